"""Layer-list ("hybrid") decoders served in their checkpoint dtype: every layer is `x += mixer(norm(x))` then optionally `x += feed_forward(norm(x))`, the mixer being
one of the registered kinds (`MIXERS`: state-space-duality recurrence, paged attention with a sliding window and kept first tokens), the feed-forward one of
`FEED_FORWARDS` (sigmoid-routed experts with a gated shared expert).  The Gekilix architecture (config.json `"architecture": "Gekilix"`) is one such list.

The step function is `HybridDecoder.forward_batch(batch)`: ONE ragged batch -- prompt portions of any length next to single decoded tokens -- through the HIP kernels of
csrc/hyb_kernels.hip and csrc/hyb_gemm.hip (C ABI, this process's current stream; PyTorch owns buffers and the stream, nothing else).  What the sequences carry between
steps lives outside the step: K / V pages addressed through the block tables of `KVCacheManager`, convolution taps and recurrent states in the slots of `StateSlotPool`
(kv_cache_manager.py).  The scheduler's engine (scheduler.PagedEngine) and the trace runner (bin/trace_run) both drive this function.

Precision: the residual stream, norms, positions and angles, attention scores / softmax / weighted sums, router scores, decays, step sizes and recurrent states are f32 in
every mode.  `dtype="bfloat16"`: weights, GEMM operands and K / V pages in bf16, f32 accumulation; `dtype="float32"`: everything f32 (the bf16 checkpoint widened exactly).
There is no CPU path: the kernels raise if libmrs_hybrid.so is missing.
"""
from __future__ import annotations

import ctypes as C
import json
import math
import os
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Sequence

import numpy as np
import torch

from . import _lib

_vp, _i, _l, _f = C.c_void_p, C.c_int32, C.c_int64, C.c_float
DTYPES = {"bfloat16": (1, torch.bfloat16), "float32": (2, torch.float32)}

_SIGS = {
    "mrs_hyb_embed": [_vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "mrs_hyb_rmsnorm": [_vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _f, _i, _i, _vp, _i, _vp],
    "mrs_hyb_conv_silu": [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "mrs_hyb_ssd_scan": [_vp] * 16 + [_i] * 10 + [_vp],
    "mrs_hyb_qk_norm_rope_cache": [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _f, _i, _vp],
    "mrs_hyb_paged_window_attn": [_vp] * 7 + [_i] * 9 + [_f, _i, _vp, _vp, _vp, _i, _i, _vp],
    "mrs_hyb_route_sigmoid_topk": [_vp, _vp, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp],
    "mrs_hyb_moe_dispatch": [_vp, _i, _i, _vp, _vp, _vp, _vp, _vp],
    "mrs_hyb_moe_gather": [_vp, _vp, _vp, _i, _vp, _i, _i, _i, _vp],
    "mrs_hyb_glu_silu": [_vp, _vp, _i, _i, _i, _vp],
    "mrs_hyb_moe_combine": [_vp, _vp, _vp, _i, _vp, _vp, _i, _i, _vp],
    "mrs_hyb_gather_rows": [_vp, _vp, _vp, _i, _i, _vp],
    "mrs_hyb_gemm": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _i, _l, _i, _vp],
    "mrs_hyb_gemv": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _l, _i, _vp, _vp, _i, _vp],
}
_fns: dict = {}
_step_stream: Optional[int] = None   # the stream handle of the step in progress (looked up once per forward_batch, not once per launch)


def _call(name: str, *args) -> None:
    """One kernel launcher of libmrs_hybrid.so on the current stream (appended as the last argument).  Tensors pass as device pointers."""
    fn = _fns.get(name)
    if fn is None:
        fn = _fns[name] = _lib.sym("hybrid", name, _SIGS[name], C.c_int)
    conv = [a.data_ptr() if isinstance(a, torch.Tensor) else a for a in args]
    if fn(*conv, _step_stream if _step_stream is not None else torch.cuda.current_stream().cuda_stream) != 0:
        err = _lib.sym("hybrid", "mrs_hyb_gemm_last_error" if "gem" in name else "mrs_hyb_last_error", [], C.c_char_p)()
        raise ValueError((err or b"").decode() or name)


# ------------------------------------------------------------------------------------------------------------------ what a step sees
@dataclass
class RaggedBatch:
    """A step's tokens as one flat row range: entry s owns rows [seq_start[s], seq_start[s + 1]) at positions seq_pos0[s] + i."""
    rows: int
    entries: int
    max_blocks: int
    tokens: torch.Tensor        # i32 [rows]
    tok_seq: torch.Tensor       # i32 [rows]  entry of the row
    tok_pos: torch.Tensor       # i32 [rows]  position in its sequence
    seq_start: torch.Tensor     # i32 [entries + 1]
    seq_pos0: torch.Tensor      # i32 [entries]  position of the entry's first row (0: the sequence starts here, its state slot counts as zero)
    seq_slot: torch.Tensor      # i32 [entries]  state slot
    block_tables: torch.Tensor  # i32 [entries, max_blocks]
    slot_mapping: torch.Tensor  # i64 [rows]  K / V page slot = block * block_size + offset
    want: torch.Tensor          # i32 [n]  rows whose logits are wanted
    # every entry's rows cut into segments of at most SEGMENT rows (linear recurrences run the segments of a long portion in parallel)
    segments: int = 0
    seg_entry: Optional[torch.Tensor] = None   # i32 [segments]
    seg_row0: Optional[torch.Tensor] = None    # i32 [segments]  first row
    seg_len: Optional[torch.Tensor] = None     # i32 [segments]
    ent_seg0: Optional[torch.Tensor] = None    # i32 [entries + 1]  first segment of every entry, then the total

    SEGMENT = int(os.environ.get("MRS_HYB_SEGMENT", "64"))   # rows per segment

    @staticmethod
    def build(entries: Sequence[dict], block_size: int, device) -> "RaggedBatch":
        """entries: dicts with `tokens`, `pos0`, `slot` (state slot or 0), `blocks` (the sequence's block ids, covering pos0 + len(tokens)), `want` (local indices)."""
        S = len(entries)
        lens = [len(e["tokens"]) for e in entries]
        T = sum(lens)
        mb = max(1, max((len(e["blocks"]) for e in entries), default=1))
        L = RaggedBatch.SEGMENT
        nseg = sum(max(1, -(-n // L)) for n in lens)
        sizes = (T, T, T, S + 1, S, S, S * mb, nseg, nseg, nseg, S + 1)
        ints = np.zeros(sum(sizes), dtype=np.int32)
        o = 0
        views = []
        for n in sizes:
            views.append(ints[o:o + n])
            o += n
        tok, tseq, tpos, sst, sp0, ssl, bt, sge, sgr, sgl, es0 = views
        z = 0
        bt = bt.reshape(S, mb)
        slots = np.zeros(T, dtype=np.int64)
        want: List[int] = []
        r = 0
        for s, e in enumerate(entries):
            n, p0 = lens[s], int(e["pos0"])
            blocks = np.asarray(e["blocks"], dtype=np.int64)
            if n and (p0 + n - 1) // block_size >= len(blocks):
                raise ValueError("RaggedBatch: the entry's blocks do not cover its last position")
            tok[r:r + n] = e["tokens"]
            tseq[r:r + n] = s
            pos = np.arange(p0, p0 + n, dtype=np.int64)
            tpos[r:r + n] = pos
            sst[s] = r
            sp0[s] = p0
            ssl[s] = int(e.get("slot") or 0)
            bt[s, :len(blocks)] = blocks
            if n:
                slots[r:r + n] = blocks[pos // block_size] * block_size + pos % block_size
            want.extend(r + int(j) for j in e.get("want", ()))
            es0[s] = z
            for a0 in range(0, max(n, 1), L):
                sge[z], sgr[z], sgl[z] = s, r + a0, min(L, n - a0)
                z += 1
            r += n
        sst[S] = T
        es0[S] = z
        dev_ints = torch.from_numpy(ints).to(device)
        o = 0
        dv = []
        for n in sizes:
            dv.append(dev_ints[o:o + n])
            o += n
        return RaggedBatch(T, S, mb, dv[0], dv[1], dv[2], dv[3], dv[4], dv[5], dv[6].view(S, mb), torch.from_numpy(slots).to(device),
                           torch.tensor(want, dtype=torch.int32, device=device), nseg, dv[7], dv[8], dv[9], dv[10])


# ------------------------------------------------------------------------------------------------------------------ layer descriptions
@dataclass
class RotarySpec:
    """Interleaved rotary on the first `dims` dimensions of a head: pair (2i, 2i + 1) turns by position * f_i, f_i = base^(-2i / dims), optionally rescaled by wavelength
    (`scaling`: factor, low, high, original -- wavelengths under original / high keep f, over original / low use f / factor, linear blend between)."""
    dims: int
    base: float
    scaling: Optional[dict] = None

    def frequencies(self) -> np.ndarray:
        i = np.arange(self.dims // 2, dtype=np.float64)
        f = np.float64(self.base) ** (-2.0 * i / self.dims)
        if self.scaling:
            fac, lo, hi, orig = (float(self.scaling[k]) for k in ("factor", "low", "high", "original"))
            wl = 2.0 * math.pi / f
            s = (orig / wl - lo) / (hi - lo)
            mid = (1.0 - s) * f / fac + s * f
            f = np.where(wl < orig / hi, f, np.where(wl > orig / lo, f / fac, mid))
        return f.astype(np.float32)


@dataclass
class AttentionSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int = 0            # 0: every earlier token
    keep_first: int = 0        # tokens at the start of the sequence that stay visible behind the window
    rotary: Optional[RotarySpec] = None
    qk_norm: bool = True       # plain-weight RMS norm over the whole query / key projection, before rotation


@dataclass
class Mamba2Spec:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state


@dataclass
class MoeSpec:
    experts: int
    top: int
    ff: int
    shared_ff: int = 0         # 0: no shared expert


@dataclass
class LayerSpec:
    kind: str
    mixer: object
    ff: Optional[MoeSpec]
    prefix: str                # tensor-name prefix of the layer


@dataclass
class HybridSpec:
    vocab: int
    width: int
    eps: float
    layers: List[LayerSpec]
    embed: str = "embed"
    final_norm: str = "final.norm"
    head: str = "head"


def gekilix_spec(cfg: dict) -> HybridSpec:
    """config.json of a Gekilix checkpoint -> the layer list.  Every size and every model-dependent constant comes from the file."""
    layers = []
    for i, L in enumerate(cfg["layers"]):
        m = L["mixer"]
        if L["type"] == "mamba2":
            mixer = Mamba2Spec(int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"]), int(m["conv"]), int(m.get("norm_groups", 1)))
        elif L["type"] == "attention":
            rot = m.get("rot")
            mask = m.get("mask") or {}
            mixer = AttentionSpec(int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), float(m["scale"]), int(mask.get("size", 0) or 0),
                                  int(mask.get("keep_first", 0) or 0),
                                  RotarySpec(int(rot["dims"]), float(rot["base"]), rot.get("scaling")) if rot and int(rot.get("dims", 0)) > 0 else None)
        else:
            raise ValueError(f"Gekilix: unknown layer type {L['type']!r}")
        f = L.get("mlp")
        ff = None
        if f:
            if f.get("kind", "moe") != "moe":
                raise ValueError(f"Gekilix: unknown feed-forward kind {f.get('kind')!r}")
            sh = f.get("shared")
            ff = MoeSpec(int(f["router"]["experts"]), int(f["router"]["top"]), int(f["expert"]["ff"]), int(sh["ff"]) if sh else 0)
        layers.append(LayerSpec(L["type"], mixer, ff, f"l{i}."))
    return HybridSpec(int(cfg["vocab"]), int(cfg["width"]), float(cfg["norm"]["eps"]), layers)


# ------------------------------------------------------------------------------------------------------------------ mixers and feed-forwards
class _Module:
    def __init__(self, model: "HybridDecoder"):
        self.m = model

    def w(self, get, name, gemm: bool):
        """A checkpoint tensor on the device: GEMM operands in the serving dtype, everything else f32."""
        t = get(name)
        return t.to(self.m.device, self.m.torch_dtype if gemm else torch.float32).contiguous()


class Mamba2Mixer(_Module):
    """in-projection -> [z | x | B | C | dt]; causal convolution + SiLU over x, B, C; dt = softplus(dt + bias); per head S <- exp(-exp(A_log) dt) S + dt B x^T,
    y = S^T C + D x; y * silu(z); RMS norm in `norm_groups` parts; out-projection.  Carries the last conv - 1 inputs and S (f32) per sequence slot."""

    def __init__(self, model, spec: Mamba2Spec, prefix: str):
        super().__init__(model)
        self.s, self.p = spec, prefix
        if spec.inner % spec.norm_groups or spec.heads % spec.groups:
            raise ValueError("mamba2: heads % groups and (heads * vdim) % norm_groups must be 0")
        slots, dev = model.state_slots, model.device
        self.conv_state = torch.zeros(slots, spec.conv_channels, max(spec.conv - 1, 1), dtype=torch.float32, device=dev)
        self.ssm_state = torch.zeros(slots, spec.heads, spec.state, spec.vdim, dtype=torch.float32, device=dev)

    def load(self, get):
        s, p = self.s, self.p
        self.w_in, self.w_o = self.w(get, p + "in", True), self.w(get, p + "o", True)
        self.conv_w, self.conv_b = self.w(get, p + "conv", False), self.w(get, p + "conv.b", False)
        self.dt_bias, self.A_log, self.D, self.norm = (self.w(get, p + n, False) for n in ("dt_bias", "A_log", "D", "norm"))
        n_in = 2 * s.inner + 2 * s.groups * s.state + s.heads
        if tuple(self.w_in.shape) != (n_in, self.m.spec.width) or tuple(self.conv_w.shape) != (s.conv_channels, s.conv):
            raise ValueError(f"{p}: tensor shapes do not match the mixer's sizes")

    def forward(self, h, x, b: RaggedBatch):
        s, m = self.s, self.m
        T = b.rows
        u = m.linear(h, self.w_in)                                         # f32 [T, z | x B C | dt]
        xbc = torch.empty(T, s.conv_channels, dtype=torch.float32, device=m.device)
        _call("mrs_hyb_conv_silu", u[:, s.inner:], u.stride(0), self.conv_w, self.conv_b, self.conv_state, b.tok_seq, b.seq_start, b.seq_pos0, b.seq_slot, xbc,
              T, b.entries, s.conv_channels, s.conv)
        y = torch.empty(T, s.inner, dtype=torch.float32, device=m.device)
        steps = torch.empty(T, s.heads, 2, dtype=torch.float32, device=m.device)
        carry = decay = None
        if b.segments > b.entries:   # some portion is longer than a segment: scratch for the segments' local end states
            carry = torch.empty(b.segments, s.heads, s.state, s.vdim, dtype=torch.float32, device=m.device)
            decay = torch.empty(b.segments, s.heads, dtype=torch.float32, device=m.device)
        _call("mrs_hyb_ssd_scan", xbc, u, self.dt_bias, self.A_log, self.D, self.ssm_state, y, b.seq_pos0, b.seq_slot, b.seg_entry, b.seg_row0, b.seg_len, b.ent_seg0,
              steps, carry, decay, T, b.entries, b.segments, s.conv_channels, u.stride(0), s.inner + s.conv_channels, s.heads, s.vdim, s.state, s.groups)
        yn = m.norm(y, self.norm, one_plus=False, parts=s.norm_groups, gate=u)   # y * silu(z) (z = the first `inner` columns of u), then the grouped norm
        m.linear(yn, self.w_o, out=x, accumulate=True)

    def state_bytes_per_slot(self) -> int:
        return 4 * (self.conv_state[0].numel() + self.ssm_state[0].numel())


class WindowAttention(_Module):
    """q, k, v projections (one product); plain-weight RMS norm over the WHOLE query and key projections; interleaved rotary on the first dims of every head; K / V into
    pages; softmax over the keys j <= i with i - j < window or j < keep_first (true positions throughout); out-projection.  Grouped heads: query head h reads key / value
    head h // (heads / kv_heads); key and value head sizes are independent."""

    def __init__(self, model, spec: AttentionSpec, prefix: str):
        super().__init__(model)
        self.s, self.p = spec, prefix
        dev, bs, nb = model.device, model.block_size, model.num_blocks
        self.k_cache = torch.zeros(nb, spec.kv_heads, bs, spec.dim, dtype=model.torch_dtype, device=dev)
        self.v_cache = torch.zeros(nb, spec.kv_heads, bs, spec.vdim, dtype=model.torch_dtype, device=dev)
        self.freq = torch.from_numpy(spec.rotary.frequencies()).to(dev) if spec.rotary else torch.zeros(1, dtype=torch.float32, device=dev)

    def load(self, get):
        s, p = self.s, self.p
        q, k, v = (get(p + n) for n in ("q", "k", "v"))
        if q.shape[0] != s.heads * s.dim or k.shape[0] != s.kv_heads * s.dim or v.shape[0] != s.kv_heads * s.vdim:
            raise ValueError(f"{p}: projection shapes do not match the mixer's sizes")
        self.w_qkv = torch.cat([q, k, v], 0).to(self.m.device, self.m.torch_dtype).contiguous()
        self.w_o = self.w(get, p + "o", True)
        self.q_norm = self.w(get, p + "q.norm", False) if s.qk_norm else None
        self.k_norm = self.w(get, p + "k.norm", False) if s.qk_norm else None

    def forward(self, h, x, b: RaggedBatch):
        s, m = self.s, self.m
        T = b.rows
        qkv = m.linear(h, self.w_qkv)
        q = torch.empty(T, s.heads * s.dim, dtype=m.torch_dtype, device=m.device)
        _call("mrs_hyb_qk_norm_rope_cache", qkv, qkv.stride(0), self.q_norm, self.k_norm, self.freq, b.tok_pos, b.slot_mapping, q, self.k_cache, self.v_cache, T,
              s.heads, s.kv_heads, s.dim, s.vdim, s.rotary.dims if s.rotary else 0, m.block_size, m.spec.eps, m.dt)
        o = torch.empty(T, s.heads * s.vdim, dtype=m.torch_dtype, device=m.device)
        _call("mrs_hyb_paged_window_attn", q, self.k_cache, self.v_cache, b.block_tables, b.tok_seq, b.tok_pos, o, T, s.heads, s.kv_heads, s.dim, s.vdim, m.block_size,
              b.max_blocks, s.window, s.keep_first, s.scale, m.dt, b.seg_entry, b.seg_row0, b.seg_len, b.segments, RaggedBatch.SEGMENT)
        m.linear(o, self.w_o, out=x, accumulate=True)


class SigmoidMoe(_Module):
    """Router logits in f32, scores = sigmoid, the `top` largest, un-renormalised; the score multiplies the expert's INPUT: out = sum_e expert_e(s_e h), expert =
    down(silu(gate h) * (up h)); plus sigmoid(sg . h) * shared(h).  All experts of a step run as grouped products over expert-sorted rows."""

    def __init__(self, model, spec: MoeSpec, prefix: str):
        super().__init__(model)
        self.s, self.p = spec, prefix

    def load(self, get):
        s, p, m = self.s, self.p, self.m
        dev, dt = m.device, m.torch_dtype
        self.w_gu = torch.stack([torch.cat([get(f"{p}e{e}.gate"), get(f"{p}e{e}.up")], 0) for e in range(s.experts)]).to(dev, dt).contiguous()   # [E, 2 ff, W]
        self.w_down = torch.stack([get(f"{p}e{e}.down") for e in range(s.experts)]).to(dev, dt).contiguous()                                      # [E, W, ff]
        if tuple(self.w_gu.shape[1:]) != (2 * s.ff, m.spec.width):
            raise ValueError(f"{p}: expert shapes do not match the layer's sizes")
        rows = [get(p + "router")]
        if s.shared_ff:
            rows.append(get(p + "shared.sg").reshape(1, -1))
            self.ws_gu = torch.cat([get(p + "shared.gate"), get(p + "shared.up")], 0).to(dev, dt).contiguous()
            self.ws_down = self.w(get, p + "shared.down", True)
        self.w_router = torch.cat(rows, 0).to(dev, torch.float32).contiguous()   # [E (+ 1), W] f32: router rows, then the shared expert's gate row

    def forward(self, h, h32, x, b: RaggedBatch):
        s, m = self.s, self.m
        T, W, dev = b.rows, m.spec.width, m.device
        R = T * s.top
        ids = torch.empty(R, dtype=torch.int32, device=dev)
        wts = torch.empty(R, dtype=torch.float32, device=dev)
        gate = torch.empty(T, dtype=torch.float32, device=dev) if s.shared_ff else None
        _call("mrs_hyb_route_sigmoid_topk", h32, self.w_router, T, W, s.experts, s.top, int(bool(s.shared_ff)), ids, wts, gate)
        meta = torch.empty(s.experts + 1 + 3 * R, dtype=torch.int32, device=dev)
        bounds, sorted_route, route_pos, sorted_expert = meta[:s.experts + 1], meta[s.experts + 1:][:R], meta[s.experts + 1 + R:][:R], meta[s.experts + 1 + 2 * R:][:R]
        _call("mrs_hyb_moe_dispatch", ids, R, s.experts, bounds, sorted_route, route_pos, sorted_expert)
        f32 = dict(dtype=torch.float32, device=dev)
        if R <= m.GROUPED_GEMV_ROWS:
            # decode-sized steps: every route streams its expert's slabs; the scaled gather and the GLU happen in the consuming product's operand load (same roundings)
            gu = torch.empty(R, 2 * s.ff, **f32)
            _call("mrs_hyb_gemv", h32, self.w_gu, gu, R, 2 * s.ff, W, h32.stride(0), W, 2 * s.ff, m.dt, 0, sorted_expert, self.w_gu.stride(0), 2, sorted_route, wts, s.top)
            d = torch.empty(R, W, **f32)
            _call("mrs_hyb_gemv", gu, self.w_down, d, R, W, s.ff, 2 * s.ff, s.ff, W, m.dt, 0, sorted_expert, self.w_down.stride(0), 1, None, None, 1)
        else:
            xs = torch.empty(R, W, dtype=m.torch_dtype, device=dev)
            _call("mrs_hyb_moe_gather", h32, sorted_route, wts, s.top, xs, R, W, m.dt)
            gu = m.grouped_linear(xs, self.w_gu, bounds, sorted_expert)
            act = torch.empty(R, s.ff, dtype=m.torch_dtype, device=dev)
            _call("mrs_hyb_glu_silu", gu, act, R, s.ff, m.dt)
            d = m.grouped_linear(act, self.w_down, bounds, sorted_expert)
        sh = None
        if s.shared_ff:
            sgu = m.linear(h, self.ws_gu)
            if T <= m.GEMV_ROWS:
                sh = torch.empty(T, W, **f32)
                _call("mrs_hyb_gemv", sgu, self.ws_down, sh, T, W, s.shared_ff, 2 * s.shared_ff, s.shared_ff, W, m.dt, 0, None, 0, 1, None, None, 1)
            else:
                sact = torch.empty(T, s.shared_ff, dtype=m.torch_dtype, device=dev)
                _call("mrs_hyb_glu_silu", sgu, sact, T, s.shared_ff, m.dt)
                sh = m.linear(sact, self.ws_down)
        _call("mrs_hyb_moe_combine", x, d, route_pos, s.top, sh, gate, T, W)


MIXERS: Dict[str, Callable] = {"mamba2": Mamba2Mixer, "attention": WindowAttention}
FEED_FORWARDS: Dict[str, Callable] = {"moe": SigmoidMoe}


class _Layer:
    def __init__(self, model, ls: LayerSpec):
        self.spec = ls
        self.mixer = MIXERS[ls.kind](model, ls.mixer, ls.prefix + "mix.")
        self.ff = FEED_FORWARDS["moe"](model, ls.ff, ls.prefix + "mlp.") if ls.ff else None
        self.norm1 = self.norm2 = None


# ------------------------------------------------------------------------------------------------------------------ the model
class HybridDecoder:
    """`num_blocks` K / V pages of `block_size` tokens per attention layer and `state_slots` recurrent-state slots per state-space layer; which sequence uses which is
    the cache managers' business (KVCacheManager / StateSlotPool), the model only follows the tables in the batch."""

    GEMV_ROWS = 8          # at most this many rows share one streamed weight pass
    GROUPED_GEMV_ROWS = 32 # expert-sorted rows up to which every row streams its own expert slab

    def __init__(self, spec: HybridSpec, device, dtype: str = "bfloat16", num_blocks: int = 64, block_size: int = 32, state_slots: int = 4):
        if dtype not in DTYPES:
            raise ValueError(f"dtype must be one of {sorted(DTYPES)}")
        _lib.load("hybrid")
        self.spec, self.device, self.dtype = spec, torch.device(device), dtype
        self.dt, self.torch_dtype = DTYPES[dtype]
        self.num_blocks, self.block_size, self.state_slots = int(num_blocks), int(block_size), int(state_slots)
        self.layers = [_Layer(self, ls) for ls in spec.layers]
        self.trace_layers: Optional[list] = None   # set to a list: forward_batch appends the residual stream after every layer (debugging / tests)

    # ---- construction
    @property
    def has_recurrent_state(self) -> bool:
        return any(isinstance(l.mixer, Mamba2Mixer) for l in self.layers)

    @property
    def has_paged_kv(self) -> bool:
        return any(isinstance(l.mixer, WindowAttention) for l in self.layers)

    def load_weights(self, get: Callable[[str], torch.Tensor]) -> None:
        sp = self.spec
        f32 = lambda n: get(n).to(self.device, torch.float32).contiguous()
        self.embed = get(sp.embed).to(self.device, self.torch_dtype).contiguous()
        self.head = get(sp.head).to(self.device, self.torch_dtype).contiguous()
        self.final_norm = f32(sp.final_norm)
        if tuple(self.embed.shape) != (sp.vocab, sp.width) or tuple(self.head.shape) != (sp.vocab, sp.width):
            raise ValueError("embedding / head shapes do not match vocab x width")
        for l in self.layers:
            l.norm1 = f32(l.spec.prefix + "norm1")
            l.mixer.load(get)
            if l.ff:
                l.norm2 = f32(l.spec.prefix + "norm2")
                l.ff.load(get)

    @classmethod
    def from_pretrained(cls, path: str, device, dtype: str = "bfloat16", **kw) -> "HybridDecoder":
        """`path`: a folder with config.json and model.safetensors."""
        from safetensors import safe_open
        with open(os.path.join(path, "config.json")) as f:
            cfg = json.load(f)
        model = cls(SPEC_READERS[cfg["architecture"]](cfg), device, dtype, **kw)
        with safe_open(os.path.join(path, "model.safetensors"), "pt") as st:
            model.load_weights(st.get_tensor)
        return model

    # ---- building blocks on the current stream
    def norm(self, x, w, one_plus: bool, parts: int = 1, want32: bool = False, gate=None):
        """RMS norm of every row (in `parts` equal pieces); gate [rows, >= width]: the row is multiplied by silu(gate) first."""
        rows, width = x.shape
        out = torch.empty(rows, width, dtype=self.torch_dtype, device=self.device)
        out32 = torch.empty(rows, width, dtype=torch.float32, device=self.device) if want32 else None
        _call("mrs_hyb_rmsnorm", x, x.stride(0), w, out, out32, None, rows, width, parts, self.spec.eps, int(one_plus), self.dt, gate, gate.stride(0) if gate is not None else 0)
        return (out, out32) if want32 else out

    def linear(self, a, w, out=None, accumulate: bool = False, dtype_code: Optional[int] = None):
        """out (f32 [M, N]) (+)= a [M, K] . w [N, K]^T"""
        M, K = a.shape
        N = w.shape[0]
        if out is None:
            out = torch.empty(M, N, dtype=torch.float32, device=self.device)
        dt = dtype_code or self.dt
        if M <= self.GEMV_ROWS:
            _call("mrs_hyb_gemv", a, w, out, M, N, K, a.stride(0), w.stride(0), out.stride(0), dt, int(accumulate), None, 0, 0, None, None, 1)
        else:
            _call("mrs_hyb_gemm", a, w, out, M, N, K, a.stride(0), w.stride(0), out.stride(0), dt, int(accumulate), None, 0, 0, 0)
        return out

    def grouped_linear(self, a, w, bounds, sorted_expert):
        """a [R, K] rows sorted by group, w [groups, N, K]: row r multiplies the slab of its group."""
        R, K = a.shape
        E, N = w.shape[0], w.shape[1]
        out = torch.empty(R, N, dtype=torch.float32, device=self.device)
        if R <= self.GROUPED_GEMV_ROWS:
            _call("mrs_hyb_gemv", a, w, out, R, N, K, a.stride(0), w.stride(1), out.stride(0), self.dt, 0, sorted_expert, w.stride(0), 0, None, None, 1)
        else:
            _call("mrs_hyb_gemm", a, w, out, R, N, K, a.stride(0), w.stride(1), out.stride(0), self.dt, 0, bounds, E, w.stride(0), R)
        return out

    # ---- the step
    def forward_batch(self, b: RaggedBatch) -> torch.Tensor:
        """Runs the batch's rows from the cache and state that earlier steps left; returns f32 logits [len(want), vocab] in the order of `want`."""
        global _step_stream
        _step_stream = torch.cuda.current_stream().cuda_stream
        try:
            return self._forward_batch(b)
        finally:
            _step_stream = None

    def _forward_batch(self, b: RaggedBatch) -> torch.Tensor:
        sp = self.spec
        T = b.rows
        if T == 0:
            return torch.empty(0, sp.vocab, dtype=torch.float32, device=self.device)
        x = torch.empty(T, sp.width, dtype=torch.float32, device=self.device)
        _call("mrs_hyb_embed", b.tokens, self.embed, x, T, sp.width, sp.vocab, self.dt)
        for l in self.layers:
            l.mixer.forward(self.norm(x, l.norm1, one_plus=True), x, b)
            if l.ff:
                h, h32 = self.norm(x, l.norm2, one_plus=True, want32=True)
                l.ff.forward(h, h32, x, b)
            if self.trace_layers is not None:
                self.trace_layers.append(x.clone())
        n = b.want.numel()
        if n == 0:
            return torch.empty(0, sp.vocab, dtype=torch.float32, device=self.device)
        xs = torch.empty(n, sp.width, dtype=torch.float32, device=self.device)
        _call("mrs_hyb_gather_rows", x, b.want, xs, n, sp.width)
        return self.linear(self.norm(xs, self.final_norm, one_plus=True), self.head)

    # ---- decode steps as a HIP graph
    def capture_decode(self, entries: int, max_blocks: int) -> "DecodeGraph":
        """One decode step for `entries` sequences (one row each), captured into a HIP graph over static batch buffers: replays cost one launch instead of one per kernel."""
        return DecodeGraph(self, entries, max_blocks)

    # ---- sizes
    def kv_bytes_per_token(self) -> int:
        e = 2 if self.dtype == "bfloat16" else 4
        return sum(e * l.mixer.s.kv_heads * (l.mixer.s.dim + l.mixer.s.vdim) for l in self.layers if isinstance(l.mixer, WindowAttention))

    def state_bytes_per_slot(self) -> int:
        return sum(l.mixer.state_bytes_per_slot() for l in self.layers if isinstance(l.mixer, Mamba2Mixer))


class DecodeGraph:
    """A captured decode step (role of pipeline/cuda_graph.rs in the reference): the batch description lives in static device buffers that `replay` refreshes with two
    small host -> device copies; every kernel argument besides those buffers (row counts, table width) is fixed at capture.  Logits of all rows come back as a view of a
    static buffer: consume them before the next replay."""

    def __init__(self, model: HybridDecoder, entries: int, max_blocks: int):
        self.m, self.n, self.mb = model, int(entries), int(max_blocks)
        dev, n, mb = model.device, self.n, self.mb
        self._ints = torch.zeros(3 * n + (n + 1) + 2 * n + n * mb, dtype=torch.int32, device=dev)
        self._slots = torch.zeros(n, dtype=torch.int64, device=dev)
        v, o = [], 0
        for k in (n, n, n, n + 1, n, n, n * mb):
            v.append(self._ints[o:o + k])
            o += k
        rows = torch.arange(n + 1, dtype=torch.int32, device=dev)   # one row = one segment per entry
        self.batch = RaggedBatch(n, n, mb, v[0], v[1], v[2], v[3], v[4], v[5], v[6].view(n, mb), self._slots, rows[:n].clone(), n, rows[:n], rows[:n],
                                 torch.ones(n, dtype=torch.int32, device=dev), rows)
        self._host = np.zeros(self._ints.numel(), dtype=np.int32)
        self._host[3 * n:3 * n + n + 1] = np.arange(n + 1)          # seq_start: one row per entry
        self._host[2 * n:3 * n] = 1                                  # positions >= 1 during warm-up: the slots' states are read, nothing is reset
        self._host[n:2 * n] = np.arange(n)                           # tok_seq
        self._ints.copy_(torch.from_numpy(self._host))
        # warm-up outside capture (lazy module loads).  It really runs -- on state slot 0 and page slot 0, which may belong to a live sequence: put both back afterwards
        keep = []
        for l in model.layers:
            mx = l.mixer
            keep += [(t, t[0].clone()) for t in ((mx.conv_state, mx.ssm_state) if isinstance(mx, Mamba2Mixer) else (mx.k_cache, mx.v_cache))]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            model.forward_batch(self.batch)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        for t, saved in keep:
            t[0].copy_(saved)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.logits = model.forward_batch(self.batch)

    def replay(self, entries: Sequence[dict]) -> torch.Tensor:
        """entries as for RaggedBatch.build, one token each (`pos0` = the token's position)."""
        n, mb, h = self.n, self.mb, self._host
        if len(entries) != n:
            raise ValueError(f"DecodeGraph: captured for {n} sequences, got {len(entries)}")
        slots = np.zeros(n, dtype=np.int64)
        bt = h[3 * n + (n + 1) + 2 * n:].reshape(n, mb)
        bs = self.m.block_size
        for s, e in enumerate(entries):
            p, blocks = int(e["pos0"]), e["blocks"]
            if len(e["tokens"]) != 1 or len(blocks) > mb or p // bs >= len(blocks):
                raise ValueError("DecodeGraph: one token per entry, its page inside the captured table width")
            h[s], h[2 * n + s] = e["tokens"][0], p
            h[3 * n + (n + 1) + s], h[3 * n + (n + 1) + n + s] = p, int(e.get("slot") or 0)
            bt[s, :len(blocks)] = blocks
            slots[s] = blocks[p // bs] * bs + p % bs
        self._ints.copy_(torch.from_numpy(h))
        self._slots.copy_(torch.from_numpy(slots))
        self.graph.replay()
        return self.logits


def synthetic_weights(spec: HybridSpec, device, seed: int = 0) -> Callable[[str], torch.Tensor]:
    """`get(name)` for HybridDecoder.load_weights that draws every tensor on the device when it is asked for (benchmarks: there is no network for checkpoints).
    Projections N(0, 1 / fan_in), norm weights around their neutral value, decays and step sizes in the range trained state-space models use."""
    W = spec.width
    g = torch.Generator(device=device).manual_seed(seed)
    shapes: Dict[str, tuple] = {spec.embed: (spec.vocab, W), spec.head: (spec.vocab, W), spec.final_norm: (W,)}
    for ls in spec.layers:
        p, m = ls.prefix, ls.mixer
        shapes[p + "norm1"] = (W,)
        if isinstance(m, Mamba2Spec):
            shapes.update({p + "mix.in": (2 * m.inner + 2 * m.groups * m.state + m.heads, W), p + "mix.conv": (m.conv_channels, m.conv), p + "mix.conv.b": (m.conv_channels,),
                           p + "mix.dt_bias": (m.heads,), p + "mix.A_log": (m.heads,), p + "mix.D": (m.heads,), p + "mix.norm": (m.inner,), p + "mix.o": (W, m.inner)})
        else:
            shapes.update({p + "mix.q": (m.heads * m.dim, W), p + "mix.k": (m.kv_heads * m.dim, W), p + "mix.v": (m.kv_heads * m.vdim, W), p + "mix.q.norm": (m.heads * m.dim,),
                           p + "mix.k.norm": (m.kv_heads * m.dim,), p + "mix.o": (W, m.heads * m.vdim)})
        if ls.ff:
            f = ls.ff
            shapes[p + "norm2"], shapes[p + "mlp.router"] = (W,), (f.experts, W)
            for e in range(f.experts):
                shapes.update({f"{p}mlp.e{e}.gate": (f.ff, W), f"{p}mlp.e{e}.up": (f.ff, W), f"{p}mlp.e{e}.down": (W, f.ff)})
            if f.shared_ff:
                shapes.update({p + "mlp.shared.gate": (f.shared_ff, W), p + "mlp.shared.up": (f.shared_ff, W), p + "mlp.shared.down": (W, f.shared_ff), p + "mlp.shared.sg": (1, W)})

    def get(name: str) -> torch.Tensor:
        shape = shapes[name]
        r = torch.randn(*shape, device=device, generator=g)
        last = name.rsplit(".", 1)[-1]
        if name.endswith(("q.norm", "k.norm")) or last == "D" or name.endswith("mix.norm"):
            r = 1.0 + 0.1 * r
        elif last in ("norm1", "norm2") or name == spec.final_norm:
            r = 0.1 * r
        elif last == "dt_bias":
            r = -2.0 + 0.5 * r
        elif last == "A_log":
            r = 0.5 * r
        elif last == "b":
            r = 0.1 * r
        elif last == "conv":
            r = 0.4 * r
        elif name != spec.embed:
            r = r * (shape[-1] ** -0.5)
        return r.to(torch.bfloat16)
    return get


SPEC_READERS: Dict[str, Callable[[dict], HybridSpec]] = {"Gekilix": gekilix_spec}


class HybridCache:
    """What live sequences hold between steps, for a HybridDecoder: K / V blocks from the paged `KVCacheManager` and one state slot each from `StateSlotPool`.
    `reserve` grows a request to `total_tokens` (admitting it on first use), `entry` describes its next rows for `RaggedBatch.build`, `release` gives everything back.
    Prefix caching stays off when the model has recurrent layers: a cached K / V block does not bring the recurrent state of its last token with it."""

    def __init__(self, model: HybridDecoder, enable_prefix_caching: bool = False):
        from .kv_cache_manager import KVCacheManager, StateSlotPool
        self.model = model
        self.kv = KVCacheManager(model.num_blocks, model.block_size, enable_prefix_caching and not model.has_recurrent_state, [0])
        self.slots = StateSlotPool(model.state_slots)

    def reserve(self, request_id: int, total_tokens: int) -> bool:
        if self.slots.allocate(request_id) is None:
            return False
        if self.kv.allocate_slots(request_id, total_tokens, []) is None:
            if not self.kv.has_request(request_id):
                self.slots.free(request_id)
            return False
        return True

    def entry(self, request_id: int, tokens: Sequence[int], pos0: int, want: Sequence[int] = ()) -> dict:
        return {"tokens": list(tokens), "pos0": pos0, "slot": self.slots.slot_of(request_id), "blocks": self.kv.get_block_ids(request_id) or [], "want": list(want)}

    def release(self, request_id: int) -> None:
        self.kv.free(request_id)
        self.slots.free(request_id)
