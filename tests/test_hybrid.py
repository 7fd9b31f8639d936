"""Layer-list decoders (mistralrs_amd.hybrid, csrc/hyb_*.hip) against the plain float64 restatement in tests/hybrid_oracle.py.

Every test builds its own small configuration with random bf16-representable weights (so the bf16 and the all-f32 serving modes read identical numbers).  The sharp
comparisons run in the f32 mode (a wrong key, a window one token off or a lost state is an O(1) error there, rounding is 1e-6); the bf16 mode is held to a rounding-sized bar.
CPU tests cover what needs no device: the state slot pool, the batch description, the config reader, the scheduler with state slots.
"""
import copy
import json
import math
import os

import numpy as np
import pytest
import torch

import mistralrs_amd  # noqa: F401
from mistralrs_amd import _lib
from tests import hybrid_oracle as O

HYB = os.path.exists(_lib.path("hybrid"))
needs_lib = pytest.mark.skipif(not HYB, reason="libmrs_hybrid.so not built (python mistral.rs_amd/build.py --only libmrs_hybrid.so)")


# ---------------------------------------------------------------------------------------------------------------- configurations and weights
def attn_layer(heads=4, kv_heads=2, dim=16, vdim=8, size=12, keep=2, rot=8, scaling=True, mlp=True, experts=5, top=2, ff=24, shared=16):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": 1.0 / math.sqrt(dim), "mask": {"size": size, "keep_first": keep}}
    if rot:
        m["rot"] = {"dims": rot, "base": 10000.0}
        if scaling:
            m["rot"]["scaling"] = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}
    return {"type": "attention", "mixer": m, "mlp": moe(experts, top, ff, shared) if mlp else None}


def mamba_layer(heads=4, vdim=8, state=12, groups=2, conv=4, norm_groups=2, mlp=True, experts=5, top=2, ff=24, shared=16):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups},
            "mlp": moe(experts, top, ff, shared) if mlp else None}


def moe(experts, top, ff, shared):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}, "shared": {"ff": shared} if shared else None}


def config(layers, vocab=96, width=40, eps=1e-5):
    return {"architecture": "Gekilix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


def weights(cfg, seed=0, peaky=3.0):
    """name -> bf16 tensor.  `peaky` scales the query norm weights so that single keys carry visible softmax mass."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    w = {}

    def rnd(*shape, scale=1.0, shift=0.0):
        return (torch.randn(*shape, generator=g) * scale + shift).to(torch.bfloat16)
    w["embed"], w["head"], w["final.norm"] = rnd(cfg["vocab"], W), rnd(cfg["vocab"], W, scale=W ** -0.5), rnd(W, scale=0.1)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        w[p + "norm1"] = rnd(W, scale=0.1)
        if L["type"] == "mamba2":
            inner, gn = m["heads"] * m["vdim"], m["groups"] * m["state"]
            w[p + "mix.in"] = rnd(2 * inner + 2 * gn + m["heads"], W, scale=W ** -0.5)
            w[p + "mix.conv"], w[p + "mix.conv.b"] = rnd(inner + 2 * gn, m["conv"], scale=0.4), rnd(inner + 2 * gn, scale=0.1)
            w[p + "mix.dt_bias"] = rnd(m["heads"], scale=0.5, shift=-1.0)
            w[p + "mix.A_log"] = rnd(m["heads"], scale=0.5, shift=-0.5)
            w[p + "mix.D"] = rnd(m["heads"], scale=0.3, shift=1.0)
            w[p + "mix.norm"] = rnd(inner, scale=0.2, shift=1.0)
            w[p + "mix.o"] = rnd(W, inner, scale=inner ** -0.5)
        else:
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            w[p + "mix.q"], w[p + "mix.k"], w[p + "mix.v"] = rnd(H * D, W, scale=W ** -0.5), rnd(G * D, W, scale=W ** -0.5), rnd(G * Dv, W, scale=W ** -0.5)
            w[p + "mix.q.norm"], w[p + "mix.k.norm"] = rnd(H * D, scale=0.2, shift=peaky), rnd(G * D, scale=0.2, shift=1.0)
            w[p + "mix.o"] = rnd(W, H * Dv, scale=(H * Dv) ** -0.5)
        f = L.get("mlp")
        if f:
            w[p + "norm2"] = rnd(W, scale=0.1)
            ff = f["expert"]["ff"]
            for e in range(f["router"]["experts"]):
                w[f"{p}mlp.e{e}.gate"], w[f"{p}mlp.e{e}.up"], w[f"{p}mlp.e{e}.down"] = rnd(ff, W, scale=W ** -0.5), rnd(ff, W, scale=W ** -0.5), rnd(W, ff, scale=ff ** -0.5)
            w[p + "mlp.router"] = rnd(f["router"]["experts"], W, scale=2.0 * W ** -0.5)
            if f.get("shared"):
                sf = f["shared"]["ff"]
                w[p + "mlp.shared.gate"], w[p + "mlp.shared.up"], w[p + "mlp.shared.down"] = rnd(sf, W, scale=W ** -0.5), rnd(sf, W, scale=W ** -0.5), rnd(W, sf, scale=sf ** -0.5)
                w[p + "mlp.shared.sg"] = rnd(1, W, scale=W ** -0.5)
    return w


def f64(w):
    return {k: v.to(torch.float64) for k, v in w.items()}


MIXED = [mamba_layer(), attn_layer(), mamba_layer(norm_groups=1, groups=4, top=1, shared=0), attn_layer(kv_heads=4, vdim=16, keep=0, size=7, rot=16, scaling=False, top=1)]


class Served:
    """A model on the device with its caches, stepped the way the engine and the trace runner step it."""

    def __init__(self, cfg, w, dev, dtype="float32", max_tokens=512, slots=4, block_size=32):
        from mistralrs_amd.hybrid import HybridCache, HybridDecoder, gekilix_spec
        self.bs = block_size
        self.m = HybridDecoder(gekilix_spec(cfg), dev, dtype, num_blocks=-(-max_tokens // block_size) + slots + 1, block_size=block_size, state_slots=slots)
        self.m.load_weights(w.__getitem__)
        self.cache = HybridCache(self.m)
        self.len = {}

    def step(self, parts):
        """parts: [(request id, tokens)]; logits of every row, split per part"""
        from mistralrs_amd.hybrid import RaggedBatch
        entries = []
        for rid, toks in parts:
            p0 = self.len.get(rid, 0)
            assert self.cache.reserve(rid, p0 + len(toks)), "out of pages / slots"
            entries.append(self.cache.entry(rid, toks, p0, range(len(toks))))
            self.len[rid] = p0 + len(toks)
        out = self.m.forward_batch(RaggedBatch.build(entries, self.bs, self.m.device)).double().cpu()
        res, r = [], 0
        for _, toks in parts:
            res.append(out[r:r + len(toks)])
            r += len(toks)
        return res

    def end(self, rid):
        self.cache.release(rid)
        self.len.pop(rid, None)


def rel(a, b):
    return float((a - b).norm() / (b.norm() + 1e-30))


def close(a, b, bar):
    """f32 mode (bar < 1e-3): the whole tensor within `bar`.  bf16 mode: rounding can move a router's close call in these narrow models, which changes single rows by
    much more than rounding does -- so the typical row is held to `bar` and at most one row in ten may exceed five times that."""
    if bar < 1e-3:
        return rel(a, b) < bar
    rows = (a - b).reshape(-1, a.shape[-1]).norm(dim=1) / (b.reshape(-1, b.shape[-1]).norm(dim=1) + 1e-30)
    return float(rows.median()) < bar and float((rows > 5 * bar).double().mean()) <= 0.1


def toks(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


# ---------------------------------------------------------------------------------------------------------------- host-side pieces (no GPU)
@needs_lib
def test_state_slot_pool_reuses_slots():
    from mistralrs_amd.kv_cache_manager import StateSlotPool
    p = StateSlotPool(3)
    assert p.capacity() == 3 and p.num_free_slots() == 3
    a, b, c = p.allocate(10), p.allocate(11), p.allocate(12)
    assert sorted((a, b, c)) == [0, 1, 2] and p.allocate(13) is None and p.num_free_slots() == 0
    assert p.allocate(11) == b and p.slot_of(11) == b and p.slot_of(99) is None
    p.free(11)
    p.free(11)  # idempotent
    assert p.num_free_slots() == 1 and p.allocate(13) == b  # the freed slot is the next one out
    p.free(10); p.free(12); p.free(13)
    assert p.num_free_slots() == 3


def test_ragged_batch_description():
    from mistralrs_amd.hybrid import RaggedBatch
    b = RaggedBatch.build([{"tokens": [5, 6, 7], "pos0": 30, "slot": 2, "blocks": [4, 9], "want": [0, 2]},
                           {"tokens": [8], "pos0": 0, "slot": 0, "blocks": [1], "want": [0]}], 32, "cpu")
    assert b.rows == 4 and b.entries == 2 and b.max_blocks == 2
    assert b.tok_seq.tolist() == [0, 0, 0, 1] and b.tok_pos.tolist() == [30, 31, 32, 0] and b.seq_start.tolist() == [0, 3, 4]
    assert b.seq_pos0.tolist() == [30, 0] and b.seq_slot.tolist() == [2, 0]
    assert b.slot_mapping.tolist() == [4 * 32 + 30, 4 * 32 + 31, 9 * 32 + 0, 1 * 32 + 0]  # the third row crosses into the second page
    assert b.block_tables.tolist() == [[4, 9], [1, 0]] and b.want.tolist() == [0, 2, 3]
    with pytest.raises(ValueError):
        RaggedBatch.build([{"tokens": [1, 2], "pos0": 31, "slot": 0, "blocks": [3], "want": []}], 32, "cpu")


def test_config_reader_takes_every_size_from_the_file():
    from mistralrs_amd.hybrid import AttentionSpec, Mamba2Spec, gekilix_spec
    cfg = config([mamba_layer(heads=6, vdim=10, state=20, groups=3, conv=3, norm_groups=5, mlp=False), attn_layer(heads=6, kv_heads=3, dim=20, vdim=12, size=9, keep=1, rot=6)],
                 vocab=77, width=50, eps=3e-6)
    s = gekilix_spec(json.loads(json.dumps(cfg)))
    assert (s.vocab, s.width, s.eps) == (77, 50, 3e-6) and [l.kind for l in s.layers] == ["mamba2", "attention"] and s.layers[0].ff is None
    m, a = s.layers[0].mixer, s.layers[1].mixer
    assert isinstance(m, Mamba2Spec) and (m.heads, m.vdim, m.state, m.groups, m.conv, m.norm_groups, m.inner, m.conv_channels) == (6, 10, 20, 3, 3, 5, 60, 180)
    assert isinstance(a, AttentionSpec) and (a.heads, a.kv_heads, a.dim, a.vdim, a.window, a.keep_first, a.rotary.dims) == (6, 3, 20, 12, 9, 1, 6)
    assert (s.layers[1].ff.experts, s.layers[1].ff.top, s.layers[1].ff.ff, s.layers[1].ff.shared_ff) == (5, 2, 24, 16)
    with pytest.raises(ValueError):
        gekilix_spec(config([{"type": "lstm", "mixer": {}, "mlp": None}]))


def test_rotary_frequencies_match_the_restatement():
    from mistralrs_amd.hybrid import RotarySpec
    for dims, base, sc in ((8, 10000.0, None), (32, 500000.0, {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 2048}), (16, 100.0, {"factor": 3.0, "low": 2.0, "high": 8.0, "original": 80})):
        got, want = RotarySpec(dims, base, sc).frequencies(), O.rope_frequencies(dims, base, sc).numpy()
        assert np.allclose(got, want, rtol=1e-6, atol=0)
    sc = {"factor": 3.0, "low": 2.0, "high": 8.0, "original": 80}
    f, plain = O.rope_frequencies(16, 100.0, sc).numpy(), O.rope_frequencies(16, 100.0, None).numpy()
    assert f[0] == plain[0] and np.isclose(f[-1], plain[-1] / 3.0) and np.any((f != plain) & ~np.isclose(f, plain / 3.0))  # all three branches are exercised


@needs_lib
def test_scheduler_hands_out_and_takes_back_state_slots():
    from mistralrs_amd.kv_cache_manager import KVCacheManager, StateSlotPool
    from mistralrs_amd.scheduler import PagedAttentionScheduler, SchedulerConfig, Sequence, DONE
    kv, pool = KVCacheManager(32, 8, True, [0]), StateSlotPool(2)
    s = PagedAttentionScheduler(SchedulerConfig(max_num_seqs=4, max_num_batched_tokens=64, uniform_prompt_batches=False), kv, prefix_caching=True, state_pool=pool)
    assert not s.prefix_caching_enabled  # a cached block does not carry the recurrent state
    seqs = [Sequence(id=i + 1, tokens=list(range(5 + 3 * i)), max_new_tokens=2) for i in range(3)]
    for q in seqs:
        s.add_seq(q)
    out = s.schedule()
    assert out.kind == "prompt" and [q.id for q in out.scheduled] == [1, 2]  # unequal lengths in one batch; the third finds pages but no slot
    assert pool.slot_of(1) is not None and pool.slot_of(2) is not None and pool.slot_of(3) is None and s.waiting_len() == 1
    for q in out.scheduled:
        q.num_computed_tokens = len(q)
    seqs[0].state = DONE
    s.free_finished_sequence_groups()
    assert pool.slot_of(1) is None and pool.num_free_slots() == 1 and not kv.has_request(1)
    seqs[1].state = "running_completion"  # what the engine does when the prompt's last token has produced the first new one
    seqs[1].tokens.append(7)
    assert s.schedule().kind == "completion"  # a decode step comes first (one must have run before a waiting prompt interrupts)
    seqs[1].num_computed_tokens = len(seqs[1])
    seqs[1].tokens.append(8)
    out = s.schedule()
    assert out.kind == "prompt" and [q.id for q in out.scheduled] == [3] and pool.slot_of(3) is not None
    s._preempt(seqs[2])
    assert pool.slot_of(3) is None and seqs[2].num_computed_tokens == 0  # preempted: slot back, restart from position 0


def test_registry_knows_the_architectures():
    from mistralrs_amd import registry
    assert {"Gekilix", "llama"} <= set(registry.ARCHITECTURES)


# ---------------------------------------------------------------------------------------------------------------- mechanisms alone (GPU)
def _one_layer(layer, dev, dtype="float32", seed=1, **kw):
    cfg = config([layer], **kw)
    w = weights(cfg, seed)
    return cfg, w, Served(cfg, w, dev, dtype)


def _batch_of(sv, n, rid=1):
    from mistralrs_amd.hybrid import RaggedBatch
    assert sv.cache.reserve(rid, n)
    return RaggedBatch.build([sv.cache.entry(rid, [0] * n, 0, [])], sv.bs, sv.m.device)


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", [(1, 37, 40), (3, 64, 24), (8, 130, 72), (9, 65, 33), (70, 129, 96), (200, 31, 256), (300, 260, 96), (257, 128, 41)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_linear_products(dev, M, N, K, dtype):
    """out (+)= a . w^T through the row kernel (M <= 8) and the tile kernel, odd sizes included (K = 33: the element-wise load path)"""
    _, _, sv = _one_layer(mamba_layer(mlp=False), dev, dtype)
    g = torch.Generator().manual_seed(M * 1000 + N)
    a, w = torch.randn(M, K, generator=g).to(torch.bfloat16), torch.randn(N, K, generator=g).to(torch.bfloat16)
    base = torch.randn(M, N, generator=g)
    want = a.double() @ w.double().T
    td = sv.m.torch_dtype
    got = sv.m.linear(a.to(dev, td), w.to(dev, td))
    assert rel(got.double().cpu(), want) < 2e-6
    acc = base.to(dev).clone()
    sv.m.linear(a.to(dev, td), w.to(dev, td), out=acc, accumulate=True)
    assert rel(acc.double().cpu(), want + base.double()) < 2e-6


@pytest.mark.gpu
@pytest.mark.parametrize("R", [5, 32, 33, 150, 900])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_grouped_products(dev, R, dtype):
    """rows sorted by group, one weight slab per group; empty groups and groups larger than a tile"""
    _, _, sv = _one_layer(mamba_layer(mlp=False), dev, dtype)
    E, N, K = (6, 50, 40) if R < 900 else (4, 136, 72)   # 900 rows over 4 groups: the 128-row tile form
    g = torch.Generator().manual_seed(R)
    grp = torch.sort(torch.randint(0, E, (R,), generator=g)).values
    grp[grp == 2] = 3  # group 2 stays empty
    a, w = torch.randn(R, K, generator=g).to(torch.bfloat16), torch.randn(E, N, K, generator=g).to(torch.bfloat16)
    bounds = torch.tensor([int((grp < e).sum()) for e in range(E + 1)], dtype=torch.int32)
    want = torch.stack([a[r].double() @ w[grp[r]].double().T for r in range(R)])
    td = sv.m.torch_dtype
    got = sv.m.grouped_linear(a.to(dev, td), w.to(dev, td).contiguous(), bounds.to(dev), grp.to(torch.int32).to(dev))
    assert rel(got.double().cpu(), want) < 2e-6


@pytest.mark.gpu
@pytest.mark.parametrize("parts,one_plus", [(1, True), (1, False), (4, False)])
def test_rms_norm(dev, parts, one_plus):
    _, _, sv = _one_layer(mamba_layer(mlp=False), dev)
    g = torch.Generator().manual_seed(3)
    x, w = torch.randn(7, 48, generator=g) * 3, torch.randn(48, generator=g) * 0.2
    u = O.rms_unit(x.double().view(7, parts, 48 // parts), sv.m.spec.eps).reshape(7, 48)
    want = u * (1 + w.double()) if one_plus else u * w.double()
    assert rel(sv.m.norm(x.to(dev), w.to(dev), one_plus=one_plus, parts=parts).double().cpu(), want) < 1e-6


@pytest.mark.gpu
@pytest.mark.parametrize("layer", [mamba_layer(mlp=False), mamba_layer(heads=3, vdim=5, state=7, groups=1, conv=2, norm_groups=3, mlp=False),
                                   mamba_layer(heads=2, vdim=20, state=70, groups=2, conv=5, norm_groups=1, mlp=False),
                                   mamba_layer(heads=2, vdim=4, state=150, groups=1, conv=1, norm_groups=2, mlp=False)], ids=["base", "odd", "wide", "state150-conv1"])
def test_state_space_mixer_alone(dev, layer):
    cfg, w, sv = _one_layer(layer, dev)
    T, W = 21, cfg["width"]
    h = torch.randn(T, W, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16)
    want = O.mamba2_mixer(h.double(), layer["mixer"], f64(w), "l0.mix.", cfg["norm"]["eps"])
    x = torch.zeros(T, W, device=dev)
    sv.m.layers[0].mixer.forward(h.to(dev, torch.float32), x, _batch_of(sv, T))
    assert rel(x.double().cpu(), want) < 2e-5


@pytest.mark.gpu
@pytest.mark.parametrize("layer", [attn_layer(mlp=False), attn_layer(heads=3, kv_heads=3, dim=10, vdim=70, size=5, keep=0, rot=10, scaling=False, mlp=False),
                                   attn_layer(heads=6, kv_heads=1, dim=24, vdim=4, size=1000, keep=3, rot=0, mlp=False),
                                   attn_layer(heads=2, kv_heads=2, dim=8, vdim=8, size=1, keep=1, rot=4, mlp=False)], ids=["base", "mha-widev", "mqa-norot", "window1"])
def test_attention_mixer_alone(dev, layer):
    cfg, w, sv = _one_layer(layer, dev)
    T, W = 75, cfg["width"]
    h = torch.randn(T, W, generator=torch.Generator().manual_seed(6)).to(torch.bfloat16)
    want = O.attention_mixer(h.double(), layer["mixer"], f64(w), "l0.mix.", cfg["norm"]["eps"])
    x = torch.zeros(T, W, device=dev)
    sv.m.layers[0].mixer.forward(h.to(dev, torch.float32), x, _batch_of(sv, T))
    assert rel(x.double().cpu(), want) < 2e-5


@pytest.mark.gpu
@pytest.mark.parametrize("experts,top,shared", [(5, 2, 16), (1, 1, 0), (12, 1, 8), (7, 7, 0), (40, 3, 24)])
def test_routed_experts_alone(dev, experts, top, shared):
    layer = mamba_layer(mlp=True, experts=experts, top=top, ff=24, shared=shared)
    cfg, w, sv = _one_layer(layer, dev)
    T, W = 45, cfg["width"]
    h = torch.randn(T, W, generator=torch.Generator().manual_seed(7)).to(torch.bfloat16)
    want = O.moe_ffn(h.double(), layer["mlp"], f64(w), "l0.mlp.")
    x = torch.zeros(T, W, device=dev)
    hf = h.to(dev, torch.float32)
    sv.m.layers[0].ff.forward(hf, hf, x, _batch_of(sv, T))
    assert rel(x.double().cpu(), want) < 2e-5


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_planted_keys_at_every_edge(dev, dtype):
    """One key gets a score far above the rest, so whether the kernel sees it decides the output: just inside and just outside the window, the last kept first token and the
    first one that is not kept, both sides of a page border, a key hundreds of tokens back -- for a prompt pass and for single decoded rows reading the pages."""
    from mistralrs_amd.hybrid import RaggedBatch, _call
    H, G, D, Dv, size, keep, bs, T = 2, 1, 8, 4, 40, 3, 32, 300
    _, _, sv = _one_layer(attn_layer(heads=H, kv_heads=G, dim=D, vdim=Dv, size=size, keep=keep, mlp=False), dev, dtype)
    m, td = sv.m, sv.m.torch_dtype
    att = m.layers[0].mixer
    assert sv.cache.reserve(1, T)
    blocks = sv.cache.kv.get_block_ids(1)
    g = torch.Generator().manual_seed(11)
    v = torch.randn(T, G, Dv, generator=g).to(torch.bfloat16)
    cases = []  # (query position, planted key)
    for i in (60, 64, 95, 96, 299):
        for j in (i - size, i - size + 1, keep - 1, keep, 0, i, 31, 32, i - 1):
            if 0 <= j <= i:
                cases.append((i, j))
    for i, j in cases:
        k = torch.randn(T, G, D, generator=g).to(torch.bfloat16) * 0.05
        k[j, 0, 0] = 6.0
        q = torch.zeros(1, H, D, dtype=torch.bfloat16)
        q[0, :, 0] = 6.0
        want = O.windowed_attention(q.double(), k.double(), v.double(), 1.0, size, keep, pos_q=[i])
        seen = O.visible(i, j, size, keep)
        # the planted key decides: with it visible the output is (nearly) its value row
        assert (rel(want[0, 0], v[j, 0].double()) < 0.05) == seen
        for t in range(T):  # pages through the block table, as the cache-write kernel lays them out
            att.k_cache[blocks[t // bs], :, t % bs] = k[t].to(dev, td)
            att.v_cache[blocks[t // bs], :, t % bs] = v[t].to(dev, td)
        for rows in ("decode", "prompt"):
            p0 = i if rows == "decode" else max(0, i - 20)
            n = i - p0 + 1
            b = RaggedBatch.build([{"tokens": [0] * n, "pos0": p0, "slot": 0, "blocks": blocks, "want": []}], bs, dev)
            qq = torch.zeros(n, H * D, dtype=td, device=dev)
            qq[n - 1] = q.reshape(-1).to(dev, td)
            out = torch.empty(n, H * Dv, dtype=td, device=dev)
            _call("mrs_hyb_paged_window_attn", qq, att.k_cache, att.v_cache, b.block_tables, b.tok_seq, b.tok_pos, out, n, H, G, D, Dv, bs, b.max_blocks, size, keep, 1.0, m.dt,
                  b.seg_entry, b.seg_row0, b.seg_len, b.segments, RaggedBatch.SEGMENT)
            got = out[n - 1].double().cpu().view(H, Dv)
            assert rel(got, want[0]) < (1e-5 if dtype == "float32" else 1e-2), (i, j, rows, seen)
    sv.end(1)


# ---------------------------------------------------------------------------------------------------------------- whole models (GPU)
@pytest.mark.gpu
@pytest.mark.parametrize("dtype,bar", [("float32", 3e-5), ("bfloat16", 4e-2)])
def test_whole_prompt_every_layer(dev, dtype, bar):
    cfg = config(MIXED)
    w = weights(cfg, 2)
    t = toks(90, cfg["vocab"], 1)
    want, trail = O.forward(cfg, f64(w), t, keep_layers=True)
    sv = Served(cfg, w, dev, dtype)
    sv.m.trace_layers = []
    got = sv.step([(1, t)])[0]
    for i, x in enumerate(sv.m.trace_layers):
        assert close(x.double().cpu(), trail[i], bar), f"residual stream after layer {i} ({cfg['layers'][i]['type']})"
    assert close(got, want, bar)


@pytest.mark.gpu
def test_portions_and_decoding_equal_the_whole_prompt(dev):
    """the same 150 tokens: at once; in portions of changing size down to two tokens (crossing pages and the window); one by one"""
    cfg = config(MIXED)
    w = weights(cfg, 3)
    t = toks(150, cfg["vocab"], 2)
    want = O.forward(cfg, f64(w), t)
    sv = Served(cfg, w, dev)
    whole = sv.step([(1, t)])[0]
    assert rel(whole, want) < 3e-5
    cuts, at, sizes = [], 0, [37, 2, 17, 3, 31, 2, 33, 1, 5, 64]
    while at < len(t):
        n = sizes[len(cuts) % len(sizes)]
        cuts.append(t[at:at + n])
        at += n
    got = torch.cat([sv.step([(2, c)])[0] for c in cuts])
    assert rel(got, want) < 3e-5 and rel(got, whole) < 1e-5
    one = torch.cat([sv.step([(3, [x])])[0] for x in t])
    assert rel(one, want) < 3e-5 and rel(one, whole) < 1e-5


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,bar", [("float32", 3e-5), ("bfloat16", 4e-2)])
def test_mixed_batches_with_reused_pages_and_slots(dev, dtype, bar):
    """six unequal requests through four slots and a pool too small for all of them: portions of some beside single tokens of others; every row against the request alone"""
    cfg = config(MIXED)
    w = weights(cfg, 4)
    lens = [70, 9, 33, 1, 50, 41]
    reqs = {i + 1: toks(n, cfg["vocab"], 10 + i) for i, n in enumerate(lens)}
    want = {r: O.forward(cfg, f64(w), t) for r, t in reqs.items()}
    sv = Served(cfg, w, dev, dtype, max_tokens=192, slots=4)
    at, got = {r: 0 for r in reqs}, {r: [] for r in reqs}
    waiting, live, step = list(reqs), [], 0
    sizes = [16, 2, 1, 30, 3, 1, 1, 25]
    while waiting or live:
        while waiting and len(live) < 4 and sum(-(-len(reqs[r]) // 32) for r in live + waiting[:1]) * 32 <= 192:
            live.append(waiting.pop(0))
        parts = []
        for n, r in enumerate(live):
            if (step + n) % 3 == 2 and len(live) > 1:
                continue  # left out of this step, goes on later
            k = sizes[(step + 2 * n) % len(sizes)]
            parts.append((r, reqs[r][at[r]:at[r] + k]))
        step += 1
        if not parts:
            continue
        for (r, tk), lg in zip(parts, sv.step(parts)):
            got[r].append(lg)
            at[r] += len(tk)
        for r in [r for r in live if at[r] == len(reqs[r])]:
            live.remove(r)
            sv.end(r)
    for r in reqs:
        assert close(torch.cat(got[r]), want[r], bar), f"request {r}"


@pytest.mark.gpu
def test_long_decoding_past_the_window_with_kept_first_tokens(dev):
    """a short prompt, then 260 single steps: the window (12 / 7) slides over decoded tokens across eight pages, the kept first tokens stay, the recurrent state carries on"""
    cfg = config([mamba_layer(top=1), attn_layer(top=1), attn_layer(keep=0, size=7, top=1)])
    w = weights(cfg, 5)
    t = toks(270, cfg["vocab"], 3)
    want = O.forward(cfg, f64(w), t)
    sv = Served(cfg, w, dev)
    got = torch.cat([sv.step([(1, t[:10])])[0]] + [sv.step([(1, [x])])[0] for x in t[10:]])
    assert rel(got, want) < 3e-5
    assert rel(got[-1], want[-1]) < 3e-5 and rel(got[9], want[9]) < 3e-5


@pytest.mark.gpu
def test_sizes_that_coincide_or_equal_one(dev):
    """head counts, groups and parts of 1, key size == value size == rotary size, one expert, no feed-forward, a window longer than the text"""
    layers = [mamba_layer(heads=1, vdim=16, state=4, groups=1, conv=2, norm_groups=1, experts=1, top=1, ff=8, shared=0),
              attn_layer(heads=1, kv_heads=1, dim=16, vdim=16, size=500, keep=0, rot=16, scaling=False, mlp=False),
              mamba_layer(heads=5, vdim=3, state=9, groups=5, conv=3, norm_groups=5, experts=3, top=3, ff=10, shared=6)]
    cfg = config(layers, vocab=50, width=24, eps=1e-6)
    w = weights(cfg, 6)
    t = toks(40, 50, 4)
    want = O.forward(cfg, f64(w), t)
    sv = Served(cfg, w, dev)
    assert rel(sv.step([(1, t)])[0], want) < 3e-5
    assert rel(torch.cat([sv.step([(2, t[:3])])[0], sv.step([(2, t[3:5])])[0], sv.step([(2, t[5:])])[0]]), want) < 3e-5


@pytest.mark.gpu
@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
def test_greedy_generation_through_scheduler_and_engine(dev, graphs):
    """the package's own entry point: scheduler (pages + state slots), engine, sampler (top-1 kernels); five prompts through three slots, against greedy decoding of the restatement"""
    from mistralrs_amd.cli import make_engine
    from mistralrs_amd.hybrid import HybridDecoder, gekilix_spec
    from mistralrs_amd.sampler import SequenceSampler
    from mistralrs_amd.scheduler import Sequence
    cfg = config([mamba_layer(top=1), attn_layer(top=1, size=9, keep=2)])
    w = weights(cfg, 7)
    m = HybridDecoder(gekilix_spec(cfg), dev, "float32", num_blocks=12, block_size=32, state_slots=3)
    m.load_weights(w.__getitem__)
    core = os.path.exists(_lib.path("core"))
    eng = make_engine(m, 12 * 32, 3, sampler=SequenceSampler(cfg["vocab"], dev, top_k=1) if core else None, max_batched_tokens=48, use_graphs=graphs)
    prompts = [toks(n, cfg["vocab"], 20 + n) for n in (5, 40, 1, 23, 60)]
    seqs = [Sequence(id=i + 1, tokens=list(p), max_new_tokens=6) for i, p in enumerate(prompts)]
    for s in seqs:
        eng.s.add_seq(s)
    eng.run()
    wd = f64(w)
    for p, s in zip(prompts, seqs):
        ref = list(p)
        for _ in range(6):
            lg = O.forward(cfg, wd, ref)[-1]
            top2 = torch.topk(lg, 2).values
            if float(top2[0] - top2[1]) < 1e-3:
                break  # a tie within rounding: the comparison stops here
            ref.append(int(lg.argmax()))
        assert s.error is None and s.generated[:len(ref) - len(p)] == ref[len(p):], (s.id, s.generated, ref[len(p):])
    assert eng.s.state_pool.num_free_slots() == 3 and eng.steps["prompt"] >= 2 and eng.steps["completion"] >= 6
    assert bool(eng._graphs) == graphs


@pytest.mark.gpu
def test_captured_decode_steps_equal_eager_steps(dev):
    """a HIP graph of one decode step for three sequences, captured while two of them are live: every replay (eager work and synchronisation between replays) against the
    eager step function on a second copy of the model, and the states the warm-up touched are intact"""
    cfg = config(MIXED)
    w = weights(cfg, 8)
    a, b = Served(cfg, w, dev), Served(cfg, w, dev)
    prompts = {1: toks(37, cfg["vocab"], 31), 2: toks(3, cfg["vocab"], 32), 3: toks(64, cfg["vocab"], 33)}
    for sv in (a, b):
        sv.step([(1, prompts[1]), (2, prompts[2])])
    g = a.m.capture_decode(3, 8)
    for sv in (a, b):
        sv.step([(3, prompts[3])])
    nxt = {r: toks(12, cfg["vocab"], 40 + r) for r in prompts}
    for i in range(12):
        parts = [(r, [nxt[r][i]]) for r in (1, 2, 3)]
        want = torch.cat(b.step(parts))
        entries = []
        for r, tk in parts:
            assert a.cache.reserve(r, a.len[r] + 1)
            entries.append(a.cache.entry(r, tk, a.len[r]))
            a.len[r] += 1
        got = g.replay(entries).double().cpu()
        assert rel(got, want) < 1e-6, f"replay {i}"
        torch.cuda.synchronize()


@pytest.mark.gpu
def test_checkpoint_folder_through_registry_command_line_and_trace_replay(dev, tmp_path, monkeypatch, capsys):
    """config.json + model.safetensors on disk -> registry -> `generate` (scheduler, engine, sampler) and `trace` (steps from standard input, logits to files, pages and
    slots given back and reused) -- both against the restatement"""
    import io
    from safetensors.torch import save_file
    from mistralrs_amd import cli, registry, trace
    cfg = config([mamba_layer(top=1), attn_layer(top=2, size=10, keep=1)])
    w = weights(cfg, 9)
    folder = tmp_path / "model"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in w.items()}, str(folder / "model.safetensors"))
    assert registry.architecture_of(str(folder)) == "Gekilix"
    wd = f64(w)
    # ---- trace replay: three requests through two state slots and a pool of 128 tokens, portions beside single tokens, an empty `want`
    reqs = {"a": toks(45, cfg["vocab"], 51), "b": toks(20, cfg["vocab"], 52), "c": toks(33, cfg["vocab"], 53)}
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": reqs["a"][:30], "want": [0, 29]}, {"id": "b", "tokens": reqs["b"][:19], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": reqs["a"][30:31], "want": [0]}, {"id": "b", "tokens": reqs["b"][19:], "want": [0]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "c", "tokens": reqs["c"][:2], "want": [1]}, {"id": "a", "tokens": reqs["a"][31:], "want": [13]}], "end": ["a"]},
             {"step": 3, "entries": [{"id": "c", "tokens": reqs["c"][2:], "want": [0, 30]}], "end": ["c"]}]
    out = tmp_path / "out"
    monkeypatch.setattr("sys.stdin", io.StringIO("\n".join(json.dumps(s) for s in steps) + "\n"))
    assert trace.main(["--model", str(folder), "--dtype", "float32", "--out", str(out), "--max-tokens", "128", "--state-slots", "2"]) == 0
    printed = capsys.readouterr().out.split("\n")
    assert [l for l in printed if l.startswith("done")] == [f"done {i}" for i in range(4)]
    full = {r: O.forward(cfg, wd, t) for r, t in reqs.items()}
    want = {0: [full["a"][0], full["a"][29]], 1: [full["a"][30], full["b"][19]], 2: [full["c"][1], full["a"][44]], 3: [full["c"][2], full["c"][32]]}
    for n, rows in want.items():
        got = torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(len(rows), cfg["vocab"]).astype(np.float64))
        assert rel(got, torch.stack(rows)) < 3e-5, f"step {n}"
    # ---- generate: greedy, two prompts
    prompts = [toks(12, cfg["vocab"], 61), toks(3, cfg["vocab"], 62)]
    args = ["generate", "--model", str(folder), "--dtype", "float32", "--max-new-tokens", "4", "--max-tokens", "256", "--max-seqs", "2"]
    for p in prompts:
        args += ["--prompt-ids", ",".join(map(str, p))]
    if not os.path.exists(_lib.path("core")):
        pytest.skip("the sampler's library is not built")
    assert cli.main(args) == 0
    lines = [json.loads(l) for l in capsys.readouterr().out.split("\n") if l.startswith("{")]
    assert len(lines) == 2
    for p, line in zip(prompts, lines):
        ref = list(p)
        for _ in range(4):
            lg = O.forward(cfg, wd, ref)[-1]
            t2 = torch.topk(lg, 2).values
            if float(t2[0] - t2[1]) < 1e-3:
                break
            ref.append(int(lg.argmax()))
        assert line["error"] is None and line["tokens"][:len(ref) - len(p)] == ref[len(p):]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,bar", [("float32", 3e-5), ("bfloat16", 5e-2)])
def test_sizes_off_every_vector_width(dev, dtype, bar):
    """a width of 30, an odd value size, a key size of 6, expert sizes of 10 and 7, a state size of 9: nothing is a multiple of 4 or 8, so every kernel runs its element-wise
    path -- whole prompt, portions and single steps (whose products build their operands in the load)"""
    layers = [mamba_layer(heads=3, vdim=5, state=9, groups=1, conv=3, norm_groups=3, experts=4, top=2, ff=10, shared=7),
              attn_layer(heads=4, kv_heads=2, dim=6, vdim=5, size=11, keep=2, rot=4, experts=3, top=1, ff=7, shared=0),
              attn_layer(heads=2, kv_heads=1, dim=8, vdim=3, size=200, keep=0, rot=8, scaling=False, mlp=False)]
    cfg = config(layers, vocab=51, width=30, eps=1e-6)
    w = weights(cfg, 12)
    t = toks(80, 51, 9)
    want = O.forward(cfg, f64(w), t)
    sv = Served(cfg, w, dev, dtype)
    assert close(sv.step([(1, t)])[0], want, bar)
    got = torch.cat([sv.step([(2, t[:70])])[0]] + [sv.step([(2, [x])])[0] for x in t[70:]])
    assert close(got, want, bar)
    mixed = sv.step([(3, t[:9]), (4, t[:1])])
    assert close(mixed[0], want[:9], bar) and close(mixed[1], want[:1], bar)
