"""Sobunex decoders (mistralrs_amd.hybrid: TalkSigmoidAttention, XieluFeedForward, ClampedSoftmaxMoe, layer norms around every sublayer; csrc/hyb_attn_talk.hip and the
kernels added to csrc/hyb_kernels.hip / hyb_gemm.hip) against the plain float64 restatement in tests/sobunex_oracle.py.

Every test builds its own small configuration with random bf16-representable weights.  The sharp comparisons run in the all-f32 mode (a wrong key, a window one token
off, a page of the wrong layer is an O(1) error there, rounding is 1e-6); the bf16 mode is held to a rounding-sized bar.  CPU tests cover what needs no device.
"""
import io
import json
import math
import os

import numpy as np
import pytest
import torch

import mistralrs_amd  # noqa: F401
from mistralrs_amd import _lib
from tests import sobunex_oracle as O


# ---------------------------------------------------------------------------------------------------------------- configurations and weights
def dense(ff=56):
    return {"kind": "dense", "ff": ff}


def moe(experts=5, top=2, ff=24, shared=16, scale=1.25, limit=1.5, shared_limit=0.75):
    return {"kind": "moe", "router": {"experts": experts, "top": top, "scale": scale}, "expert": {"ff": ff, "limit": limit},
            "shared": {"ff": shared, "limit": shared_limit} if shared else None}


def layer(heads=4, kv_heads=2, dim=16, vdim=8, size=12, coef=0.25, every=16, kv_from=None, mlp="dense"):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": 1.0 / math.sqrt(dim)}
    if size:
        m["mask"] = {"size": size}
    if coef:
        m["q_temp"] = {"coef": coef, "every": every}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": dense() if mlp == "dense" else (moe() if mlp == "moe" else mlp)}


def config(layers, vocab=96, width=40, eps=1e-5):
    return {"architecture": "Sobunex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


def weights(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    w = {}

    def rnd(*shape, scale=1.0, shift=0.0):
        return (torch.randn(*shape, generator=g) * scale + shift).to(torch.bfloat16)

    def norm(name):
        w[name], w[name + ".b"] = rnd(W, scale=0.2, shift=1.0), rnd(W, scale=0.1)
    w["embed"], w["head"] = rnd(cfg["vocab"], W), rnd(cfg["vocab"], W, scale=W ** -0.5)
    norm("final.norm")
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        norm(p + "norm1"), norm(p + "norm1b")
        w[p + "mix.q"], w[p + "mix.q.b"] = rnd(H * D, W, scale=1.5 * W ** -0.5), rnd(H * D, scale=0.3)
        if m.get("kv_from") is None:
            w[p + "mix.k"], w[p + "mix.k.b"] = rnd(G * D, W, scale=1.5 * W ** -0.5), rnd(G * D, scale=0.3)
            w[p + "mix.v"], w[p + "mix.v.b"] = rnd(G * Dv, W, scale=W ** -0.5), rnd(G * Dv, scale=0.3)
        w[p + "mix.talk"] = (torch.eye(H) + 0.3 * torch.randn(H, H, generator=g)).to(torch.bfloat16)
        w[p + "mix.pb"], w[p + "mix.g"] = rnd(H, shift=-1.0), rnd(H, W, scale=2.0 * W ** -0.5)
        w[p + "mix.o"], w[p + "mix.o.b"] = rnd(W, H * Dv, scale=(H * Dv) ** -0.5), rnd(W, scale=0.2)
        f = L.get("mlp")
        if not f:
            continue
        norm(p + "norm2"), norm(p + "norm2b")
        if f["kind"] == "dense":
            w[p + "mlp.up"], w[p + "mlp.up.b"] = rnd(f["ff"], W, scale=W ** -0.5), rnd(f["ff"], scale=0.3)
            w[p + "mlp.down"], w[p + "mlp.down.b"] = rnd(W, f["ff"], scale=f["ff"] ** -0.5), rnd(W, scale=0.2)
            w[p + "mlp.act"] = rnd(2, scale=0.7)
        else:
            ff = f["expert"]["ff"]
            for e in range(f["router"]["experts"]):
                w[f"{p}mlp.e{e}.gate"], w[f"{p}mlp.e{e}.up"], w[f"{p}mlp.e{e}.down"] = rnd(ff, W, scale=2 * W ** -0.5), rnd(ff, W, scale=2 * W ** -0.5), rnd(W, ff, scale=ff ** -0.5)
            w[p + "mlp.router"] = rnd(f["router"]["experts"], W, scale=2.0 * W ** -0.5)
            if f.get("shared"):
                sf = f["shared"]["ff"]
                w[p + "mlp.shared.gate"], w[p + "mlp.shared.up"], w[p + "mlp.shared.down"] = rnd(sf, W, scale=2 * W ** -0.5), rnd(sf, W, scale=2 * W ** -0.5), rnd(W, sf, scale=sf ** -0.5)
    return w


def f64(w):
    return {k: v.to(torch.float64) for k, v in w.items()}


STACK = [layer(mlp="dense"), layer(kv_from=0, mlp="moe"), layer(heads=6, kv_heads=3, dim=8, vdim=12, size=7, every=5, mlp=None), layer(kv_from=0, size=20, coef=0.0, mlp="moe"),
         layer(heads=6, kv_heads=3, dim=8, vdim=12, kv_from=2, size=0, mlp="dense")]


class Served:
    """A model on the device with its caches, stepped the way the engine and the trace runner step it."""

    def __init__(self, cfg, w, dev, dtype="float32", max_tokens=512, slots=4, block_size=32):
        from mistralrs_amd.hybrid import SPEC_READERS, HybridCache, HybridDecoder
        self.bs = block_size
        self.m = HybridDecoder(SPEC_READERS[cfg["architecture"]](cfg), dev, dtype, num_blocks=-(-max_tokens // block_size) + slots + 1, block_size=block_size, state_slots=slots)
        self.m.load_weights(w.__getitem__)
        self.cache = HybridCache(self.m)
        self.len = {}

    def step(self, parts):
        """parts: [(request id, tokens)]; logits of every row, split per part"""
        from mistralrs_amd.hybrid import RaggedBatch
        entries = []
        for rid, tk in parts:
            p0 = self.len.get(rid, 0)
            assert self.cache.reserve(rid, p0 + len(tk)), "out of pages / slots"
            entries.append(self.cache.entry(rid, tk, p0, range(len(tk))))
            self.len[rid] = p0 + len(tk)
        out = self.m.forward_batch(RaggedBatch.build(entries, self.bs, self.m.device)).double().cpu()
        res, r = [], 0
        for _, tk in parts:
            res.append(out[r:r + len(tk)])
            r += len(tk)
        return res

    def end(self, rid):
        self.cache.release(rid)
        self.len.pop(rid, None)


def rel(a, b):
    return float((a - b).norm() / (b.norm() + 1e-30))


def close(a, b, bar):
    """f32 mode (bar < 1e-3): the whole tensor within `bar`.  bf16 mode: rounding can move a router's close call in these narrow models, which changes single rows by much
    more than rounding does -- so the typical row is held to `bar` and at most one row in ten may exceed five times that."""
    if bar < 1e-3:
        return rel(a, b) < bar
    rows = (a - b).reshape(-1, a.shape[-1]).norm(dim=1) / (b.reshape(-1, b.shape[-1]).norm(dim=1) + 1e-30)
    return float(rows.median()) < bar and float((rows > 5 * bar).double().mean()) <= 0.1


def toks(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


# ---------------------------------------------------------------------------------------------------------------- no device needed
def test_config_reader_takes_every_size_and_constant_from_the_file():
    from mistralrs_amd.hybrid import ClampedMoeSpec, DenseSpec, sobunex_spec
    cfg = config([layer(heads=6, kv_heads=3, dim=10, vdim=14, size=33, coef=0.5, every=9, mlp=dense(77)),
                  layer(heads=6, kv_heads=3, dim=10, vdim=14, size=0, coef=0.0, kv_from=0, mlp=moe(11, 4, 20, 0, scale=2.5, limit=3.0)),
                  layer(mlp=moe(3, 1, 8, 12, scale=1.0, limit=0.5, shared_limit=2.0)), layer(mlp=None)], vocab=123, width=56, eps=3e-4)
    sp = sobunex_spec(cfg)
    assert (sp.vocab, sp.width, sp.eps, sp.norm, sp.post_norms) == (123, 56, 3e-4, "layer", True)
    a, b, c, d = sp.layers
    assert (a.mixer.heads, a.mixer.kv_heads, a.mixer.dim, a.mixer.vdim, a.mixer.window, a.mixer.temp_coef, a.mixer.temp_every, a.mixer.kv_from) == (6, 3, 10, 14, 33, 0.5, 9, None)
    assert isinstance(a.ff, DenseSpec) and a.ff.ff == 77
    assert (b.mixer.window, b.mixer.temp_every, b.mixer.kv_from) == (0, 0, 0)
    assert isinstance(b.ff, ClampedMoeSpec) and (b.ff.experts, b.ff.top, b.ff.ff, b.ff.limit, b.ff.route_scale, b.ff.shared_ff) == (11, 4, 20, 3.0, 2.5, 0)
    assert (c.ff.shared_ff, c.ff.shared_limit, c.ff.limit) == (12, 2.0, 0.5) and d.ff is None
    assert [l.prefix for l in sp.layers] == ["l0.", "l1.", "l2.", "l3."]
    for bad in ([layer(kv_from=0)], [layer(), layer(kv_from=1)], [layer(), layer(kv_from=0), layer(kv_from=1)], [layer(), layer(dim=8, kv_from=0)]):
        with pytest.raises(ValueError):
            sobunex_spec(config(bad))


def test_registry_and_synthetic_weights_know_the_architecture():
    from mistralrs_amd import registry
    from mistralrs_amd.hybrid import FEED_FORWARDS, MIXERS, SPEC_READERS, sobunex_spec, synthetic_weights
    assert "Sobunex" in registry.ARCHITECTURES and "Sobunex" in SPEC_READERS
    assert {"talk_attention"} <= set(MIXERS) and {"dense_xielu", "moe_softmax_clamped"} <= set(FEED_FORWARDS)
    cfg = config(STACK)
    get = synthetic_weights(sobunex_spec(cfg), "cpu", 1)
    for name, t in weights(cfg).items():
        assert tuple(get(name).shape) == tuple(t.shape), name
    with pytest.raises(KeyError):
        get("l1.mix.k")   # a layer that reads another layer's pages has no key projection


def test_restatement_pieces():
    """the oracle's own building blocks on hand-computed values"""
    x = torch.tensor([[1.0, 2.0, 3.0, 6.0]], dtype=torch.float64)
    y = O.layer_norm(x, torch.ones(4, dtype=torch.float64), torch.zeros(4, dtype=torch.float64), 0.0)
    assert abs(float(y.mean())) < 1e-12 and abs(float((y * y).mean()) - 1.0) < 1e-12
    assert abs(float(O.xielu(torch.tensor(2.0, dtype=torch.float64), 0.0, 0.0)) - (math.log(2.0) * 4 + 1.0)) < 1e-12
    assert abs(float(O.xielu(torch.tensor(-1.0, dtype=torch.float64), 0.0, 0.0)) - ((0.5 + math.log(2.0)) * (math.exp(-1.0) - 1 + 1) - 0.5)) < 1e-12
    assert O.query_temperature(12, 0.5, 4).tolist() == [1.0] * 3 + [1 + 0.5 * math.log(2)] * 4 + [1 + 0.5 * math.log(3)] * 4 + [1 + 0.5 * math.log(4)]
    assert O.visible(5, 2).tolist() == [[j in (i, i - 1) and j >= 0 for j in range(5)] for i in range(5)]
    assert abs(float(O.head_slopes(4)[1]) - 2.0 ** -4) < 1e-15


# ---------------------------------------------------------------------------------------------------------------- mechanisms alone (GPU)
def _model(layers, dev, dtype="float32", seed=1, **kw):
    cfg = config(layers, **{k: v for k, v in kw.items() if k in ("vocab", "width", "eps")})
    w = weights(cfg, seed)
    return cfg, w, Served(cfg, w, dev, dtype, **{k: v for k, v in kw.items() if k in ("max_tokens", "slots", "block_size")})


@pytest.mark.gpu
@pytest.mark.parametrize("width", [40, 37, 300])
def test_layer_norm_kernel(dev, width):
    from mistralrs_amd.hybrid import _call
    _, _, sv = _model([layer(mlp=None)], dev, width=40)
    g = torch.Generator().manual_seed(width)
    x, w, b, ib, res = (torch.randn(*s, generator=g) for s in ((9, width), (width,), (width,), (width,), (9, width)))
    x = x * 3 + 1.5
    want = O.layer_norm(x.double(), w.double(), b.double(), 1e-5)
    out32 = torch.empty(9, width, device=dev)
    out = torch.empty(9, width, device=dev)
    _call("mrs_hyb_layernorm", x.to(dev), width, None, w.to(dev), b.to(dev), out, out32, None, 0, 9, width, 1e-5, 2)
    assert rel(out32.double().cpu(), want) < 2e-6 and rel(out.double().cpu(), want) < 2e-6
    r = res.to(dev)
    _call("mrs_hyb_layernorm", x.to(dev), width, ib.to(dev), w.to(dev), b.to(dev), None, None, r, width, 9, width, 1e-5, 2)
    new = res.double() + O.layer_norm((x + ib).double(), w.double(), b.double(), 1e-5)
    assert rel(r.double().cpu(), new) < 2e-6
    # the norm behind a sublayer and the norm in front of the next one in one launch
    w2, b2 = torch.randn(width, generator=g), torch.randn(width, generator=g)
    r = res.to(dev)
    _call("mrs_hyb_layernorm_pair", x.to(dev), width, ib.to(dev), w.to(dev), b.to(dev), r, width, w2.to(dev), b2.to(dev), out, out32, 9, width, 1e-5, 2)
    assert rel(r.double().cpu(), new) < 2e-6 and rel(out32.double().cpu(), O.layer_norm(new, w2.double(), b2.double(), 1e-5)) < 3e-6 and rel(out.double().cpu(), out32.double().cpu()) == 0


@pytest.mark.gpu
def test_activation_kernels(dev):
    from mistralrs_amd.hybrid import _call
    _, _, sv = _model([layer(mlp=None)], dev)
    g = torch.Generator().manual_seed(3)
    rows, ff = 7, 45
    u, b = torch.randn(rows, ff, generator=g) * 3, torch.randn(ff, generator=g)
    p, q = 0.3, -0.6
    out = torch.empty(rows, ff, device=dev)
    _call("mrs_hyb_bias_xielu", u.to(dev), ff, b.to(dev), out, rows, ff, O.softplus(p), 0.5 + O.softplus(q), 2)
    assert rel(out.double().cpu(), O.xielu((u + b).double(), p, q)) < 2e-6
    gu = torch.randn(rows, 2 * ff, generator=g) * 2
    _call("mrs_hyb_glu_clamped", gu.to(dev), out, rows, ff, 0.8, 1.702, 2)
    gg, uu = torch.clamp(gu[:, :ff].double(), max=0.8), torch.clamp(gu[:, ff:].double(), -0.8, 0.8)
    assert rel(out.double().cpu(), gg * torch.sigmoid(1.702 * gg) * (uu + 1)) < 2e-6
    assert float(out.max()) <= 0.8 * 1.8 + 1e-6


@pytest.mark.gpu
@pytest.mark.parametrize("E,top", [(5, 2), (1, 1), (70, 3), (9, 9)])
def test_softmax_router(dev, E, top):
    from mistralrs_amd.hybrid import _call
    _, _, sv = _model([layer(mlp=None)], dev)
    g = torch.Generator().manual_seed(E)
    T, W = 11, 52
    h, wr = torch.randn(T, W, generator=g), torch.randn(E, W, generator=g) * 0.4
    ids = torch.empty(T * top, dtype=torch.int32, device=dev)
    wts = torch.empty(T * top, device=dev)
    _call("mrs_hyb_route_softmax_topk", h.to(dev), wr.to(dev), T, W, E, top, 1.75, ids, wts)
    idx, val = O.route_softmax(h.double(), wr.double(), top, 1.75)
    assert ids.cpu().view(T, top).tolist() == idx.tolist()
    assert rel(wts.double().cpu().view(T, top), val) < 2e-6


@pytest.mark.gpu
def test_projection_biases_query_temperature_and_page_write(dev):
    from mistralrs_amd.hybrid import RaggedBatch, _call
    H, G, D, Dv, bs = 3, 1, 6, 5, 32
    _, _, sv = _model([layer(heads=H, kv_heads=G, dim=D, vdim=Dv, mlp=None)], dev)
    att = sv.m.layers[0].mixer
    assert sv.cache.reserve(1, 70)
    blocks = sv.cache.kv.get_block_ids(1)
    p0, n = 27, 40                       # positions 27 .. 66: over a page border and over several steps of the temperature
    b = RaggedBatch.build([{"tokens": [0] * n, "pos0": p0, "slot": 0, "blocks": blocks, "want": []}], bs, dev)
    g = torch.Generator().manual_seed(5)
    ld = H * D + G * D + G * Dv + H
    u = torch.randn(n, ld, generator=g)
    qb, kb, vb = torch.randn(H * D, generator=g), torch.randn(G * D, generator=g), torch.randn(G * Dv, generator=g)
    q = torch.empty(n, H * D, device=dev)
    _call("mrs_hyb_qkv_bias_temp_cache", u.to(dev), ld, qb.to(dev), kb.to(dev), vb.to(dev), b.tok_pos, b.slot_mapping, q, att.k_cache, att.v_cache, n, H, G, D, Dv, bs, 0.4, 8, 2)
    f = torch.tensor([1 + 0.4 * math.log((p + 1) // 8 + 1) for p in range(p0, p0 + n)], dtype=torch.float64)
    assert rel(q.double().cpu(), (u[:, :H * D] + qb).double() * f[:, None]) < 1e-6
    for i in (0, 4, 5, 39):
        pos = p0 + i
        kk = att.k_cache[blocks[pos // bs], :, pos % bs].double().cpu().reshape(-1)
        vv = att.v_cache[blocks[pos // bs], :, pos % bs].double().cpu().reshape(-1)
        assert rel(kk, (u[i, H * D:H * D + G * D] + kb).double()) < 1e-6 and rel(vv, (u[i, H * D + G * D:H * D + G * D + G * Dv] + vb).double()) < 1e-6
    sv.end(1)


ATTN_SHAPES = [dict(), dict(heads=3, kv_heads=3, dim=10, vdim=7, size=5, every=3), dict(heads=6, kv_heads=2, dim=24, vdim=40, size=70, every=50),
               dict(heads=2, kv_heads=1, dim=8, vdim=4, size=0, coef=0.0), dict(heads=8, kv_heads=4, dim=16, vdim=160, size=33), dict(heads=5, kv_heads=1, dim=9, vdim=3, size=64, every=1),
               dict(heads=16, kv_heads=4, dim=32, vdim=130, size=20)]


@pytest.mark.gpu
@pytest.mark.parametrize("shape", ATTN_SHAPES, ids=lambda s: "-".join(f"{k}{v}" for k, v in s.items()) or "default")
@pytest.mark.parametrize("dtype,bar", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_attention_mixer_alone(dev, shape, dtype, bar):
    """one layer without a feed-forward: a prompt of 150 tokens (tiles of several queries, several passes of 64 keys), then 30 decoded tokens one by one"""
    cfg, w, sv = _model([layer(mlp=None, **shape)], dev, dtype, seed=2)
    t = toks(180, cfg["vocab"], 9)
    want = O.forward(cfg, f64(w), t)
    got = sv.step([(1, t[:150])])[0]
    assert close(got, want[:150], bar)
    got = torch.cat([sv.step([(1, [t[i]])])[0] for i in range(150, 180)])
    assert close(got, want[150:], bar)


@pytest.mark.gpu
@pytest.mark.parametrize("mlp", [dense(56), dense(9), dense(300), moe(), moe(1, 1, 8, 0), moe(12, 1, 16, 8), moe(7, 7, 24, 0, scale=0.5, limit=0.3), moe(40, 3, 20, 24, limit=7.0)],
                         ids=lambda f: f["kind"] + "-" + "-".join(str(v) for v in (f.get("router") or {"ff": f.get("ff")}).values()))
def test_feed_forwards_alone(dev, mlp):
    """one layer whose attention sees only the token itself, so the feed-forward decides: 70 rows at once (grouped products) and 3 rows (the streamed products of decode steps)"""
    cfg, w, sv = _model([layer(size=1, coef=0.0, mlp=mlp)], dev, seed=4)
    t = toks(70, cfg["vocab"], 10)
    want = O.forward(cfg, f64(w), t)
    assert rel(sv.step([(1, t)])[0], want) < 2e-5
    sv.end(1)
    assert rel(sv.step([(2, t[:1])])[0], want[:1]) < 2e-5
    got = torch.cat(sv.step([(2, [t[1]]), (3, [t[0]]), (4, [t[0]])]))   # a window of one token: a row's logits depend on its token and (through the temperature) nothing else
    assert rel(got, torch.stack([want[1], want[0], want[0]])) < 2e-5


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_planted_keys_at_every_edge(dev, dtype):
    """One key gets a score far above the rest and the head biases push every other weight to nothing, so whether the kernel sees the key decides the output (its value row, or
    zero): just inside and just outside the window, both sides of a page border, the first token, the query itself, a key hundreds of tokens back under a wide window -- for
    prompt tiles and for single decoded rows reading the pages; the mixing matrix moves head 1's score into head 0."""
    from mistralrs_amd.hybrid import RaggedBatch, _call
    H, G, D, Dv, bs, T = 2, 1, 8, 4, 32, 300
    _, _, sv = _model([layer(heads=H, kv_heads=G, dim=D, vdim=Dv, mlp=None)], dev, dtype)
    m, td = sv.m, sv.m.torch_dtype
    att = m.layers[0].mixer
    assert sv.cache.reserve(1, T)
    blocks = sv.cache.kv.get_block_ids(1)
    g = torch.Generator().manual_seed(11)
    v = torch.randn(T, G, Dv, generator=g).to(torch.bfloat16)
    talk = torch.tensor([[0.0, 1.0], [1.0, 0.0]])            # the heads swap scores
    pb = torch.tensor([-20.0, -20.0])
    slopes = torch.zeros(H)
    zeros_gate = torch.zeros(64, H, device=dev)               # sigmoid(0) = 1 / 2 on every head output
    blk, off = torch.tensor([blocks[t // bs] for t in range(T)], device=dev), torch.arange(T, device=dev) % bs
    for size in (37, 290):
        cases = []
        for i in (60, 64, 95, 96, 299):
            for j in (i - size, i - size + 1, 0, i, 31, 32, i - 1, i - 64, i - 65):
                if 0 <= j <= i:
                    cases.append((i, j))
        for i, j in cases:
            k = torch.randn(T, G, D, generator=g).to(torch.bfloat16) * 0.05
            k[j, 0, 0] = 6.0
            q = torch.zeros(H, D, dtype=torch.bfloat16)
            q[1, 0] = 6.0                                    # only head 1 asks; after the swap only head 0 answers
            seen = i - j < size
            want = torch.zeros(H, Dv, dtype=torch.float64)
            if seen:
                want[0] = 0.5 * v[j, 0].double() / (1 + math.exp(-(36.0 - 20.0)))
            att.k_cache[blk, :, off] = k.to(dev, td)        # pages through the block table, as the cache-write kernel lays them out
            att.v_cache[blk, :, off] = v.to(dev, td)
            for rows in ("decode", "prompt"):
                p0 = i if rows == "decode" else max(0, i - 20)
                n = i - p0 + 1
                b = RaggedBatch.build([{"tokens": [0] * n, "pos0": p0, "slot": 0, "blocks": blocks, "want": []}], bs, dev)
                qq = torch.zeros(n, H * D, dtype=td, device=dev)
                qq[n - 1] = q.reshape(-1).to(dev, td)
                out = torch.empty(n, H * Dv, dtype=td, device=dev)
                ks = 5 if (rows == "decode" or i == 64) else 0            # the keys dealt to several workgroups, or all to one
                scratch = torch.full((max(ks, 1), n, H * Dv), float("nan"), device=dev)
                _call("mrs_hyb_paged_talk_sigmoid_attn", qq, att.k_cache, att.v_cache, b.block_tables, b.tok_pos, talk.to(dev), pb.to(dev), slopes.to(dev), zeros_gate, H, out,
                      n, H, G, D, Dv, bs, b.max_blocks, size, 1.0, m.dt, b.seg_entry, b.seg_row0, b.seg_len, b.segments, b.seg_rows, scratch if ks else None, ks)
                got = out[n - 1].double().cpu().view(H, Dv)
                assert float((got - want).abs().max()) < (1e-4 if dtype == "float32" else 2e-2), (size, i, j, rows, seen)
    sv.end(1)


@pytest.mark.gpu
def test_distance_bias_and_head_mixing_against_the_restatement(dev):
    """queries and keys scaled up so that the distance bias and the mixing matrix move weights between 0 and 1 (a forgotten slope, a transposed matrix or a bias added before the
    mixing shows as an O(1) error)"""
    cfg = config([layer(heads=4, kv_heads=2, dim=8, vdim=8, size=50, coef=0.8, every=7, mlp=None)])
    w = weights(cfg, 12)
    w["l0.mix.q"] = (w["l0.mix.q"].float() * 3).to(torch.bfloat16)
    w["l0.mix.talk"] = torch.tensor([[1.0, -0.5, 0.0, 2.0], [0.25, 1.0, 0.5, 0.0], [-1.0, 0.0, 1.5, 0.5], [0.0, 3.0, -0.25, 1.0]]).to(torch.bfloat16)
    w["l0.mix.pb"] = torch.tensor([0.5, -2.0, 1.0, -0.5]).to(torch.bfloat16)
    sv = Served(cfg, w, dev)
    t = toks(120, cfg["vocab"], 13)
    lo = []
    want = O.forward(cfg, f64(w), t, lo)
    sv.m.trace_layers = []
    got = sv.step([(1, t)])[0]
    assert rel(sv.m.trace_layers[0].double().cpu(), lo[0]) < 2e-5 and rel(got, want) < 2e-5


# ---------------------------------------------------------------------------------------------------------------- whole models (GPU)
@pytest.mark.gpu
@pytest.mark.parametrize("dtype,bar", [("float32", 3e-5), ("bfloat16", 4e-2)])
def test_whole_prompt_every_layer(dev, dtype, bar):
    cfg = config(STACK)
    w = weights(cfg, 5)
    sv = Served(cfg, w, dev, dtype)
    t = toks(150, cfg["vocab"], 14)
    lo = []
    want = O.forward(cfg, f64(w), t, lo)
    sv.m.trace_layers = []
    got = sv.step([(1, t)])[0]
    for i, (a, b) in enumerate(zip(sv.m.trace_layers, lo)):
        assert close(a.double().cpu(), b, bar), f"residual stream after layer {i}"
    assert close(got, want, bar)


@pytest.mark.gpu
def test_portions_and_decoding_equal_the_whole_prompt(dev):
    """the same 200 tokens: whole; in portions of changing sizes down to two tokens and single tokens; token by token from the start"""
    cfg = config(STACK)
    w = weights(cfg, 6)
    t = toks(200, cfg["vocab"], 15)
    want = O.forward(cfg, f64(w), t)
    sv = Served(cfg, w, dev)
    assert rel(sv.step([(1, t)])[0], want) < 3e-5
    cuts = [2, 3, 1, 64, 2, 31, 1, 1, 65, 7, 2, 21]
    assert sum(cuts) == 200
    got, at = [], 0
    for c in cuts:
        got += sv.step([(2, t[at:at + c])])
        at += c
    assert rel(torch.cat(got), want) < 3e-5
    got = [sv.step([(3, [x])])[0] for x in t[:80]]
    assert rel(torch.cat(got), want[:80]) < 3e-5


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,bar", [("float32", 3e-5), ("bfloat16", 4e-2)])
def test_mixed_batches_with_reused_pages_and_slots(dev, dtype, bar):
    """five requests of unequal length through a pool of 192 tokens and three slots: portions beside single tokens, a request left out of a step, pages and slots of finished
    requests taken by later ones -- every row against the request alone in the restatement"""
    cfg = config(STACK)
    w = weights(cfg, 7)
    wd = f64(w)
    sv = Served(cfg, w, dev, dtype, max_tokens=192, slots=3)
    req = {r: toks(n, cfg["vocab"], 20 + r) for r, n in ((1, 70), (2, 9), (3, 64), (4, 33), (5, 90))}
    full = {r: O.forward(cfg, wd, t) for r, t in req.items()}
    plan = [[(1, 40), (2, 1)], [(1, 1), (2, 3), (3, 33)], [(2, 5), (3, 1)], [(1, 29), (3, 30)], [(4, 2), (3, 0)], [(4, 31), (5, 60)], [(5, 1), (4, 0)], [(5, 29)]]
    at = {r: 0 for r in req}
    for step in plan:
        parts = [(r, req[r][at[r]:at[r] + n]) for r, n in step if n]
        outs = sv.step(parts)
        for (r, tk), o in zip(parts, outs):
            assert close(o, full[r][at[r]:at[r] + len(tk)], bar), (r, at[r])
            at[r] += len(tk)
            if at[r] == len(req[r]):
                sv.end(r)
    assert at == {r: len(t) for r, t in req.items()}


@pytest.mark.gpu
def test_long_decoding_past_windows_and_temperature_steps(dev):
    cfg = config([layer(size=9, every=11), layer(kv_from=0, size=45, every=64, mlp="moe")])
    w = weights(cfg, 8)
    t = toks(260, cfg["vocab"], 16)
    want = O.forward(cfg, f64(w), t)
    sv = Served(cfg, w, dev)
    got = sv.step([(1, t[:5])]) + [sv.step([(1, [x])])[0] for x in t[5:]]
    assert rel(torch.cat(got), want) < 3e-5


@pytest.mark.gpu
def test_sizes_that_coincide_or_equal_one(dev):
    """one head, one expert of which one is used, a window of one token, a temperature step at every token, key and value sizes equal to the width, one-token prompts"""
    for layers, kw in (([layer(heads=1, kv_heads=1, dim=24, vdim=24, size=1, every=1, mlp=moe(1, 1, 24, 24, scale=1.0))], dict(width=24, vocab=24)),
                       ([layer(heads=2, kv_heads=2, dim=2, vdim=1, size=2, every=2, mlp=dense(1)), layer(heads=2, kv_heads=2, dim=2, vdim=1, size=3, kv_from=0, mlp=None)], dict(width=8, vocab=5))):
        cfg = config(layers, **kw)
        w = weights(cfg, 9)
        t = toks(40, cfg["vocab"], 17)
        want = O.forward(cfg, f64(w), t)
        sv = Served(cfg, w, dev)
        assert rel(sv.step([(1, t[:1])])[0], want[:1]) < 3e-5
        got = sv.step([(2, t[:1])]) + sv.step([(2, t[1:3])]) + sv.step([(2, t[3:])])
        assert rel(torch.cat(got), want) < 3e-5


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,bar", [("float32", 3e-5), ("bfloat16", 5e-2)])
def test_sizes_off_every_vector_width(dev, dtype, bar):
    """width, vocabulary, head sizes, feed-forward and expert sizes that no 16-byte load divides: the element-wise paths of every kernel, prompt and decode"""
    cfg = config([layer(heads=3, kv_heads=1, dim=11, vdim=13, size=19, every=7, mlp=dense(27)), layer(heads=3, kv_heads=1, dim=11, vdim=13, size=70, kv_from=0, mlp=moe(6, 3, 15, 21)),
                  layer(heads=5, kv_heads=5, dim=6, vdim=9, size=0, mlp=moe(3, 2, 7, 0))], vocab=77, width=50)
    w = weights(cfg, 13)
    t = toks(100, cfg["vocab"], 18)
    want = O.forward(cfg, f64(w), t)
    sv = Served(cfg, w, dev, dtype)
    got = sv.step([(1, t[:67])]) + sv.step([(1, t[67:90])]) + [sv.step([(1, [x])])[0] for x in t[90:]]
    assert close(torch.cat(got), want, bar)


@pytest.mark.gpu
@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
def test_greedy_generation_through_scheduler_and_engine(dev, graphs):
    """the package's own entry point: scheduler (pages + slots), engine, sampler; five prompts through three slots, against greedy decoding of the restatement"""
    from mistralrs_amd.cli import make_engine
    from mistralrs_amd.hybrid import HybridDecoder, sobunex_spec
    from mistralrs_amd.sampler import SequenceSampler
    from mistralrs_amd.scheduler import Sequence
    cfg = config([layer(size=9), layer(kv_from=0, size=30, mlp="moe"), layer(heads=2, kv_heads=1, mlp=None)])
    w = weights(cfg, 10)
    m = HybridDecoder(sobunex_spec(cfg), dev, "float32", num_blocks=12, block_size=32, state_slots=3)
    m.load_weights(w.__getitem__)
    core = os.path.exists(_lib.path("core"))
    eng = make_engine(m, 12 * 32, 3, sampler=SequenceSampler(cfg["vocab"], dev, top_k=1) if core else None, max_batched_tokens=48, use_graphs=graphs)
    prompts = [toks(n, cfg["vocab"], 30 + n) for n in (5, 40, 1, 23, 60)]
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
    assert eng.steps["prompt"] >= 2 and eng.steps["completion"] >= 6 and bool(eng._graphs) == graphs


@pytest.mark.gpu
def test_captured_decode_steps_equal_eager_steps(dev):
    """a HIP graph of one decode step for three sequences, captured while two of them are live: every replay (eager work and synchronisation between replays) against the
    eager step function on a second copy of the model, and the pages the warm-up touched are intact"""
    cfg = config(STACK)
    w = weights(cfg, 11)
    a, b = Served(cfg, w, dev), Served(cfg, w, dev)
    prompts = {1: toks(37, cfg["vocab"], 41), 2: toks(3, cfg["vocab"], 42), 3: toks(64, cfg["vocab"], 43)}
    for sv in (a, b):
        sv.step([(1, prompts[1]), (2, prompts[2])])
    g = a.m.capture_decode(3, 8)
    for sv in (a, b):
        sv.step([(3, prompts[3])])
    nxt = {r: toks(12, cfg["vocab"], 50 + r) for r in prompts}
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
    """config.json + model.safetensors on disk -> registry -> `trace` (steps from standard input, logits to files, pages given back and reused) and `generate` (scheduler,
    engine, sampler) -- both against the restatement"""
    from safetensors.torch import save_file
    from mistralrs_amd import cli, registry, trace
    cfg = config([layer(size=10), layer(kv_from=0, size=25, mlp="moe")])
    w = weights(cfg, 12)
    folder = tmp_path / "model"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in w.items()}, str(folder / "model.safetensors"))
    assert registry.architecture_of(str(folder)) == "Sobunex"
    wd = f64(w)
    reqs = {"a": toks(45, cfg["vocab"], 61), "b": toks(20, cfg["vocab"], 62), "c": toks(33, cfg["vocab"], 63)}
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
    if not os.path.exists(_lib.path("core")):
        pytest.skip("the sampler's library is not built")
    prompts = [toks(12, cfg["vocab"], 71), toks(3, cfg["vocab"], 72)]
    args = ["generate", "--model", str(folder), "--dtype", "float32", "--max-new-tokens", "4", "--max-tokens", "256", "--max-seqs", "2"]
    for p in prompts:
        args += ["--prompt-ids", ",".join(map(str, p))]
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
