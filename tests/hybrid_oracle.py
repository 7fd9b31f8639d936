"""TEST INFRASTRUCTURE: a plain, slow restatement of the hybrid decoder family (state-space-duality mixers, windowed attention with kept first tokens,
sigmoid-routed experts with a gated shared expert), one function per mechanism, in float64 on the CPU.  Shares no code with the product path
(mistral.rs_amd/hybrid.py and csrc/hyb_*.hip): every function below is written from the equations in its docstring.

A model is `(cfg, w)`: `cfg` the parsed config dictionary, `w` a dict name -> float64 torch tensor.
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    """Layer norm of the family: unit RMS, then (1 + w) (weights are kept as offsets from one)."""
    return rms_unit(x, eps) * (1.0 + w)


def norm_plain(x, w, eps):
    return rms_unit(x, eps) * w


def rope_frequencies(dims, base, scaling=None):
    """f_i = base^(-2i/dims), i < dims/2; optional wavelength-dependent scaling: wavelengths below original/high keep f, above original/low use f/factor,
    in between a linear blend in s = (original/l - low) / (high - low)."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            fac, lo, hi, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            l = 2.0 * math.pi / f
            if l < orig / hi:
                pass
            elif l > orig / lo:
                f = f / fac
            else:
                s = (orig / l - lo) / (hi - lo)
                f = (1.0 - s) * f / fac + s * f
        out.append(f)
    return torch.tensor(out, dtype=F)


def rope_interleaved(x, pos, freqs):
    """x [T, heads, dim]; the pair (x[2i], x[2i+1]), i < len(freqs), is turned by pos * f_i; the remaining dimensions pass."""
    x = x.clone()
    r = 2 * len(freqs)
    ang = pos.to(F)[:, None] * freqs[None, :]          # [T, r/2]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., 0:r:2].clone(), x[..., 1:r:2].clone()
    x[..., 0:r:2] = u * c - v * s
    x[..., 1:r:2] = v * c + u * s
    return x


def visible(i, j, size, keep_first):
    """Window with kept first tokens: query i sees key j."""
    return j <= i and (i - j < size or j < keep_first)


def windowed_attention(q, k, v, scale, size, keep_first, pos_q=None):
    """q [Tq, H, D], k [Tk, G, D], v [Tk, G, Dv]; key j sits at position j, query row r at pos_q[r] (default r).  Softmax over the visible keys, one (query, head) at a time."""
    Tq, H, _ = q.shape
    G, Dv = k.shape[1], v.shape[2]
    pos_q = list(range(Tq)) if pos_q is None else [int(p) for p in pos_q]
    out = torch.zeros(Tq, H, Dv, dtype=F)
    for hh in range(H):
        g = hh // (H // G)
        for r, i in enumerate(pos_q):
            js = [j for j in range(min(i + 1, k.shape[0])) if visible(i, j, size if size > 0 else i + 1, keep_first)]
            s = (k[js, g] @ q[r, hh]) * scale
            pr = torch.softmax(s, 0)
            out[r, hh] = pr @ v[js, g]
    return out


def attention_mixer(h, m, w, p, eps):
    """h [T, width] of ONE sequence from position 0.  m: the mixer's config."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = h @ w[p + "q"].T, h @ w[p + "k"].T, h @ w[p + "v"].T
    q = norm_plain(q, w[p + "q.norm"], eps).view(T, H, D)   # over the whole projection, before the split into heads
    k = norm_plain(k, w[p + "k.norm"], eps).view(T, G, D)
    v = v.view(T, G, Dv)
    rot = m.get("rot")
    pos = torch.arange(T)
    if rot:
        fr = rope_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q, k = rope_interleaved(q, pos, fr), rope_interleaved(k, pos, fr)
    out = windowed_attention(q, k, v, m["scale"], m["mask"]["size"], m["mask"]["keep_first"])
    return out.reshape(T, H * Dv) @ w[p + "o"].T


def mamba2_mixer(h, m, w, p, eps):
    """State-space-duality mixer on ONE sequence from a zero state.  h [T, width]."""
    T = h.shape[0]
    Hh, P, N, G, taps, ng = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"], m["norm_groups"]
    inner = Hh * P
    u = h @ w[p + "in"].T
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N:]
    assert dt.shape[1] == Hh
    cw, cb = w[p + "conv"], w[p + "conv.b"]
    pad = torch.cat([torch.zeros(taps - 1, xbc.shape[1], dtype=F), xbc], 0)
    conv = torch.stack([(pad[t:t + taps].T * cw).sum(1) + cb for t in range(T)])      # the last tap multiplies the current token
    conv = silu(conv)
    x = conv[:, :inner].view(T, Hh, P)
    B = conv[:, inner:inner + G * N].view(T, G, N)
    Cc = conv[:, inner + G * N:].view(T, G, N)
    dt = torch.nn.functional.softplus(dt + w[p + "dt_bias"], threshold=1e9)
    A = -torch.exp(w[p + "A_log"])
    y = torch.zeros(T, Hh, P, dtype=F)
    for hh in range(Hh):
        g = hh // (Hh // G)
        S = torch.zeros(N, P, dtype=F)
        for t in range(T):
            S = torch.exp(A[hh] * dt[t, hh]) * S + dt[t, hh] * torch.outer(B[t, g], x[t, hh])
            y[t, hh] = S.T @ Cc[t, g] + w[p + "D"][hh] * x[t, hh]
    y = y.reshape(T, inner) * silu(z)                      # the gate comes before the norm
    y = rms_unit(y.view(T, ng, inner // ng), eps).reshape(T, inner) * w[p + "norm"]
    return y @ w[p + "o"].T


def expert(h, w, p):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def moe_ffn(h, f, w, p):
    """Sigmoid router, the `top` largest scores, un-renormalised, applied to the expert's INPUT; plus a shared expert times sigmoid(W_sg h)."""
    T = h.shape[0]
    E, top = f["router"]["experts"], f["router"]["top"]
    s = torch.sigmoid(h @ w[p + "router"].T)
    out = torch.zeros(T, w[p + "e0.down"].shape[0], dtype=F)
    for t in range(T):
        order = sorted(range(E), key=lambda e: (-float(s[t, e]), e))[:top]
        for e in order:
            out[t] += expert(s[t, e] * h[t:t + 1], w, f"{p}e{e}.")[0]
    if f.get("shared"):
        out = out + torch.sigmoid(h @ w[p + "shared.sg"].T) * expert(h, w, p + "shared.")
    return out


def forward(cfg, w, tokens, keep_layers=False):
    """Logits [T, vocab] of one sequence; with keep_layers also the residual stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    trail = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        hn = norm_one_plus(x, w[p + "norm1"], eps)
        mixer = {"mamba2": mamba2_mixer, "attention": attention_mixer}[layer["type"]]
        x = x + mixer(hn, layer["mixer"], w, p + "mix.", eps)
        if layer.get("mlp"):
            x = x + moe_ffn(norm_one_plus(x, w[p + "norm2"], eps), layer["mlp"], w, p + "mlp.")
        trail.append(x.clone())
    logits = norm_one_plus(x, w["final.norm"], eps) @ w["head"].T
    return (logits, torch.stack(trail)) if keep_layers else logits
