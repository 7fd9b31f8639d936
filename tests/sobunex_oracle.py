"""TEST INFRASTRUCTURE: a plain, slow restatement of the Sobunex decoder (layer norms around every sublayer, sigmoid attention with a distance bias, mixed head scores,
a query temperature and a per-head output gate, optionally reading another layer's keys and values; dense xIELU and softmax-routed clamped-GLU feed-forwards), one
function per mechanism, in float64 on the CPU.  Shares no code with the product path (mistral.rs_amd/hybrid.py and csrc/hyb_*.hip).

A model is `(cfg, w)`: `cfg` the parsed config dictionary, `w` a dict name -> float64 torch tensor.  Everything works on one whole sequence [T, ...], positions 0 .. T-1.
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def layer_norm(x, w, b, eps):
    """(x - mean) / sqrt(var + eps) * w + b over the last axis, var = mean of squared deviations."""
    mu = x.mean(-1, keepdim=True)
    d = x - mu
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * w + b


def softplus(v):
    return math.log1p(math.exp(-abs(v))) + max(v, 0.0)


def xielu(z, p, q):
    """z > 0: softplus(p) z^2 + z/2;  z <= 0: (1/2 + softplus(q)) (e^z - 1 - z) + z/2."""
    ap, aq = softplus(float(p)), 0.5 + softplus(float(q))
    pos = ap * z * z + 0.5 * z
    neg = aq * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z
    return torch.where(z > 0, pos, neg)


def query_temperature(T, coef, every):
    """Factor on the query at position p: 1 + coef ln(floor((p + 1) / every) + 1)."""
    return torch.tensor([1.0 + coef * math.log((p + 1) // every + 1) for p in range(T)], dtype=F)


def head_slopes(H):
    """slope_h = 2^(-8 (h + 1) / H)."""
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], dtype=F)


def visible(T, size):
    """[T, T] bool: query i sees key j when 0 <= i - j < size (size <= 0: every j <= i)."""
    i = torch.arange(T).view(T, 1)
    j = torch.arange(T).view(1, T)
    m = j <= i
    if size and size > 0:
        m = m & (i - j < size)
    return m


def project_kv(h, w, p, m):
    """Keys [T, G, D] and values [T, G, Dv] of the layer with prefix p from its input h."""
    T = h.shape[0]
    k = (h @ w[p + "k"].T + w[p + "k.b"]).view(T, m["kv_heads"], m["dim"])
    v = (h @ w[p + "v"].T + w[p + "v.b"]).view(T, m["kv_heads"], m["vdim"])
    return k, v


def sigmoid_attention(h, k, v, w, p, m):
    """The mixer after its keys and values are known.  Per head g: s_g[i, j] = scale (q_g[i] . k[j]) - slope_g (i - j); heads are mixed, s'_h = sum_g talk[h, g] s_g;
    the weight of a visible key is sigmoid(s'_h + pb_h) (no normalisation over keys); head outputs are scaled by sigmoid(g_h . input), then projected."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T + w[p + "q.b"]).view(T, H, D)
    qt = m.get("q_temp")
    if qt:
        q = q * query_temperature(T, float(qt["coef"]), int(qt["every"])).view(T, 1, 1)
    rep = H // G
    dist = (torch.arange(T).view(T, 1) - torch.arange(T).view(1, T)).to(F)
    slopes = head_slopes(H)
    s = torch.stack([(q[:, g] @ k[:, g // rep].T) * float(m["scale"]) - slopes[g] * dist for g in range(H)])     # [H, T, T]
    s = torch.einsum("hg,gij->hij", w[p + "talk"], s)
    wt = torch.sigmoid(s + w[p + "pb"].view(H, 1, 1)) * visible(T, int((m.get("mask") or {}).get("size", 0) or 0)).to(F)
    o = torch.stack([wt[hh] @ v[:, hh // rep] for hh in range(H)], 1)                                            # [T, H, Dv]
    gate = torch.sigmoid(h @ w[p + "g"].T)                                                                      # [T, H]
    o = o * gate.view(T, H, 1)
    return o.reshape(T, H * Dv) @ w[p + "o"].T + w[p + "o.b"]


def dense_ff(h, w, p):
    u = h @ w[p + "up"].T + w[p + "up.b"]
    a = xielu(u, w[p + "act"][0], w[p + "act"][1])
    return a @ w[p + "down"].T + w[p + "down.b"]


def clamped_glu_expert(h, w, p, limit):
    """g = min(Wg h, limit), u = clamp(Wu h, -limit, limit); Wd (g sigmoid(1.702 g) (u + 1))."""
    g = torch.clamp(h @ w[p + "gate"].T, max=limit)
    u = torch.clamp(h @ w[p + "up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def route_softmax(h, wr, top, scale):
    """softmax over all experts; the `top` largest; weights = the chosen scores * scale, not renormalised.  Returns (ids [T, top], weights [T, top])."""
    s = torch.softmax(h @ wr.T, -1)
    val, idx = torch.topk(s, top, dim=-1)
    return idx, val * scale


def moe_ff(h, w, p, f):
    r = f["router"]
    idx, wt = route_softmax(h, w[p + "router"], int(r["top"]), float(r.get("scale", 1.0)))
    out = torch.zeros(h.shape[0], w[p + "e0.down"].shape[0], dtype=F)
    lim = float(f["expert"]["limit"])
    for t in range(h.shape[0]):
        for k in range(idx.shape[1]):
            e = int(idx[t, k])
            out[t] += wt[t, k] * clamped_glu_expert(h[t:t + 1], w, f"{p}e{e}.", lim)[0]
    if f.get("shared"):
        out = out + clamped_glu_expert(h, w, p + "shared.", float(f["shared"]["limit"]))
    return out


def forward(cfg, w, tokens, layers_out=None):
    """Logits [T, vocab] of one whole sequence."""
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    kv = {}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        ln = lambda name, v: layer_norm(v, w[p + name], w[p + name + ".b"], eps)
        h = ln("norm1", x)
        if m.get("kv_from") is not None:
            k, v = kv[int(m["kv_from"])]
        else:
            k, v = kv[i] = project_kv(h, w, p + "mix.", m)
        x = x + ln("norm1b", sigmoid_attention(h, k, v, w, p + "mix.", m))
        f = L.get("mlp")
        if f:
            h = ln("norm2", x)
            y = dense_ff(h, w, p + "mlp.") if f["kind"] == "dense" else moe_ff(h, w, p + "mlp.", f)
            x = x + ln("norm2b", y)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = layer_norm(x, w["final.norm"], w["final.norm.b"], eps)
    return x @ w["head"].T
