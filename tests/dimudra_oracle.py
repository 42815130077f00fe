"""Plain float64 restatement of the Dimudra decoder: one function per mechanism, whole sequences only, dense masks, explicit
token loops for the recurrences.  No cache, no state hand-over, no packed weights - nothing is shared with the product path.

Notation: h [T, width] the input of a sublayer, W [out, in] applied as h @ W.T, p the position (0-based) of a token.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms(y, eps):
    return y / torch.sqrt((y * y).mean(dim=-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    """RMS norm whose weight is ONE number"""
    return rms(x, eps) * g


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def causal_conv(h, w, bias=None):
    """h [T, C], w [C, taps]: out_t = sum_j w[:, j] * h_(t - taps + 1 + j), zeros before the first token (the last column
    of w meets the token itself)"""
    T, taps = h.shape[0], w.shape[1]
    out = torch.zeros_like(h)
    for j in range(taps):
        back = taps - 1 - j
        if back < T:
            out[back:] += h[: T - back] * w[:, j]
    return out if bias is None else out + bias


def rotate_half_partial(x, dims, base):
    """x [T, heads, D]: the pair (i, i + dims / 2), i < dims / 2, turns by p * base^(-2 i / dims); dimensions >= dims pass"""
    if not dims:
        return x
    T, half = x.shape[0], dims // 2
    f = torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    ang = torch.arange(T, dtype=F64)[:, None] * f[None]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def softmax_attention(q, k, v, scale, window=0, sink=False):
    """q [T, H, D], k [T, G, D], v [T, G, Dv] -> [T, H, Dv].  Query i sees key j when 0 <= i - j (< window when window > 0).
    sink: one more term exp(0) in the denominator that carries no value."""
    T, H, _ = q.shape
    G = k.shape[1]
    i = torch.arange(T)
    dist = i[:, None] - i[None, :]
    seen = dist >= 0
    if window > 0:
        seen &= dist < window
    out = torch.zeros(T, H, v.shape[-1], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~seen, -math.inf)
        m = s.max(dim=-1, keepdim=True).values
        if sink:
            m = torch.clamp(m, min=0.0)
        e = torch.exp(s - m)
        den = e.sum(dim=-1, keepdim=True) + (torch.exp(-m) if sink else 0.0)
        out[:, h] = (e / den) @ v[:, g]
    return out


def windowed_attention_mixer(h, W, p, m, eps):
    """the left half of a 'parallel' mixer: biased projections, RMS norm over the WHOLE q (and k) row with a weight, no
    positions, sliding window, sigmoid gate on the concatenated heads"""
    T = h.shape[0]
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = rms(h @ W[p + "q"].T + W[p + "q.b"], eps) * W[p + "q.norm"]
    k = rms(h @ W[p + "k"].T + W[p + "k.b"], eps) * W[p + "k.norm"]
    v = h @ W[p + "v"].T + W[p + "v.b"]
    o = softmax_attention(q.view(T, H, D), k.view(T, G, D), v.view(T, G, Dv), float(m["scale"]), window=int((m.get("mask") or {}).get("size") or 0))
    return (o.reshape(T, H * Dv) * torch.sigmoid(h @ W[p + "g"].T)) @ W[p + "o"].T


def selective_scan_mixer(h, W, p, m):
    """the right half of a 'parallel' mixer: S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n,  y_c = S[c, :] . C + D_c x_c"""
    T = h.shape[0]
    inner, N, R = int(m["inner"]), int(m["state"]), int(m["dt_rank"])
    xz = h @ W[p + "in"].T
    x, z = xz[:, :inner], xz[:, inner:]
    x = silu(causal_conv(x, W[p + "conv"], W[p + "conv.b"]))
    dbc = x @ W[p + "x"].T
    dt = softplus(dbc[:, :R] @ W[p + "dt"].T + W[p + "dt.b"])
    B, C = dbc[:, R: R + N], dbc[:, R + N: R + 2 * N]
    A = -torch.exp(W[p + "A_log"])
    S = torch.zeros(inner, N, dtype=F64)
    y = torch.zeros(T, inner, dtype=F64)
    for t in range(T):
        S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + W[p + "D"] * x[t]
    return (y * silu(z)) @ W[p + "o"].T


def parallel_mixer(h, W, p, m, eps):
    left = windowed_attention_mixer(h, W, p + "left.", m["left"], eps)
    right = selective_scan_mixer(h, W, p + "right.", m["right"])
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right


def hgrn2_mixer(h, W, p, m, eps):
    """per head S <- diag(f) S + (1 - f) v^T, o = S^T q; the forget gate is bounded from below by `lower`"""
    T = h.shape[0]
    H, D, Dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = silu(h @ W[p + "q"].T).view(T, H, D)
    v = (h @ W[p + "v"].T).view(T, H, Dv)
    lo = W[p + "lower"]
    f = (lo + (1.0 - lo) * torch.sigmoid(h @ W[p + "f"].T + W[p + "f.b"])).view(T, H, D)
    S = torch.zeros(H, D, Dv, dtype=F64)
    o = torch.zeros(T, H, Dv, dtype=F64)
    for t in range(T):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    o = rms(o, eps) * W[p + "norm"]
    return o.reshape(T, H * Dv) @ W[p + "o"].T


def attention_mixer(h, W, p, m, eps):
    """rotated (rotate-half, partial), then unit-RMS q and k per head; causal; a sink in the softmax; sigmoid gate"""
    T = h.shape[0]
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    rot = m.get("rot") or {}
    dims, base = int(rot.get("dims", 0)), float(rot.get("base", 10000.0))
    q = rms(rotate_half_partial((h @ W[p + "q"].T).view(T, H, D), dims, base), eps)
    k = rms(rotate_half_partial((h @ W[p + "k"].T).view(T, G, D), dims, base), eps)
    v = (h @ W[p + "v"].T).view(T, G, Dv)
    o = softmax_attention(q, k, v, float(m["scale"]), window=0, sink=True)
    return (o.reshape(T, H * Dv) * torch.sigmoid(h @ W[p + "g"].T)) @ W[p + "o"].T


def glu_expert(h, W, p):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def route(z, correction, top, count, keep):
    """z [T, E] router logits -> (chosen [T, top] indices, weights [T, top]).  Scores sigmoid(z); the choice uses scores +
    correction, inside the `keep` groups (of `count` equal groups of neighbours) whose two best choice scores add up highest;
    weights are the chosen scores without correction, normalised."""
    T, E = z.shape
    s = torch.sigmoid(z)
    c = s + correction
    gs = E // count
    grp = c.view(T, count, gs)
    gscore = grp.topk(min(2, gs), dim=-1).values.sum(dim=-1)
    kept = torch.zeros(T, count, dtype=torch.bool)
    kept.scatter_(1, gscore.topk(keep, dim=-1).indices, True)
    allowed = kept[:, :, None].expand(T, count, gs).reshape(T, E)
    chosen = c.masked_fill(~allowed, -math.inf).topk(top, dim=-1).indices
    w = s.gather(1, chosen)
    return chosen, w / (w.sum(dim=-1, keepdim=True) + 1e-20)


def moe(h, W, p, mlp):
    r = mlp["router"]
    E, top = int(r["experts"]), int(r["top"])
    g = r.get("groups") or {}
    count = int(g.get("count", 1))
    keep = int(g.get("keep", count))
    corr = W[p + "correction"] if p + "correction" in W else torch.zeros(E, dtype=F64)
    chosen, w = route(h @ W[p + "router"].T, corr, top, count, keep)
    out = torch.zeros_like(h)
    for e in range(E):
        sel = (chosen == e)
        rows = sel.any(dim=-1)
        if rows.any():
            out[rows] += glu_expert(h[rows], W, p + f"e{e}.") * (w * sel)[rows].sum(dim=-1, keepdim=True)
    if mlp.get("shared"):
        out = out + glu_expert(h, W, p + "shared.") * torch.sigmoid(h @ W[p + "shared.sg"].T)
    return out


MIXERS = {"parallel": parallel_mixer, "hgrn2": hgrn2_mixer, "attention": attention_mixer}


def layer_runs(cfg):
    """the order in which layers run: the looped span `times` times in a row -> [(layer, first of a later pass)]"""
    n = len(cfg["layers"])
    loop = cfg.get("loop") or {}
    a, b, times = int(loop.get("start", 0)), int(loop.get("stop", 0)), int(loop.get("times", 1))
    if b <= a or times <= 1:
        return [(i, False) for i in range(n)]
    runs = [(i, False) for i in range(a)]
    for rep in range(times):
        runs += [(i, rep > 0 and i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def forward(cfg, W, tokens):
    """-> (logits [T, vocab], [stream after every layer run])   W: {name: float64 tensor}"""
    eps = float(cfg["norm"]["eps"])
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    canon = bool((cfg.get("canon") or {}).get("taps", 0))
    x0 = x.clone()
    streams = []
    for i, readd in layer_runs(cfg):
        L, p = cfg["layers"][i], f"l{i}."
        if readd:
            x = x + x0
        h = scalar_norm(x, W[p + "norm1"], eps)
        if canon:
            h = h + causal_conv(h, W[p + "canon1"])
        if L["type"] == "parallel":
            x = x + parallel_mixer(h, W, p + "mix.", L["mixer"], eps)
        elif L["type"] == "hgrn2":
            x = x + hgrn2_mixer(h, W, p + "mix.", L["mixer"], eps)
        else:
            x = x + attention_mixer(h, W, p + "mix.", L["mixer"], eps)
        if L.get("mlp"):
            x = x + moe(scalar_norm(x, W[p + "norm2"], eps), W, p + "mlp.", L["mlp"])
        streams.append(x.clone())
    return scalar_norm(x, W["final.norm"], eps) @ W["head"].T, streams
