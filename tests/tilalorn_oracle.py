"""Plain restatement of the Tilalorn decoder for the tests: one function per mechanism, whole prompts, dense masks, per-head
keys and values written out (no absorbed maps, no cache, no pages), in the dtype it is given (float64 in the tests).  It
shares no code with the product path.

Notation: x [T, W] the residual stream, p the positions 0..T-1, eps the norm constant, m the residual multiplier.
    norm(x, w)   = x / sqrt(mean(x^2) + eps) * (1 + w)
    layer        : x <- x + m * mixer(norm(x, w1));   x <- x + m * ff(norm(x, w2))   (the second step only with a feed-forward)
    logits       = norm(x, w_final) E^T   with the embedding table E
"""
from __future__ import annotations

import math

import torch


def unit_rms(y, eps):
    return y / torch.sqrt(y.pow(2).mean(-1, keepdim=True) + eps)


def norm(x, w, eps):
    return unit_rms(x, eps) * (1.0 + w)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotate_half(y, pos, dims, base):
    """y [T, ..., D]: dimension i < dims / 2 is paired with i + dims / 2, angle pos * base^(-2 i / dims); the rest passes"""
    if not dims:
        return y
    half = dims // 2
    f = torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(half)], dtype=y.dtype)
    a = pos.to(y.dtype).view(-1, *([1] * (y.dim() - 2)), 1) * f
    u, v = y[..., :half], y[..., half:dims]
    return torch.cat([u * torch.cos(a) - v * torch.sin(a), v * torch.cos(a) + u * torch.sin(a), y[..., dims:]], -1)


def visible(T, window):
    """[T, T] bool: query i sees key j when 0 <= i - j (< window when there is one)"""
    d = torch.arange(T).view(-1, 1) - torch.arange(T).view(1, -1)
    return (d >= 0) & ((d < window) if window else torch.ones_like(d, dtype=torch.bool))


def softmax_read(scores, vis, v):
    """scores [H, T, T], v [T, H, Dv] -> [T, H, Dv]"""
    w = torch.softmax(scores.masked_fill(~vis, float("-inf")), -1)
    return torch.einsum("hij,jhd->ihd", w, v)


def attention_mixer(W, p, m, h, eps, kv=None):
    """grouped-head attention; kv: (normed keys [T, G, D], values [T, G, Dv]) of the layer it borrows from -> (out, kv)"""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m.get("vdim", m["dim"])
    pos = torch.arange(T)
    q = unit_rms((h @ W[p + "q"].T + W[p + "q.b"]).view(T, H, D), eps)
    if kv is None:
        k = unit_rms((h @ W[p + "k"].T + W[p + "k.b"]).view(T, G, D), eps)
        v = (h @ W[p + "v"].T + W[p + "v.b"]).view(T, G, Dv)
        kv = (k, v)
    k, v = kv
    qt = m.get("q_temp")
    if qt:
        q = q * (1.0 + qt["coef"] * torch.log(torch.floor((pos + 1) / qt["every"]) + 1.0)).to(h.dtype).view(T, 1, 1)
    k, v = k.repeat_interleave(H // G, 1), v.repeat_interleave(H // G, 1)        # query head a reads key head a // (H / G)
    s = torch.einsum("ihd,jhd->hij", q, k) * m["scale"]
    if m.get("softcap"):
        s = m["softcap"] * torch.tanh(s / m["softcap"])
    o = softmax_read(s, visible(T, (m.get("mask") or {}).get("size")), v)
    o = o * torch.sigmoid(h @ W[p + "g"].T).view(T, H, 1)
    return o.reshape(T, H * Dv) @ W[p + "o"].T, kv


def latent_mixer(W, p, m, h, eps):
    T = h.shape[0]
    H, D, Dr, Dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    base = (m.get("rot") or {}).get("base", 1.0)
    q = (h @ W[p + "q"].T).view(T, H, D + Dr)
    d = h @ W[p + "dkv"].T
    c = unit_rms(d[:, :R], eps) * W[p + "dkv.norm"]
    k_rot = rotate_half(d[:, R:], pos, Dr, base)                                # [T, Dr], one for all heads
    q_rot = rotate_half(q[..., D:], pos, Dr, base)
    k = (c @ W[p + "uk"].T).view(T, H, D)
    v = (c @ W[p + "uv"].T).view(T, H, Dv)
    s = (torch.einsum("ihd,jhd->hij", q[..., :D], k) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * m["scale"]
    o = softmax_read(s, visible(T, (m.get("mask") or {}).get("size")), v).reshape(T, H * Dv)
    return (o * torch.sigmoid(h @ W[p + "g"].T)) @ W[p + "o"].T


def dense_ff(W, p, h):
    return (gelu_tanh(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def route(z, r):
    """router logits z [T, E] -> [T, E] weights: scores = softmax over all experts; consecutive experts are cut into `count` blocks
    of one size, a block ranks by its best score, `keep` blocks stay; the `top` best experts inside them get score * scale, every
    other expert 0 (lowest index wins a tie)"""
    T, E = z.shape
    s = torch.softmax(z, -1)
    g = r.get("groups") or {}
    count = g.get("count", 1)
    keep = g.get("keep", count)
    out = torch.zeros_like(s)
    for t in range(T):
        gs = [max(s[t, e].item() for e in range(c * (E // count), (c + 1) * (E // count))) for c in range(count)]
        groups = sorted(range(count), key=lambda c: (-gs[c], c))[:keep]
        cand = [e for e in range(E) if e // (E // count) in groups]
        for e in sorted(cand, key=lambda e: (-s[t, e].item(), e))[: r["top"]]:
            out[t, e] = s[t, e] * r.get("scale", 1.0)
    return out


def moe_ff(W, p, ml, h):
    w = route(h @ W[p + "router"].T, ml["router"])
    out = torch.zeros_like(h)
    for e in range(ml["router"]["experts"]):
        rows = torch.nonzero(w[:, e]).view(-1)
        if rows.numel():
            he = h[rows]
            y = (torch.nn.functional.silu(he @ W[p + f"e{e}.gate"].T) * (he @ W[p + f"e{e}.up"].T)) @ W[p + f"e{e}.down"].T
            out[rows] += w[rows, e].view(-1, 1) * y
    return out


class Oracle:
    def __init__(self, cfg, W, dtype=torch.float64):
        self.cfg, self.dtype = cfg, dtype
        self.W = {k: v.to(dtype) for k, v in W.items()}

    def forward(self, ids, layers_out=None):
        """ids [T] -> logits [T, vocab]; layers_out (a list) receives the stream after every layer"""
        cfg, W = self.cfg, self.W
        eps, mult = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
        x = W["embed"][torch.as_tensor(ids).long()]
        kvs = {}
        for i, L in enumerate(cfg["layers"]):
            p, m = f"l{i}.", L["mixer"]
            h = norm(x, W[p + "norm1"], eps)
            if L["type"] == "attention":
                src = m.get("kv_from")
                y, kvs[i] = attention_mixer(W, p + "mix.", m, h, eps, None if src is None else kvs[src])
            else:
                y = latent_mixer(W, p + "mix.", m, h, eps)
            x = x + mult * y
            if L.get("mlp"):
                h = norm(x, W[p + "norm2"], eps)
                y = moe_ff(W, p + "mlp.", L["mlp"], h) if L["mlp"].get("kind") == "moe" else dense_ff(W, p + "mlp.", h)
                x = x + mult * y
            if layers_out is not None:
                layers_out.append(x.clone())
        return norm(x, W["final.norm"], eps) @ W["embed"].T
