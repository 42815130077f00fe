"""Small random Dimudra checkpoints for the tests: config dicts, bf16 weights with the checkpoint's tensor names, a folder on
disk for the loader.  Sizes are deliberately unequal (heads != kv_heads, dim != vdim, inner != width, short windows, groups of
experts, a looped span that does not start at layer 0) so that a swapped size shows."""
from __future__ import annotations

import math

import torch

from tests.garesun_helpers import rel_rms, write_checkpoint  # noqa: F401


def moe(experts=6, top=2, ff=16, groups=3, keep=2, shared=24):
    m = dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top, groups=dict(count=groups, keep=keep)))
    if shared:
        m["shared"] = dict(ff=shared)
    return m


def _mlp(mlp):
    return moe() if mlp == "moe" else mlp


def parallel(heads=4, kv_heads=2, dim=12, vdim=20, scale=0.3, window=9, inner=40, state=6, dt_rank=5, conv=3, left_scale=0.8,
             right_scale=1.3, mlp="moe"):
    left = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if window:
        left["mask"] = dict(size=window)
    return dict(type="parallel", mixer=dict(left=left, left_scale=left_scale, right=dict(inner=inner, state=state, dt_rank=dt_rank, conv=conv),
                                            right_scale=right_scale), mlp=_mlp(mlp))


def hgrn2(heads=3, dim=10, vdim=14, mlp="moe"):
    return dict(type="hgrn2", mixer=dict(heads=heads, dim=dim, vdim=vdim), mlp=_mlp(mlp))


def attention(heads=6, kv_heads=2, dim=16, vdim=12, scale=0.35, rot_dims=6, base=300.0, mlp="moe"):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if rot_dims:
        m["rot"] = dict(base=base, dims=rot_dims)
    return dict(type="attention", mixer=m, mlp=_mlp(mlp))


def config(layers, vocab=101, width=56, eps=1e-5, taps=4, escale=3.0, loop=None):
    cfg = dict(architecture="Dimudra", vocab=vocab, width=width, layers=layers, norm=dict(eps=eps), embedding=dict(scale=escale))
    if taps:
        cfg["canon"] = dict(taps=taps)
    if loop:
        cfg["loop"] = dict(start=loop[0], stop=loop[1], times=loop[2])
    return cfg


def weights(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    W, width = {}, cfg["width"]
    taps = (cfg.get("canon") or {}).get("taps", 0)

    def lin(name, out, inn, s=1.0):
        W[name] = (torch.randn(out, inn, generator=g) * (s / inn ** 0.5)).to(torch.bfloat16)

    def vec(name, n, center=0.0, s=0.2):
        W[name] = (center + s * torch.randn(n, generator=g)).to(torch.bfloat16)

    def one(name):
        W[name] = (1.0 + 0.3 * torch.randn((), generator=g)).to(torch.bfloat16)

    def attn(p, m, biased):
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m.get("vdim", m["dim"])
        lin(p + "q", H * D, width, 2.0)
        lin(p + "k", G * D, width, 2.0)
        lin(p + "v", G * Dv, width, 2.0)
        lin(p + "g", H * Dv, width, 3.0)
        lin(p + "o", width, H * Dv)
        if biased:
            vec(p + "q.b", H * D, 0.0, 0.5)
            vec(p + "k.b", G * D, 0.0, 0.5)
            vec(p + "v.b", G * Dv, 0.0, 0.5)
            vec(p + "q.norm", H * D, 1.0, 0.3)
            vec(p + "k.norm", G * D, 1.0, 0.3)

    W["embed"] = (torch.randn(cfg["vocab"], width, generator=g) * 0.4).to(torch.bfloat16)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        one(p + "norm1")
        if taps:
            W[p + "canon1"] = (0.4 * torch.randn(width, taps, generator=g)).to(torch.bfloat16)
        if L["type"] == "parallel":
            attn(p + "mix.left.", m["left"], True)
            r = m["right"]
            C, N, R, ct = r["inner"], r["state"], r["dt_rank"], r["conv"]
            pr = p + "mix.right."
            lin(pr + "in", 2 * C, width, 1.0)
            W[pr + "conv"] = (0.5 * torch.randn(C, ct, generator=g)).to(torch.bfloat16)
            vec(pr + "conv.b", C, 0.0, 0.3)
            lin(pr + "x", R + 2 * N, C, 1.0)
            lin(pr + "dt", C, R, 1.5)
            vec(pr + "dt.b", C, -2.0, 1.0)
            W[pr + "A_log"] = torch.log(1.0 + torch.arange(N, dtype=torch.float32)).repeat(C, 1).add(0.3 * torch.randn(C, N, generator=g)).to(torch.bfloat16)
            vec(pr + "D", C, 1.0, 0.3)
            lin(pr + "o", width, C, 1.5)
        elif L["type"] == "hgrn2":
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            lin(p + "mix.q", H * D, width, 2.0)
            lin(p + "mix.f", H * D, width, 3.0)
            vec(p + "mix.f.b", H * D, 0.5, 1.0)
            W[p + "mix.lower"] = (0.9 * torch.rand(H * D, generator=g)).to(torch.bfloat16)
            lin(p + "mix.v", H * Dv, width, 2.0)
            vec(p + "mix.norm", Dv, 1.0, 0.3)
            lin(p + "mix.o", width, H * Dv)
        else:
            attn(p + "mix.", m, False)
        ml = L.get("mlp")
        if ml:
            one(p + "norm2")
            E, ff = ml["router"]["experts"], ml["expert"]["ff"]
            lin(p + "mlp.router", E, width, 1.5)                 # logits inside the sigmoid's open range: saturated scores would all but tie
            W[p + "mlp.correction"] = (0.3 * torch.randn(E, generator=g)).to(torch.bfloat16)
            names = [f"e{e}" for e in range(E)] + (["shared"] if ml.get("shared") else [])
            for n in names:
                f = ml["shared"]["ff"] if n == "shared" else ff
                lin(p + f"mlp.{n}.gate", f, width, 1.5)
                lin(p + f"mlp.{n}.up", f, width, 1.5)
                lin(p + f"mlp.{n}.down", width, f)
            if ml.get("shared"):
                lin(p + "mlp.shared.sg", 1, width, 3.0)
    one("final.norm")
    lin("head", cfg["vocab"], width, 2.0)
    return W


def as_f64(W):
    return {k: v.to(torch.float64) for k, v in W.items()}


def mixed_layers():
    """every mixer with and without a feed-forward, a window longer than a page, every expert chosen, one group, no shared
    expert, full and no rotation, kv_heads = heads and = 1"""
    return [hgrn2(),
            parallel(),
            attention(),
            parallel(heads=2, kv_heads=2, dim=8, vdim=8, window=70, inner=24, state=3, dt_rank=2, conv=2, mlp=moe(experts=4, top=4, groups=1, keep=1, shared=0)),
            attention(heads=3, kv_heads=1, dim=8, vdim=40, rot_dims=8, mlp=None),
            hgrn2(heads=1, dim=40, vdim=8, mlp=None)]


def mixed_config(**kw):
    """layers 1..3 run twice in a row (the span starts after layer 0): 9 runs"""
    return config(mixed_layers(), loop=(1, 4, 2), **kw)
