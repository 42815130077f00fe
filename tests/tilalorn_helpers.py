"""Small random Tilalorn checkpoints for the tests: config dicts, bf16 weights with the checkpoint's tensor names, a folder
on disk for the loader.  Sizes are deliberately unequal (heads != kv_heads, dim != vdim != rot_dim, short windows, groups of
experts) so that a swapped size shows."""
from __future__ import annotations

import torch

from tests.garesun_helpers import rel_rms, write_checkpoint  # noqa: F401


def dense(ff=40):
    return dict(kind="dense", ff=ff)


def moe(experts=6, top=2, ff=16, groups=3, keep=2, scale=1.7):
    return dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top, scale=scale, groups=dict(count=groups, keep=keep)))


def attention(heads=4, kv_heads=2, dim=24, vdim=16, scale=0.2, softcap=7.0, coef=0.25, every=5, kv_from=None, mlp="dense", window=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if softcap:
        m["softcap"] = softcap
    if every:
        m["q_temp"] = dict(coef=coef, every=every)
    if kv_from is not None:
        m["kv_from"] = kv_from
    if window:
        m["mask"] = dict(size=window)
    return dict(type="attention", mixer=m, mlp=(dense() if mlp == "dense" else mlp))


def latent(heads=3, dim=16, rot_dim=8, vdim=24, kv_rank=40, scale=0.3, window=9, base=500.0, mlp="moe"):
    m = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, scale=scale, rot=dict(base=base, dims=rot_dim))
    if window:
        m["mask"] = dict(size=window)
    return dict(type="latent_attention", mixer=m, mlp=(moe() if mlp == "moe" else (dense() if mlp == "dense" else mlp)))


def config(layers, vocab=101, width=56, mult=0.6, eps=1e-5):
    return dict(architecture="Tilalorn", vocab=vocab, width=width, layers=layers, norm=dict(eps=eps), residual_mult=mult)


def weights(cfg, seed=0, gain=1.0):
    g = torch.Generator().manual_seed(seed)
    W, width = {}, cfg["width"]

    def lin(name, out, inn, s=1.0):
        W[name] = (torch.randn(out, inn, generator=g) * (s * gain / inn ** 0.5)).to(torch.bfloat16)

    def vec(name, n, center=0.0, s=0.2):
        W[name] = (center + s * torch.randn(n, generator=g)).to(torch.bfloat16)

    W["embed"] = (torch.randn(cfg["vocab"], width, generator=g) * 0.7).to(torch.bfloat16)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        vec(p + "norm1", width)
        if L["type"] == "attention":
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m.get("vdim", m["dim"])
            lin(p + "mix.q", H * D, width, 2.0)
            vec(p + "mix.q.b", H * D, 0.0, 0.5)
            if m.get("kv_from") is None:
                lin(p + "mix.k", G * D, width, 2.0)
                vec(p + "mix.k.b", G * D, 0.0, 0.5)
                lin(p + "mix.v", G * Dv, width, 2.0)
                vec(p + "mix.v.b", G * Dv, 0.0, 0.5)
            lin(p + "mix.g", H, width, 3.0)
            lin(p + "mix.o", width, H * Dv)
        else:
            H, D, Dr, Dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            lin(p + "mix.q", H * (D + Dr), width, 2.0)
            lin(p + "mix.dkv", R + Dr, width, 2.0)
            vec(p + "mix.dkv.norm", R, 1.0, 0.2)
            lin(p + "mix.uk", H * D, R, 2.0)
            lin(p + "mix.uv", H * Dv, R, 2.0)
            lin(p + "mix.g", H * Dv, width, 3.0)
            lin(p + "mix.o", width, H * Dv)
        ml = L.get("mlp")
        if ml:
            vec(p + "norm2", width)
            if ml["kind"] == "moe":
                lin(p + "mlp.router", ml["router"]["experts"], width, 6.0)           # spread logits: few near ties between experts
                for e in range(ml["router"]["experts"]):
                    lin(p + f"mlp.e{e}.gate", ml["expert"]["ff"], width, 1.5)
                    lin(p + f"mlp.e{e}.up", ml["expert"]["ff"], width, 1.5)
                    lin(p + f"mlp.e{e}.down", width, ml["expert"]["ff"])
            else:
                lin(p + "mlp.gate", ml["ff"], width, 1.5)
                lin(p + "mlp.up", ml["ff"], width, 1.5)
                lin(p + "mlp.down", width, ml["ff"])
    vec("final.norm", width)
    return W


def mixed_layers():
    """both mixers with both feed-forwards and none, a layer that reads an earlier (not the previous) layer's keys and values,
    a window longer than a page, every expert chosen, one group"""
    return [latent(), attention(), latent(heads=2, dim=8, rot_dim=16, vdim=8, kv_rank=24, window=70, mlp="dense"),
            attention(heads=6, kv_heads=2, dim=24, vdim=16, kv_from=1, softcap=None, every=64, mlp=moe(experts=4, top=4, groups=1, keep=1)),
            latent(heads=5, dim=8, rot_dim=2, vdim=40, kv_rank=16, window=3, mlp=None),
            attention(heads=2, kv_heads=2, dim=40, vdim=72, every=None, mlp=None)]
