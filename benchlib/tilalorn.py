"""`bench.py --workload tilalorn-compare`: prefill and decode throughput of the Tilalorn design (grouped-head attention with
unit-RMS queries / keys, capped scores and shared key / value caches; latent attention with rotary positions inside a sliding
window; dense gated-gelu and group-limited silu expert feed-forwards; pre-norm fp32 residual stream) next to the framework's
closest model, Garesun (latent attention and mixtures of experts on the same ragged step), at the same width, depth, head
count, head size and feed-forward work per token - random weights, synthetic token ids, bf16.  Not the headline metric: one
JSON line of its own."""
from __future__ import annotations

import torch

from benchlib.garesun import SIZES, _measure, garesun_cfg, garesun_weights


def tilalorn_cfg(s, window=1024):
    H, hd, W = s["heads"], s["hd"], s["width"]
    # the comparison model runs 2 of 8 experts + a shared one of inter / 4 each with two matrices per expert; here an expert has
    # three: 2 of 8 gated experts of inter / 4, or one dense gated layer of inter / 2, are the same work per token
    dense = dict(kind="dense", ff=s["inter"] // 2 // 8 * 8)
    moe = dict(kind="moe", expert=dict(ff=s["inter"] // 4 // 8 * 8), router=dict(experts=8, top=2, scale=2.0, groups=dict(count=4, keep=2)))
    att = dict(heads=H, kv_heads=s["kv_heads"], dim=hd, vdim=hd, scale=hd ** -0.5, softcap=30.0, q_temp=dict(coef=0.1, every=1024))
    lat = dict(heads=H, dim=hd, rot_dim=64, vdim=hd, kv_rank=512, scale=(hd + 64) ** -0.5, rot=dict(base=500000.0, dims=64), mask=dict(size=window))
    pattern = [("attention", att, dense), ("latent_attention", lat, moe), ("latent_attention", lat, dense), ("attention", att, moe),
               ("attention", dict(att, kv_from=3), dense), ("latent_attention", lat, moe)]
    layers = []
    for i in range(s["layers"]):
        t, m, ml = pattern[i % 6]
        m = dict(m)
        if "kv_from" in m:
            m["kv_from"] = i - 1
        layers.append(dict(type=t, mixer=m, mlp=ml))
    return dict(architecture="Tilalorn", vocab=s["vocab"], width=W, layers=layers, norm=dict(eps=1e-6), residual_mult=0.5)


def tilalorn_weights(cfg, dev, seed=0):
    g = torch.Generator(device=dev).manual_seed(seed)
    W, width = {}, cfg["width"]

    def lin(name, o, i):
        W[name] = (torch.randn(o, i, generator=g, device=dev, dtype=torch.float32) * i ** -0.5).to(torch.bfloat16)

    def const(name, n, v=0.0):
        W[name] = torch.full((n,), v, dtype=torch.bfloat16, device=dev)

    lin("embed", cfg["vocab"], width)
    const("final.norm", width)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        const(p + "norm1", width)
        H = m["heads"]
        if L["type"] == "attention":
            lin(p + "mix.q", H * m["dim"], width)
            const(p + "mix.q.b", H * m["dim"])
            if m.get("kv_from") is None:
                lin(p + "mix.k", m["kv_heads"] * m["dim"], width)
                const(p + "mix.k.b", m["kv_heads"] * m["dim"])
                lin(p + "mix.v", m["kv_heads"] * m["vdim"], width)
                const(p + "mix.v.b", m["kv_heads"] * m["vdim"])
            lin(p + "mix.g", H, width)
        else:
            lin(p + "mix.q", H * (m["dim"] + m["rot_dim"]), width)
            lin(p + "mix.dkv", m["kv_rank"] + m["rot_dim"], width)
            const(p + "mix.dkv.norm", m["kv_rank"], 1.0)
            lin(p + "mix.uk", H * m["dim"], m["kv_rank"])
            lin(p + "mix.uv", H * m["vdim"], m["kv_rank"])
            lin(p + "mix.g", H * m["vdim"], width)
        lin(p + "mix.o", width, H * m["vdim"])
        ml = L["mlp"]
        const(p + "norm2", width)
        if ml["kind"] == "moe":
            lin(p + "mlp.router", ml["router"]["experts"], width)
            for e in range(ml["router"]["experts"]):
                for n in ("gate", "up"):
                    lin(p + f"mlp.e{e}.{n}", ml["expert"]["ff"], width)
                lin(p + f"mlp.e{e}.down", width, ml["expert"]["ff"])
        else:
            for n in ("gate", "up"):
                lin(p + "mlp." + n, ml["ff"], width)
            lin(p + "mlp.down", width, ml["ff"])
    return W


def workload_tilalorn_compare(args):
    from mlx_vlm_amd.models import garesun, tilalorn

    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    prompt_lens, rows, ctx, steps = (512, 2048), (1, 8), 512, max(8, int(args.steps) * 8)
    ids_in = lambda ids: (torch.as_tensor(ids, dtype=torch.int32, device=dev).reshape(-1, 1), None)      # noqa: E731
    res = {}
    for name, s in SIZES.items():
        cfg = tilalorn_cfg(s)
        tm = tilalorn.Model(tilalorn.ModelConfig.from_dict(cfg), device=dev, dtype="bfloat16", kv_pool_tokens=16384, max_seqs=12)
        tm.load_weights(tilalorn_weights(cfg, dev))
        r = {"tilalorn": _measure(tm.language_model, ids_in, s["vocab"], prompt_lens, rows, ctx, steps)}
        del tm
        torch.cuda.empty_cache()
        cfg = garesun_cfg(s)
        gm = garesun.Model(garesun.ModelConfig.from_dict(cfg), device=dev, dtype="bfloat16", kv_pool_tokens=16384, max_seqs=12)
        gm.load_weights(garesun_weights(cfg, dev))
        r["garesun"] = _measure(gm.language_model, ids_in, s["vocab"], prompt_lens, rows, ctx, steps)
        del gm
        torch.cuda.empty_cache()
        r["ratio_tilalorn_over_garesun"] = {
            "prefill_" + k: round(r["tilalorn"]["prefill"][k]["tokens_per_s"] / r["garesun"]["prefill"][k]["tokens_per_s"], 3) for k in r["garesun"]["prefill"]}
        r["ratio_tilalorn_over_garesun"].update({
            "decode_" + k: round(r["tilalorn"]["decode"][k]["tokens_per_s"] / r["garesun"]["decode"][k]["tokens_per_s"], 3) for k in r["garesun"]["decode"]})
        res[name] = dict(sizes=s, **r)
    return {"metric": "tilalorn_vs_garesun", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic", "n_gpus": 1,
            "config": {"layers": "6 per model: (attention, latent_attention, latent_attention, attention, attention reading the layer "
                                 "before it, latent_attention), feed-forwards alternately dense gated-gelu of half the dense intermediate "
                                 "and 8-expert top-2 group-limited silu experts | (mlstm, latent_attention, retention) x 2 with 8-expert "
                                 "top-2 MoE + shared expert", "window": 1024, "prompt_lens": list(prompt_lens), "decode_rows": list(rows),
                       "decode_context": ctx},
            "results": res}
