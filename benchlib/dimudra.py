"""`bench.py --workload dimudra-compare`: prefill and decode throughput of the Dimudra design (input convolutions on every layer,
sliding-window attention side by side with a selective state-space scan, a row-gated matrix-state recurrence, sink attention
with partial rotary positions, sigmoid-routed group-limited silu experts with a gated shared expert; three layers whose span
runs twice) next to the framework's closest model, Garesun (matrix-state recurrences, attention and mixtures of experts with a
shared expert on the same ragged step), at the same width, number of layer runs, head count, head size and feed-forward work per
token - random weights, synthetic token ids, bf16.  Not the headline metric: one JSON line of its own."""
from __future__ import annotations

import torch

from benchlib.garesun import SIZES, _measure, garesun_cfg, garesun_weights


def dimudra_cfg(s, window=1024):
    H, hd, W = s["heads"], s["hd"], s["width"]
    # the comparison model runs 2 of 8 experts + a shared one of inter / 4 each with two matrices per expert; here an expert has
    # three, so 2 of 8 + a shared one of inter / 6 are the same work per token
    ff = s["inter"] // 6 // 8 * 8
    mlp = dict(kind="moe", expert=dict(ff=ff), router=dict(experts=8, top=2, groups=dict(count=4, keep=2)), shared=dict(ff=ff))
    att = dict(heads=H, kv_heads=s["kv_heads"], dim=hd, vdim=hd, scale=hd ** -0.5)
    kinds = [dict(type="parallel", mixer=dict(left=dict(att, mask=dict(size=window)), left_scale=1.1,
                                              right=dict(inner=2 * W, state=16, dt_rank=W // 16, conv=4), right_scale=0.7)),
             dict(type="hgrn2", mixer=dict(heads=H, dim=hd, vdim=hd)),
             dict(type="attention", mixer=dict(att, rot=dict(base=500000.0, dims=hd // 2)))]
    n = max(1, s["layers"] // 2)
    layers = [dict(kinds[i % 3], mlp=mlp) for i in range(n)]
    return dict(architecture="Dimudra", vocab=s["vocab"], width=W, layers=layers, norm=dict(eps=1e-6), embedding=dict(scale=W ** 0.5),
                canon=dict(taps=4), loop=dict(start=0, stop=n, times=2))


def dimudra_weights(cfg, dev, seed=0):
    g = torch.Generator(device=dev).manual_seed(seed)
    W, width, taps = {}, cfg["width"], cfg["canon"]["taps"]

    def lin(name, o, i, s=1.0):
        W[name] = (torch.randn(o, i, generator=g, device=dev, dtype=torch.float32) * (s * i ** -0.5)).to(torch.bfloat16)

    def const(name, n, v=1.0):
        W[name] = torch.full((n,) if n else (), v, dtype=torch.bfloat16, device=dev)

    def attn(p, m):
        lin(p + "q", m["heads"] * m["dim"], width)
        lin(p + "k", m["kv_heads"] * m["dim"], width)
        lin(p + "v", m["kv_heads"] * m["vdim"], width)
        lin(p + "g", m["heads"] * m["vdim"], width)
        lin(p + "o", width, m["heads"] * m["vdim"])

    lin("embed", cfg["vocab"], width)
    lin("head", cfg["vocab"], width)
    const("final.norm", 0)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        const(p + "norm1", 0)
        const(p + "norm2", 0)
        W[p + "canon1"] = (0.2 * torch.randn(width, taps, generator=g, device=dev)).to(torch.bfloat16)
        if L["type"] == "parallel":
            a, r = m["left"], m["right"]
            attn(p + "mix.left.", a)
            for n, k in (("q", a["heads"] * a["dim"]), ("k", a["kv_heads"] * a["dim"])):
                const(p + f"mix.left.{n}.b", k, 0.0)
                const(p + f"mix.left.{n}.norm", k, 1.0)
            const(p + "mix.left.v.b", a["kv_heads"] * a["vdim"], 0.0)
            C, N, R = r["inner"], r["state"], r["dt_rank"]
            pr = p + "mix.right."
            lin(pr + "in", 2 * C, width)
            W[pr + "conv"] = (0.3 * torch.randn(C, r["conv"], generator=g, device=dev)).to(torch.bfloat16)
            const(pr + "conv.b", C, 0.0)
            lin(pr + "x", R + 2 * N, C)
            lin(pr + "dt", C, R)
            const(pr + "dt.b", C, -3.0)
            W[pr + "A_log"] = torch.log(1.0 + torch.arange(N, dtype=torch.float32, device=dev)).repeat(C, 1).to(torch.bfloat16)
            const(pr + "D", C, 1.0)
            lin(pr + "o", width, C)
        elif L["type"] == "hgrn2":
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            lin(p + "mix.q", H * D, width)
            lin(p + "mix.f", H * D, width)
            const(p + "mix.f.b", H * D, 1.0)
            const(p + "mix.lower", H * D, 0.5)
            lin(p + "mix.v", H * Dv, width)
            const(p + "mix.norm", Dv, 1.0)
            lin(p + "mix.o", width, H * Dv)
        else:
            attn(p + "mix.", m)
        ml = L["mlp"]
        E = ml["router"]["experts"]
        lin(p + "mlp.router", E, width)
        const(p + "mlp.correction", E, 0.0)
        for n, f in [(f"e{e}", ml["expert"]["ff"]) for e in range(E)] + [("shared", ml["shared"]["ff"])]:
            lin(p + f"mlp.{n}.gate", f, width)
            lin(p + f"mlp.{n}.up", f, width)
            lin(p + f"mlp.{n}.down", width, f)
        lin(p + "mlp.shared.sg", 1, width)
    return W


def workload_dimudra_compare(args):
    from mlx_vlm_amd.models import dimudra, garesun

    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    prompt_lens, rows, ctx, steps = (512, 2048), (1, 8), 512, max(8, int(args.steps) * 8)
    ids_in = lambda ids: (torch.as_tensor(ids, dtype=torch.int32, device=dev).reshape(-1, 1), None)      # noqa: E731
    res = {}
    for name, s in SIZES.items():
        cfg = dimudra_cfg(s)
        dm = dimudra.Model(dimudra.ModelConfig.from_dict(cfg), device=dev, dtype="bfloat16", kv_pool_tokens=16384, max_seqs=12)
        dm.load_weights(dimudra_weights(cfg, dev))
        r = {"dimudra": _measure(dm.language_model, ids_in, s["vocab"], prompt_lens, rows, ctx, steps)}
        del dm
        torch.cuda.empty_cache()
        cfg = garesun_cfg(s)
        gm = garesun.Model(garesun.ModelConfig.from_dict(cfg), device=dev, dtype="bfloat16", kv_pool_tokens=16384, max_seqs=12)
        gm.load_weights(garesun_weights(cfg, dev))
        r["garesun"] = _measure(gm.language_model, ids_in, s["vocab"], prompt_lens, rows, ctx, steps)
        del gm
        torch.cuda.empty_cache()
        r["ratio_dimudra_over_garesun"] = {
            "prefill_" + k: round(r["dimudra"]["prefill"][k]["tokens_per_s"] / r["garesun"]["prefill"][k]["tokens_per_s"], 3) for k in r["garesun"]["prefill"]}
        r["ratio_dimudra_over_garesun"].update({
            "decode_" + k: round(r["dimudra"]["decode"][k]["tokens_per_s"] / r["garesun"]["decode"][k]["tokens_per_s"], 3) for k in r["garesun"]["decode"]})
        res[name] = dict(sizes=s, **r)
    return {"metric": "dimudra_vs_garesun", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic", "n_gpus": 1,
            "config": {"layers": "6 layer runs per model: (parallel [windowed attention | selective scan], hgrn2, sink attention), the span run "
                                 "twice, each with 8-expert top-2 group-limited silu experts + gated shared expert and a 4-tap input "
                                 "convolution | (mlstm, latent_attention, retention) x 2 with 8-expert top-2 MoE + shared expert",
                       "window": 1024, "prompt_lens": list(prompt_lens), "decode_rows": list(rows), "decode_context": ctx},
            "results": res}
