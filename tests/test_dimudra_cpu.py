"""Host side of the Dimudra model package (no GPU): config parsing, its defaults and refusals, the order of layer runs of a
looped span, the registry lookup by config.json, weight loading with its shape checks and the per-run caches / states / carried
inputs on the CPU device, and the plain oracle against itself (causality, the window's edge, the convolution's reach, the sink,
the router's group limit and its choice-only correction)."""
import copy

import numpy as np
import pytest
import torch

from tests import dimudra_helpers as H
from tests import dimudra_oracle as O

F64 = torch.float64


def test_config_reads_every_size_and_refuses_what_the_design_does_not_have():
    from mlx_vlm_amd.models.dimudra import ModelConfig
    from mlx_vlm_amd.models.dimudra.config import attention_constants

    cfg = H.mixed_config(vocab=123, width=56, eps=3e-4, taps=5, escale=2.5)
    mc = ModelConfig.from_dict(cfg)
    assert (mc.vocab, mc.width, mc.norm_eps, mc.canon_taps, mc.embedding_scale, len(mc.layers), mc.loop) == (123, 56, 3e-4, 5, 2.5, 6, (1, 4, 2))
    assert [i for i, _ in mc.runs()] == [0, 1, 2, 3, 1, 2, 3, 4, 5] and [r for _, r in mc.runs()] == [False] * 4 + [True] + [False] * 4
    assert mc.runs() == O.layer_runs(cfg)
    assert attention_constants(mc.layers[1].mixer["left"]) == (4, 2, 12, 20, 0.3, 9, 0, 10000.0)
    assert attention_constants(mc.layers[2].mixer) == (6, 2, 16, 12, 0.35, 0, 6, 300.0)
    assert mc.layers[0].router == (6, 2, 3, 2) and mc.layers[3].router == (4, 4, 1, 1)
    assert (mc.layers[0].ff, mc.layers[0].shared_ff, mc.layers[3].shared_ff, mc.layers[4].ff) == (16, 24, 0, 0) and mc.layers[4].mlp is None
    plain = H.config([H.attention(rot_dims=0)], taps=0)
    del plain["embedding"], plain["layers"][0]["mixer"]["vdim"]
    mp = ModelConfig.from_dict(plain)                                             # what a config leaves out
    assert mp.embedding_scale == 1.0 and mp.canon_taps == 0 and mp.layers[0].mixer["vdim"] == 16 and mp.runs() == [(0, False)]
    assert ModelConfig.from_dict(H.config(H.mixed_layers(), loop=(0, 6, 3))).runs()[6] == (0, True)
    assert all(not r for _, r in ModelConfig.from_dict(H.config(H.mixed_layers(), loop=(2, 4, 1))).runs())
    bad = H.config([H.attention()])
    bad["layers"][0]["type"] = "convolution"
    with pytest.raises(ValueError):
        ModelConfig.from_dict(bad)
    for layers in ([H.attention(heads=5, kv_heads=2)], [H.attention(rot_dims=5)], [H.attention(rot_dims=18)], [H.parallel(window=-3)],
                   [H.parallel(state=0)], [H.parallel(conv=0)],
                   [H.hgrn2(mlp=H.moe(experts=6, top=7))], [H.hgrn2(mlp=H.moe(experts=6, groups=4))],
                   [H.hgrn2(mlp=H.moe(experts=6, top=3, groups=3, keep=1))], [H.hgrn2(mlp=H.moe(groups=3, keep=4))],
                   [H.hgrn2(mlp=dict(kind="dense", ff=8))]):
        with pytest.raises(ValueError):
            ModelConfig.from_dict(H.config(layers))
    for loop in ((2, 1, 2), (0, 7, 2), (0, 2, 0)):
        with pytest.raises(ValueError):
            ModelConfig.from_dict(H.config(H.mixed_layers(), loop=loop))
    lean = H.config([H.hgrn2()])
    del lean["layers"][0]["mixer"]["vdim"]
    with pytest.raises(ValueError):
        ModelConfig.from_dict(lean)


def test_registry_finds_the_package_by_architecture():
    from mlx_vlm_amd.utils import get_model_and_args

    arch, name = get_model_and_args({"architecture": "Dimudra"})
    assert name == "dimudra" and hasattr(arch, "Model") and hasattr(arch, "ModelConfig") and "selective_scan" in arch.HIP_SOURCES


def test_weights_load_on_the_cpu_device_with_shape_checks_and_per_run_state():
    from mlx_vlm_amd.models.cache import PAGE, RecurrentCache, RowCache
    from mlx_vlm_amd.models.dimudra import LanguageModel, ModelConfig

    cfg = H.mixed_config()
    W = H.weights(cfg, seed=3)
    for dtype, T in (("bfloat16", torch.bfloat16), ("float32", torch.float32)):
        lm = LanguageModel(ModelConfig.from_dict(copy.deepcopy(cfg)), device="cpu", dtype=dtype, kv_pool_tokens=5 * PAGE, max_seqs=3)
        lm.load_weights(dict(W, unused=torch.zeros(3)))                           # a tensor nobody asks for is left alone
        pool = lm.pool
        # runs: 0 hgrn2 | 1 parallel, 2 attention, 3 parallel | 4 parallel, 5 attention, 6 parallel | 7 attention, 8 hgrn2
        assert sorted(pool.rows) == sorted((r, n) for r in (1, 2, 3, 4, 5, 6, 7) for n in "kv")
        assert pool.rows[(1, "k")].dtype == torch.float32 and pool.rows[(1, "v")].dtype == T
        assert pool.rows[(1, "k")].shape == (5, PAGE, 2 * 12) and pool.rows[(4, "v")].shape == (5, PAGE, 2 * 20) and pool.rows[(2, "k")].shape == (5, PAGE, 2 * 16)
        assert sorted(pool.state) == [0, 1, 3, 4, 6, 8] and pool.state[0].shape == (3, 3, 10, 14) and pool.state[4].shape == (3, 1, 40, 6)
        assert pool.state[8].shape == (3, 1, 40, 8) and all(t.dtype == torch.float32 for t in pool.state.values())
        assert sorted(pool.aux, key=str) == sorted([(r, "canon") for r in range(9)] + [(r, "conv") for r in (1, 3, 4, 6)], key=str)
        assert pool.aux[(0, "canon")].shape == (3, 3, 56) and pool.aux[(1, "conv")].shape == (3, 2, 40) and pool.aux[(3, "conv")].shape == (3, 1, 24)
        L0, L1 = lm._L[0], lm._L[1]
        assert L0.norm1.shape == (56,) and torch.all(L0.norm1 == W["l0.norm1"].to(T)) and lm._w["final_norm"].shape == (56,)
        assert torch.equal(L0.router[:6], W["l0.mlp.router"].to(T)) and torch.equal(L0.router[6:], W["l0.mlp.shared.sg"].to(T))
        assert L0.correction.dtype == torch.float32
        # every expert's gate rows, then its up rows, expert after expert, the shared expert behind them; the down projections side by side
        assert torch.equal(L0.wff[16:32], W["l0.mlp.e0.up"].to(T)) and torch.equal(L0.wff[32:48], W["l0.mlp.e1.gate"].to(T))
        assert torch.equal(L0.wff[192:216], W["l0.mlp.shared.gate"].to(T)) and torch.equal(L0.down[:, 16:32], W["l0.mlp.e1.down"].to(T))
        assert torch.equal(L0.down[:, 96:120], W["l0.mlp.shared.down"].to(T)) and lm._L[3].router.shape == (4, 56)
        assert torch.equal(L1.wproj[L1.off["in"]: L1.off["in"] + 80], W["l1.mix.right.in"].to(T))
        assert torch.equal(L0.normw, W["l0.mix.norm"].to(T).repeat(3))
        caches = lm.make_cache()
        assert len(caches) == 9 and [type(c) for c in caches] == [RecurrentCache] + [RecurrentCache, RowCache, RecurrentCache] * 2 + [RowCache, RecurrentCache]
        caches[0]._seq.reserve(70)
        caches[0]._seq.offset = 70
        assert caches[2].state.shape == (70, 32) and [tuple(t.shape) for t in caches[1].state] == [(1, 40, 6), (3, 56), (2, 40)]
        assert [tuple(t.shape) for t in caches[0].state] == [(3, 10, 14), (3, 56)] and not caches[0].is_trimmable()
        caches[0]._seq.release()
    short = dict(W)
    short["l1.mix.right.A_log"] = short["l1.mix.right.A_log"][:, :-1]
    with pytest.raises(ValueError):
        LanguageModel(ModelConfig.from_dict(copy.deepcopy(cfg)), device="cpu").load_weights(short)
    vector = dict(W)
    vector["l2.norm1"] = torch.ones(56)                                           # a norm's weight is one number
    with pytest.raises(ValueError):
        LanguageModel(ModelConfig.from_dict(copy.deepcopy(cfg)), device="cpu").load_weights(vector)
    missing = {k: v for k, v in W.items() if k != "l1.mix.left.q.b"}
    with pytest.raises(KeyError):
        LanguageModel(ModelConfig.from_dict(copy.deepcopy(cfg)), device="cpu").load_weights(missing)


def test_oracle_is_causal_windowed_and_its_convolution_reaches_taps_tokens():
    cfg = H.mixed_config()
    W = H.as_f64(H.weights(cfg, seed=9))
    ids = np.arange(60) % cfg["vocab"]
    a, _ = O.forward(cfg, W, ids)
    ids2 = ids.copy()
    ids2[40:] = (ids2[40:] + 7) % cfg["vocab"]
    b, _ = O.forward(cfg, W, ids2)
    assert torch.allclose(a[:40], b[:40], rtol=0, atol=1e-11) and not torch.allclose(a[40:], b[40:])     # (experts gather other rows: last bits)
    # the attention half of a parallel layer alone, window 4, input convolution of 3 taps: token 10 reaches the inputs of
    # tokens 10..12, which are seen by rows up to 15
    one = H.config([H.parallel(window=4, right_scale=0.0, mlp=None)], taps=3)
    W1 = H.as_f64(H.weights(one, seed=2))
    x, _ = O.forward(one, W1, ids)
    ids3 = ids.copy()
    ids3[10] = (ids3[10] + 1) % one["vocab"]
    y, _ = O.forward(one, W1, ids3)
    assert [t for t in range(60) if not torch.allclose(x[t], y[t], rtol=0, atol=1e-11)] == [10, 11, 12, 13, 14, 15]
    h = torch.randn(9, 4, dtype=F64)
    w = torch.randn(4, 3, dtype=F64)
    c = O.causal_conv(h, w)
    assert torch.allclose(c[0], w[:, 2] * h[0]) and torch.allclose(c[5], w[:, 0] * h[3] + w[:, 1] * h[4] + w[:, 2] * h[5])
    # rotation: the pair of dimension i is i + dims / 2, angle position * base^(-2 i / dims); the rest passes
    v = torch.zeros(3, 1, 6, dtype=F64)
    v[..., 0], v[..., 5] = 1.0, 2.0
    r = O.rotate_half_partial(v, 4, 100.0)[:, 0]
    ang = torch.tensor([0.0, 1.0, 2.0], dtype=F64)
    assert torch.allclose(r[:, 0], torch.cos(ang)) and torch.allclose(r[:, 2], torch.sin(ang)) and torch.equal(r[:, 4:], v[:, 0, 4:]) and torch.all(r[:, 1] == 0)


def test_oracle_sink_takes_weight_without_a_value():
    q = torch.zeros(2, 1, 4, dtype=F64)
    k = torch.zeros(2, 1, 4, dtype=F64)
    v = torch.ones(2, 1, 3, dtype=F64)
    o = O.softmax_attention(q, k, v, 1.0, sink=True)                              # every score 0: weights 1 / (1 + visible keys)
    assert torch.allclose(o[0], torch.full((1, 3), 0.5, dtype=F64)) and torch.allclose(o[1], torch.full((1, 3), 2 / 3, dtype=F64))
    assert torch.allclose(O.softmax_attention(q, k, v, 1.0), torch.ones(2, 1, 3, dtype=F64))


def test_oracle_router_ranks_groups_by_two_members_and_corrects_the_choice_only():
    z = torch.tensor([[2.0, -4.0, 1.0, 0.9, -1.0, 1.5]], dtype=F64)              # groups {0,1} {2,3} {4,5}
    s = torch.sigmoid(z)
    zero = torch.zeros(6, dtype=F64)
    # sums of the two best: .88 + .02, .73 + .71, .27 + .82 -> groups 1 and 2 stay although expert 0 scores highest
    chosen, w = O.route(z, zero, 2, 3, 2)
    assert sorted(chosen[0].tolist()) == [2, 5] and torch.allclose(w.sum(), torch.tensor(1.0, dtype=F64))
    assert torch.allclose(w[0], s[0, chosen[0]] / s[0, chosen[0]].sum())
    chosen, _ = O.route(z, zero, 3, 3, 2)
    assert sorted(chosen[0].tolist()) == [2, 3, 5]
    chosen, _ = O.route(z, zero, 3, 1, 1)
    assert sorted(chosen[0].tolist()) == [0, 2, 5]
    corr = torch.tensor([0.0, 0.0, 0.0, 0.0, 2.0, 0.0], dtype=F64)               # lifts expert 4 into the choice, not into the weights
    chosen, w = O.route(z, corr, 2, 3, 2)
    assert sorted(chosen[0].tolist()) == [4, 5] and torch.allclose(w[0], s[0, chosen[0]] / s[0, chosen[0]].sum())
    neg = torch.full((6,), -5.0, dtype=F64)                                       # every choice score negative: a group that is out stays out
    chosen, _ = O.route(z, neg, 3, 3, 2)
    assert sorted(chosen[0].tolist()) == [2, 3, 5]
