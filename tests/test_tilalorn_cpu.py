"""Host side of the Tilalorn model package (no GPU): config parsing and its refusals, the registry lookup by config.json, the
row-cache facades of layers that read another layer's cache, weight loading and its shape checks on the CPU device, and the
plain oracle against itself (causality, the window's edge, the group limit of the router, borrowed keys and values)."""
import copy

import numpy as np
import pytest
import torch

from tests import tilalorn_helpers as H
from tests import tilalorn_oracle as O

F64 = torch.float64


def test_config_reads_every_size_and_refuses_what_the_design_does_not_have():
    from mlx_vlm_amd.models.tilalorn import ModelConfig

    cfg = H.config(H.mixed_layers(), vocab=123, width=56, mult=0.45, eps=3e-4)
    mc = ModelConfig.from_dict(cfg)
    assert (mc.vocab, mc.width, mc.residual_mult, mc.norm_eps, len(mc.layers)) == (123, 56, 0.45, 3e-4, 6)
    assert [l.window for l in mc.layers] == [9, 0, 70, 0, 3, 0] and [l.kv_from for l in mc.layers] == [None, None, None, 1, None, None]
    assert mc.layers[4].mlp is None and mc.layers[4].ff == 0 and mc.layers[2].ff == 40 and not mc.layers[2].moe
    assert mc.layers[0].moe and mc.layers[0].router == (6, 2, 3, 2, 1.7) and mc.layers[3].router == (4, 4, 1, 1, 1.7)
    assert mc.layers[1].mixer["q_temp"] == dict(coef=0.25, every=5) and "softcap" not in mc.layers[3].mixer
    plain = H.config([H.attention()])
    del plain["residual_mult"], plain["layers"][0]["mixer"]["vdim"]
    mp = ModelConfig.from_dict(plain)
    assert mp.residual_mult == 1.0 and mp.layers[0].mixer["vdim"] == 24          # what an entry leaves out
    chain = ModelConfig.from_dict(H.config([H.attention(), H.attention(kv_from=0), H.latent(), H.attention(kv_from=1)]))
    assert [l.kv_from for l in chain.layers] == [None, 0, None, 0]                # a borrowing source is followed to the owner
    lean = H.config([H.attention(vdim=40), H.attention(kv_from=0, vdim=40)])
    del lean["layers"][1]["mixer"]["kv_heads"], lean["layers"][1]["mixer"]["vdim"]      # left to the entry of the layer it reads
    ml = ModelConfig.from_dict(lean)
    assert ml.layers[1].mixer["kv_heads"] == 2 and ml.layers[1].mixer["vdim"] == 40
    bad = H.config([H.attention()])
    bad["layers"][0]["type"] = "convolution"
    with pytest.raises(ValueError):
        ModelConfig.from_dict(bad)
    for layers in ([H.attention(kv_from=0)],                                      # names itself
                   [H.attention(kv_from=1), H.attention()],                       # a later layer: its cache is not written yet
                   [H.latent(), H.attention(kv_from=0)],                          # another kind of cache
                   [H.attention(), H.attention(kv_from=0, dim=16)],               # other cache sizes
                   [H.attention(heads=5, kv_heads=2)], [H.attention(softcap=-1.0)],
                   [H.attention(window=-3)], [H.latent(rot_dim=5)], [H.latent(window=-1)],
                   [H.latent(mlp=H.moe(experts=6, top=7))], [H.latent(mlp=H.moe(experts=6, groups=4))],
                   [H.latent(mlp=H.moe(experts=6, top=3, groups=3, keep=1))], [H.latent(mlp=H.moe(groups=3, keep=4))],
                   [H.latent(mlp=dict(kind="conv", ff=8))]):
        with pytest.raises(ValueError):
            ModelConfig.from_dict(H.config(layers))
    never = H.config([H.attention()])
    never["layers"][0]["mixer"]["q_temp"]["every"] = 0
    with pytest.raises(ValueError):
        ModelConfig.from_dict(never)
    odd = H.config([H.latent()])
    odd["layers"][0]["mixer"]["rot"]["dims"] = 4                                  # the rotated part is rot_dim wide
    with pytest.raises(ValueError):
        ModelConfig.from_dict(odd)


def test_registry_finds_the_package_by_architecture():
    from mlx_vlm_amd.utils import get_model_and_args

    arch, name = get_model_and_args({"architecture": "Tilalorn"})
    assert name == "tilalorn" and hasattr(arch, "Model") and hasattr(arch, "ModelConfig")


def test_weights_load_on_the_cpu_device_with_shape_checks_and_typed_caches():
    from mlx_vlm_amd.models.cache import PAGE
    from mlx_vlm_amd.models.tilalorn import LanguageModel, ModelConfig

    cfg = H.config(H.mixed_layers())
    W = H.weights(cfg, seed=3)
    for dtype, T in (("bfloat16", torch.bfloat16), ("float32", torch.float32)):
        lm = LanguageModel(ModelConfig.from_dict(copy.deepcopy(cfg)), device="cpu", dtype=dtype, kv_pool_tokens=5 * PAGE, max_seqs=3)
        lm.load_weights(dict(W, unused=torch.zeros(3)))                           # a tensor nobody asks for is left alone
        rows = lm.pool.rows
        assert sorted(rows) == [(0, "c"), (1, "k"), (1, "v"), (2, "c"), (4, "c"), (5, "k"), (5, "v")]      # layer 3 has no cache of its own
        assert rows[(1, "k")].dtype == torch.float32 and rows[(1, "v")].dtype == T and rows[(0, "c")].dtype == T
        assert rows[(1, "k")].shape == (5, PAGE, 2 * 24) and rows[(1, "v")].shape == (5, PAGE, 2 * 16) and rows[(0, "c")].shape == (5, PAGE, 48)
        L0, L3 = lm._L[0], lm._L[3]
        assert L3.src == 1 and "k" not in L3.off and L0.uk_t.shape == (3, 40, 16) and L0.uv.shape == (3, 24, 40)
        # every expert's gate rows, then its up rows, expert after expert; the down projections side by side
        assert torch.equal(L0.wff[16:32], W["l0.mlp.e0.up"].to(T)) and torch.equal(L0.wff[32:48], W["l0.mlp.e1.gate"].to(T))
        assert torch.equal(L0.down[:, 16:32], W["l0.mlp.e1.down"].to(T))
        caches = lm.make_cache()
        assert len(caches) == 6 and caches[3]._shared and not caches[1]._shared and caches[3]._layer == (1, "k")
        caches[0]._seq.reserve(70)
        caches[0]._seq.offset = 70
        assert caches[3].state.shape == (70, 48) and caches[0].state.shape == (70, 48) and caches[3].trim(5) == 5 and caches[0].offset == 70
        assert caches[0].trim(5) == 5 and caches[1].offset == 65                  # only the first owner moves the shared offset
        caches[0]._seq.release()
    short = dict(W)
    short["l1.mix.k"] = short["l1.mix.k"][:-1]
    with pytest.raises(ValueError):
        LanguageModel(ModelConfig.from_dict(copy.deepcopy(cfg)), device="cpu").load_weights(short)
    missing = {k: v for k, v in W.items() if k != "l1.mix.q.b"}
    with pytest.raises(KeyError):
        LanguageModel(ModelConfig.from_dict(copy.deepcopy(cfg)), device="cpu").load_weights(missing)


def test_oracle_is_causal_windowed_and_reads_borrowed_caches():
    cfg = H.config(H.mixed_layers())
    W = H.weights(cfg, seed=9)
    ids = np.arange(60) % cfg["vocab"]
    a = O.Oracle(cfg, W, F64).forward(ids)
    ids2 = ids.copy()
    ids2[40:] = (ids2[40:] + 7) % cfg["vocab"]
    b = O.Oracle(cfg, W, F64).forward(ids2)
    assert torch.equal(a[:40], b[:40]) and not torch.allclose(a[40:], b[40:])
    # one latent layer with a window of 4: token 10 moves rows 10..13 and no other
    one = H.config([H.latent(window=4, mlp=None)])
    W1 = H.weights(one, seed=2)
    x = O.Oracle(one, W1, F64).forward(ids)
    ids3 = ids.copy()
    ids3[10] = (ids3[10] + 1) % one["vocab"]
    y = O.Oracle(one, W1, F64).forward(ids3)
    changed = [t for t in range(60) if not torch.equal(x[t], y[t])]
    assert changed == [10, 11, 12, 13]
    # rotation: the pair of dimension i is i + dims / 2, angle position * base^(-2 i / dims)
    v = torch.zeros(3, 6, dtype=F64)
    v[:, 0], v[:, 5] = 1.0, 2.0
    r = O.rotate_half(v, torch.tensor([0, 1, 2]), 4, 100.0)
    assert torch.allclose(r[:, 0], torch.cos(torch.tensor([0.0, 1.0, 2.0], dtype=F64))) and torch.allclose(r[:, 2], torch.sin(torch.tensor([0.0, 1.0, 2.0], dtype=F64)))
    assert torch.equal(r[:, 4:], v[:, 4:]) and torch.all(r[:, 1] == 0)


def test_oracle_router_keeps_the_best_groups_and_does_not_renormalise():
    z = torch.tensor([[5.0, 0.0, 4.0, 3.9, 1.0, 4.5]], dtype=F64)                 # groups {0,1} {2,3} {4,5}: best members 5, 4, 4.5
    w = O.route(z, dict(experts=6, top=2, scale=2.0, groups=dict(count=3, keep=2)))
    s = torch.softmax(z, -1)
    assert torch.nonzero(w[0]).view(-1).tolist() == [0, 5] and torch.allclose(w[0, [0, 5]], 2.0 * s[0, [0, 5]])
    w = O.route(z, dict(experts=6, top=3, scale=1.0, groups=dict(count=3, keep=2)))
    assert torch.nonzero(w[0]).view(-1).tolist() == [0, 4, 5]                     # expert 2 scores higher than 4 but its group is out
    w = O.route(z, dict(experts=6, top=3, scale=1.0))
    assert torch.nonzero(w[0]).view(-1).tolist() == [0, 2, 5]
