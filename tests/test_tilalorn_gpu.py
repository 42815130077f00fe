"""Tilalorn on MI355X against the plain restatement in tests/tilalorn_oracle.py (float64 on the CPU, dense masks).

Small random checkpoints with unequal sizes (tests/tilalorn_helpers.py) are written to disk and loaded through
`utils.load_model` (registry by config.json, safetensors reader, weight packing).  float32 serving is compared tightly,
bfloat16 within the rounding of a 16-bit projection chain.  Covered: every mechanism alone (operator level and as a one-
layer model); whole prompts against portions of several sizes (down to two tokens) and against token-by-token decoding;
batches of unequal requests against each alone; pages and slots freed and used again; keys at page, tile and window borders,
just inside and just outside the window and far back among hundreds, in prompts and decoding, with one score made to stand
out; the first tokens; long decoding; sizes that are equal or 1 elsewhere; greedy generation through generate_step and the
continuous batch generator; replay of a scheduled trace; captured decode steps."""
import numpy as np
import pytest
import torch

from tests import tilalorn_helpers as H
from tests import tilalorn_oracle as O

pytestmark = pytest.mark.gpu
F64 = torch.float64
TOL = {"float32": 4e-5, "bfloat16": 4e-2}


def _close(got, want, dtype):
    """float32: every row within TOL (six layers of fp32 sums behind sharp softmaxes; a wrong key, window or expert moves a
    row by 1e-2 and more).  bfloat16: eight rows in ten within TOL - with random router weights a choice of experts can sit
    inside the rounding of a 16-bit activation and pick another expert for that token, which moves that row widely"""
    if dtype == "float32":
        return H.rel_rms(got, want) < TOL[dtype]
    return H.rel_rms(got, want, 0.8) < TOL[dtype]


def _load(tmp_path, cfg, W, dtype, tokens=4096, seqs=6, name="m"):
    from mlx_vlm_amd.utils import load_model

    return load_model(H.write_checkpoint(str(tmp_path / name), cfg, W), dtype=dtype, kv_pool_tokens=tokens, max_seqs=seqs)


def _ids(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).numpy().astype(np.int32)


def _whole(lm, ids):
    c = lm.make_cache()
    lg = lm.step([(c[0]._seq, ids)], want="all").cpu()
    c[0]._seq.release()
    return lg


def _portions(lm, ids, sizes):
    """the prompt in portions of the given sizes (cycled), every row's logits"""
    c, out, o, j = lm.make_cache(), [], 0, 0
    while o < len(ids):
        n = min(sizes[j % len(sizes)], len(ids) - o)
        out.append(lm.step([(c[0]._seq, ids[o:o + n])], want="all").cpu())
        o, j = o + n, j + 1
    c[0]._seq.release()
    return torch.cat(out)


# ------------------------------------------------------------------------------------------------ operators
def test_residual_step_with_the_next_norm_and_gated_products():
    from mlx_vlm_amd import ops

    g = torch.Generator().manual_seed(2)
    for T in (torch.float32, torch.bfloat16):
        tol = 1e-5 if T == torch.float32 else 1e-2
        x = torch.randn(7, 50, generator=g)
        y = torch.randn(7, 60, generator=g).to(T)                                  # a view with a pitch of 60
        w = (0.3 * torch.randn(50, generator=g)).to(T)
        xs = x.clone().cuda()
        h = ops.scaled_add_rms_(xs, y.cuda()[:, :50], 0.3, w=w.cuda(), w_offset=1.0, eps=1e-5)
        want = x.double() + 0.3 * y.double()[:, :50]
        assert (xs.cpu().double() - want).abs().max() < 1e-6
        assert (h.float().cpu().double() - O.norm(want, w.double(), 1e-5)).abs().max() < tol * 5
        xs2 = x.clone().cuda()
        assert ops.scaled_add_rms_(xs2, y.cuda()[:, :50], 0.3) is None and torch.equal(xs2, xs)          # add only
        h2 = ops.scaled_add_rms_(xs2, w=w.cuda(), w_offset=1.0, eps=1e-5)                                # norm only
        assert torch.equal(h2, h) and torch.equal(xs2, xs)
        a, b = torch.randn(5, 40, generator=g).to(T), torch.randn(5, 44, generator=g).to(T)
        for act, f in ((ops.GLU_GELU_TANH, O.gelu_tanh), (ops.GLU_SILU, torch.nn.functional.silu), (ops.GLU_SIGMOID, torch.sigmoid)):
            out = torch.empty(5, 33, dtype=T, device="cuda")
            ops.glu_rows(a.cuda()[:, 3:], b.cuda()[:, 1:], act, out=out)
            assert (out.float().cpu().double() - f(a.double()[:, 3:36]) * b.double()[:, 1:34]).abs().max() < tol * 10
        # stacked experts: expert e's gate columns at e * 14, its up columns 7 further, weights from a route table with zeros
        gu = torch.randn(5, 3 * 14 + 2, generator=g).to(T)
        route = torch.tensor([[0.5, 0, 1.5], [0, 0, 2.0], [1, 1, 1], [0, 0.25, 0], [0.1, 0.2, 0]])
        gu[1, :28] = float("nan")                                                  # columns of experts nobody chose are never read
        out = ops.glu_rows(gu.cuda(), gu.cuda()[:, 7:], ops.GLU_SILU, route=route.cuda(), E=3, ff=7, estride=14)
        G3 = gu.double()[:, :42].view(5, 3, 14)
        want = torch.nan_to_num(torch.nn.functional.silu(G3[..., :7]) * G3[..., 7:]) * route.double().view(5, 3, 1)
        assert (out.float().cpu().double().view(5, 3, 7) - want).abs().max() < tol * 10


@pytest.mark.parametrize("E,top,groups,keep", [(8, 3, 4, 2), (6, 2, 3, 2), (12, 4, 1, 1), (5, 5, 5, 5), (9, 1, 3, 1), (130, 6, 10, 3)])
def test_router_scores_groups_and_weights(E, top, groups, keep):
    from mlx_vlm_amd import ops

    z = torch.randn(40, E, generator=torch.Generator().manual_seed(E + top)) * 2
    z[3] = z[3, 0]                                                                 # every expert tied: the lowest indices win
    z[4, : E // groups] = z[4, E // groups: 2 * (E // groups)] if groups > 1 else z[4, : E // groups]
    gate, idx, wgt = ops.moe_route_scored(z.cuda(), top, groups, keep, 1.7)
    want = O.route(z.double(), dict(experts=E, top=top, scale=1.7, groups=dict(count=groups, keep=keep)))
    assert (gate.cpu().double() - want).abs().max() < 1e-6
    assert ((gate != 0).sum(-1) == top).all()
    for t in range(40):
        assert sorted(idx[t].tolist()) == sorted(torch.nonzero(want[t]).view(-1).tolist())
        assert (wgt[t].cpu().double().sort().values - want[t][want[t] != 0].sort().values).abs().max() < 1e-6


def test_headnorm_rows_bias_unit_norm_position_multiplier_and_value_rows():
    from mlx_vlm_amd import ops
    from mlx_vlm_amd.models.cache import PAGE

    g = torch.Generator().manual_seed(4)
    Hh, D, Dv = 3, 14, 6
    for T in (torch.float32, torch.bfloat16):
        x = torch.randn(9, Hh * D + 5, generator=g).to(T)
        v = torch.randn(9, Hh * Dv + 3, generator=g).to(T)
        b, vb = torch.randn(Hh * D, generator=g).to(T), torch.randn(Hh * Dv, generator=g).to(T)
        pos = torch.tensor([0, 1, 63, 64, 65, 700, 5, 6, 7], dtype=torch.int32)
        seq = torch.tensor([0] * 6 + [1] * 3, dtype=torch.int32)
        bt = torch.zeros(2, 12, dtype=torch.int32)
        bt[0] = torch.arange(12, dtype=torch.int32).flip(0) + 1
        base = O.unit_rms((x.double()[:, : Hh * D] + b.double()).view(9, Hh, D), 1e-5)
        mult = 1 + 0.3 * torch.log(torch.floor((pos + 1) / 3) + 1).double()
        dense = torch.zeros(9, Hh * D, device="cuda")
        ops.headnorm_rows(x.cuda()[:, : Hh * D], Hh, D, pos.cuda(), dense, eps=1e-5, bias=b.cuda(), temp=(0.3, 3))
        assert (dense.cpu().double().view(9, Hh, D) - base * mult.view(9, 1, 1)).abs().max() < 1e-5
        kp = torch.zeros(13, PAGE, Hh * D, device="cuda")
        vp = torch.zeros(13, PAGE, Hh * Dv, dtype=T, device="cuda")
        ops.headnorm_rows(x.cuda()[:, : Hh * D], Hh, D, pos.cuda(), kp, eps=1e-5, bias=b.cuda(), tok_seq=seq.cuda(), block_table=bt.cuda(),
                          raw=v.cuda()[:, : Hh * Dv], raw_dim=Dv, raw_bias=vb.cuda(), raw_pool=vp)
        for t in range(9):
            page, slot = int(bt[seq[t], pos[t] // PAGE]), int(pos[t]) % PAGE
            assert (kp[page, slot].cpu().double().view(Hh, D) - base[t]).abs().max() < 1e-5
            assert (vp[page, slot].float().cpu().double() - (v.double()[t, : Hh * Dv] + vb.double())).abs().max() < (1e-6 if T == torch.float32 else 3e-2)


@pytest.mark.parametrize("D,Dv", [(20, 12), (24, 16), (136, 72)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_grouped_attention_capped_scores_head_gates_against_a_dense_softmax(dtype, D, Dv):
    """two sequences at different offsets on scattered pages (one 1890 tokens deep), query blocks that end inside a key tile,
    value size unequal to the key size, capped scores, one gate per head, with and without a window"""
    from mlx_vlm_amd import ops
    from mlx_vlm_amd.models.cache import PAGE

    Hh, G = 6, 2
    g = torch.Generator().manual_seed(9)
    bt = torch.zeros(3, 32, dtype=torch.int32)
    bt[1, :31] = torch.randperm(31, generator=g).to(torch.int32) + 1
    kpool = torch.randn(32, PAGE, G * D, generator=g) * 0.7
    vpool = torch.randn(32, PAGE, G * Dv, generator=g).to(dtype)
    tok_seq = torch.tensor([1] * 37 + [2] * 5, dtype=torch.int32)
    tok_pos = torch.tensor(list(range(1890, 1927)) + list(range(5)), dtype=torch.int32)
    q = torch.randn(42, Hh * D, generator=g)
    gate = torch.randn(42, Hh + 8, generator=g).to(dtype)
    qb_start = torch.tensor([0, 16, 32, 37], dtype=torch.int32).cuda()
    qb_count = torch.tensor([16, 16, 5, 5], dtype=torch.int32).cuda()
    rows = {sq: (kpool[bt[sq].long()].reshape(-1, G, D).double(), vpool[bt[sq].long()].reshape(-1, G, Dv).double()) for sq in (1, 2)}
    for window, cap in ((0, 3.0), (0, 0.0), (17, 3.0), (1025, 50.0)):
        want = torch.zeros(42, Hh, Dv, dtype=F64)
        for t in range(42):
            sq, pos = int(tok_seq[t]), int(tok_pos[t])
            lo = max(0, pos - window + 1) if window > 0 else 0
            for h in range(Hh):
                kh = h // (Hh // G)
                s = rows[sq][0][lo:pos + 1, kh] @ q[t, h * D:(h + 1) * D].double() * 0.3
                s = cap * torch.tanh(s / cap) if cap else s
                want[t, h] = (torch.softmax(s, 0) @ rows[sq][1][lo:pos + 1, kh]) * torch.sigmoid(gate[t, h].double())
        args = (tok_seq.cuda(), tok_pos.cuda(), bt.cuda(), Hh, G, D, Dv, 0.3)
        a = torch.zeros(42, Hh * Dv, dtype=dtype, device="cuda")
        b = torch.zeros(42, Hh * Dv, dtype=dtype, device="cuda")
        kw = dict(window=window, gate=gate.cuda()[:, :Hh], cap=cap, gate_head=True)
        ops.window_attn_rows(q.cuda(), kpool.cuda(), vpool.cuda(), *args, a, **kw)
        ops.window_attn_blocks(q.cuda(), kpool.cuda(), vpool.cuda(), qb_start, qb_count, *args, b, **kw)
        tol = 2e-5 if dtype == torch.float32 else 2e-2
        assert (a.cpu().double().view(42, Hh, Dv) - want).abs().max() < tol, (window, cap)
        assert (b.cpu().double().view(42, Hh, Dv) - want).abs().max() < tol, (window, cap)


@pytest.mark.parametrize("R,Dr", [(24, 8), (21, 6), (264, 2)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_latent_attention_windows_both_forms_against_a_dense_softmax(dtype, R, Dr):
    from mlx_vlm_amd import ops
    from mlx_vlm_amd.models.cache import PAGE

    Hh = 3
    g = torch.Generator().manual_seed(R)
    deep = 1890 if R < 100 else 890                     # 1890: the decode form walks more than one chunk of 1024 keys
    npg = (deep + 37) // PAGE + 2
    bt = torch.zeros(3, npg, dtype=torch.int32)
    bt[1, : npg - 1] = torch.randperm(npg - 1, generator=g).to(torch.int32) + 1
    pool = (torch.randn(npg, PAGE, R + Dr, generator=g) * 0.5).to(dtype)
    tok_seq = torch.tensor([1] * 37 + [2] * 5, dtype=torch.int32)
    tok_pos = torch.tensor(list(range(deep, deep + 37)) + list(range(5)), dtype=torch.int32)
    q = torch.randn(42, Hh, R + Dr, generator=g) * 0.5
    qb_start = torch.tensor([0, 16, 32, 37], dtype=torch.int32).cuda()
    qb_count = torch.tensor([16, 16, 5, 5], dtype=torch.int32).cuda()
    rows = {sq: pool[bt[sq].long()].reshape(-1, R + Dr).double() for sq in (1, 2)}
    for window in (0, 1, 2, 16, 17, 37, 64, 65, 255, 256, 257, 600, 1024, 1025, 1800):
        want = torch.zeros(42, Hh, R, dtype=F64)
        for t in range(42):
            sq, pos = int(tok_seq[t]), int(tok_pos[t])
            lo = max(0, pos - window + 1) if window > 0 else 0
            c = rows[sq][lo:pos + 1]
            for h in range(Hh):
                want[t, h] = torch.softmax(c @ q[t, h].double() * 0.2, 0) @ c[:, :R]
        args = (tok_seq.cuda(), tok_pos.cuda(), bt.cuda(), Hh, R, Dr, 0.2)
        a = ops.latent_attn(q.cuda(), pool.cuda(), *args, window=window)
        b = ops.latent_attn_blocks(q.cuda(), pool.cuda(), qb_start, qb_count, *args, window=window)
        assert (a.cpu().double() - want).abs().max() < 2e-5, window
        assert (b.cpu().double() - want).abs().max() < 2e-5, window


def test_latent_rows_and_query_parts_rotate_half():
    from mlx_vlm_amd import ops
    from mlx_vlm_amd.models.cache import PAGE

    g = torch.Generator().manual_seed(6)
    R, Dr, Hh, D = 10, 6, 2, 5
    d = torch.randn(6, R + Dr + 3, generator=g)
    w = torch.randn(R, generator=g)
    pos = torch.tensor([0, 1, 63, 64, 700, 2], dtype=torch.int32)
    seq = torch.tensor([0] * 5 + [1], dtype=torch.int32)
    bt = torch.zeros(2, 12, dtype=torch.int32)
    bt[0] = torch.arange(12, dtype=torch.int32).flip(0) + 1
    inv = torch.tensor([300.0 ** (-2 * i / Dr) for i in range(Dr // 2)])
    pool = torch.zeros(13, PAGE, R + Dr, device="cuda")
    ops.latent_kv_write(d.cuda(), w.cuda(), R, Dr, inv.cuda(), seq.cuda(), pos.cuda(), bt.cuda(), pool, 1e-5, rot_half=True)
    want = torch.cat([O.unit_rms(d.double()[:, :R], 1e-5) * w.double(), O.rotate_half(d.double()[:, R:R + Dr], pos, Dr, 300.0)], -1)
    for t in range(6):
        got = pool[int(bt[seq[t], pos[t] // PAGE]), int(pos[t]) % PAGE].cpu().double()
        assert (got - want[t]).abs().max() < 2e-4                                  # fp32 angles at position 700
    q = torch.randn(6, Hh * (D + Dr), generator=g)
    out = torch.zeros(6, Hh * (R + Dr), device="cuda")
    ops.rope_pairs_rows(q.cuda()[:, D:], D + Dr, Hh, Dr, inv.cuda(), pos.cuda(), out[:, R:], R + Dr, rot_half=True)
    wq = O.rotate_half(q.double().view(6, Hh, D + Dr)[..., D:], pos, Dr, 300.0)
    assert (out.cpu().double().view(6, Hh, R + Dr)[..., R:] - wq).abs().max() < 2e-4


# ------------------------------------------------------------------------------------------------ one-layer models
ONE = {"latent_moe": [H.latent()], "latent_dense_no_window": [H.latent(window=None, mlp="dense")],
       "latent_window_1_no_ff": [H.latent(heads=1, window=1, mlp=None)],
       "latent_wide": [H.latent(heads=2, dim=72, rot_dim=40, vdim=136, kv_rank=264, window=33, mlp="dense")],
       "latent_rank_beyond_the_block_form": [H.latent(heads=2, dim=8, rot_dim=4, vdim=8, kv_rank=520, window=20, mlp=None)],
       "attention": [H.attention()], "attention_equal_heads_plain": [H.attention(heads=3, kv_heads=3, softcap=None, every=None, mlp=None)],
       "attention_one_kv_head_window": [H.attention(heads=5, kv_heads=1, dim=12, vdim=20, window=11, every=1, mlp=H.moe(experts=3, top=1, groups=1, keep=1))],
       "attention_wide": [H.attention(heads=2, kv_heads=1, dim=136, vdim=72, every=64, mlp=H.moe(experts=8, top=3, ff=24, groups=4, keep=2))]}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", sorted(ONE))
def test_each_mixer_alone(tmp_path, kind, dtype):
    cfg = H.config(ONE[kind])
    W = H.weights(cfg, seed=3)
    ids = _ids(150, cfg["vocab"], 5)
    got = _whole(_load(tmp_path, cfg, W, dtype, tokens=512).language_model, ids)
    assert _close(got, O.Oracle(cfg, W, F64).forward(ids), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_match_layer_by_layer(tmp_path, dtype):
    cfg = H.config(H.mixed_layers())
    W = H.weights(cfg, seed=11)
    ids = _ids(90, cfg["vocab"], 6)
    lm = _load(tmp_path, cfg, W, dtype, tokens=512).language_model
    lm._trace = []
    c = lm.make_cache()
    lm.step([(c[0]._seq, ids)], want="all")
    ref = []
    O.Oracle(cfg, W, F64).forward(ids, ref)
    assert len(lm._trace) == len(ref) == 6
    for i, (a, b) in enumerate(zip(lm._trace, ref)):
        assert _close(a.cpu(), b, dtype), i
    lm._trace = None
    c[0]._seq.release()


# ------------------------------------------------------------------------------------------------ schedules
@pytest.fixture(scope="module")
def mixed32(tmp_path_factory):
    cfg = H.config(H.mixed_layers())
    W = H.weights(cfg, seed=21)
    model = _load(tmp_path_factory.mktemp("mixed32"), cfg, W, "float32", tokens=1024, seqs=4)
    return cfg, W, model.language_model


def test_portions_and_token_by_token_equal_the_whole_prompt(mixed32):
    cfg, W, lm = mixed32
    ids = _ids(200, cfg["vocab"], 7)
    whole = _whole(lm, ids)
    assert H.rel_rms(whole, O.Oracle(cfg, W, F64).forward(ids)) < TOL["float32"]
    for sizes in ([1], [2], [3, 1, 2], [37], [61, 2, 1], [63], [64], [65, 1, 1, 1, 2], [9, 70]):
        assert torch.equal(_portions(lm, ids, sizes), whole), sizes           # float32 serving: one summation order per token


def test_bf16_portions_and_decode(tmp_path):
    cfg = H.config(H.mixed_layers())
    W = H.weights(cfg, seed=22)
    lm = _load(tmp_path, cfg, W, "bfloat16", tokens=1024).language_model
    ids = _ids(140, cfg["vocab"], 8)
    want = O.Oracle(cfg, W, F64).forward(ids)
    for sizes in ([1], [2], [5, 1, 1, 40], [64, 3]):
        assert _close(_portions(lm, ids, sizes), want, "bfloat16"), sizes


def test_unequal_batch_equals_each_alone_and_pages_and_slots_are_reused(mixed32):
    cfg, W, lm = mixed32
    rng = np.random.default_rng(3)
    reqs = [_ids(n, cfg["vocab"], 30 + n) for n in (130, 2, 75, 1, 64, 199, 33)]
    alone = [_whole(lm, r) for r in reqs]
    free0 = lm.pool.free_pages
    live, waiting, got = {}, list(range(len(reqs))), {i: [] for i in range(len(reqs))}
    used_slots, used_pages = [], []
    while waiting or live:
        while waiting and len(live) < 4:
            i = waiting.pop(0)
            live[i] = [lm.make_cache(), 0]
            used_slots.append(live[i][0][0]._seq.seq)
        entries, who = [], []
        for i, (c, o) in live.items():
            if rng.random() < 0.25 and len(live) > 1:
                continue                                                     # left out of this step
            n = min(int(rng.choice([1, 1, 2, 3, 17, 64, 70])), len(reqs[i]) - o)
            entries.append((c[0]._seq, reqs[i][o:o + n]))
            who.append((i, n))
        if not entries:
            continue
        lg = lm.step(entries, want="all").cpu()
        o = 0
        for i, n in who:
            got[i].append(lg[o:o + n])
            o += n
            live[i][1] += n
            if live[i][1] == len(reqs[i]):
                c = live.pop(i)[0]
                used_pages += list(c[0]._seq.pages)
                c[0]._seq.release()
    for i in range(len(reqs)):
        assert torch.equal(torch.cat(got[i]), alone[i]), i
    assert lm.pool.free_pages == free0 and len(set(used_slots)) < len(used_slots) and len(set(used_pages)) < len(used_pages)


def test_pool_exhaustion_is_an_error_not_a_fault(tmp_path):
    cfg = H.config([H.latent(), H.attention()])
    lm = _load(tmp_path, cfg, H.weights(cfg, seed=1), "float32", tokens=128, seqs=2).language_model
    c = lm.make_cache()
    lm.step([(c[0]._seq, _ids(128, cfg["vocab"], 1))])
    with pytest.raises(RuntimeError):
        lm.step([(c[0]._seq, _ids(1, cfg["vocab"], 2))])
    c[0]._seq.release()
    c = lm.make_cache()
    lm.step([(c[0]._seq, _ids(100, cfg["vocab"], 3))])
    c[0]._seq.release()


# ------------------------------------------------------------------------------------------------ edges made visible
def _marked_embedding(W):
    """token 1 (`mark`) lives on stream direction 0 alone, token 2 (the asking token) on direction 1 alone; no other token
    has a component along either"""
    emb = W["embed"].float()
    emb[:, :2] = 0
    emb[1], emb[2] = 0, 0
    emb[1, 0], emb[2, 1] = 4.0, 4.0
    W["embed"] = emb.to(torch.bfloat16)
    W["l0.norm1"] = torch.zeros_like(W["l0.norm1"])


def _check_probe(lm, orc, cfg, dtype, n, ask, dist, seen, portions):
    ids = 3 + _ids(n, cfg["vocab"] - 3, 40 + ask + dist)
    ids[ask - dist], ids[ask] = 1, 2
    want = orc.forward(ids)
    other = ids.copy()
    other[ask - dist] = 5
    moved = H.rel_rms(orc.forward(other)[ask:ask + 1], want[ask:ask + 1])
    if seen:                                              # the probe is sharp: with and without `mark` in view differ widely
        assert moved > 0.05, (ask, dist, moved)
    else:
        assert moved < 1e-9, (ask, dist, moved)           # out of view: the asked row does not know the token at all
    for sizes in portions:
        sizes = [n for n in sizes if n > 0]
        got = _portions(lm, ids, sizes)
        assert H.rel_rms(got[ask:ask + 1], want[ask:ask + 1]) < (2.5 if dtype == "bfloat16" else 1) * TOL[dtype], (ask, dist, sizes)
        assert _close(got, want, dtype), (ask, dist, sizes)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("window", [1, 2, 16, 17, 64, 65, 130])
def test_latent_window_edge_in_prompt_and_decoding(tmp_path, window, dtype):
    """token `mark` appears once, at distance window - 1 (just inside) or window (just outside) of the asked position; the
    latent of `mark` and the query of the asking token are made so that their score stands out.  Whole prompt, portions cut
    at the edge and at the asked token, and decoding token by token must agree with the oracle."""
    cfg = H.config([H.latent(heads=2, dim=8, rot_dim=4, vdim=8, kv_rank=16, window=window, scale=1.0, mlp=None)], width=48, vocab=64)
    W = H.weights(cfg, seed=5)
    _marked_embedding(W)
    dkv, q, uk = W["l0.mix.dkv"].float(), W["l0.mix.q"].float(), W["l0.mix.uk"].float()
    dkv[:, 0], q[:, 1] = 0, 0
    dkv[0, 0] = 6.0                                       # `mark` fills latent channel 0 (and, after the norm, little else)
    uk[:, 0] = 0
    uk[0, 0], uk[8, 0] = 2.0, 2.0                         # key dimension 0 of both heads reads latent channel 0
    q[0, 1], q[12, 1] = 3.0, 3.0                          # unrotated query dimension 0 of both heads reads the asking token
    W["l0.mix.dkv"], W["l0.mix.q"], W["l0.mix.uk"] = dkv.to(torch.bfloat16), q.to(torch.bfloat16), uk.to(torch.bfloat16)
    lm = _load(tmp_path, cfg, W, dtype, tokens=1024).language_model
    orc = O.Oracle(cfg, W, F64)
    n = 2 * window + 70
    for ask in (window + 3, n - 1):
        for dist in (window - 1, window):
            if ask - dist < 0 or dist == 0:
                continue
            _check_probe(lm, orc, cfg, dtype, n, ask, dist, dist < window,
                         ([n], [ask - dist + 1, 1000], [ask, 1], [ask - 1, 2], [ask - dist, 1, 1000], [3, 1]))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_far_key_among_hundreds_and_at_page_borders(tmp_path, dtype):
    """causal grouped attention: one key whose score towers over all others, at the first positions, around page borders and
    hundreds of tokens back; seen from its own position's successor and from far away, in a prompt, at a portion's first
    token and decoded token by token"""
    cfg = H.config([H.attention(heads=2, kv_heads=1, dim=16, vdim=16, scale=1.0, softcap=40.0, coef=0.1, every=64, mlp=None)], width=48, vocab=64)
    W = H.weights(cfg, seed=5)
    _marked_embedding(W)
    k, q = W["l0.mix.k"].float(), W["l0.mix.q"].float()
    k[:, 0], q[:, 1] = 0, 0
    k[:, 0] = 3.0                                         # key of `mark`: the all-ones direction
    q[:, 1] = 3.0                                         # query of the asking token: the same direction, both heads
    alt = torch.tensor([1.0, -1.0] * 8)                   # every other key leans to a direction orthogonal to it
    W["l0.mix.k"], W["l0.mix.q"] = k.to(torch.bfloat16), q.to(torch.bfloat16)
    W["l0.mix.k.b"] = (2.0 * alt).to(torch.bfloat16)
    W["l0.mix.q.b"] = torch.zeros(32).to(torch.bfloat16)
    lm = _load(tmp_path, cfg, W, dtype, tokens=1024).language_model
    orc = O.Oracle(cfg, W, F64)
    n = 700
    for at in (0, 1, 63, 64, 65, 255, 256, 511, 640):
        for ask in sorted({at + 1, min(at + 130, n - 1), n - 1}):
            dist = ask - at
            _check_probe(lm, orc, cfg, dtype, n, ask, dist, True, ([n], [at + 1, 1000], [ask, 1], [ask - 1, 2]) + (([at, 1, 1000],) if at else ()))


def test_borrowed_keys_and_values_matter_and_follow_the_source(tmp_path):
    """a layer that reads the cache of an earlier layer (not the one before it) with its own queries, gate and constants"""
    layers = [H.attention(), H.latent(mlp="dense"), H.attention(heads=6, kv_heads=2, dim=24, vdim=16, kv_from=0, scale=0.2, softcap=None, every=3)]
    cfg = H.config(layers)
    W = H.weights(cfg, seed=41)
    assert "l2.mix.k" not in W and "l2.mix.v.b" not in W
    ids = _ids(120, cfg["vocab"], 43)
    want = O.Oracle(cfg, W, F64).forward(ids)
    own = H.config([layers[0], layers[1], H.attention(heads=6, kv_heads=2, dim=24, vdim=16, scale=0.2, softcap=None, every=3)])
    W2 = dict(H.weights(own, seed=44), **W)
    assert H.rel_rms(O.Oracle(own, W2, F64).forward(ids), want) > 1e-2              # whose keys it reads shows in the logits
    for dtype in ("float32", "bfloat16"):
        lm = _load(tmp_path, cfg, W, dtype, tokens=256, name=dtype).language_model
        assert _close(_whole(lm, ids), want, dtype), dtype
        assert _close(_portions(lm, ids, [7, 1, 30, 2]), want, dtype), dtype


def test_first_tokens_and_a_one_token_request(mixed32):
    cfg, W, lm = mixed32
    for n in (1, 2, 3, 4, 5):                                       # shorter than the windows
        ids = _ids(n, cfg["vocab"], 90 + n)
        want = O.Oracle(cfg, W, F64).forward(ids)
        assert H.rel_rms(_whole(lm, ids), want) < TOL["float32"]
        assert H.rel_rms(_portions(lm, ids, [1]), want) < TOL["float32"]


def test_long_decoding_crosses_pages_windows_and_multiplier_steps(tmp_path):
    cfg = H.config([H.latent(window=70), H.attention(every=64), H.latent(window=5, mlp="dense"), H.attention(kv_from=1, every=7, mlp=None)])
    W = H.weights(cfg, seed=17)
    ids = _ids(400, cfg["vocab"], 19)
    want = O.Oracle(cfg, W, F64).forward(ids)
    for dtype in ("float32", "bfloat16"):
        lm = _load(tmp_path, cfg, W, dtype, tokens=1024, name=dtype).language_model
        got = _portions(lm, ids, [20] + [1] * 380)
        assert _close(got, want, dtype)
        assert H.rel_rms(got[-1:], want[-1:]) < 2.5 * TOL[dtype]


def test_other_sizes(tmp_path):
    """widths, head sizes and expert sizes that are not multiples of 8, an odd vocabulary, multiplier 1, every expert chosen,
    one expert chosen, groups that all stay, a window on the grouped attention, one rotated pair"""
    layers = [H.attention(heads=3, kv_heads=1, dim=10, vdim=7, scale=0.7, softcap=2.5, coef=1.0, every=2, window=50,
                          mlp=H.moe(experts=5, top=5, ff=9, groups=5, keep=5, scale=0.5)),
              H.latent(heads=5, dim=6, rot_dim=2, vdim=9, kv_rank=13, window=1000, base=7.0, mlp=H.moe(experts=10, top=1, ff=12, groups=2, keep=1, scale=3.0)),
              H.attention(heads=4, kv_heads=4, dim=9, vdim=11, mlp=H.dense(ff=25)),
              H.latent(heads=1, dim=20, rot_dim=12, vdim=5, kv_rank=30, window=2, mlp=H.dense(ff=17))]
    cfg = H.config(layers, vocab=301, width=60, mult=1.0, eps=3e-4)
    W = H.weights(cfg, seed=23)
    ids = _ids(100, cfg["vocab"], 29)
    want = O.Oracle(cfg, W, F64).forward(ids)
    for dtype in ("float32", "bfloat16"):
        lm = _load(tmp_path, cfg, W, dtype, tokens=256, name=dtype).language_model
        assert _close(_whole(lm, ids), want, dtype), dtype
        assert _close(_portions(lm, ids, [50, 1, 2]), want, dtype), dtype


# ------------------------------------------------------------------------------------------------ generation
def _greedy_oracle(cfg, W, prompt, n):
    orc, ids, toks, margins = O.Oracle(cfg, W, F64), list(prompt), [], []
    for _ in range(n):
        lg = orc.forward(np.asarray(ids))[-1]
        top = torch.topk(lg, 2).values
        toks.append(int(lg.argmax()))
        margins.append(float((top[0] - top[1]) / lg.std()))
        ids.append(toks[-1])
    return toks, margins


def test_greedy_generation_through_generate_step_and_the_batch_generator(tmp_path):
    from mlx_vlm_amd.batch import BatchGenerator
    from mlx_vlm_amd.generate import generate_step

    cfg = H.config(H.mixed_layers()[:4])
    W = H.weights(cfg, seed=51)
    W["embed"] = (W["embed"].float() * 3).to(torch.bfloat16)        # wide margins: greedy choices survive bf16 logits
    model = _load(tmp_path, cfg, W, "float32", tokens=2048, seqs=8)
    prompts = [_ids(n, cfg["vocab"], 60 + n) for n in (9, 70, 33)]
    refs = [_greedy_oracle(cfg, W, p, 12) for p in prompts]

    def agree(got, ref):
        toks, margins = ref
        for a, b, m in zip(got, toks, margins):
            if a != b:
                assert m < 0.05, (got, toks, margins)            # a tie within the bf16 rounding of the sampler's logits
                return
    for p, ref in zip(prompts, refs):
        got = [t for t, _ in generate_step(p[None], model, None, None, max_tokens=12, temperature=0.0)]
        assert len(got) == 12
        agree(got, ref)
    gen = BatchGenerator(model, None, max_tokens=12, completion_batch_size=2, prefill_batch_size=2, compute_logprobs=True)
    uids = gen.insert([p for p in prompts])
    out = {u: [] for u in uids}
    while gen.has_work:
        _, rs = gen.next()
        for r in rs:
            out[r.uid].append(r.token)
    gen.close()
    for u, ref in zip(uids, refs):
        assert len(out[u]) == 12
        agree(out[u], ref)
    assert len(model.language_model.pool._free_seqs) >= 7         # rows gave their slots back (the scratch row keeps one)


def test_trace_session_replays_mixed_steps(tmp_path):
    from mlx_vlm_amd.batch import TraceSession

    cfg = H.config(H.mixed_layers()[:4])
    W = H.weights(cfg, seed=61)
    model = _load(tmp_path, cfg, W, "float32", tokens=256, seqs=4)
    a, b = _ids(100, cfg["vocab"], 1), _ids(30, cfg["vocab"], 2)
    wa, wb = O.Oracle(cfg, W, F64).forward(a), O.Oracle(cfg, W, F64).forward(b)
    s = TraceSession(model)
    assert s.step([("a", a[:64].tolist(), [])]) is None
    lg = s.step([("a", a[64:99].tolist(), [0, 34]), ("b", b[:29].tolist(), [28])])
    assert H.rel_rms(lg, torch.stack([wa[64], wa[98], wb[28]])) < TOL["float32"]
    lg = s.step([("b", b[29:].tolist(), [0]), ("a", a[99:].tolist(), [0])], end=["a", "b"])
    assert H.rel_rms(lg, torch.stack([wb[29], wa[99]])) < TOL["float32"]
    assert model.language_model.pool.free_pages == 4


def test_captured_decode_steps_equal_eager_ones(tmp_path):
    """a captured decode step is replayed many times, with eager work (another request's prompt, a release, synchronisations)
    between the replays; every replay's logits and token must equal the eager step's"""
    from mlx_vlm_amd.sample_utils import make_sampler

    cfg = H.config(H.mixed_layers())
    W = H.weights(cfg, seed=71)
    lm = _load(tmp_path, cfg, W, "bfloat16", tokens=2048, seqs=6).language_model
    sargs = make_sampler().engine_args()
    prompts = [_ids(n, cfg["vocab"], 80 + n) for n in (40, 7, 66)]

    def run(use_graph):
        caches = lm.make_cache_batch(3)
        lg = lm.prefill(torch.cat([torch.as_tensor(p) for p in prompts]).cuda().reshape(-1, 1), None, caches, [len(p) for p in prompts])
        st = lm.decode_begin(caches, lg.argmax(-1), np.zeros((3, 1)), max_new_tokens=80)
        out = []
        for i in range(70):                                          # crosses a page border and the windows in every row
            lm.decode_run(st, 1, sargs, use_graph=use_graph)
            out.append((st.tok.cpu().clone(), st.logits.float().cpu().clone()))
            if i % 9 == 4:                                           # eager work between replays
                other = lm.make_cache()
                lm.step([(other[0]._seq, _ids(30 + i, cfg["vocab"], i))])
                torch.cuda.synchronize()
                other[0]._seq.release()
        for c in caches:
            c[0]._seq.release()
        return out
    eager, graph = run(False), run(True)
    assert any(isinstance(v, tuple) for v in lm._graphs.values())            # a graph was captured and used
    for i, ((t0, l0), (t1, l1)) in enumerate(zip(eager, graph)):
        assert torch.equal(t0, t1) and torch.equal(l0, l1), i


def test_sampled_generation_uses_the_device_sampler_and_refuses_what_is_not_built(tmp_path):
    from mlx_vlm_amd.generate import generate_step

    cfg = H.config(H.mixed_layers()[:3])
    model = _load(tmp_path, cfg, H.weights(cfg, seed=91), "bfloat16", tokens=1024, seqs=4)
    p = _ids(20, cfg["vocab"], 5)
    runs = [[t for t, _ in generate_step(p[None], model, None, None, max_tokens=16, temperature=0.8, top_p=0.9, seed=7)] for _ in range(2)]
    assert runs[0] == runs[1] and len(runs[0]) == 16 and all(0 <= t < cfg["vocab"] for t in runs[0])
    with pytest.raises(NotImplementedError):
        list(generate_step(p[None], model, None, None, max_tokens=4, repetition_penalty=1.3))
    assert len(model.language_model.pool._free_seqs) == 4           # every generation gave its slot back
