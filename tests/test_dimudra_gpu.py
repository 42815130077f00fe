"""Dimudra on MI355X against the plain restatement in tests/dimudra_oracle.py (float64 on the CPU, dense masks, token loops).

Small random checkpoints with unequal sizes (tests/dimudra_helpers.py) are written to disk and loaded through
`utils.load_model` (registry by config.json, safetensors reader, weight packing).  float32 serving is compared tightly,
bfloat16 within the rounding of a 16-bit projection chain.  Covered: every mechanism alone (operator level and as a one-layer
model); looped spans; whole prompts against portions of several sizes (down to two tokens and one) and against token-by-token
decoding; batches of unequal requests against each alone; pages, state slots and carried convolution inputs freed and used
again; keys at page, tile and window borders, just inside and just outside the window and far back among hundreds, in prompts
and decoding, with one score made to stand out; recurrent states that remember hundreds of tokens; the first tokens; long
decoding; sizes that are equal or 1 elsewhere; greedy generation through generate_step and the continuous batch generator;
replay of a scheduled trace, also through the command line program; captured decode steps."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import dimudra_helpers as H
from tests import dimudra_oracle as O

pytestmark = pytest.mark.gpu
F64 = torch.float64
TOL = {"float32": 4e-5, "bfloat16": 4e-2}
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _close(got, want, dtype):
    """float32: every row within TOL.  bfloat16: the median row within TOL and eight rows in ten within twice that - with random
    router weights a choice of experts can sit inside the rounding of a 16-bit activation and pick another expert for that
    token, and a looped span meets such choices several times"""
    if dtype == "float32":
        return H.rel_rms(got, want) < TOL[dtype]
    return H.rel_rms(got, want, 0.5) < TOL[dtype] and H.rel_rms(got, want, 0.8) < 2 * TOL[dtype]


def _load(tmp_path, cfg, W, dtype, tokens=4096, seqs=6, name="m"):
    from mlx_vlm_amd.utils import load_model

    return load_model(H.write_checkpoint(str(tmp_path / name), cfg, W), dtype=dtype, kv_pool_tokens=tokens, max_seqs=seqs)


def _ids(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).numpy().astype(np.int32)


def _oracle(cfg, W, ids, streams=False):
    lg, st = O.forward(cfg, H.as_f64(W), ids)
    return (lg, st) if streams else lg


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


def _segments(lens, slots, pos0):
    """the tables of a ragged step"""
    i32 = torch.int32
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=i32).cuda()
    tok_seq = torch.cat([torch.full((n,), s, dtype=i32) for n, s in zip(lens, slots)]).cuda()
    tok_pos = torch.cat([torch.arange(p, p + n, dtype=i32) for n, p in zip(lens, pos0)]).cuda()
    return tok_seq, tok_pos, cu, torch.tensor(slots, dtype=i32).cuda(), torch.tensor(pos0, dtype=i32).cuda()


# ------------------------------------------------------------------------------------------------ operators
def test_residual_step_with_two_addends_and_an_fp32_norm_row():
    from mlx_vlm_amd import ops

    g = torch.Generator().manual_seed(2)
    for T in (torch.float32, torch.bfloat16):
        x = torch.randn(7, 50, generator=g)
        y, y2 = torch.randn(7, 60, generator=g).to(T), torch.randn(7, 52, generator=g).to(T)
        w = torch.full((50,), 1.25).to(T)
        xs = x.clone().cuda()
        h = ops.scaled_add_rms_(xs, y.cuda()[:, :50], 0.8, w=w.cuda(), eps=1e-5, y2=y2.cuda()[:, :50], mult2=1.3, h_dtype=torch.float32)
        want = x.double() + 0.8 * y.double()[:, :50] + 1.3 * y2.double()[:, :50]
        assert h.dtype == torch.float32 and (xs.cpu().double() - want).abs().max() < 2e-6
        assert (h.cpu().double() - O.scalar_norm(want, 1.25, 1e-5)).abs().max() < 1e-5
        hT = ops.scaled_add_rms_(xs, w=w.cuda(), eps=1e-5)                           # norm only, in the serving dtype
        assert hT.dtype == T and (hT.float().cpu() - h.cpu()).abs().max() < (1e-6 if T == torch.float32 else 3e-2)


@pytest.mark.parametrize("taps", [1, 2, 4, 7])
@pytest.mark.parametrize("T", [torch.float32, torch.bfloat16])
def test_short_convolution_carries_its_inputs_across_portions_and_reused_slots(T, taps):
    """three sequences in portions down to one token, two of them side by side in one launch; then a new sequence in a slot
    whose carry still holds the old one's inputs"""
    from mlx_vlm_amd import ops

    g = torch.Generator().manual_seed(taps)
    C = 70
    w, b = (0.5 * torch.randn(C, taps, generator=g)).to(T), torch.randn(C, generator=g).to(T)
    seqs = {s: torch.randn(n, C + 3, generator=g).to(T) for s, n in ((0, 29), (2, 11), (1, 5))}
    carry = torch.full((3, max(taps - 1, 1), C), float("nan")).cuda()[:, : taps - 1].contiguous() if taps > 1 else None
    for act, residual, bias in ((False, True, None), (True, False, b)):
        want = {}
        for s, x in seqs.items():
            y = O.causal_conv(x.double()[:, :C], w.double(), None if bias is None else bias.double())
            y = y + x.double()[:, :C] if residual else y
            want[s] = O.silu(y) if act else y
        got = {s: [] for s in seqs}
        at = {s: 0 for s in seqs}
        plan = [[(0, 5)], [(0, 1), (2, 3)], [(2, 1), (0, 1)], [(0, 2), (2, 7)], [(0, 20), (1, 5)]]
        for step in plan:
            lens, slots, pos0 = [n for _, n in step], [s for s, _ in step], [at[s] for s, _ in step]
            rows = torch.cat([seqs[s][at[s]: at[s] + n] for s, n in step]).cuda()
            out = ops.short_conv_rows(rows[:, :C], w.cuda(), carry, *_segments(lens, slots, pos0), bias=None if bias is None else bias.cuda(),
                                      act=act, residual=residual, out_dtype=torch.float32)
            o = 0
            for s, n in step:
                got[s].append(out[o:o + n].cpu())
                o, at[s] = o + n, at[s] + n
        for s in seqs:
            assert (torch.cat(got[s]).double() - want[s]).abs().max() < (1e-5 if T == torch.float32 else 2e-2), (s, act)
        # slot 0 again, from position 0: nothing of the old sequence may show
        x = seqs[2][:4]
        out = ops.short_conv_rows(x.cuda()[:, :C], w.cuda(), carry, *_segments([4], [0], [0]), bias=None if bias is None else bias.cuda(),
                                  act=act, residual=residual, out_dtype=torch.float32)
        assert (out.cpu().double() - want[2][:4]).abs().max() < (1e-5 if T == torch.float32 else 2e-2)


@pytest.mark.parametrize("C,N", [(70, 6), (40, 16), (33, 1), (10, 70), (9, 130)])
@pytest.mark.parametrize("T", [torch.float32, torch.bfloat16])
def test_selective_scan_against_a_token_loop_in_portions_and_reused_slots(T, C, N):
    from mlx_vlm_amd import _lib, ops

    g = torch.Generator().manual_seed(C + N)
    n = 45
    x, z = torch.randn(n, C + 5, generator=g).to(T), torch.randn(n, C + 1, generator=g).to(T)
    dt_pre, Bm, Cm = torch.randn(n, C, generator=g), torch.randn(n, N + 2, generator=g), torch.randn(n, N + 2, generator=g)
    dt_b, A_log, D = torch.randn(C, generator=g).to(T), (0.5 * torch.randn(C, N, generator=g)).to(T), torch.randn(C, generator=g).to(T)
    A = -torch.exp(A_log.double())
    S, want = torch.zeros(C, N, dtype=F64), torch.zeros(n, C, dtype=F64)
    for t in range(n):
        dt = O.softplus(dt_pre[t].double() + dt_b.double())
        xv = x[t, :C].double()
        S = torch.exp(dt[:, None] * A) * S + (dt * xv)[:, None] * Bm[t, :N].double()[None]
        want[t] = (S @ Cm[t, :N].double() + D.double() * xv) * O.silu(z[t, :C].double())
    state = torch.full((3, 1, C, N), float("nan")).cuda()

    R = 7
    low, wdt = torch.randn(n, R + 3, generator=g), torch.randn(C, R, generator=g).to(T)
    want_fused = None

    def run(lo, hi, slot, fused=False):
        out = torch.empty(hi - lo, C, dtype=T, device="cuda")
        xs, zs, dp, bs, cs = (t[lo:hi].cuda() for t in (x, z, dt_pre, Bm, Cm))
        keep = [t.cuda() for t in (dt_b, A_log, D)]
        _, _, cu, sl, p0 = _segments([hi - lo], [slot], [lo])
        a = _lib.SelectiveScanArgs()
        a.x, a.ldx, a.z, a.ldz = xs.data_ptr(), xs.stride(0), zs.data_ptr(), zs.stride(0)
        a.dt_pre, a.lddt, a.B, a.Cm, a.ldbc = dp.data_ptr(), dp.stride(0), bs.data_ptr(), cs.data_ptr(), bs.stride(0)
        if fused:                                                       # the step-size projection inside the scan
            lw, wd = low[lo:hi].cuda(), wdt.cuda()
            keep += [lw, wd]
            a.dt_pre, a.dt_low, a.dt_w, a.R, a.lddt = None, lw.data_ptr(), wd.data_ptr(), R, lw.stride(0)
        a.dt_bias, a.A_log, a.D = (k.data_ptr() for k in keep[:3])
        a.seg_start, a.seg_slot, a.seg_pos0 = cu.data_ptr(), sl.data_ptr(), p0.data_ptr()
        a.state, a.out, a.ldo, a.C, a.N = state.data_ptr(), out.data_ptr(), out.stride(0), C, N
        ops.selective_scan(a, 1, hi - lo, T == torch.float32)
        torch.cuda.synchronize()
        return out.float().cpu()
    tol = 2e-4 if T == torch.float32 else 6e-2
    scale = want.abs().max()
    whole = run(0, n, 1)
    assert (whole.double() - want).abs().max() < tol * scale
    cuts = [0, 17, 18, 20, 36, n]
    parts = torch.cat([run(a, b, 2) for a, b in zip(cuts, cuts[1:])])
    assert torch.equal(parts, whole)                                    # token-by-token arithmetic: the cut does not show
    assert torch.equal(run(0, n, 2), whole)                             # a used slot, from position 0
    assert (state[2, 0].cpu().double() - S).abs().max() < 2e-4 * S.abs().max().clamp_min(1.0)
    pre = (low[:, :R].double() @ wdt.double().T).float()
    dt_pre.copy_(pre)
    given, fused = run(0, n, 1), run(0, n, 1, fused=True)
    assert (fused.double() - given.double()).abs().max() < tol * scale
    assert torch.equal(torch.cat([run(a, b, 0, fused=True) for a, b in zip(cuts, cuts[1:])]), fused)


@pytest.mark.parametrize("E,top,groups,keep", [(8, 3, 4, 2), (6, 2, 3, 2), (12, 4, 1, 1), (5, 5, 5, 5), (9, 1, 3, 1), (130, 6, 10, 3), (6, 2, 6, 3)])
def test_router_sigmoid_scores_correction_group_sums_and_weights(E, top, groups, keep):
    from mlx_vlm_amd import ops

    g = torch.Generator().manual_seed(E + top)
    z = torch.randn(40, E + 2, generator=g) * 2
    for corr in (torch.randn(E, generator=g) * 0.4, -3.0 - torch.rand(E, generator=g), None):     # (all choice scores negative: a
        gate, idx, wgt, ex = ops.moe_route_sigmoid(z.cuda(), E, top, groups, keep, correction=None if corr is None else corr.cuda(), extra=1)
        chosen, w = O.route(z[:, :E].double(), torch.zeros(E, dtype=F64) if corr is None else corr.double(), top, groups, keep)
        for t in range(40):                                                                      # group that is out stays out)
            assert sorted(idx[t].tolist()) == sorted(chosen[t].tolist()), t
            dense = torch.zeros(E, dtype=F64)
            dense[chosen[t]] = w[t]
            assert (gate[t].cpu().double() - dense).abs().max() < 1e-6
            assert abs(float(wgt[t].sum()) - 1.0) < 1e-5
        assert (ex[:, 0].cpu().double() - torch.sigmoid(z[:, E].double())).abs().max() < 1e-6


def test_headnorm_rotate_half_then_unit_rms_and_whole_row_norm_with_bias():
    from mlx_vlm_amd import ops
    from mlx_vlm_amd.models.cache import PAGE

    g = torch.Generator().manual_seed(4)
    Hh, D = 3, 14
    x = torch.randn(9, Hh * D + 5, generator=g)
    pos = torch.tensor([0, 1, 63, 64, 65, 700, 5, 6, 7], dtype=torch.int32)
    seq = torch.tensor([0] * 6 + [1] * 3, dtype=torch.int32)
    bt = torch.zeros(2, 12, dtype=torch.int32)
    bt[0] = torch.arange(12, dtype=torch.int32).flip(0) + 1
    for dims in (0, 2, 6, 14):
        inv = torch.tensor([50.0 ** (-2 * i / dims) for i in range(dims // 2)]).cuda() if dims else None
        want = torch.zeros(9, Hh, D, dtype=F64)
        for t in range(9):                                        # the oracle turns by the row index: one row at a time, at its position
            full = torch.zeros(int(pos[t]) + 1, Hh, D, dtype=F64)
            full[-1] = x[t, : Hh * D].double().view(Hh, D)
            want[t] = O.rms(O.rotate_half_partial(full, dims, 50.0), 1e-5)[-1]
        dense = torch.zeros(9, Hh * D, device="cuda")
        ops.headnorm_rows(x.cuda()[:, : Hh * D], Hh, D, pos.cuda(), dense, eps=1e-5, rot_dims=dims, inv_freq=inv, rot_half=True)
        assert (dense.cpu().double().view(9, Hh, D) - want).abs().max() < 3e-4                   # fp32 angles at position 700
        kp = torch.zeros(13, PAGE, Hh * D, device="cuda")
        ops.headnorm_rows(x.cuda()[:, : Hh * D], Hh, D, pos.cuda(), kp, eps=1e-5, rot_dims=dims, inv_freq=inv, rot_half=True,
                          tok_seq=seq.cuda(), block_table=bt.cuda())
        for t in range(9):
            assert (kp[int(bt[seq[t], pos[t] // PAGE]), int(pos[t]) % PAGE].cpu().double().view(Hh, D) - want[t]).abs().max() < 3e-4
    # one norm over all heads of the row, bias first, a weight per coordinate
    b, w = torch.randn(Hh * D, generator=g), 1 + 0.3 * torch.randn(Hh * D, generator=g)
    dense = torch.zeros(9, Hh * D, device="cuda")
    ops.headnorm_rows(x.cuda()[:, : Hh * D], 1, Hh * D, pos.cuda(), dense, eps=1e-5, w=w.cuda(), bias=b.cuda())
    assert (dense.cpu().double() - O.rms(x.double()[:, : Hh * D] + b.double(), 1e-5) * w.double()).abs().max() < 1e-5


@pytest.mark.parametrize("D,Dv", [(20, 12), (24, 16), (136, 72)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_with_a_sink_against_a_dense_softmax(dtype, D, Dv):
    """two sequences at different offsets on scattered pages (one 1890 tokens deep), value size unequal to the key size, an
    elementwise gate; the sink with and without a window, both forms"""
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
    gate = torch.randn(42, Hh * Dv + 8, generator=g).to(dtype)
    qb_start = torch.tensor([0, 16, 32, 37], dtype=torch.int32).cuda()
    qb_count = torch.tensor([16, 16, 5, 5], dtype=torch.int32).cuda()
    rows = {sq: (kpool[bt[sq].long()].reshape(-1, G, D).double(), vpool[bt[sq].long()].reshape(-1, G, Dv).double()) for sq in (1, 2)}
    for window, sink, scale in ((0, True, 0.3), (0, False, 0.3), (17, True, 0.3), (1025, True, 0.05), (0, True, -0.4)):
        want = torch.zeros(42, Hh, Dv, dtype=F64)
        for t in range(42):
            sq, pos = int(tok_seq[t]), int(tok_pos[t])
            lo = max(0, pos - window + 1) if window > 0 else 0
            for h in range(Hh):
                kh = h // (Hh // G)
                e = torch.exp(rows[sq][0][lo:pos + 1, kh] @ q[t, h * D:(h + 1) * D].double() * scale)
                want[t, h] = (e / (e.sum() + (1.0 if sink else 0.0))) @ rows[sq][1][lo:pos + 1, kh]
        want = want * torch.sigmoid(gate.double()[:, : Hh * Dv]).view(42, Hh, Dv)
        args = (tok_seq.cuda(), tok_pos.cuda(), bt.cuda(), Hh, G, D, Dv, scale)
        a = torch.zeros(42, Hh * Dv, dtype=dtype, device="cuda")
        b = torch.zeros(42, Hh * Dv, dtype=dtype, device="cuda")
        kw = dict(window=window, gate=gate.cuda()[:, : Hh * Dv], sink=sink)
        ops.window_attn_rows(q.cuda(), kpool.cuda(), vpool.cuda(), *args, a, **kw)
        ops.window_attn_blocks(q.cuda(), kpool.cuda(), vpool.cuda(), qb_start, qb_count, *args, b, **kw)
        tol = 2e-5 if dtype == torch.float32 else 2e-2
        assert (a.cpu().double().view(42, Hh, Dv) - want).abs().max() < tol, (window, sink)
        assert (b.cpu().double().view(42, Hh, Dv) - want).abs().max() < tol, (window, sink)


# ------------------------------------------------------------------------------------------------ one-layer models
ONE = {"hgrn2_moe": [H.hgrn2()], "hgrn2_one_wide_head_no_ff": [H.hgrn2(heads=1, dim=72, vdim=136, mlp=None)],
       "hgrn2_many_small_heads": [H.hgrn2(heads=7, dim=3, vdim=5, mlp=H.moe(experts=3, top=1, groups=1, keep=1, shared=8))],
       "parallel": [H.parallel()], "parallel_window_1_one_tap": [H.parallel(heads=1, kv_heads=1, window=1, conv=1, state=1, dt_rank=1, mlp=None)],
       "parallel_no_window_wide": [H.parallel(heads=2, kv_heads=1, dim=136, vdim=72, window=None, inner=130, state=70, dt_rank=9, conv=5,
                                              mlp=H.moe(experts=8, top=3, ff=24, groups=4, keep=2, shared=0))],
       "parallel_left_only": [H.parallel(right_scale=0.0)], "parallel_right_only": [H.parallel(left_scale=0.0, mlp=None)],
       "attention": [H.attention()], "attention_equal_heads_no_rotation": [H.attention(heads=3, kv_heads=3, rot_dims=0, mlp=None)],
       "attention_one_kv_head_full_rotation": [H.attention(heads=5, kv_heads=1, dim=12, vdim=20, rot_dims=12, mlp=H.moe(experts=4, top=2, groups=2, keep=1))],
       "attention_wide": [H.attention(heads=2, kv_heads=1, dim=136, vdim=72, rot_dims=64, base=10000.0)]}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", sorted(ONE))
def test_each_mixer_alone(tmp_path, kind, dtype):
    cfg = H.config(ONE[kind], taps=1 if "one_tap" in kind else (0 if "wide" in kind else 3))
    W = H.weights(cfg, seed=3)
    ids = _ids(150, cfg["vocab"], 5)
    got = _whole(_load(tmp_path, cfg, W, dtype, tokens=512).language_model, ids)
    assert _close(got, _oracle(cfg, W, ids), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_runs_match_run_by_run_through_a_looped_span(tmp_path, dtype):
    cfg = H.mixed_config()
    W = H.weights(cfg, seed=11)
    ids = _ids(90, cfg["vocab"], 6)
    lm = _load(tmp_path, cfg, W, dtype, tokens=512).language_model
    lm._trace = []
    c = lm.make_cache()
    lm.step([(c[0]._seq, ids)], want="all")
    _, ref = _oracle(cfg, W, ids, streams=True)
    assert len(lm._trace) == len(ref) == 9 and len(c) == 9
    for i, (a, b) in enumerate(zip(lm._trace, ref)):
        assert _close(a.cpu(), b, dtype), i
    lm._trace = None
    c[0]._seq.release()


@pytest.mark.parametrize("loop", [None, (0, 6, 2), (0, 1, 3), (5, 6, 2), (2, 4, 1), (3, 3, 4)])
def test_loop_spans(tmp_path, loop):
    """no loop, the whole stack, the first layer alone, the last layer alone, a span that runs once, an empty span"""
    cfg = H.config(H.mixed_layers(), loop=loop)
    W = H.weights(cfg, seed=13)
    ids = _ids(70, cfg["vocab"], 3)
    lm = _load(tmp_path, cfg, W, "float32", tokens=256).language_model
    assert len(lm.make_cache()) == len(O.layer_runs(cfg))
    assert _close(_whole(lm, ids), _oracle(cfg, W, ids), "float32")


# ------------------------------------------------------------------------------------------------ schedules
@pytest.fixture(scope="module")
def mixed32(tmp_path_factory):
    cfg = H.mixed_config()
    W = H.weights(cfg, seed=21)
    model = _load(tmp_path_factory.mktemp("mixed32"), cfg, W, "float32", tokens=1024, seqs=4)
    return cfg, W, model.language_model


def test_portions_and_token_by_token_equal_the_whole_prompt(mixed32):
    cfg, W, lm = mixed32
    ids = _ids(200, cfg["vocab"], 7)
    whole = _whole(lm, ids)
    assert H.rel_rms(whole, _oracle(cfg, W, ids)) < TOL["float32"]
    for sizes in ([1], [2], [3, 1, 2], [37], [61, 2, 1], [63], [64], [65, 1, 1, 1, 2], [9, 70]):
        assert torch.equal(_portions(lm, ids, sizes), whole), sizes           # float32 serving: one summation order per token


def test_bf16_portions_and_decode(tmp_path):
    cfg = H.mixed_config()
    W = H.weights(cfg, seed=22)
    lm = _load(tmp_path, cfg, W, "bfloat16", tokens=1024).language_model
    ids = _ids(140, cfg["vocab"], 8)
    want = _oracle(cfg, W, ids)
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
    cfg = H.config([H.parallel(), H.attention()])
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
def _marked(W):
    """token 1 (`mark`) lives on stream direction 0 alone, token 2 (the asking token) on direction 1 alone; no other token has
    a component along either.  The input convolution is switched off by its weights (the kernel still runs and carries), so
    that a token shows in no neighbour's input."""
    emb = W["embed"].float()
    emb[:, :2] = 0
    emb[1], emb[2] = 0, 0
    emb[1, 0], emb[2, 1] = 4.0, 4.0
    W["embed"] = emb.to(torch.bfloat16)
    W["l0.canon1"] = torch.zeros_like(W["l0.canon1"])


def _towering(W, p, n_q, n_k):
    """the key of `mark` and the query of the asking token point along the all-ones direction; every other key leans to a
    direction orthogonal to it"""
    k, q = W[p + "k"].float(), W[p + "q"].float()
    k[:, 0], q[:, 1] = 3.0, 3.0
    W[p + "k"], W[p + "q"] = k.to(torch.bfloat16), q.to(torch.bfloat16)
    if p + "k.b" in W:
        W[p + "k.b"] = (2.0 * torch.tensor([1.0, -1.0] * (n_k // 2))).to(torch.bfloat16)
        W[p + "q.b"] = torch.zeros(n_q).to(torch.bfloat16)
        W[p + "k.norm"], W[p + "q.norm"] = torch.ones(n_k).to(torch.bfloat16), torch.ones(n_q).to(torch.bfloat16)


def _check_probe(lm, cfg, W, dtype, n, ask, dist, seen, portions):
    ids = 3 + _ids(n, cfg["vocab"] - 3, 40 + ask + dist)
    ids[ask - dist], ids[ask] = 1, 2
    want = _oracle(cfg, W, ids)
    other = ids.copy()
    other[ask - dist] = 5
    moved = H.rel_rms(_oracle(cfg, W, other)[ask:ask + 1], want[ask:ask + 1])
    if seen:                                              # the probe is sharp: with and without `mark` in view differ widely
        assert moved > 0.05, (ask, dist, moved)
    else:
        assert moved < 1e-9, (ask, dist, moved)           # out of view: the asked row does not know the token at all
    for sizes in portions:
        sizes = [s for s in sizes if s > 0]
        got = _portions(lm, ids, sizes)
        assert H.rel_rms(got[ask:ask + 1], want[ask:ask + 1]) < (2.5 if dtype == "bfloat16" else 1) * TOL[dtype], (ask, dist, sizes)
        assert _close(got, want, dtype), (ask, dist, sizes)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("window", [1, 2, 16, 17, 64, 65, 130])
def test_window_edge_in_prompt_and_decoding(tmp_path, window, dtype):
    """token `mark` appears once, at distance window - 1 (just inside) or window (just outside) of the asked position, and its
    key towers over all others.  Whole prompt, portions cut at the edge and at the asked token, and decoding token by token
    must agree with the oracle.  (The scan beside the attention is weighted 0: it would remember the token anyway.)"""
    cfg = H.config([H.parallel(heads=2, kv_heads=1, dim=8, vdim=8, scale=1.0, window=window, right_scale=0.0, mlp=None)], width=48, vocab=64, taps=3)
    W = H.weights(cfg, seed=5)
    _marked(W)
    _towering(W, "l0.mix.left.", 16, 8)
    lm = _load(tmp_path, cfg, W, dtype, tokens=1024).language_model
    n = 2 * window + 70
    for ask in (window + 3, n - 1):
        for dist in (window - 1, window):
            if ask - dist < 0 or dist == 0:
                continue
            _check_probe(lm, cfg, W, dtype, n, ask, dist, dist < window,
                         ([n], [ask - dist + 1, 1000], [ask, 1], [ask - 1, 2], [ask - dist, 1, 1000], [3, 1]))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_far_key_among_hundreds_and_at_page_borders(tmp_path, dtype):
    """causal attention with a sink: one key whose score towers over all others, at the first positions, around page borders
    and hundreds of tokens back; seen from its own position's successor and from far away, in a prompt, at a portion's first
    token and decoded token by token"""
    cfg = H.config([H.attention(heads=2, kv_heads=1, dim=16, vdim=16, scale=1.0, rot_dims=2, mlp=None)], width=48, vocab=64, taps=2)
    W = H.weights(cfg, seed=5)
    _marked(W)
    _towering(W, "l0.mix.", 32, 16)
    lm = _load(tmp_path, cfg, W, dtype, tokens=1024).language_model
    n = 700
    for at in (0, 1, 63, 64, 65, 255, 256, 511, 640):
        for ask in sorted({at + 1, min(at + 130, n - 1), n - 1}):
            _check_probe(lm, cfg, W, dtype, n, ask, ask - at, True, ([n], [at + 1, 1000], [ask, 1], [ask - 1, 2]) + (([at, 1, 1000],) if at else ()))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recurrent_states_remember_hundreds_of_tokens(tmp_path, dtype):
    """forget gates held near one (a lower bound of 0.998; slow decays and small steps in the scan): tokens 40..43 still move
    the logits 300 and 650 tokens later - whole, in portions, and decoded from a state that crossed many steps"""
    cfg = H.config([H.hgrn2(heads=2, dim=8, vdim=8, mlp=None), H.parallel(heads=2, kv_heads=1, dim=8, vdim=8, window=4, inner=24, state=4, mlp=None)],
                   width=48, vocab=64, taps=2)
    W = H.weights(cfg, seed=7)
    W["l0.mix.lower"] = torch.full_like(W["l0.mix.lower"], 0.998)
    W["l1.mix.right.A_log"] = torch.full_like(W["l1.mix.right.A_log"], -6.0)
    W["l1.mix.right.dt.b"] = torch.full_like(W["l1.mix.right.dt.b"], -3.0)
    n = 700
    ids = _ids(n, cfg["vocab"], 3)
    want = _oracle(cfg, W, ids)
    other = ids.copy()
    other[40:44] = (other[40:44] + 9) % cfg["vocab"]
    moved = _oracle(cfg, W, other)
    for ask in (340, 699):
        assert H.rel_rms(moved[ask:ask + 1], want[ask:ask + 1]) > 1e-2, ask
    lm = _load(tmp_path, cfg, W, dtype, tokens=1024).language_model
    for sizes in ([n], [44, 1000], [41, 2, 300, 1], [64], [600] + [1] * 100):
        got = _portions(lm, ids, sizes)
        # (states that average hundreds of values: fp32 sums over 700 tokens are a few times less exact than elsewhere)
        assert H.rel_rms(got, want) < 2e-4 if dtype == "float32" else _close(got, want, dtype), sizes
        assert H.rel_rms(got[[340, 699]], want[[340, 699]]) < 2.5 * TOL[dtype], sizes


def test_first_tokens_and_a_one_token_request(mixed32):
    cfg, W, lm = mixed32
    for n in (1, 2, 3, 4, 5):                                       # shorter than the windows and the convolutions
        ids = _ids(n, cfg["vocab"], 90 + n)
        want = _oracle(cfg, W, ids)
        assert H.rel_rms(_whole(lm, ids), want) < TOL["float32"]
        assert H.rel_rms(_portions(lm, ids, [1]), want) < TOL["float32"]


def test_long_decoding_crosses_pages_and_windows(tmp_path):
    cfg = H.config([H.parallel(window=70), H.attention(), H.hgrn2(), H.parallel(window=5, mlp=None)], loop=(0, 2, 2))
    W = H.weights(cfg, seed=17)
    ids = _ids(400, cfg["vocab"], 19)
    want = _oracle(cfg, W, ids)
    for dtype in ("float32", "bfloat16"):
        lm = _load(tmp_path, cfg, W, dtype, tokens=1024, name=dtype).language_model
        got = _portions(lm, ids, [20] + [1] * 380)
        assert _close(got, want, dtype)
        assert H.rel_rms(got[-1:], want[-1:]) < 2.5 * TOL[dtype]


def test_other_sizes(tmp_path):
    """widths, head sizes, channel counts and expert sizes that are not multiples of 8, an odd vocabulary, every expert chosen,
    one expert chosen, groups of one expert, groups that all stay, branch scales of 1, one rotated pair, a window beyond the prompt"""
    layers = [H.parallel(heads=3, kv_heads=1, dim=10, vdim=7, scale=0.7, window=1000, inner=21, state=5, dt_rank=3, conv=2, left_scale=1.0,
                         right_scale=1.0, mlp=H.moe(experts=5, top=5, ff=9, groups=5, keep=5, shared=11)),
              H.attention(heads=5, kv_heads=5, dim=6, vdim=9, rot_dims=2, base=7.0, mlp=H.moe(experts=10, top=1, ff=12, groups=2, keep=1, shared=0)),
              H.hgrn2(heads=4, dim=9, vdim=11, mlp=H.moe(experts=6, top=2, ff=7, groups=6, keep=3, shared=5)),
              H.parallel(heads=1, kv_heads=1, dim=20, vdim=5, window=2, inner=17, state=33, dt_rank=1, conv=6, mlp=H.moe(experts=3, top=2, ff=17, groups=1, keep=1))]
    cfg = H.config(layers, vocab=301, width=60, eps=3e-4, taps=5, escale=4.0, loop=(1, 3, 2))
    W = H.weights(cfg, seed=23)
    ids = _ids(100, cfg["vocab"], 29)
    want = _oracle(cfg, W, ids)
    for dtype in ("float32", "bfloat16"):
        lm = _load(tmp_path, cfg, W, dtype, tokens=256, name=dtype).language_model
        assert _close(_whole(lm, ids), want, dtype), dtype
        assert _close(_portions(lm, ids, [50, 1, 2]), want, dtype), dtype


# ------------------------------------------------------------------------------------------------ generation
def _greedy_oracle(cfg, W, prompt, n):
    ids, toks, margins = list(prompt), [], []
    for _ in range(n):
        lg = _oracle(cfg, W, np.asarray(ids))[-1]
        top = torch.topk(lg, 2).values
        toks.append(int(lg.argmax()))
        margins.append(float((top[0] - top[1]) / lg.std()))
        ids.append(toks[-1])
    return toks, margins


def test_greedy_generation_through_generate_step_and_the_batch_generator(tmp_path):
    from mlx_vlm_amd.batch import BatchGenerator
    from mlx_vlm_amd.generate import generate_step

    cfg = H.config(H.mixed_layers()[:4], loop=(1, 3, 2))
    W = H.weights(cfg, seed=51)
    W["head"] = (W["head"].float() * 3).to(torch.bfloat16)          # wide margins: greedy choices survive bf16 logits
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

    cfg = H.config(H.mixed_layers()[:4], loop=(0, 2, 2))
    W = H.weights(cfg, seed=61)
    model = _load(tmp_path, cfg, W, "float32", tokens=256, seqs=4)
    a, b = _ids(100, cfg["vocab"], 1), _ids(30, cfg["vocab"], 2)
    wa, wb = _oracle(cfg, W, a), _oracle(cfg, W, b)
    s = TraceSession(model)
    assert s.step([("a", a[:64].tolist(), [])]) is None
    lg = s.step([("a", a[64:99].tolist(), [0, 34]), ("b", b[:29].tolist(), [28])])
    assert H.rel_rms(lg, torch.stack([wa[64], wa[98], wb[28]])) < TOL["float32"]
    lg = s.step([("b", b[29:].tolist(), [0]), ("a", a[99:].tolist(), [0])], end=["a", "b"])
    assert H.rel_rms(lg, torch.stack([wb[29], wa[99]])) < TOL["float32"]
    assert model.language_model.pool.free_pages == 4


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_program_writes_the_asked_logits(tmp_path, dtype):
    """bin/trace_run as a child process: steps on its standard input, `done <step>` lines and logits files back"""
    cfg = H.config(H.mixed_layers()[:3], loop=(1, 3, 2))
    W = H.weights(cfg, seed=63)
    folder = H.write_checkpoint(str(tmp_path / "m"), cfg, W)
    a, b = _ids(70, cfg["vocab"], 1), _ids(9, cfg["vocab"], 2)
    wa, wb = _oracle(cfg, W, a), _oracle(cfg, W, b)
    steps = [dict(step=0, entries=[dict(id="a", tokens=a[:66].tolist(), want=[0, 65])], end=[]),
             dict(step=1, entries=[dict(id="a", tokens=a[66:67].tolist(), want=[]), dict(id="b", tokens=b[:2].tolist(), want=[1])], end=[]),
             dict(step=2, entries=[dict(id="b", tokens=b[2:].tolist(), want=[6]), dict(id="a", tokens=a[67:].tolist(), want=[0, 2])], end=["a", "b"]),
             dict(step=3, entries=[dict(id="c", tokens=b.tolist(), want=[8])], end=["c"])]
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", str(out),
                        "--max-tokens", "192"], input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2", "done 3"]
    want = {0: wa[[0, 65]], 1: wb[[1]], 2: torch.cat([wb[[8]], wa[[67, 69]]]), 3: wb[[8]]}
    for n, w in want.items():
        got = torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(-1, cfg["vocab"]))
        assert got.shape == w.shape and H.rel_rms(got, w) < 2.5 * TOL[dtype], n


def test_captured_decode_steps_equal_eager_ones(tmp_path):
    """a captured decode step is replayed many times, with eager work (another request's prompt, a release, synchronisations)
    between the replays; every replay's logits and token must equal the eager step's"""
    from mlx_vlm_amd.sample_utils import make_sampler

    cfg = H.mixed_config()
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
