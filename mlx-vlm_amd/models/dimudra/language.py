"""Dimudra language model on the HIP operator library (the ragged step of models/ragged.py).

Pre-norm layers on an fp32 residual stream x; a norm's weight is ONE number g (kept as a vector of equal entries):
    n = rms(x) * g1 (fp32)      h = n + conv(n)  over time, per channel, inputs carried per sequence      -> serving dtype
    proj = h @ [mixer projections]^T                                     one GEMM (rows packed at load)
    parallel  : left  = biased q / k / v, RMS norm over the whole q (k) row with a weight, keys into the paged fp32 cache, values
                        into theirs, sliding-window softmax attention without positions, elementwise sigmoid gate, W_o
                right = [x | z] -> short convolution + silu on x (inputs carried) -> [dt | B | C] in fp32 -> selective scan over
                        the sequence's fp32 state (step sizes softplus(W_dt dt + b) evaluated in its staging), times silu(z), W_o
                x += left_scale * left + right_scale * right
    hgrn2     : matrix-state recurrence whose forget gate per state row (bounded below) also sets the write strength,
                q = silu(.), per-head RMS norm with a weight shared by the heads, W_o
    attention : rotate-half positions on the first rot.dims dimensions, then unit-RMS q / k per head, causal softmax with a sink
                (one more exp(0) in the denominator), elementwise sigmoid gate, W_o
    x += mixer and the second norm, one kernel
    moe       : fp32 router logits (+ the shared expert's gate logit as one more row) -> sigmoid scores, choice on scores +
                correction inside the best groups, normalised weights; ONE GEMM over every expert's [gate | up] rows and the
                shared expert's, silu(gate) * up * weight (exact zeros for experts a token did not choose), ONE GEMM over the
                stacked W_down - the sum over experts and the shared expert is its k loop
    x += ff and the next run's first norm, one kernel
A span of layers may run several times in a row: a RUN is one execution of a layer; runs of one layer share its tensors and
have caches / states / carried inputs of their own (the pool is keyed by run).  Before every pass but the first the embedding
output is added to the stream.  Final norm of the wanted rows, logits = rows @ head^T.
"""
from __future__ import annotations

from types import SimpleNamespace
from typing import Dict

import torch

from ... import _lib, ops
from ..cache import HybridPool, PagedSequence, RecurrentCache, RowCache
from ..ragged import RaggedLanguageModel, _al8, inv_freq, pack_cols, pack_rows
from .config import ModelConfig, attention_constants


class LanguageModel(RaggedLanguageModel):
    NAME = "Dimudra"

    def __init__(self, config: ModelConfig, **kwargs):
        super().__init__(config, **kwargs)

    @property
    def layers(self):
        return list(range(len(self._runs))) if getattr(self, "_runs", None) else list(range(len(self.config.runs())))

    # ------------------------------------------------------------------ weights
    def load_weights(self, W: Dict[str, torch.Tensor]):
        cfg, dev, T = self.config, self.device, self.dtype
        f32 = torch.float32

        def g(name, shape, dtype=None):
            if name not in W:
                raise KeyError(f"Dimudra checkpoint: tensor {name!r} missing")
            t = W[name]
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"Dimudra checkpoint: {name} is {tuple(t.shape)}, the config says {tuple(shape)}")
            return t.to(device=dev, dtype=dtype or T).contiguous()

        Wd, taps = cfg.width, cfg.canon_taps

        def one(name):           # a norm whose weight is one number, as the vector the norm kernels take
            return g(name, ()).reshape(1).expand(Wd).contiguous()

        self._w = dict(embed=g("embed", (cfg.vocab, Wd)), final_norm=one("final.norm"), head=g("head", (cfg.vocab, Wd)))
        self._L = []
        for i, L in enumerate(cfg.layers):
            p, m = f"l{i}.", L.mixer
            ns = SimpleNamespace(type=L.type, norm1=one(p + "norm1"))
            ns.canon = g(p + "canon1", (Wd, taps)) if taps else None
            if L.type == "parallel":
                a, r = m["left"], m["right"]
                pl, pr = p + "mix.left.", p + "mix.right."
                ns.H, ns.G, ns.D, ns.Dv, ns.scale, ns.window, _, _ = attention_constants(a)
                ns.inner, ns.N, ns.R, ns.ctaps = int(r["inner"]), int(r["state"]), int(r["dt_rank"]), int(r["conv"])
                ns.left_scale, ns.right_scale = float(m["left_scale"]), float(m["right_scale"])
                H, G, D, Dv = ns.H, ns.G, ns.D, ns.Dv
                parts = [("q", g(pl + "q", (H * D, Wd))), ("k", g(pl + "k", (G * D, Wd))), ("v", g(pl + "v", (G * Dv, Wd))),
                         ("g", g(pl + "g", (H * Dv, Wd))), ("in", g(pr + "in", (2 * ns.inner, Wd)))]
                ns.qb, ns.kb, ns.vb = g(pl + "q.b", (H * D,)), g(pl + "k.b", (G * D,)), g(pl + "v.b", (G * Dv,))
                ns.qnorm, ns.knorm = g(pl + "q.norm", (H * D,)), g(pl + "k.norm", (G * D,))
                ns.left_o = g(pl + "o", (Wd, H * Dv))
                ns.conv, ns.conv_b = g(pr + "conv", (ns.inner, ns.ctaps)), g(pr + "conv.b", (ns.inner,))
                ns.wx = g(pr + "x", (ns.R + 2 * ns.N, ns.inner))
                ns.wdt, ns.dt_b = g(pr + "dt", (ns.inner, ns.R)), g(pr + "dt.b", (ns.inner,))
                ns.A_log, ns.Dskip = g(pr + "A_log", (ns.inner, ns.N)), g(pr + "D", (ns.inner,))
                ns.right_o = g(pr + "o", (Wd, ns.inner))
            elif L.type == "hgrn2":
                H, D, Dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
                ns.H, ns.D, ns.Dv = H, D, Dv
                parts = [("q", g(p + "mix.q", (H * D, Wd))), ("f", g(p + "mix.f", (H * D, Wd))), ("v", g(p + "mix.v", (H * Dv, Wd)))]
                ns.fb, ns.lower = g(p + "mix.f.b", (H * D,)), g(p + "mix.lower", (H * D,))
                # (one weight of vdim for every head: laid out per head for the finish pass)
                ns.normw = g(p + "mix.norm", (Dv,)).repeat(H).contiguous()
                ns.wo = g(p + "mix.o", (Wd, H * Dv))
            else:
                ns.H, ns.G, ns.D, ns.Dv, ns.scale, ns.window, ns.rot_dims, base = attention_constants(m)
                H, G, D, Dv = ns.H, ns.G, ns.D, ns.Dv
                ns.inv_freq = inv_freq(ns.rot_dims, base, dev) if ns.rot_dims else None
                parts = [("q", g(p + "mix.q", (H * D, Wd))), ("g", g(p + "mix.g", (H * Dv, Wd))), ("k", g(p + "mix.k", (G * D, Wd))),
                         ("v", g(p + "mix.v", (G * Dv, Wd)))]
                ns.wo = g(p + "mix.o", (Wd, H * Dv))
            ns.wproj, ns.off = pack_rows(parts, T, dev)
            ns.ff, ns.sff = L.ff, L.shared_ff
            if L.mlp is not None:
                ns.norm2 = one(p + "norm2")
                ns.E, ns.top, ns.groups, ns.keep = L.router
                E, ff, sff = ns.E, ns.ff, ns.sff
                rows = [g(p + "mlp.router", (E, Wd))] + ([g(p + "mlp.shared.sg", (1, Wd))] if sff else [])
                ns.router = torch.cat(rows, dim=0).contiguous()            # the shared expert's gate logit rides as row E
                ns.correction = g(p + "mlp.correction", (E,), f32) if p + "mlp.correction" in W else None
                # expert e's rows: [gate_e | up_e], 2 ff rows side by side, so that a step of few rows can skip whole experts
                ex = torch.cat([t for e in range(E) for t in (g(p + f"mlp.e{e}.gate", (ff, Wd)), g(p + f"mlp.e{e}.up", (ff, Wd)))], dim=0)
                up = [("experts", ex)]
                down = [("experts", torch.cat([g(p + f"mlp.e{e}.down", (Wd, ff)) for e in range(E)], dim=1))]
                if sff:
                    up.append(("shared", torch.cat([g(p + "mlp.shared.gate", (sff, Wd)), g(p + "mlp.shared.up", (sff, Wd))], dim=0)))
                    down.append(("shared", g(p + "mlp.shared.down", (Wd, sff))))
                ns.wff, ns.foff = pack_rows(up, T, dev)
                ns.down, ns.doff = pack_cols(down, T, dev)
                if ns.down.shape[1] % 64:           # whole K tiles for the matrix-core kernel's staging: zero columns meet zero activations
                    ns.down = torch.nn.functional.pad(ns.down, (0, 64 - ns.down.shape[1] % 64)).contiguous()
            self._L.append(ns)
        # caches, states and carried inputs: one set per RUN of a layer
        self._runs = cfg.runs()
        self._x0 = any(readd for _, readd in self._runs)
        rows, states, aux = {}, {}, {}
        for r, (i, _) in enumerate(self._runs):
            ns = self._L[i]
            if taps > 1:
                aux[(r, "canon")] = (taps - 1, Wd)
            if ns.type in ("parallel", "attention"):
                rows[(r, "k")] = (ns.G * ns.D, f32)                       # normed keys, never rounded
                rows[(r, "v")] = (ns.G * ns.Dv, T)
            if ns.type == "parallel":
                states[r] = (1, ns.inner, ns.N, False)
                if ns.ctaps > 1:
                    aux[(r, "conv")] = (ns.ctaps - 1, ns.inner)
            elif ns.type == "hgrn2":
                states[r] = (ns.H, ns.D, ns.Dv, False)
        self.pool = HybridPool(len(self._runs), rows, states, self._kv_pool_tokens, self._max_seqs, device=dev, dtype=T, aux_layers=aux)
        return self

    # ------------------------------------------------------------------ cache
    def make_cache(self):
        seq = PagedSequence(self.pool)
        return [RowCache(seq, (r, "k")) if self._L[i].type == "attention" else RecurrentCache(seq, r) for r, (i, _) in enumerate(self._runs)]

    def make_cache_batch(self, n: int):
        return [self.make_cache() for _ in range(n)]

    # ------------------------------------------------------------------ mixers
    def _softmax_attention(self, ns, proj, pl, r, keep, whole_row_norm):
        """-> [tokens, heads * vdim] in the serving dtype: gated attention read-outs.  whole_row_norm: the left half of a parallel
        mixer (bias, one RMS norm over all heads of q / k with a weight, a window, no positions); else the attention mixer
        (positions, unit RMS per head, a sink)"""
        Tn, H, G, D, Dv, dev = pl.Tn, ns.H, ns.G, ns.D, ns.Dv, self.device
        col = lambda name: proj[:, ns.off[name]:]          # noqa: E731   (2-D view: data_ptr at the column, stride(0) = pitch)
        pool, eps = self.pool, self.config.norm_eps
        kpool, vpool = pool.rows[(r, "k")], pool.rows[(r, "v")]
        q = torch.empty(Tn, H * D, dtype=torch.float32, device=dev)
        paged = dict(tok_seq=pl.tok_seq, block_table=pool.block_table, raw=col("v"), raw_pool=vpool)
        if whole_row_norm:
            ops.headnorm_rows(col("k"), 1, G * D, pl.tok_pos, kpool, eps=eps, w=ns.knorm, bias=ns.kb, raw_dim=G * Dv, raw_bias=ns.vb, **paged)
            ops.headnorm_rows(col("q"), 1, H * D, pl.tok_pos, q, eps=eps, w=ns.qnorm, bias=ns.qb)
        else:
            rot = dict(rot_dims=ns.rot_dims, inv_freq=ns.inv_freq, rot_half=True)
            ops.headnorm_rows(col("k"), G, D, pl.tok_pos, kpool, eps=eps, raw_dim=Dv, **rot, **paged)
            ops.headnorm_rows(col("q"), H, D, pl.tok_pos, q, eps=eps, **rot)
        out = torch.empty(Tn, _al8(H * Dv), dtype=self.dtype, device=dev)[:, : H * Dv]
        # prompt form wherever a step brings more than decode rows, and always in float32 serving - one kernel there, so that
        # a token's bits do not depend on the schedule (shapes its LDS tiles cannot take run the row form everywhere)
        DP = (D + 3) & ~3
        nacc = 4 if Dv <= 64 else (8 if Dv <= 128 else 16)
        blocks_fit = Dv <= 256 and (16 * DP + 16 * (DP + 4) + 16 * nacc * 16 + 16 * 17 + 48) * 4 <= 48 * 1024
        args = dict(window=ns.window, gate=col("g"), sink=not whole_row_norm)
        if (self.dtype == torch.float32 or Tn > 8) and blocks_fit:
            ops.window_attn_blocks(q, kpool, vpool, pl.qb_start, pl.qb_count, pl.tok_seq, pl.tok_pos, pool.block_table, H, G, D, Dv,
                                   ns.scale, out, **args)
        else:
            ops.window_attn_rows(q, kpool, vpool, pl.tok_seq, pl.tok_pos, pool.block_table, H, G, D, Dv, ns.scale, out, **args)
        keep.append(q)
        return out

    def _selective_scan(self, ns, proj, pl, r, keep):
        """-> [tokens, inner] in the serving dtype: the scan's read-out times silu(z)"""
        Tn, C_, N, R, dev, T = pl.Tn, ns.inner, ns.N, ns.R, self.device, self.dtype
        f32 = torch.float32
        xz = proj[:, ns.off["in"]:]
        xc = torch.empty(Tn, _al8(C_), dtype=T, device=dev)[:, :C_]
        ops.short_conv_rows(xz, ns.conv, self.pool.aux.get((r, "conv")), pl.tok_seq, pl.tok_pos, pl.cu, pl.slot, pl.pos0, bias=ns.conv_b,
                            act=True, out=xc)
        # what enters the recurrence after the projections stays fp32: step-size logits, B and C
        dbc = self._linear(xc, ns.wx, out_dtype=f32)
        out = torch.empty(Tn, _al8(C_), dtype=T, device=dev)[:, :C_]
        a = _lib.SelectiveScanArgs()
        a.x, a.ldx, a.z, a.ldz = xc.data_ptr(), xc.stride(0), xz[:, C_:].data_ptr(), xz.stride(0)
        a.dt_low, a.dt_w, a.R, a.lddt = dbc.data_ptr(), ns.wdt.data_ptr(), R, dbc.stride(0)     # W_dt is applied inside the scan's staging
        a.B, a.Cm, a.ldbc = dbc[:, R:].data_ptr(), dbc[:, R + N:].data_ptr(), dbc.stride(0)
        a.dt_bias, a.A_log, a.D = ns.dt_b.data_ptr(), ns.A_log.data_ptr(), ns.Dskip.data_ptr()
        a.seg_start, a.seg_slot, a.seg_pos0 = pl.cu.data_ptr(), pl.slot.data_ptr(), pl.pos0.data_ptr()
        a.state, a.out, a.ldo, a.C, a.N = self.pool.state[r].data_ptr(), out.data_ptr(), out.stride(0), C_, N
        ops.selective_scan(a, pl.nseg, Tn, T == f32)
        keep += [xc, dbc]
        return out

    def _hgrn2(self, ns, proj, pl, r, keep):
        """-> [tokens, heads * vdim] in the serving dtype: head-normed read-outs"""
        Tn, H, D, Dv, dev = pl.Tn, ns.H, ns.D, ns.Dv, self.device
        col = lambda name: proj[:, ns.off[name]:]          # noqa: E731
        raw = torch.empty(Tn, H, Dv, dtype=torch.float32, device=dev)
        out = torch.empty(Tn, _al8(H * Dv), dtype=self.dtype, device=dev)[:, : H * Dv]
        a = _lib.RecurrenceArgs()
        a.q, a.k, a.v = col("q").data_ptr(), col("f").data_ptr(), col("v").data_ptr()
        a.ldq = a.ldk = a.ldv = proj.stride(0)
        a.gated, a.q_act, a.fbias, a.lower = 2, 1, ns.fb.data_ptr(), ns.lower.data_ptr()
        a.normw, a.gate_act, a.eps = ns.normw.data_ptr(), 2, self.config.norm_eps
        a.seg_start, a.seg_slot, a.seg_pos0 = pl.cu.data_ptr(), pl.slot.data_ptr(), pl.pos0.data_ptr()
        a.state, a.raw, a.out, a.ldo = self.pool.state[r].data_ptr(), raw.data_ptr(), out.data_ptr(), out.stride(0)
        a.H, a.D, a.Dv = H, D, Dv
        ops.linear_recurrence(a, pl.nseg, Tn, self.dtype == torch.float32)
        keep.append(raw)
        return out

    # ------------------------------------------------------------------ the device side of a step
    def _run(self, pl, logits_dtype=torch.float32):
        """Nothing here looks at host data that changes between two steps of the same shape, so a decode step can be
        captured once and replayed."""
        cfg, dev, T = self.config, self.device, self.dtype
        eps, Tn, f32 = cfg.norm_eps, pl.Tn, torch.float32
        few = Tn <= self.STREAM_ROWS and T != f32       # decode rows over bf16 weights: weight-streaming projections
        x = ops.embed_scale_f32(pl.ids, self._w["embed"], cfg.embedding_scale)
        x0 = x.clone() if self._x0 else None
        keep = [pl.md, pl.ids, x0]
        pending = None           # (y, mult, y2, mult2): a sublayer's result that the next reader's norm kernel adds to the stream

        def add_norm(w, h_dtype=None):
            nonlocal pending
            y, mult, y2, mult2 = pending or (None, 1.0, None, 1.0)
            pending = None
            return ops.scaled_add_rms_(x, y, mult, w=w, eps=eps, y2=y2, mult2=mult2, h_dtype=h_dtype)

        for r, (i, readd) in enumerate(self._runs):
            ns = self._L[i]
            if readd:
                if pending:
                    add_norm(None)
                ops.stream_add_(x, x0)
            if ns.canon is not None:
                n1 = add_norm(ns.norm1, f32)
                h = torch.empty(Tn, _al8(cfg.width), dtype=T, device=dev)[:, : cfg.width]
                ops.short_conv_rows(n1, ns.canon, self.pool.aux.get((r, "canon")), pl.tok_seq, pl.tok_pos, pl.cu, pl.slot, pl.pos0,
                                    residual=True, out=h)
                keep.append(n1)
            else:
                h = add_norm(ns.norm1)
            proj = self._linear(h, ns.wproj)
            if ns.type == "parallel":
                ol = self._softmax_attention(ns, proj, pl, r, keep, True)
                yl = self._linear(ol, ns.left_o)
                orr = self._selective_scan(ns, proj, pl, r, keep)
                yr = self._linear(orr, ns.right_o)
                pending = (yl, ns.left_scale, yr, ns.right_scale)
                keep += [ol, orr]
            else:
                o = self._hgrn2(ns, proj, pl, r, keep) if ns.type == "hgrn2" else self._softmax_attention(ns, proj, pl, r, keep, False)
                pending = (self._linear(o, ns.wo), 1.0, None, 1.0)
                keep.append(o)
            keep += [h, proj, pending]
            if ns.ff:
                E, ff, sff = ns.E, ns.ff, ns.sff
                h2 = add_norm(ns.norm2)
                z = self._linear(h2, ns.router, out_dtype=f32)
                route, _, _, sgate = ops.moe_route_sigmoid(z, E, ns.top, ns.groups, ns.keep, correction=ns.correction, extra=1 if sff else 0)
                skip = dict(skip_gate=route, skip_col0=0, E=E, ff=2 * ff) if few else None
                gu = self._linear(h2, ns.wff, skip=skip)
                K = ns.down.shape[1]
                act = (torch.empty if K == E * ff + sff else torch.zeros)(Tn, K, dtype=T, device=dev)
                ops.glu_rows(gu, gu[:, ff:], ops.GLU_SILU, out=act[:, : E * ff], route=route, E=E, ff=ff, estride=2 * ff)
                if sff:
                    so, do = ns.foff["shared"], ns.doff["shared"]
                    ops.glu_rows(gu[:, so:], gu[:, so + sff:], ops.GLU_SILU, out=act[:, do: do + sff], route=sgate, E=1, ff=sff, estride=sff)
                pending = (self._linear(act, ns.down), 1.0, None, 1.0)
                keep += [h2, z, route, sgate, gu, act, pending]
            if self._trace is not None:
                add_norm(None)
                self._trace.append(x.clone())
        if pending:
            add_norm(None)
        self._keep = keep
        if pl.rows.size == 0:
            return None
        xl = x if pl.all_rows else x.index_select(0, pl.rows_d.long())
        hn = ops.scaled_add_rms_(xl, w=self._w["final_norm"], eps=eps)
        # rows at a pitch of vocab rounded up to 8: 16-byte aligned bf16 rows for the samplers, whatever the vocabulary
        out = torch.empty(hn.shape[0], _al8(cfg.vocab), dtype=logits_dtype, device=dev)[:, : cfg.vocab]
        return self._linear(hn, self._w["head"], out=out)
