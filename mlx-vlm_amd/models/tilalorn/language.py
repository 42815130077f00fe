"""Tilalorn language model on the HIP operator library (the ragged step of models/ragged.py).

Pre-norm layers on an fp32 residual stream x; a norm weight is kept as its offset from one (`rms(x) * (1 + w)`), every sublayer's
result enters the stream times one model-wide multiplier m:
    h = norm1(x)        proj = h @ [mixer projections]^T                         one GEMM (rows packed at load)
    attention        : bias + unit RMS per head on q and k (k into the paged fp32 key cache, v + bias into the value cache in
                       the same launch), q times 1 + coef * ln(floor((pos + 1) / every) + 1), grouped-head causal softmax
                       attention with capped scores, one sigmoid gate per head.  A layer with `kv_from` has no key / value
                       projections and reads the named layer's caches with its own queries
    latent_attention : absorbed form over ONE cached row per token [normed latent | rotated key part]: q' = U_k^T q per head,
                       rotate-half positions on the rotated parts, softmax attention inside a sliding window straight over
                       the rows, U_v per head, elementwise sigmoid gate
    x += m * (o @ W_o^T)        and the next reader's norm, one kernel
    dense ff  : norm2(x) @ [W_gate | W_up]^T, gelu_tanh(gate) * up, W_down
    moe ff    : router logits (fp32) -> softmax over all experts, the `top` best inside the best expert groups, weights =
                scores * scale; ONE GEMM over every expert's [gate | up] rows, silu(gate) * up * weight (exact zeros for the
                experts a token did not choose), ONE GEMM over the stacked W_down - the sum over experts is its k loop
    x += m * ff        and the next layer's norm1, one kernel
Final norm of the wanted rows, logits = rows @ embed^T.
"""
from __future__ import annotations

from types import SimpleNamespace
from typing import Dict

import torch

from ... import ops
from ..cache import HybridPool, PagedSequence, RowCache
from ..ragged import RaggedLanguageModel, _al8, inv_freq, pack_rows
from .config import ModelConfig


class LanguageModel(RaggedLanguageModel):
    NAME = "Tilalorn"

    def __init__(self, config: ModelConfig, **kwargs):
        super().__init__(config, **kwargs)

    # ------------------------------------------------------------------ weights
    def load_weights(self, W: Dict[str, torch.Tensor]):
        cfg, dev, T = self.config, self.device, self.dtype

        def g(name, shape):
            if name not in W:
                raise KeyError(f"Tilalorn checkpoint: tensor {name!r} missing")
            t = W[name]
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"Tilalorn checkpoint: {name} is {tuple(t.shape)}, the config says {tuple(shape)}")
            return t.to(device=dev, dtype=T).contiguous()

        Wd = cfg.width
        self._w = dict(embed=g("embed", (cfg.vocab, Wd)), final_norm=g("final.norm", (Wd,)))
        rows = {}
        self._L = []
        for i, L in enumerate(cfg.layers):
            p, m = f"l{i}.", L.mixer
            ns = SimpleNamespace(type=L.type, norm1=g(p + "norm1", (Wd,)), window=L.window, scale=float(m["scale"]))
            ns.src = i if L.kv_from is None else L.kv_from
            if L.type == "attention":
                H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
                ns.H, ns.G, ns.D, ns.Dv = H, G, D, Dv
                ns.cap = float(m["softcap"]) if m.get("softcap") is not None else 0.0
                qt = m.get("q_temp")
                ns.q_temp = (float(qt["coef"]), int(qt["every"])) if qt is not None else None
                parts = [("q", g(p + "mix.q", (H * D, Wd))), ("g", g(p + "mix.g", (H, Wd)))]
                ns.qb = g(p + "mix.q.b", (H * D,))
                if ns.src == i:
                    parts += [("k", g(p + "mix.k", (G * D, Wd))), ("v", g(p + "mix.v", (G * Dv, Wd)))]
                    ns.kb, ns.vb = g(p + "mix.k.b", (G * D,)), g(p + "mix.v.b", (G * Dv,))
                    rows[(i, "k")] = (G * D, torch.float32)           # unit-RMS keys, never rounded
                    rows[(i, "v")] = (G * Dv, T)
                ns.kmix = H * Dv
            else:
                H, D, Dr, Dv, R = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
                ns.H, ns.D, ns.Dr, ns.Dv, ns.R = H, D, Dr, Dv, R
                ns.inv_freq = inv_freq(Dr, m["rot"]["base"], dev) if Dr else None
                parts = [("q", g(p + "mix.q", (H * (D + Dr), Wd))), ("g", g(p + "mix.g", (H * Dv, Wd)))]
                if ns.src == i:
                    parts.append(("dkv", g(p + "mix.dkv", (R + Dr, Wd))))
                    ns.dkv_norm = g(p + "mix.dkv.norm", (R,))
                    rows[(i, "c")] = R + Dr
                # per-head maps of the latent, moved to the query side (transposed) and the output side
                ns.uk_t = g(p + "mix.uk", (H * D, R)).view(H, D, R).transpose(1, 2).contiguous()          # [H, R, D]
                ns.uv = g(p + "mix.uv", (H * Dv, R)).view(H, Dv, R).contiguous()                           # [H, Dv, R]
                ns.kmix = H * Dv
            ns.wproj, ns.off = pack_rows(parts, T, dev)
            ns.wo = g(p + "mix.o", (Wd, ns.kmix))
            ns.ff, ns.moe = L.ff, L.moe
            if L.mlp is not None:
                ns.norm2 = g(p + "norm2", (Wd,))
                if ns.moe:
                    ns.E, ns.top, ns.groups, ns.keep, ns.rscale = L.router
                    ns.router = g(p + "mlp.router", (ns.E, Wd))
                    # expert e's rows: [gate_e | up_e], 2 ff rows side by side, so that a step of few rows can skip whole experts
                    ns.wff = torch.cat([t for e in range(ns.E) for t in (g(p + f"mlp.e{e}.gate", (ns.ff, Wd)), g(p + f"mlp.e{e}.up", (ns.ff, Wd)))], dim=0)
                    ns.wff, _ = pack_rows([("experts", ns.wff)], T, dev)
                    ns.down = torch.cat([g(p + f"mlp.e{e}.down", (Wd, ns.ff)) for e in range(ns.E)], dim=1).contiguous()
                else:
                    ns.wff, ns.foff = pack_rows([("gate", g(p + "mlp.gate", (ns.ff, Wd))), ("up", g(p + "mlp.up", (ns.ff, Wd)))], T, dev)
                    ns.down = g(p + "mlp.down", (Wd, ns.ff))
            self._L.append(ns)
        self.pool = HybridPool(len(cfg.layers), rows, {}, self._kv_pool_tokens, self._max_seqs, device=dev, dtype=T)
        return self

    # ------------------------------------------------------------------ cache
    def _cache_key(self, i):
        ns = self._L[i]
        return (ns.src, "k" if ns.type == "attention" else "c")

    def make_cache(self):
        seq = PagedSequence(self.pool)
        return [RowCache(seq, self._cache_key(i), shared=self._L[i].src != i) for i in range(len(self._L))]

    def make_cache_batch(self, n: int):
        return [self.make_cache() for _ in range(n)]

    # ------------------------------------------------------------------ mixers
    def _attention(self, ns, proj, pl, i, keep):
        """-> [tokens, heads * vdim] in the serving dtype: gated attention read-outs"""
        Tn, H, G, D, Dv, dev = pl.Tn, ns.H, ns.G, ns.D, ns.Dv, self.device
        col = lambda name: proj[:, ns.off[name]:]          # noqa: E731   (2-D view: data_ptr at the column, stride(0) = pitch)
        pool, eps = self.pool, self.config.norm_eps
        kpool, vpool = pool.rows[(ns.src, "k")], pool.rows[(ns.src, "v")]
        if ns.src == i:
            ops.headnorm_rows(col("k"), G, D, pl.tok_pos, kpool, eps=eps, bias=ns.kb, tok_seq=pl.tok_seq, block_table=pool.block_table,
                              raw=col("v"), raw_dim=Dv, raw_bias=ns.vb, raw_pool=vpool)
        q = torch.empty(Tn, H * D, dtype=torch.float32, device=dev)
        ops.headnorm_rows(col("q"), H, D, pl.tok_pos, q, eps=eps, bias=ns.qb, temp=ns.q_temp)
        out = torch.empty(Tn, _al8(H * Dv), dtype=self.dtype, device=dev)[:, : H * Dv]
        # prompt form wherever a step brings more than decode rows, and always in float32 serving - one kernel there, so that
        # a token's bits do not depend on the schedule (shapes its LDS tiles cannot take run the row form everywhere)
        DP = (D + 3) & ~3
        nacc = 4 if Dv <= 64 else (8 if Dv <= 128 else 16)
        blocks_fit = Dv <= 256 and (16 * DP + 16 * (DP + 4) + 16 * nacc * 16 + 16 * 17 + 48) * 4 <= 48 * 1024
        args = dict(temp=None, window=ns.window, gate=col("g"), cap=ns.cap, gate_head=True)
        if (self.dtype == torch.float32 or Tn > 8) and blocks_fit:
            ops.window_attn_blocks(q, kpool, vpool, pl.qb_start, pl.qb_count, pl.tok_seq, pl.tok_pos, pool.block_table, H, G, D, Dv,
                                   ns.scale, out, **args)
        else:
            ops.window_attn_rows(q, kpool, vpool, pl.tok_seq, pl.tok_pos, pool.block_table, H, G, D, Dv, ns.scale, out, **args)
        keep.append(q)
        return out

    def _latent_attention(self, ns, proj, pl, i, keep):
        """-> [tokens, heads * vdim] in the serving dtype"""
        Tn, H, D, Dr, Dv, R, dev = pl.Tn, ns.H, ns.D, ns.Dr, ns.Dv, ns.R, self.device
        col = lambda name: proj[:, ns.off[name]:]          # noqa: E731
        pool, bt = self.pool, self.pool.block_table
        cpool = pool.rows[(ns.src, "c")]
        if ns.src == i:
            ops.latent_kv_write(col("dkv"), ns.dkv_norm, R, Dr, ns.inv_freq, pl.tok_seq, pl.tok_pos, bt, cpool, self.config.norm_eps,
                                rot_half=True)
        qabs = torch.empty(Tn, H * (R + Dr), dtype=torch.float32, device=dev)
        # absorbed keys: q'_h = U_k,h^T q_h for every head (batch = heads, strides inside the packed rows)
        ops.linear_any(col("q"), ns.uk_t.view(H * R, D), out=qabs, M=Tn, N=R, K=D, batch=H, stride_a=D + Dr, stride_w=R * D, stride_c=R + Dr)
        if Dr:
            ops.rope_pairs_rows(proj[:, ns.off["q"] + D:], D + Dr, H, Dr, ns.inv_freq, pl.tok_pos, qabs[:, R:], R + Dr, rot_half=True)
        if (self.dtype == torch.float32 or Tn > 8) and R <= 512 and (32 * _al8(R + Dr) + 512) * 4 <= 150 * 1024:
            ol = ops.latent_attn_blocks(qabs.view(Tn, H, R + Dr), cpool, pl.qb_start, pl.qb_count, pl.tok_seq, pl.tok_pos, bt, H, R, Dr,
                                        ns.scale, window=ns.window)
        else:
            ol = ops.latent_attn(qabs.view(Tn, H, R + Dr), cpool, pl.tok_seq, pl.tok_pos, bt, H, R, Dr, ns.scale, window=ns.window)
        out = torch.empty(Tn, _al8(H * Dv), dtype=self.dtype, device=dev)[:, : H * Dv]
        ops.linear_any(ol.view(Tn, H * R), ns.uv.view(H * Dv, R), out=out, M=Tn, N=Dv, K=R, batch=H, stride_a=R, stride_w=Dv * R, stride_c=Dv)
        ops.glu_rows(col("g"), out, ops.GLU_SIGMOID, out=out)
        keep += [qabs, ol]
        return out

    # ------------------------------------------------------------------ the device side of a step
    def _run(self, pl, logits_dtype=torch.float32):
        """Nothing here looks at host data that changes between two steps of the same shape, so a decode step can be
        captured once and replayed."""
        cfg, dev, T = self.config, self.device, self.dtype
        eps, mult, Tn = cfg.norm_eps, cfg.residual_mult, pl.Tn
        few = Tn <= self.STREAM_ROWS and T != torch.float32       # decode rows over bf16 weights: weight-streaming projections
        x = ops.embed_scale_f32(pl.ids, self._w["embed"], 1.0)
        h = ops.scaled_add_rms_(x, w=self._L[0].norm1, w_offset=1.0, eps=eps) if self._L else None
        keep = [pl.md, pl.ids]
        for i, ns in enumerate(self._L):
            nxt = self._L[i + 1].norm1 if i + 1 < len(self._L) else None
            proj = self._linear(h, ns.wproj)
            o = (self._attention if ns.type == "attention" else self._latent_attention)(ns, proj, pl, i, keep)
            y = self._linear(o, ns.wo)
            h2 = ops.scaled_add_rms_(x, y, mult, w=ns.norm2 if ns.ff else nxt, w_offset=1.0, eps=eps)
            keep += [h, proj, o, y]
            if ns.ff:
                if ns.moe:
                    z = self._linear(h2, ns.router, out_dtype=torch.float32)
                    route, _, _ = ops.moe_route_scored(z, ns.top, ns.groups, ns.keep, ns.rscale)
                    skip = dict(skip_gate=route, skip_col0=0, E=ns.E, ff=2 * ns.ff) if few else None
                    gu = self._linear(h2, ns.wff, skip=skip)
                    act = torch.empty(Tn, _al8(ns.E * ns.ff), dtype=T, device=dev)[:, : ns.E * ns.ff]
                    ops.glu_rows(gu, gu[:, ns.ff:], ops.GLU_SILU, out=act, route=route, E=ns.E, ff=ns.ff, estride=2 * ns.ff)
                    keep += [z, route]
                else:
                    gu = self._linear(h2, ns.wff)
                    act = torch.empty(Tn, _al8(ns.ff), dtype=T, device=dev)[:, : ns.ff]
                    ops.glu_rows(gu[:, ns.foff["gate"]: ns.foff["gate"] + ns.ff], gu[:, ns.foff["up"]:], ops.GLU_GELU_TANH, out=act)
                y2 = self._linear(act, ns.down)
                h = ops.scaled_add_rms_(x, y2, mult, w=nxt, w_offset=1.0, eps=eps)
                keep += [h2, gu, act, y2]
            else:
                h = h2
            if self._trace is not None:
                self._trace.append(x.clone())
        keep.append(h)
        self._keep = keep
        if pl.rows.size == 0:
            return None
        xl = x if pl.all_rows else x.index_select(0, pl.rows_d.long())
        hn = ops.scaled_add_rms_(xl, w=self._w["final_norm"], w_offset=1.0, eps=eps)
        # rows at a pitch of vocab rounded up to 8: 16-byte aligned bf16 rows for the samplers, whatever the vocabulary
        out = torch.empty(hn.shape[0], _al8(cfg.vocab), dtype=logits_dtype, device=dev)[:, : cfg.vocab]
        return self._linear(hn, self._w["embed"], out=out)
