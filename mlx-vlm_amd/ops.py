"""Thin torch-tensor front end of the C ABI (include/vlm_hip.h).

torch is plumbing only here: it owns device memory and the HIP stream; every
computation below is a call into libvlm_hip.so.  Tensors must be CUDA(HIP)
resident, contiguous along the last dim and bf16 unless stated otherwise.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from . import _lib
from ._lib import check

EPI_NONE, EPI_BIAS, EPI_GELU_FAST, EPI_GELU_ERF, EPI_RESIDUAL, EPI_SWIGLU = 0, 1, 2, 4, 8, 16


def _p(t: Optional[torch.Tensor]):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dev(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise _lib.VlmHipError("libvlm_hip ops need device tensors (there is no CPU fallback)")


def gemm(a, w, bias=None, res=None, out=None, epilogue=EPI_NONE):
    """out[M,N(/2)] = epi(a[M,K] @ w[N,K].T)"""
    _dev(a, w, bias, res, out)
    M, K = a.shape
    N = w.shape[0]
    n_out = N // 2 if epilogue & EPI_SWIGLU else N
    if out is None:
        out = torch.empty(M, n_out, dtype=torch.bfloat16, device=a.device)
    check(_lib.lib().vlm_gemm_bf16(_p(a), _p(w), _p(bias), _p(res), _p(out), M, N, K, a.stride(0), w.stride(0),
                                   out.stride(0), res.stride(0) if res is not None else 0, epilogue, _stream()), "gemm")
    return out


def gemm_rope2d(a, w, bias, cos_sin, head_dim, rope_cols, out=None):
    """out = rope2d(a @ w.T + bias) on the first rope_cols columns (q / k heads with interleaved pairs), bias only on the
    rest (vlm_gemm_bf16_rope2d).  cos_sin fp32 [2, M, head_dim / 2]."""
    _dev(a, w, bias, cos_sin, out)
    M, K = a.shape
    N = w.shape[0]
    if out is None:
        out = torch.empty(M, N, dtype=torch.bfloat16, device=a.device)
    check(_lib.lib().vlm_gemm_bf16_rope2d(_p(a), _p(w), _p(bias), _p(cos_sin), _p(out), M, N, K, a.stride(0), w.stride(0),
                                          out.stride(0), int(head_dim), int(rope_cols), _stream()), "gemm_rope2d")
    return out


def gemv(x, w, bias=None, res=None, norm_w=None, out=None, eps=1e-6, epilogue=EPI_NONE):
    _dev(x, w, bias, res, norm_w, out)
    M, K = x.shape
    N = w.shape[0]
    n_out = N // 2 if epilogue & EPI_SWIGLU else N
    if out is None:
        out = torch.empty(M, n_out, dtype=torch.bfloat16, device=x.device)
    check(_lib.lib().vlm_gemv_bf16(_p(x), _p(w), _p(bias), _p(res), _p(norm_w), _p(out), M, N, K, x.stride(0),
                                   w.stride(0), out.stride(0), res.stride(0) if res is not None else 0, eps, epilogue,
                                   _stream()), "gemv")
    return out


_gemv_ws = {}


def gemv_workspace(device):
    """zero-initialised split-K workspace of the batched (5..16 row) decode projections, one per device for callers of the
    operator layer (the engine owns its own)"""
    key = torch.device(device).index or 0
    if key not in _gemv_ws:
        _gemv_ws[key] = torch.zeros(_lib.lib().vlm_gemv_workspace_bytes(), dtype=torch.uint8, device=device)
    return _gemv_ws[key]


EPI_X_TILED, EPI_Y_TILED = 64, 128      # include/vlm_hip.h: activations in the MFMA tile's layout [K / 8][16][8] between two projections


def tile_rows(x):
    """[M <= 16, K] row-major -> the tiled layout [K / 8, 16, 8] (rows M..15 zero): what EPI_X_TILED reads / EPI_Y_TILED writes"""
    M, K = x.shape
    t = torch.zeros(K // 8, 16, 8, dtype=x.dtype, device=x.device)
    t[:, :M] = x.view(M, K // 8, 8).permute(1, 0, 2)
    return t


def untile_rows(t, M):
    """inverse of tile_rows: [K / 8, 16, 8] -> [M, K]"""
    return t[:, :M].permute(1, 0, 2).reshape(M, -1).contiguous()


def gemv_ws(x, w, bias=None, res=None, norm_w=None, out=None, eps=1e-6, epilogue=EPI_NONE, M=None):
    """gemv for a batched decode step (up to 16 rows), K split over workgroups through the workspace where it pays.
    epilogue | EPI_Y_TILED: out is the tiled [N_out / 8, 16, 8] tensor; epilogue | EPI_X_TILED: x is one (pass M = rows)."""
    _dev(x, w, bias, res, norm_w, out)
    N = w.shape[0]
    n_out = N // 2 if epilogue & EPI_SWIGLU else N
    if epilogue & EPI_X_TILED:
        K, ldx = x.shape[0] * 8, 0
        assert M is not None and x.shape[1:] == (16, 8)
    else:
        M, K = x.shape
        ldx = x.stride(0)
    if out is None:
        out = (torch.full((n_out // 8, 16, 8), float("nan"), dtype=torch.bfloat16, device=x.device) if epilogue & EPI_Y_TILED
               else torch.empty(M, n_out, dtype=torch.bfloat16, device=x.device))
    ldy = 0 if epilogue & EPI_Y_TILED else out.stride(0)
    check(_lib.lib().vlm_gemv_bf16_ws(_p(x), _p(w), _p(bias), _p(res), _p(norm_w), _p(out), M, N, K, ldx,
                                      w.stride(0), ldy, res.stride(0) if res is not None else 0, eps, epilogue,
                                      _p(gemv_workspace(x.device)), _stream()), "gemv_ws")
    return out


def gemv_qkv_rope_kvwrite_ws(h, norm_w, wqkv, bqkv, Hq, Hkv, D, pos, slot, inv_freq, block_table, kpool, vpool, eps=1e-6,
                             out=None, max_pages=None):
    _dev(h, norm_w, wqkv, bqkv, pos, slot, inv_freq, block_table, kpool, vpool)
    M, K = h.shape
    if out is None:
        out = torch.zeros(M, (Hq + 2 * Hkv) * D, dtype=torch.bfloat16, device=h.device)
    check(_lib.lib().vlm_gemv_qkv_rope_kvwrite_ws(_p(h), _p(norm_w), eps, _p(wqkv), _p(bqkv), _p(out), out.stride(0), M, K,
                                                  Hq, Hkv, D, _p(pos), _p(slot), _p(inv_freq), _p(block_table),
                                                  block_table.shape[1] if block_table is not None else int(max_pages),
                                                  _p(kpool), _p(vpool), _p(gemv_workspace(h.device)), _stream()),
          "gemv_qkv_rope_kvwrite_ws")
    return out


def gemv_qkv_rope_kvwrite(h, norm_w, wqkv, bqkv, Hq, Hkv, D, pos, slot, inv_freq, block_table, kpool, vpool, eps=1e-6,
                          out=None, max_pages=None):
    """decode-step fusion: RMSNorm + qkv GEMV + bias + M-RoPE + paged KV write.  -> qkv [M, (Hq+2Hkv)*D] (q part valid)
    block_table None: identity layout (row m owns pages [m*max_pages, (m+1)*max_pages) of the pools as passed)."""
    _dev(h, norm_w, wqkv, bqkv, pos, slot, inv_freq, block_table, kpool, vpool)
    M, K = h.shape
    if out is None:
        out = torch.zeros(M, (Hq + 2 * Hkv) * D, dtype=torch.bfloat16, device=h.device)
    check(_lib.lib().vlm_gemv_qkv_rope_kvwrite(_p(h), _p(norm_w), eps, _p(wqkv), _p(bqkv), _p(out), out.stride(0), M, K,
                                               Hq, Hkv, D, _p(pos), _p(slot), _p(inv_freq), _p(block_table),
                                               block_table.shape[1] if block_table is not None else int(max_pages),
                                               _p(kpool), _p(vpool), _stream()), "gemv_qkv_rope_kvwrite")
    return out


def gemv_attn_out_(part_o, part_ml, wo, h, Hq, D):
    """h += merge(partials) @ wo.T   (in place on the residual stream)"""
    _dev(part_o, part_ml, wo, h)
    M, N = h.shape
    check(_lib.lib().vlm_gemv_attn_out(_p(part_o), _p(part_ml), part_o.shape[2], _p(wo), _p(h), h.stride(0), M, N, Hq, D,
                                       _stream()), "gemv_attn_out")
    return h


def layernorm(x, w, b, eps=1e-6, out=None):
    _dev(x, w, b)
    if out is None:
        out = torch.empty_like(x)
    check(_lib.lib().vlm_layernorm(_p(x), _p(w), _p(b), _p(out), x.shape[0], x.shape[1], eps, _stream()), "layernorm")
    return out


def rmsnorm(x, w, eps=1e-6, res=None, out=None, h_out=None):
    _dev(x, w, res)
    if out is None:
        out = torch.empty_like(x)
    check(_lib.lib().vlm_rmsnorm_residual(_p(x), _p(res), _p(w), _p(out), _p(h_out), x.shape[0], x.shape[1], eps,
                                          _stream()), "rmsnorm")
    return out


def rope2d_vision_(qkv, cos_tab, sin_tab, n_heads):
    """in place on qkv [N, 3*H*D]; cos/sin fp32 [N, D/2]"""
    _dev(qkv, cos_tab, sin_tab)
    N = qkv.shape[0]
    D = qkv.shape[1] // (3 * n_heads)
    check(_lib.lib().vlm_rope2d_vision(_p(qkv), _p(cos_tab), _p(sin_tab), N, n_heads, D, qkv.stride(0), _stream()), "rope2d")
    return qkv


def mrope_kvwrite_(qkv, Hq, Hkv, D, pos_t, pos_h, pos_w, inv_freq, sec0, sec1, kv_seq=None, kv_slot=None,
                   block_table=None, kpool=None, vpool=None, qk_scale=None):
    """qk_scale: SuScaledRoPE's typed input scale of q and k (vlm_mrope_kvwrite_scaled); None = plain"""
    _dev(qkv, pos_t, inv_freq)
    T = qkv.shape[0]
    max_pages = block_table.shape[1] if block_table is not None else 0
    if qk_scale is not None and float(qk_scale) != 1.0:
        check(_lib.lib().vlm_mrope_kvwrite_scaled(_p(qkv), qkv.stride(0), T, Hq, Hkv, D, _p(pos_t), _p(pos_h), _p(pos_w),
                                                  _p(inv_freq), sec0, sec1, _p(kv_seq), _p(kv_slot), _p(block_table),
                                                  max_pages, _p(kpool), _p(vpool), float(qk_scale), _stream()),
              "mrope_kvwrite_scaled")
        return qkv
    check(_lib.lib().vlm_mrope_kvwrite(_p(qkv), qkv.stride(0), T, Hq, Hkv, D, _p(pos_t), _p(pos_h), _p(pos_w),
                                       _p(inv_freq), sec0, sec1, _p(kv_seq), _p(kv_slot), _p(block_table), max_pages,
                                       _p(kpool), _p(vpool), _stream()), "mrope_kvwrite")
    return qkv


def kv_gather_(qkv, Hq, Hkv, D, kv_slot, block_table, kpool, vpool, kv_seq=None):
    """cached k / v of (kv_seq[t], kv_slot[t]) -> the k / v columns of row t of qkv [T, (Hq + 2 Hkv) * D] (in place)"""
    _dev(qkv, kv_slot, block_table, kpool, vpool, kv_seq)
    check(_lib.lib().vlm_kv_gather(_p(qkv), qkv.stride(0), qkv.shape[0], Hq, Hkv, D, _p(kv_seq), _p(kv_slot), _p(block_table),
                                   block_table.shape[1], _p(kpool), _p(vpool), _stream()), "kv_gather")
    return qkv


def attn_prefill(q, k, v, cu_seqlens, total_qblocks, Hq, Hkv, D, scale, causal, out=None, uniform_segments=False, q_start=None):
    """q/k/v: 2-D views [T, *] whose data_ptr points at head 0 of token 0 and stride(0) is the token stride.
    uniform_segments: placement hint (all segments the same length); results are identical.
    q_start (int32 [nseg], device): rows of segment s before q_start[s] are keys only (a cached prefix) - their rows of `out`
    are not written; total_qblocks then counts sum ceil((len_s - q_start_s) / 128)."""
    _dev(q, k, v, cu_seqlens, q_start)
    T = q.shape[0]
    if out is None:
        out = torch.empty(T, Hq * D, dtype=torch.bfloat16, device=q.device)
    nseg = cu_seqlens.numel() - 1
    flags = (1 if causal else 0) | (2 if uniform_segments else 0)
    if q_start is not None:
        cu_seqlens = torch.cat([cu_seqlens.reshape(-1).to(torch.int32), q_start.reshape(-1).to(torch.int32)])     # [cu | q_start]
        flags |= 4
    check(_lib.lib().vlm_attn_prefill(_p(q), _p(k), _p(v), _p(out), q.stride(0), k.stride(0), v.stride(0), out.stride(0),
                                      _p(cu_seqlens), nseg, total_qblocks, Hq, Hkv, D, scale, flags, _stream()), "attn_prefill")
    return out


def attn_decode_paged(q, kpool, vpool, block_table, kv_len, kv_len_add, Hq, Hkv, D, scale, nsplit, out=None,
                      merge=True, max_pages=None):
    """merge=True -> bf16 [B, Hq*D]; merge=False -> (part_o, part_ml) for gemv_attn_out_
    block_table None: identity layout (row b owns pages [b*max_pages, (b+1)*max_pages) of the pools as passed)."""
    _dev(q, kpool, vpool, block_table, kv_len)
    B = q.shape[0]
    part_o = torch.empty(B, Hq, nsplit, D, dtype=torch.float32, device=q.device)
    part_ml = torch.empty(B, Hq, nsplit, 2, dtype=torch.float32, device=q.device)
    if merge and out is None:
        out = torch.empty(B, Hq * D, dtype=torch.bfloat16, device=q.device)
    check(_lib.lib().vlm_attn_decode_paged(_p(q), q.stride(0), _p(kpool), _p(vpool), _p(block_table),
                                           block_table.shape[1] if block_table is not None else int(max_pages),
                                           _p(kv_len), kv_len_add, B, Hq, Hkv, D, scale, nsplit,
                                           _p(part_o), _p(part_ml), _p(out) if merge else None,
                                           out.stride(0) if merge else 0, _stream()), "attn_decode")
    return out if merge else (part_o, part_ml)


def gemv_attn_out_bf16_(part_o, part_ml, wo, h, Hq, D):
    """h[0] += merge(page-split partials) @ wo.T in place (one decode row)"""
    _dev(part_o, part_ml, wo, h)
    check(_lib.lib().vlm_gemv_attn_out_bf16(_p(part_o), _p(part_ml), part_o.shape[2], _p(wo), _p(h), h.stride(0), wo.shape[0],
                                            Hq, D, _stream()), "gemv_attn_out_bf16")
    return h


def attn_decode_paged_split(q, kpool, vpool, block_table, kv_len, kv_len_add, Hq, Hkv, D, scale, nsplit, out=None,
                            max_pages=None, tickets=None, merge=True, part=None):
    """page-split decode attention (one wave per page stride).  merge=True: the last arriver merges -> bf16 [B, Hq*D];
    merge=False: the partial-only form -> (part_o fp32 [B, Hq, nsplit, D], part_ml fp32 [B, Hq, nsplit, 2]) for
    gemv_attn_out_bf16_."""
    _dev(q, kpool, vpool, block_table, kv_len)
    B = q.shape[0]
    if not merge:
        if part is not None:
            part_o, part_ml = part
        else:
            part_o = torch.full((B, Hq, nsplit, D), float("nan"), dtype=torch.float32, device=q.device)   # unwritten = NaN on purpose
            part_ml = torch.empty(B, Hq, nsplit, 2, dtype=torch.float32, device=q.device)
        check(_lib.lib().vlm_attn_decode_paged_split(_p(q), q.stride(0), _p(kpool), _p(vpool), _p(block_table),
                                                     block_table.shape[1] if block_table is not None else int(max_pages),
                                                     _p(kv_len), kv_len_add, B, Hq, Hkv, D, scale, nsplit, _p(part_o),
                                                     _p(part_ml), None, None, 0, _stream()), "attn_decode_split")
        return part_o, part_ml
    part_o = torch.empty(B, Hq, nsplit, D, dtype=torch.float32, device=q.device)
    part_ml = torch.empty(B, Hq, nsplit, 2, dtype=torch.float32, device=q.device)
    if tickets is None:
        tickets = torch.zeros(B * Hkv, dtype=torch.int32, device=q.device)
    if out is None:
        out = torch.empty(B, Hq * D, dtype=torch.bfloat16, device=q.device)
    check(_lib.lib().vlm_attn_decode_paged_split(_p(q), q.stride(0), _p(kpool), _p(vpool), _p(block_table),
                                                 block_table.shape[1] if block_table is not None else int(max_pages),
                                                 _p(kv_len), kv_len_add, B, Hq, Hkv, D, scale, nsplit, _p(part_o),
                                                 _p(part_ml), _p(tickets), _p(out), out.stride(0), _stream()),
          "attn_decode_split")
    return out


class EncoderLayers:
    """The weights of a SigLIP / CLIP encoder stack as the native layer loop takes them (vlm_enc_layer array, built once at
    load from a tower's `_w` dict: keys "<i>.ln1w", "<i>.ln1b", "<i>.wqkv", "<i>.bqkv", "<i>.wo", "<i>.bo", "<i>.ln2w",
    "<i>.ln2b", "<i>.w1", "<i>.b1", "<i>.w2", "<i>.b2") + the per-call workspaces, cached by token count."""

    def __init__(self, w: dict, n_layers: int):
        self.n = n_layers
        self._keep = [w[f"{i}.{k}"].contiguous() for i in range(n_layers) for k in ("ln1w", "ln1b", "wqkv", "bqkv", "wo", "bo", "ln2w",
                                                                                    "ln2b", "w1", "b1", "w2", "b2")]
        for t in self._keep:
            if not (t.is_cuda and t.dtype == torch.bfloat16):
                raise ValueError("encoder weights must be bf16 device tensors")
        self.arr = (_lib.EncLayer * n_layers)(*[_lib.EncLayer(*[t.data_ptr() for t in self._keep[12 * i: 12 * i + 12]])
                                                for i in range(n_layers)])
        self._ws = {}

    def forward_(self, x, H, head_dim, ln_eps, act_epilogue, cu_seqlens, total_qblocks, scale, uniform_segments=True):
        """x [N, E] bf16 (device, contiguous) is the residual stream: overwritten with the output of the last layer"""
        _dev(x, cu_seqlens)
        N, E = x.shape
        MH = self._keep[8].shape[0]                 # fc1 rows
        key = (N, x.device, torch.cuda.current_stream().cuda_stream)      # (an admission prefill may run on a side stream)
        ws = self._ws.get(key)
        if ws is None:
            if len(self._ws) > 4:
                self._ws.clear()
            mk = lambda c: torch.empty(N, c, dtype=torch.bfloat16, device=x.device)   # noqa: E731
            ws = self._ws[key] = (mk(E), mk(3 * H * head_dim), mk(H * head_dim), mk(MH))
        check(_lib.lib().vlm_encoder_forward(self.arr, self.n, _p(x), _p(ws[0]), _p(ws[1]), _p(ws[2]), _p(ws[3]), N, E, H, head_dim,
                                             MH, float(ln_eps), int(act_epilogue), _p(cu_seqlens), cu_seqlens.numel() - 1,
                                             int(total_qblocks), float(scale), int(bool(uniform_segments)), _stream()),
              "encoder_forward")
        return x


def gemm_w4(a, wq, sb, bias=None, res=None, epilogue=EPI_NONE, out=None):
    """prefill GEMM over MLX 4-bit weights with the dequantisation fused into the tile staging: wq int32 [N, K/8], sb int32
    [N, K/64] (as gemv_w4)"""
    _dev(a, wq, sb, bias, res, out)
    M, K = a.shape
    N = wq.shape[0]
    n_out = N // 2 if epilogue & EPI_SWIGLU else N
    if out is None:
        out = torch.empty(M, n_out, dtype=torch.bfloat16, device=a.device)
    check(_lib.lib().vlm_gemm_w4(_p(a), _p(wq), _p(sb), _p(bias), _p(res), _p(out), M, N, K, a.stride(0), out.stride(0),
                                 res.stride(0) if res is not None else 0, epilogue, _stream()), "gemm_w4")
    return out


def kv_quantize_tokens(kpool, vpool, kpool8, vpool8, ksb, vsb, kv_seq, kv_slot, block_table, Hkv, D, n_layers=1,
                       layer_stride=0, max_pages=None):
    """KVCache.to_quantized over listed tokens: bf16 pools -> 8-bit pools (u8 + (scale | bias) words), all layers"""
    _dev(kpool, vpool, kpool8, vpool8, ksb, vsb, kv_seq, kv_slot, block_table)
    check(_lib.lib().vlm_kv_quantize_tokens(_p(kpool), _p(vpool), _p(kpool8), _p(vpool8), _p(ksb), _p(vsb), int(layer_stride),
                                            int(n_layers), _p(kv_seq), _p(kv_slot), int(kv_slot.numel()), _p(block_table),
                                            block_table.shape[1] if block_table is not None else int(max_pages), Hkv, D,
                                            _stream()), "kv_quantize_tokens")


def attn_decode_paged_q8(q, kpool16, vpool16, kpool8, vpool8, ksb, vsb, block_table, kv_len, kv_len_add, Hq, Hkv, D, scale, nsplit,
                         quantize_new=True, out=None, max_pages=None, tickets=None, merge=True):
    """page-split decode attention over the 8-bit KV pools (quantized_scaled_dot_product_attention at L == 1); merge as
    attn_decode_paged_split"""
    _dev(q, kpool16, vpool16, kpool8, vpool8, ksb, vsb, block_table, kv_len)
    B = q.shape[0]
    mp = block_table.shape[1] if block_table is not None else int(max_pages)
    if not merge:
        part_o = torch.full((B, Hq, nsplit, D), float("nan"), dtype=torch.bfloat16, device=q.device)
        part_ml = torch.empty(B, Hq, nsplit, 2, dtype=torch.float32, device=q.device)
        check(_lib.lib().vlm_attn_decode_paged_q8(_p(q), q.stride(0), _p(kpool16), _p(vpool16), _p(kpool8), _p(vpool8), _p(ksb),
                                                  _p(vsb), _p(block_table), mp, _p(kv_len), kv_len_add, B, Hq, Hkv, D, scale,
                                                  nsplit, _p(part_o), _p(part_ml), None, None, 0, int(bool(quantize_new)),
                                                  _stream()), "attn_decode_q8")
        return part_o, part_ml
    # (2 * nsplit: from 128 (row, kv head) pairs the launch runs half-page units, i.e. twice the splits)
    part_o = torch.empty(B, Hq, 2 * nsplit, D, dtype=torch.float32, device=q.device)
    part_ml = torch.empty(B, Hq, 2 * nsplit, 2, dtype=torch.float32, device=q.device)
    if tickets is None:
        tickets = torch.zeros(B * Hkv, dtype=torch.int32, device=q.device)
    if out is None:
        out = torch.empty(B, Hq * D, dtype=torch.bfloat16, device=q.device)
    check(_lib.lib().vlm_attn_decode_paged_q8(_p(q), q.stride(0), _p(kpool16), _p(vpool16), _p(kpool8), _p(vpool8), _p(ksb),
                                              _p(vsb), _p(block_table), mp, _p(kv_len), kv_len_add, B, Hq, Hkv, D, scale, nsplit,
                                              _p(part_o), _p(part_ml), _p(tickets), _p(out), out.stride(0),
                                              int(bool(quantize_new)), _stream()), "attn_decode_q8")
    return out


def embed_gather(ids, table, out=None):
    _dev(ids, table)
    T = ids.numel()
    if out is None:
        out = torch.empty(T, table.shape[1], dtype=table.dtype, device=table.device)
    check(_lib.lib().vlm_embed_gather(_p(ids), _p(table), _p(out), T, table.shape[1], out.stride(0), table.shape[0],
                                      _stream()), "embed_gather")
    return out


def scatter_rows_(src, dst_rows, dst):
    _dev(src, dst_rows, dst)
    check(_lib.lib().vlm_scatter_image_rows(_p(src), _p(dst_rows), _p(dst), src.shape[0], src.shape[1], src.stride(0),
                                            dst.stride(0), _stream()), "scatter_rows")
    return dst


def cast_pad(src_f32, ld_dst):
    _dev(src_f32)
    rows, cols = src_f32.shape
    out = torch.empty(rows, ld_dst, dtype=torch.bfloat16, device=src_f32.device)
    check(_lib.lib().vlm_cast_f32_bf16_pad(_p(src_f32), _p(out), rows, cols, src_f32.stride(0), ld_dst, _stream()), "cast_pad")
    return out


def sample_workspace(B, device):
    # zeroed: the first 256 bytes hold the arrival ticket of the fused greedy tail (csrc/sample.hip)
    return torch.zeros(_lib.lib().vlm_sample_workspace_bytes(B), dtype=torch.uint8, device=device)


def bad_argmax_rows(ws) -> int:
    """rows of fused greedy tails run over this workspace whose logits held no finite candidate (all NaN): csrc/sample.hip
    counts them behind the ticket and hands out token 0 instead of turning the sentinel into an address"""
    return int(ws[4:8].view(torch.int32).item())


def sample(logits, temperature=0.0, top_p=1.0, min_p=0.0, top_k=0, seed=0, step=None, want_logprobs=True, ws=None,
           min_tokens_to_keep=1, top_n_sigma=0.0, p_less=False, typical_p=1.0, xtc_probability=0.0, xtc_threshold=0.0,
           xtc_special_tokens=None, return_filtered=False, input_is_logprobs=False):
    """-> (tokens int32 [B], logprobs bf16 [B,V] or None[, filtered logprobs bf16 [B,V] when return_filtered]).
    vlm_sample_ex: the whole make_sampler surface (sample_utils.py:10-89), scalars handed over as python floats (doubles).
    input_is_logprobs (temperature > 0): `logits` already holds log-probs - the contract of the reference's sampler closures -
    and is filtered as it is."""
    _dev(logits)
    B, V = logits.shape
    tok = torch.empty(B, dtype=torch.int32, device=logits.device)
    lp_given = bool(input_is_logprobs) and temperature > 0
    lp = torch.empty(B, V, dtype=torch.bfloat16, device=logits.device) if ((want_logprobs or temperature > 0) and not lp_given) else None
    scratch = torch.empty(B, V, dtype=torch.bfloat16, device=logits.device) if temperature > 0 else None
    if ws is None:
        ws = sample_workspace(B, logits.device)
    sp = _lib.SamplerParams(input_is_logprobs=int(lp_given), temperature=float(temperature), top_p=float(top_p), min_p=float(min_p),
                            min_tokens_to_keep=int(min_tokens_to_keep), top_k=int(top_k), top_n_sigma=float(top_n_sigma),
                            p_less=int(bool(p_less)), typical_p=float(typical_p), xtc_probability=float(xtc_probability),
                            xtc_threshold=float(xtc_threshold), seed=int(seed) & 0xFFFFFFFF)
    keep = []
    if temperature > 0 and xtc_probability > 0 and xtc_special_tokens is not None and len(xtc_special_tokens):
        sp_tok = torch.as_tensor([int(t) for t in xtc_special_tokens], dtype=torch.int32).to(logits.device)
        keep.append(sp_tok)
        sp.xtc_special_tokens, sp.n_xtc_special = _p(sp_tok), sp_tok.numel()
    if temperature > 0 and 0.0 < typical_p < 1.0:
        sort_ws = torch.empty(_lib.lib().vlm_sample_sort_workspace_bytes(B, V), dtype=torch.uint8, device=logits.device)
        keep.append(sort_ws)
        sp.sort_workspace = _p(sort_ws)
    check(_lib.lib().vlm_sample_ex(_p(logits), logits.stride(0), B, V, _p(lp), _p(scratch), V, _p(tok), _p(ws), sp, _p(step),
                                   _stream()), "sample")
    del keep                           # (allocated and freed on the launch's own stream: the caching allocator orders reuse)
    if lp_given:
        lp = logits
    if return_filtered:
        # (no filter on: the kernel draws from the log-probs themselves and leaves the scratch row alone)
        any_filter = temperature > 0 and (0.0 < top_p < 1.0 or min_p != 0.0 or top_k > 0 or top_n_sigma > 0.0 or p_less
                                          or 0.0 < typical_p < 1.0 or xtc_probability > 0.0)
        return tok, lp, (scratch if any_filter else lp)
    return tok, lp


def sample_greedy_advance(logits, tok, ctx, pos, step, embed, h, out_ring=None, want_logprobs=True, ws=None):
    """Greedy tail of a decode step (vlm_sample_greedy_advance): tok <- argmax, ctx += 1, pos += 1, ring, step += 1,
    h <- embed[tok].  -> logprobs bf16 [B, V] or None"""
    _dev(logits, tok, ctx, pos, step, embed, h, out_ring)
    B, V = logits.shape
    lp = torch.empty(B, V, dtype=torch.bfloat16, device=logits.device) if want_logprobs else None
    if ws is None:
        ws = sample_workspace(B, logits.device)
    check(_lib.lib().vlm_sample_greedy_advance(_p(logits), logits.stride(0), B, V, _p(lp), V, _p(tok), _p(ws), _p(ctx), _p(pos),
                                               _p(out_ring), out_ring.shape[0] if out_ring is not None else 0, _p(step),
                                               _p(embed), _p(h), embed.shape[1], h.stride(0), _stream()),
          "sample_greedy_advance")
    return lp


def apply_logit_penalties(logits, pen_args, push_tok=None):
    """In place on logits [B, V] (bf16): logit_bias / repetition / presence / frequency penalties over the device token
    history (vlm_apply_logit_penalties).  pen_args: _lib.PenaltyArgs; push_tok int32 [B] is appended to the history first."""
    _dev(logits, push_tok)
    B, V = logits.shape
    check(_lib.lib().vlm_apply_logit_penalties(_p(logits), logits.stride(0), B, V, _p(push_tok), C.byref(pen_args), _stream()),
          "apply_logit_penalties")
    return logits


def gemv_w4(x, wq, sb, bias=None, res=None, norm_w=None, out=None, eps=1e-6, epilogue=EPI_NONE):
    """decode GEMV over MLX 4-bit weights: wq int32 [N, K/8] (uint32 words), sb int32 [N, K/64] (scale | bias << 16)"""
    _dev(x, wq, sb, bias, res, norm_w, out)
    M, K = x.shape
    N = wq.shape[0]
    n_out = N // 2 if epilogue & EPI_SWIGLU else N
    if out is None:
        out = torch.empty(M, n_out, dtype=torch.bfloat16, device=x.device)
    check(_lib.lib().vlm_gemv_w4(_p(x), _p(wq), _p(sb), _p(bias), _p(res), _p(norm_w), _p(out), M, N, K, x.stride(0),
                                 out.stride(0), res.stride(0) if res is not None else 0, eps, epilogue, _stream()), "gemv_w4")
    return out


def gemv_w4_qkv_rope_kvwrite(h, norm_w, wq, sb, bqkv, Hq, Hkv, D, pos, slot, inv_freq, block_table, kpool, vpool, eps=1e-6,
                             out=None, max_pages=None):
    """gemv_qkv_rope_kvwrite over 4-bit q/k/v rows (wq / sb as gemv_w4)"""
    _dev(h, norm_w, wq, sb, bqkv, pos, slot, inv_freq, block_table, kpool, vpool)
    M, K = h.shape
    if out is None:
        out = torch.zeros(M, (Hq + 2 * Hkv) * D, dtype=torch.bfloat16, device=h.device)
    check(_lib.lib().vlm_gemv_w4_qkv_rope_kvwrite(_p(h), _p(norm_w), eps, _p(wq), _p(sb), _p(bqkv), _p(out), out.stride(0), M,
                                                  K, Hq, Hkv, D, _p(pos), _p(slot), _p(inv_freq), _p(block_table),
                                                  block_table.shape[1] if block_table is not None else int(max_pages),
                                                  _p(kpool), _p(vpool), _stream()), "gemv_w4_qkv_rope_kvwrite")
    return out


def gemv_w4_ws(x, wq, sb, bias=None, res=None, norm_w=None, out=None, eps=1e-6, epilogue=EPI_NONE):
    """gemv_w4 for a batched decode step (up to 16 rows), split-K through the workspace where it pays"""
    _dev(x, wq, sb, bias, res, norm_w, out)
    M, K = x.shape
    N = wq.shape[0]
    n_out = N // 2 if epilogue & EPI_SWIGLU else N
    if out is None:
        out = torch.empty(M, n_out, dtype=torch.bfloat16, device=x.device)
    check(_lib.lib().vlm_gemv_w4_ws(_p(x), _p(wq), _p(sb), _p(bias), _p(res), _p(norm_w), _p(out), M, N, K, x.stride(0),
                                    out.stride(0), res.stride(0) if res is not None else 0, eps, epilogue,
                                    _p(gemv_workspace(x.device)), _stream()), "gemv_w4_ws")
    return out


def gemv_w4_qkv_rope_kvwrite_ws(h, norm_w, wq, sb, bqkv, Hq, Hkv, D, pos, slot, inv_freq, block_table, kpool, vpool, eps=1e-6,
                                out=None, max_pages=None):
    _dev(h, norm_w, wq, sb, bqkv, pos, slot, inv_freq, block_table, kpool, vpool)
    M, K = h.shape
    if out is None:
        out = torch.zeros(M, (Hq + 2 * Hkv) * D, dtype=torch.bfloat16, device=h.device)
    check(_lib.lib().vlm_gemv_w4_qkv_rope_kvwrite_ws(_p(h), _p(norm_w), eps, _p(wq), _p(sb), _p(bqkv), _p(out), out.stride(0), M,
                                                     K, Hq, Hkv, D, _p(pos), _p(slot), _p(inv_freq), _p(block_table),
                                                     block_table.shape[1] if block_table is not None else int(max_pages),
                                                     _p(kpool), _p(vpool), _p(gemv_workspace(h.device)), _stream()),
          "gemv_w4_qkv_rope_kvwrite_ws")
    return out


def dequant_w4(wq, sb, rows=None, out=None):
    """bf16 rows of a 4-bit matrix: all of them (rows None) or a gather (embedding lookup)"""
    _dev(wq, sb, rows, out)
    N, K = wq.shape[0], wq.shape[1] * 8
    n = N if rows is None else rows.numel()
    if out is None:
        out = torch.empty(n, K, dtype=torch.bfloat16, device=wq.device)
    check(_lib.lib().vlm_dequant_w4(_p(wq), _p(sb), _p(rows), _p(out), n, K, out.stride(0), N, _stream()), "dequant_w4")
    return out


def gemm_set_staging(mode: int):
    """0 = automatic (LDS DMA when K % 64 == 0), 1 = always register staging (test / A-B knob)."""
    check(_lib.lib().vlm_gemm_set_staging(int(mode)), "gemm_set_staging")


# ---------------------------------------------------------------------------------------------------------------------
# Operators of decoders with an fp32 residual stream (include/vlm_hip.h, second part).  "T" tensors are bf16 or fp32
# (dtype code 0 / 1 of the C ABI, taken from the tensor); the stream x and every statistic are fp32.
def _f32(t) -> int:
    if t.dtype == torch.float32:
        return 1
    if t.dtype == torch.bfloat16:
        return 0
    raise _lib.VlmHipError(f"bf16 or fp32 tensor expected, got {t.dtype}")


def linear_any(a, w, out=None, out_dtype=None, accumulate=False, batch=1, stride_a=0, stride_w=0, stride_c=0, M=None, N=None, K=None):
    """out[b][m][n] (+)= sum_k a[b][m][k] w[b][n][k] (vlm_linear_any).  Plain call: a [M, K], w [N, K] -> out [M, N] of
    out_dtype (default a's).  Batched call (per-head maps inside wider rows): pass M / N / K, `batch` and the element strides
    between batch members; a / w / out are then 2-D views whose data_ptr is member 0 and whose stride(0) is the row pitch."""
    _dev(a, w, out)
    M = a.shape[0] if M is None else int(M)
    K = a.shape[1] if K is None else int(K)
    N = w.shape[0] if N is None else int(N)
    if out is None:
        out = torch.empty(M, N, dtype=out_dtype or a.dtype, device=a.device)
    check(_lib.lib().vlm_linear_any(_p(a), _p(w), _p(out), M, N, K, a.stride(0), w.stride(0), out.stride(0), _f32(a), _f32(w),
                                    _f32(out), int(batch), int(stride_a), int(stride_w), int(stride_c), int(bool(accumulate)),
                                    _stream()), "linear_any")
    return out


def linear_rows_bf16w(a, w, out=None, out_dtype=None, accumulate=False, skip_gate=None, skip_col0=0, E=0, ff=0):
    """the decode-step form of linear_any (up to 8 rows, bf16 weights, K % 8 == 0): see vlm_linear_rows_bf16w"""
    _dev(a, w, out, skip_gate)
    M, K = a.shape
    N = w.shape[0]
    if out is None:
        out = torch.empty(M, N, dtype=out_dtype or a.dtype, device=a.device)
    check(_lib.lib().vlm_linear_rows_bf16w(_p(a), _p(w), _p(out), M, N, K, a.stride(0), w.stride(0), out.stride(0), _f32(a), _f32(out),
                                           int(bool(accumulate)), _p(skip_gate), int(skip_col0), int(E), int(ff), _stream()),
          "linear_rows_bf16w")
    return out


def embed_scale_f32(ids, table, scale, out=None):
    """x [T, D] fp32 = table[ids] * scale"""
    _dev(ids, table, out)
    T, D = ids.numel(), table.shape[1]
    if out is None:
        out = torch.empty(T, D, dtype=torch.float32, device=table.device)
    check(_lib.lib().vlm_embed_scale_f32(_p(ids), _p(table), float(scale), _p(out), T, D, table.shape[0], _f32(table), _stream()),
          "embed_scale_f32")
    return out


def layernorm_nobias(x, w, eps, out=None):
    """LayerNorm with a weight and no bias over the fp32 stream x [T, D] -> T-typed (w's dtype)"""
    _dev(x, w, out)
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise _lib.VlmHipError("layernorm_nobias: contiguous fp32 stream expected")
    if out is None:
        out = torch.empty(x.shape, dtype=w.dtype, device=x.device)
    check(_lib.lib().vlm_layernorm_nobias(_p(x), _p(w), _p(out), x.shape[0], x.shape[1], out.stride(0), float(eps), _f32(w),
                                          _stream()), "layernorm_nobias")
    return out


def stream_add_(x, a, b=None):
    """x += a (+ b): fp32 stream x [T, D], T-typed a / b (views with a row pitch)"""
    _dev(x, a, b)
    check(_lib.lib().vlm_stream_add(_p(x), _p(a), a.stride(0), _p(b), b.stride(0) if b is not None else 0, x.shape[0], x.shape[1],
                                    _f32(a), _stream()), "stream_add")
    return x


def unit_rms_add_(x, y, w, eps):
    """x += y * rsqrt(mean(y^2) + eps) * w"""
    _dev(x, y, w)
    check(_lib.lib().vlm_unit_rms_add(_p(x), _p(y), y.stride(0), _p(w), x.shape[0], x.shape[1], float(eps), _f32(y), _stream()),
          "unit_rms_add")
    return x


def gelu_tanh_gate_rows(g, table, ids, col0, out=None):
    """out[t, j] = gelu_tanh(g[t, j]) * table[ids[t], col0 + j]"""
    _dev(g, table, ids, out)
    rows, dim = g.shape
    if out is None:
        out = torch.empty(rows, dim, dtype=g.dtype, device=g.device)
    check(_lib.lib().vlm_gelu_tanh_gate_rows(_p(g), g.stride(0), _p(table), table.stride(0), _p(ids), int(col0), _p(out),
                                             out.stride(0), rows, dim, table.shape[0], _f32(g), _stream()), "gelu_tanh_gate_rows")
    return out


def linear_recurrence(args: "_lib.RecurrenceArgs", nseg: int, ntok: int, dtype_f32: bool):
    check(_lib.lib().vlm_linear_recurrence(C.byref(args), int(nseg), int(ntok), int(bool(dtype_f32)), _stream()), "linear_recurrence")


def latent_kv_write(d, w, R, Dr, inv_freq, tok_seq, tok_pos, block_table, pool, eps, rot_half=False):
    """rows of d [T, >= R + Dr] -> (normed latent | rotated key part) at each token's (sequence, position) of the paged pool;
    rot_half: the rotated pairs are (i, i + Dr / 2) instead of (2 i, 2 i + 1)"""
    _dev(d, w, inv_freq, tok_seq, tok_pos, block_table, pool)
    check(_lib.lib().vlm_latent_kv_write(_p(d), d.stride(0), _p(w), int(R), int(Dr), _p(inv_freq), _p(tok_seq), _p(tok_pos),
                                         _p(block_table), block_table.shape[1], _p(pool), float(eps), int(bool(rot_half)), d.shape[0],
                                         _f32(d), _stream()), "latent_kv_write")


def rope_pairs_rows(q, head_stride, H, Dr, inv_freq, tok_pos, out, out_head_stride, rot_half=False):
    """rotation of a Dr-wide part of every head (pairs (2 i, 2 i + 1), or (i, i + Dr / 2) with rot_half): q / out are 2-D views
    at the part's first column"""
    _dev(q, inv_freq, tok_pos, out)
    check(_lib.lib().vlm_rope_pairs_rows(_p(q), q.stride(0), int(head_stride), int(H), int(Dr), _p(inv_freq), _p(tok_pos), _p(out),
                                         out.stride(0), int(out_head_stride), int(bool(rot_half)), q.shape[0], _f32(q), _stream()),
          "rope_pairs_rows")


def latent_attn(q, pool, tok_seq, tok_pos, block_table, H, R, Dr, scale, gate=None, out=None, window=0):
    """q fp32 [T, H, R + Dr] over the latent pool -> fp32 [T, H, R] (times sigmoid(gate[t, h]) when given); window > 0: a query
    reaches back window - 1 tokens"""
    _dev(q, pool, tok_seq, tok_pos, block_table, gate, out)
    T = q.shape[0]
    if out is None:
        out = torch.empty(T, H, R, dtype=torch.float32, device=q.device)
    check(_lib.lib().vlm_latent_attn(_p(q), _p(pool), _p(tok_seq), _p(tok_pos), _p(block_table), block_table.shape[1], int(H), int(R),
                                     int(Dr), float(scale), int(window), _p(gate), gate.stride(0) if gate is not None else 0, _p(out), T,
                                     _f32(pool), _stream()), "latent_attn")
    return out


def latent_attn_blocks(q, pool, qb_start, qb_count, tok_seq, tok_pos, block_table, H, R, Dr, scale, gate=None, out=None, window=0):
    """latent_attn over query blocks (qb_start / qb_count int32 [n]: first token and number of consecutive tokens of one
    sequence, at most 16): the prompt form, key tiles staged once per block"""
    _dev(q, pool, qb_start, qb_count, tok_seq, tok_pos, block_table, gate, out)
    T = q.shape[0]
    if out is None:
        out = torch.empty(T, H, R, dtype=torch.float32, device=q.device)
    check(_lib.lib().vlm_latent_attn_blocks(_p(q), _p(pool), _p(qb_start), _p(qb_count), qb_start.numel(), _p(tok_seq), _p(tok_pos),
                                            _p(block_table), block_table.shape[1], int(H), int(R), int(Dr), float(scale), int(window),
                                            _p(gate), gate.stride(0) if gate is not None else 0, _p(out), _f32(pool), _stream()),
          "latent_attn_blocks")
    return out


def moe_route(logits, top):
    """fp32 logits [T, E] -> (dense gate table fp32 [T, E], chosen indices int32 [T, top], their weights fp32 [T, top])"""
    _dev(logits)
    T, E = logits.shape
    gate = torch.empty(T, E, dtype=torch.float32, device=logits.device)
    idx = torch.empty(T, top, dtype=torch.int32, device=logits.device)
    wgt = torch.empty(T, top, dtype=torch.float32, device=logits.device)
    check(_lib.lib().vlm_moe_route(_p(logits), T, E, int(top), _p(gate), _p(idx), _p(wgt), _stream()), "moe_route")
    return gate, idx, wgt


def moe_route_scored(logits, top, groups=1, keep=1, scale=1.0):
    """moe_route with the weights of the softmax over ALL experts times `scale` (no second normalisation), the choice made among
    the experts of the `keep` top-ranked of `groups` equally sized blocks of consecutive experts (a block ranks by its best expert)"""
    _dev(logits)
    T, E = logits.shape
    gate = torch.empty(T, E, dtype=torch.float32, device=logits.device)
    idx = torch.empty(T, top, dtype=torch.int32, device=logits.device)
    wgt = torch.empty(T, top, dtype=torch.float32, device=logits.device)
    check(_lib.lib().vlm_moe_route_scored(_p(logits), T, E, int(top), int(groups), int(keep), float(scale), _p(gate), _p(idx), _p(wgt),
                                          _stream()), "moe_route_scored")
    return gate, idx, wgt


GLU_GELU_TANH, GLU_SILU, GLU_SIGMOID = 0, 1, 2


def glu_rows(g, u, act, out=None, route=None, E=0, ff=0, estride=0):
    """out = act(g) * u over 2-D views with a row pitch (dim: out's columns, else g's); with route (fp32 [T, E]): out [T, E * ff], expert e reads the
    columns e * estride .. + ff of g and u, times route[t, e]"""
    _dev(g, u, out, route)
    rows = g.shape[0]
    dim = int(E) * int(ff) if route is not None else (out.shape[1] if out is not None else g.shape[1])
    if out is None:
        out = torch.empty(rows, dim, dtype=g.dtype, device=g.device)
    check(_lib.lib().vlm_glu_rows(_p(g), g.stride(0), _p(u), u.stride(0), _p(route), int(E), int(ff), int(estride or ff), int(act),
                                  _p(out), out.stride(0), rows, dim, _f32(g), _stream()), "glu_rows")
    return out


def scaled_add_rms_(x, y=None, mult=1.0, w=None, w_offset=0.0, eps=1e-6, h=None, y2=None, mult2=1.0, h_dtype=None):
    """x += mult * y (+ mult2 * y2) on the fp32 stream (y None: no add); then, with w: h = rms(x) * (w_offset + w) -> h (None
    without w), in w's dtype, or in fp32 with h_dtype=torch.float32 (a reader that goes on in fp32).  One pass: the residual step
    of a sublayer and the norm of the next reader."""
    _dev(x, y, y2, w, h)
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise _lib.VlmHipError("scaled_add_rms: contiguous fp32 stream expected")
    if w is not None and h is None:
        h = torch.empty(x.shape, dtype=h_dtype or w.dtype, device=x.device)
    t = y if y is not None else w
    if y2 is not None and (y is None or y2.dtype != y.dtype):
        raise _lib.VlmHipError("scaled_add_rms: the second addend comes with a first one of the same dtype")
    check(_lib.lib().vlm_scaled_add_rms(_p(x), _p(y), y.stride(0) if y is not None else 0, float(mult), _p(y2),
                                        y2.stride(0) if y2 is not None else 0, float(mult2), _p(w), float(w_offset), _p(h),
                                        h.stride(0) if h is not None else 0, int(h is not None and h.dtype == torch.float32), x.shape[0],
                                        x.shape[1], float(eps), _f32(t), _stream()), "scaled_add_rms")
    return h


def moe_route_sigmoid(logits, E, top, groups=1, keep=1, group_top=2, correction=None, normalise=True, scale=1.0, extra=0):
    """fp32 logits [T, >= E + extra] -> (gate table fp32 [T, E], chosen int32 [T, top], weights fp32 [T, top], sigmoid of the extra
    columns fp32 [T, extra] or None).  Scores sigmoid(z); the choice on scores + correction inside the `keep` best of `groups`
    blocks of neighbouring experts (a block ranks by the sum of its group_top best choice scores); weights from the scores alone."""
    _dev(logits, correction)
    if logits.dtype != torch.float32 or (correction is not None and correction.dtype != torch.float32):
        raise _lib.VlmHipError("moe_route_sigmoid: fp32 logits and correction expected")
    T = logits.shape[0]
    gate = torch.empty(T, E, dtype=torch.float32, device=logits.device)
    idx = torch.empty(T, top, dtype=torch.int32, device=logits.device)
    wgt = torch.empty(T, top, dtype=torch.float32, device=logits.device)
    ex = torch.empty(T, extra, dtype=torch.float32, device=logits.device) if extra else None
    check(_lib.lib().vlm_moe_route_sigmoid(_p(logits), logits.stride(0), T, int(E), int(top), int(groups), int(keep), int(group_top),
                                           _p(correction), int(bool(normalise)), float(scale), int(extra), _p(ex), _p(gate), _p(idx), _p(wgt),
                                           _stream()), "moe_route_sigmoid")
    return gate, idx, wgt, ex


def moe_relu2_gate(up, gate, E, ff, shared, out):
    """out[t, c] = relu(up[t, c])^2 * gate[t, c // ff] over the E * ff expert columns, relu^2 alone over the `shared` ones"""
    _dev(up, gate, out)
    check(_lib.lib().vlm_moe_relu2_gate(_p(up), up.stride(0), _p(gate), int(E), int(ff), int(shared), _p(out), out.stride(0),
                                        up.shape[0], _f32(up), _stream()), "moe_relu2_gate")
    return out


# ---------------------------------------------------------------------------------------------------------------------
# Sublayers that read the fp32 stream un-normed and norm / gate their result; delta-rule recurrences; windowed attention.
def stream_cast(x, dtype, out=None):
    """fp32 stream x [T, D] -> the serving dtype (one rounding)"""
    _dev(x, out)
    if out is None:
        out = torch.empty(x.shape, dtype=dtype, device=x.device)
    check(_lib.lib().vlm_stream_cast(_p(x), _p(out), x.shape[0], x.shape[1], _f32(out), _stream()), "stream_cast")
    return out


def rms_rows(x, w, eps, out=None):
    """RMS norm (weight, no mean) over the fp32 stream x [T, D] -> w's dtype"""
    _dev(x, w, out)
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise _lib.VlmHipError("rms_rows: contiguous fp32 stream expected")
    if out is None:
        out = torch.empty(x.shape, dtype=w.dtype, device=x.device)
    check(_lib.lib().vlm_rms_rows(_p(x), _p(w), _p(out), x.shape[0], x.shape[1], out.stride(0), float(eps), _f32(w), _stream()),
          "rms_rows")
    return out


def gated_rms_add_(x, a, w, eps, gate=None, gate_bias=None, b=None, wa=None, wb=None, h=None):
    """x += rms(y * sigmoid(gate + gate_bias)) * w with y = a, or (rms(a) wa + rms(b) wb) / 2 for two branches; h (same shape
    as x, serving dtype) receives the rounded updated stream"""
    _dev(x, a, w, gate, gate_bias, b, wa, wb, h)
    if x.dtype != torch.float32 or not x.is_contiguous() or (h is not None and not h.is_contiguous()):
        raise _lib.VlmHipError("gated_rms_add: contiguous fp32 stream expected")
    check(_lib.lib().vlm_gated_rms_add(_p(x), _p(a), a.stride(0), _p(wa), _p(b), b.stride(0) if b is not None else 0, _p(wb), _p(gate),
                                       gate.stride(0) if gate is not None else 0, _p(gate_bias), _p(w), _p(h), x.shape[0], x.shape[1],
                                       float(eps), _f32(a), _stream()), "gated_rms_add")
    return x


def relu2_rows(up, out=None):
    """out = max(up, 0)^2 (2-D views with a row pitch)"""
    _dev(up, out)
    if out is None:
        out = torch.empty(up.shape, dtype=up.dtype, device=up.device)
    check(_lib.lib().vlm_relu2_rows(_p(up), up.stride(0), _p(out), out.stride(0), up.shape[0], up.shape[1], _f32(up), _stream()),
          "relu2_rows")
    return out


def delta_prep_general(args: "_lib.DeltaPrepGeneralArgs", ntok: int, dtype_f32: bool):
    check(_lib.lib().vlm_delta_prep_general(C.byref(args), int(ntok), int(bool(dtype_f32)), _stream()), "delta_prep_general")


def delta_prep_gated(args: "_lib.DeltaPrepGatedArgs", nseg: int, ntok: int, dtype_f32: bool):
    check(_lib.lib().vlm_delta_prep_gated(C.byref(args), int(nseg), int(ntok), int(bool(dtype_f32)), _stream()), "delta_prep_gated")


def delta_rule(args: "_lib.DeltaRuleArgs", nseg: int, ntok: int, dtype_f32: bool):
    check(_lib.lib().vlm_delta_rule(C.byref(args), int(nseg), int(ntok), int(bool(dtype_f32)), _stream()), "delta_rule")


def headnorm_rope_rows(x, heads, D, w, eps, rot_dims, inv_freq, tok_pos, out, tok_seq=None, block_table=None, raw_pool=None):
    """x: 2-D view at the first head's column (row pitch = stride(0)).  Per head: RMS norm with w [D] (None: no norm), pair
    rotation of the first rot_dims dimensions -> fp32 `out`: dense [T, heads * D], or (with block_table) the paged pool
    [pages, 64, heads * D]; raw_pool: the un-normed rows in x's dtype, same paging"""
    _dev(x, w, inv_freq, tok_pos, out, tok_seq, block_table, raw_pool)
    if out.dtype != torch.float32:
        raise _lib.VlmHipError("headnorm_rope_rows: fp32 output expected")
    check(_lib.lib().vlm_headnorm_rope_rows(_p(x), x.stride(0), int(heads), int(D), _p(w), float(eps), int(rot_dims), _p(inv_freq),
                                            _p(tok_pos), _p(tok_seq), _p(block_table),
                                            block_table.shape[1] if block_table is not None else 0, _p(out), _p(raw_pool), x.shape[0],
                                            _f32(x), _stream()), "headnorm_rope_rows")
    return out


def headnorm_rows(x, heads, D, tok_pos, out, eps=0.0, norm=True, w=None, bias=None, rot_dims=0, inv_freq=None, temp=None, tok_seq=None,
                  block_table=None, raw=None, raw_dim=0, raw_bias=None, raw_pool=None, rot_half=False):
    """headnorm_rope_rows with a bias added first, a norm without a weight (norm=True, w=None), a position multiplier
    temp = (coef, every): 1 + coef * ln(floor((pos + 1) / every) + 1), and value rows `raw` (2-D view [T, heads * raw_dim],
    + raw_bias) copied into `raw_pool` in the same launch; rot_half: the rotated pairs are (i, i + rot_dims / 2) and the rotation comes
    before the norm"""
    _dev(x, w, bias, inv_freq, tok_pos, out, tok_seq, block_table, raw, raw_bias, raw_pool)
    if out.dtype != torch.float32:
        raise _lib.VlmHipError("headnorm_rows: fp32 output expected")
    a = _lib.HeadnormArgs()
    a.x, a.ldx, a.heads, a.D, a.bias, a.w, a.norm, a.eps = _p(x), x.stride(0), int(heads), int(D), _p(bias), _p(w), int(bool(norm)), float(eps)
    a.rot_dims, a.inv_freq, a.rot_half = int(rot_dims), _p(inv_freq), int(bool(rot_half))
    if temp is not None:
        a.temp_coef, a.temp_every = float(temp[0]), int(temp[1])
    a.tok_pos, a.tok_seq, a.block_table = _p(tok_pos), _p(tok_seq), _p(block_table)
    a.max_pages = block_table.shape[1] if block_table is not None else 0
    a.out = _p(out)
    if raw_pool is not None:
        if raw.dtype != x.dtype or raw_pool.dtype != x.dtype:
            raise _lib.VlmHipError("headnorm_rows: value rows and their pool have the dtype of x")
        a.raw, a.ldraw, a.Draw, a.raw_bias, a.raw_pool = _p(raw), raw.stride(0), int(raw_dim), _p(raw_bias), _p(raw_pool)
    check(_lib.lib().vlm_headnorm_rows(C.byref(a), x.shape[0], _f32(x), _stream()), "headnorm_rows")
    return out


def window_attn_blocks(q, kpool, vpool, qb_start, qb_count, tok_seq, tok_pos, block_table, H, KH, D, Dv, scale, out, temp=None, window=0,
                       gate=None, cap=0.0, gate_head=False, sink=False):
    """prompt form of the windowed attention: q fp32 [T, H * D]; out / gate: 2-D views [T, H * Dv] in vpool's dtype (gate_head:
    gate [T, H], one number per head); cap > 0: scores pass cap * tanh(. / cap); sink: one more term exp(0) in the softmax's denominator"""
    _dev(q, kpool, vpool, qb_start, qb_count, tok_seq, tok_pos, block_table, out, temp, gate)
    check(_lib.lib().vlm_window_attn_blocks(_p(q), _p(kpool), _p(vpool), _p(qb_start), _p(qb_count), qb_start.numel(), _p(tok_seq),
                                            _p(tok_pos), _p(block_table), block_table.shape[1], int(H), int(KH), int(D), int(Dv),
                                            float(scale), _p(temp), int(window), float(cap), int(bool(sink)), _p(gate),
                                            gate.stride(0) if gate is not None else 0, int(bool(gate_head)), _p(out), out.stride(0),
                                            _f32(vpool), _stream()), "window_attn_blocks")
    return out


def window_attn_rows(q, kpool, vpool, tok_seq, tok_pos, block_table, H, KH, D, Dv, scale, out, temp=None, window=0, gate=None, cap=0.0,
                     gate_head=False, sink=False):
    """decode form of the windowed attention (one workgroup per token and head)"""
    _dev(q, kpool, vpool, tok_seq, tok_pos, block_table, out, temp, gate)
    check(_lib.lib().vlm_window_attn_rows(_p(q), _p(kpool), _p(vpool), _p(tok_seq), _p(tok_pos), _p(block_table), block_table.shape[1],
                                          int(H), int(KH), int(D), int(Dv), float(scale), _p(temp), int(window), float(cap), int(bool(sink)),
                                          _p(gate), gate.stride(0) if gate is not None else 0, int(bool(gate_head)), _p(out), out.stride(0),
                                          q.shape[0], _f32(vpool), _stream()), "window_attn_rows")
    return out


# ---------------------------------------------------------------------------------------------------------------------
# Short convolutions with carried inputs and the selective state-space scan.
def short_conv_rows(x, w, carry, tok_seq, tok_pos, cu, slot, pos0, bias=None, act=False, residual=False, out=None, out_dtype=None):
    """Causal convolution over time on every channel of the rows x [T, >= C] (fp32 or w's dtype; a 2-D view with a row pitch):
    out = (x if residual) + bias + sum_j w[:, j] * x(t - taps + 1 + j), silu when act.  carry fp32 [slots, taps - 1, C] holds each
    sequence's last inputs; it is read for the tokens before the step's first one and then moved to the end of the segments
    (cu / slot / pos0: the step's segment tables)."""
    _dev(x, w, carry, tok_seq, tok_pos, cu, slot, pos0, bias, out)
    C_, taps = w.shape
    if out is None:
        out = torch.empty(x.shape[0], C_, dtype=out_dtype or w.dtype, device=x.device)
    if taps > 1 and (carry is None or carry.dtype != torch.float32 or tuple(carry.shape[1:]) != (taps - 1, C_)):
        raise _lib.VlmHipError("short_conv_rows: fp32 carry [slots, taps - 1, channels] expected")
    a = _lib.ShortConvArgs()
    a.in_, a.ldin, a.in_f32 = _p(x), x.stride(0), int(x.dtype == torch.float32)
    a.w, a.bias, a.C, a.taps, a.act, a.residual = _p(w), _p(bias), int(C_), int(taps), int(bool(act)), int(bool(residual))
    a.carry, a.tok_seq, a.tok_pos = _p(carry), _p(tok_seq), _p(tok_pos)
    a.seg_start, a.seg_slot, a.seg_pos0 = _p(cu), _p(slot), _p(pos0)
    a.out, a.ldo, a.out_f32 = _p(out), out.stride(0), int(out.dtype == torch.float32)
    f32 = _f32(w)
    if f32 and not (a.in_f32 and a.out_f32):
        raise _lib.VlmHipError("short_conv_rows: fp32 weights come with fp32 rows")
    check(_lib.lib().vlm_short_conv_rows(C.byref(a), x.shape[0], f32, _stream()), "short_conv_rows")
    check(_lib.lib().vlm_short_conv_carry(C.byref(a), slot.numel(), f32, _stream()), "short_conv_carry")
    return out


def selective_scan(args: "_lib.SelectiveScanArgs", nseg: int, ntok: int, dtype_f32: bool):
    check(_lib.lib().vlm_selective_scan(C.byref(args), int(nseg), int(ntok), int(bool(dtype_f32)), _stream()), "selective_scan")
