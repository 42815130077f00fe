// Matrix-state linear recurrences (linear attention without softmax), carried per sequence in fp32:
//
//     S_t = a_t * S_(t-1) + b_t * k_t v_t^T            o_t = S_t^T q_t                      S: [D, Dv] per head
//
//   * fixed decay ("retention"): a_t = decay[h], b_t = 1, rotary positions on q and k (rotate-half pairing on the first
//     rot_dims dimensions), k scaled after the rotation;
//   * gated ("mLSTM"): log input gate i_t = cap * tanh((i~ + bias) / cap), log forget gate f_t = logsigmoid(cap * tanh((f~ +
//     bias) / cap)), running maximum m_t = max(f_t + m_(t-1), i_t) with m_0 = 0, a_t = exp(f_t + m_(t-1) - m_t),
//     b_t = exp(i_t - m_t); the normaliser n_t = a_t n_(t-1) + b_t k_t rides along as one more COLUMN of S (v extended by a
//     constant 1), so n_t . q_t is one more output; o_t is divided by max(|n_t . q_t|, exp(-m_t)) + 1e-6;
//   * gate per state row ("HGRN2"): S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T with f_t = lower + (1 - lower) * sigmoid(f~_t + bias)
//     per head and row - the forget gate is bounded from below and also decides what is written (no separate key); q may pass
//     silu first.  The gate's pre-activation rows come in through `k`; gate and 1 - gate are evaluated in fp32 on the way into LDS.
//
// One kernel serves a whole prompt, a portion of one and a single decoded token: a segment is `len` consecutive tokens of one
// sequence; its state is read from the sequence's slot (zero when the segment starts at position 0 - a slot that is used
// again needs no clearing), advanced token by token with the same arithmetic wherever the prompt was cut, and written back.
// vlm_linear_recurrence writes the raw o (and n . q) in fp32; vlm_recurrence_finish then applies the denominator, the
// per-head unit-RMS norm, an optional weight and the output gate (silu or sigmoid of a projection) into a T-typed row.
//
// Work split: workgroup = (segment, head, tile of 64 state columns); lane c of part p holds rows [32 p, 32 p + 32) of column
// c in registers.  Tokens are staged 4 / 8 / 16 at a time through LDS (q, k rotated and scaled on the way in).
#include "common.hpp"
#include "../../include/vlm_hip.h"
#include "recurrence_finish.hpp"

namespace {

constexpr int DR = 32;       // state rows per lane
constexpr int CT = 64;       // state columns per workgroup

__device__ __forceinline__ float logsigmoid_f(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

template <typename T, int MODE>
__global__ __launch_bounds__(1024) void linear_recurrence_kernel(vlm_recurrence_args p, int P, int TB) {
  constexpr bool GATED = MODE == 1, ROWGATE = MODE == 2;
  extern __shared__ __align__(16) float smem[];
  const int seg = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * CT;
  const int D = p.D, Dv = p.Dv, C = Dv + (GATED ? 1 : 0), DP = P * DR;
  const int tid = threadIdx.x, nthr = blockDim.x;
  const int part = tid / CT, col = c0 + (tid % CT), row0 = part * DR;
  float* qs = smem;                       // [TB][DP]
  float* ks = qs + TB * DP;               // [TB][DP]
  float* vs = ks + TB * DP;               // [TB][CT]
  float* ab = vs + TB * CT;               // [TB][4]: a, b, (gated) i, f / scratch
  float* po = ab + TB * 4;                // [TB][P][CT]
  float* fs = po + TB * P * CT;           // [TB][DP] (ROWGATE): the forget gate per state row; ks holds 1 - f
  const int t_begin = p.seg_start[seg], t_end = p.seg_start[seg + 1];
  const int slot = p.seg_slot[seg], pos0 = p.seg_pos0[seg];
  const T* q = (const T*)p.q + (long)h * D;
  const T* k = (const T*)p.k + (long)h * D;
  const T* v = (const T*)p.v + (long)h * Dv;
  float* S = p.state + ((long)slot * p.H + h) * (long)D * C;
  float s[DR];
#pragma unroll
  for (int r = 0; r < DR; ++r) {
    const int row = row0 + r;
    s[r] = (pos0 > 0 && row < D && col < C) ? S[(long)row * C + col] : 0.f;
  }
  // (GATED: meaningful in lane 0; the maximum the segment starts from was saved by gate_max_kernel, which has already
  //  moved the slot's own value to the end of the segment - every column tile must see the OLD one)
  float m_run = GATED ? p.mprev[(long)seg * p.H + h] : 0.f;
  const int half = p.rot_dims / 2;
  const float dec = MODE == 0 ? p.decay[h] : 0.f;

  for (int t0 = t_begin; t0 < t_end; t0 += TB) {
    const int nb = min(TB, t_end - t0);
    for (int idx = tid; idx < nb * DP; idx += nthr) {
      const int t = idx / DP, i = idx % DP;
      float qv = 0.f, kv = 0.f;
      if (i < D) {
        const long tok = t0 + t;
        qv = ld_f(q + tok * p.ldq + i);
        kv = ld_f(k + tok * p.ldk + i);
        if (i < p.rot_dims) {
          const int j = i < half ? i + half : i - half;
          const float ang = (float)(pos0 + (t0 - t_begin) + t) * p.inv_freq[i < half ? i : i - half];
          float sn, cs;
          sincosf(ang, &sn, &cs);
          const float qo = ld_f(q + tok * p.ldq + j), ko = ld_f(k + tok * p.ldk + j);
          // (u, v) -> (u cos - v sin, v cos + u sin): the first half holds u, the second v
          qv = i < half ? qv * cs - qo * sn : qv * cs + qo * sn;
          kv = i < half ? kv * cs - ko * sn : kv * cs + ko * sn;
        }
        if (ROWGATE) {
          if (p.q_act == 1) qv = qv / (1.f + expf(-qv));
          const float lo = p.lower ? ld_f((const T*)p.lower + (long)h * D + i) : 0.f;
          const float f = lo + (1.f - lo) / (1.f + expf(-(kv + (p.fbias ? ld_f((const T*)p.fbias + (long)h * D + i) : 0.f))));
          fs[idx] = f;
          kv = 1.f - f;
        } else {
          qv *= p.qscale;
          kv *= p.kscale;
        }
      } else if (ROWGATE) {
        fs[idx] = 0.f;
      }
      qs[idx] = qv;
      ks[idx] = kv;
    }
    for (int idx = tid; idx < nb * CT; idx += nthr) {
      const int t = idx / CT, c = c0 + idx % CT;
      vs[idx] = c < Dv ? ld_f(v + (long)(t0 + t) * p.ldv + c) : (c == Dv && GATED ? 1.f : 0.f);
    }
    if (GATED) {
      if (tid < nb) {
        const long tok = t0 + tid;
        const float iv = ld_f((const T*)p.ipre + tok * p.ldi + h) + ld_f((const T*)p.ib + h);
        const float fv = ld_f((const T*)p.fpre + tok * p.ldf + h) + ld_f((const T*)p.fb + h);
        ab[tid * 4 + 2] = p.cap * tanhf(iv / p.cap);
        ab[tid * 4 + 3] = logsigmoid_f(p.cap * tanhf(fv / p.cap));
      }
      __syncthreads();
      if (tid == 0) {                     // the scalar scan: adds and maxima only; the exponentials follow in parallel
        for (int t = 0; t < nb; ++t) {
          const float ig = ab[t * 4 + 2], fg = ab[t * 4 + 3];
          const float m_new = fmaxf(fg + m_run, ig);
          ab[t * 4 + 0] = fg + m_run - m_new;
          ab[t * 4 + 1] = ig - m_new;
          m_run = m_new;
        }
      }
      __syncthreads();
      if (tid < nb) {
        ab[tid * 4 + 0] = expf(ab[tid * 4 + 0]);
        ab[tid * 4 + 1] = expf(ab[tid * 4 + 1]);
      }
    }
    __syncthreads();
    for (int t = 0; t < nb; ++t) {
      const float a = GATED ? ab[t * 4 + 0] : dec, b = GATED ? ab[t * 4 + 1] : 1.f;
      const float bv = b * vs[t * CT + (tid % CT)];
      // (k and q of the token are the same for every lane of the wave: 16-byte broadcast reads, rows ascending)
      const float4* kr = reinterpret_cast<const float4*>(ks + t * DP + row0);
      const float4* qr = reinterpret_cast<const float4*>(qs + t * DP + row0);
      float acc = 0.f;
      if (ROWGATE) {
        const float4* fr = reinterpret_cast<const float4*>(fs + t * DP + row0);
#pragma unroll
        for (int r = 0; r < DR / 4; ++r) {
          const float4 kk = kr[r], qq = qr[r], ff = fr[r];
          s[4 * r + 0] = fmaf(ff.x, s[4 * r + 0], kk.x * bv);
          acc = fmaf(s[4 * r + 0], qq.x, acc);
          s[4 * r + 1] = fmaf(ff.y, s[4 * r + 1], kk.y * bv);
          acc = fmaf(s[4 * r + 1], qq.y, acc);
          s[4 * r + 2] = fmaf(ff.z, s[4 * r + 2], kk.z * bv);
          acc = fmaf(s[4 * r + 2], qq.z, acc);
          s[4 * r + 3] = fmaf(ff.w, s[4 * r + 3], kk.w * bv);
          acc = fmaf(s[4 * r + 3], qq.w, acc);
        }
      } else
#pragma unroll
      for (int r = 0; r < DR / 4; ++r) {
        const float4 kk = kr[r], qq = qr[r];
        s[4 * r + 0] = fmaf(a, s[4 * r + 0], kk.x * bv);
        acc = fmaf(s[4 * r + 0], qq.x, acc);
        s[4 * r + 1] = fmaf(a, s[4 * r + 1], kk.y * bv);
        acc = fmaf(s[4 * r + 1], qq.y, acc);
        s[4 * r + 2] = fmaf(a, s[4 * r + 2], kk.z * bv);
        acc = fmaf(s[4 * r + 2], qq.z, acc);
        s[4 * r + 3] = fmaf(a, s[4 * r + 3], kk.w * bv);
        acc = fmaf(s[4 * r + 3], qq.w, acc);
      }
      po[(t * P + part) * CT + (tid % CT)] = acc;
    }
    __syncthreads();
    for (int idx = tid; idx < nb * CT; idx += nthr) {
      const int t = idx / CT, cc = idx % CT;
      if (c0 + cc < C) {
        float o = 0.f;
        for (int pp = 0; pp < P; ++pp) o += po[(t * P + pp) * CT + cc];
        p.raw[((long)(t0 + t) * p.H + h) * C + c0 + cc] = o;
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int r = 0; r < DR; ++r) {
    const int row = row0 + r;
    if (row < D && col < C) S[(long)row * C + col] = s[r];
  }
}

// the running maximum m_t per (token, head) for the finish pass, and the slot's maximum moved to the end of the segment: one
// wave per (segment, head).  64 tokens at a time: every lane evaluates the gates of its token (the transcendental part, in
// parallel), then the scan itself - a maximum and an add per token - walks the 64 lanes in order, the same sequence of
// operations as a token-by-token loop.
template <typename T>
__global__ __launch_bounds__(64) void gate_max_kernel(vlm_recurrence_args p, int nseg) {
  const int i = blockIdx.x, lane = threadIdx.x;
  const int seg = i / p.H, h = i % p.H;
  float* ms = p.mstate + (long)p.seg_slot[seg] * p.H + h;
  float m = p.seg_pos0[seg] > 0 ? *ms : 0.f;
  if (lane == 0) p.mprev[i] = m;
  const int t_end = p.seg_start[seg + 1];
  for (int t0 = p.seg_start[seg]; t0 < t_end; t0 += 64) {
    const int tok = t0 + lane;
    float ig = 0.f, fg = 0.f;
    if (tok < t_end) {
      const float iv = ld_f((const T*)p.ipre + (long)tok * p.ldi + h) + ld_f((const T*)p.ib + h);
      const float fv = ld_f((const T*)p.fpre + (long)tok * p.ldf + h) + ld_f((const T*)p.fb + h);
      ig = p.cap * tanhf(iv / p.cap);
      fg = logsigmoid_f(p.cap * tanhf(fv / p.cap));
    }
    const int nb = min(64, t_end - t0);
    float mine = 0.f;
    for (int t = 0; t < nb; ++t) {          // (t is wave-uniform: a broadcast read of lane t)
      const float it = __shfl(ig, t), ft = __shfl(fg, t);
      m = fmaxf(ft + m, it);
      if (lane == t) mine = m;
    }
    if (tok < t_end) p.mtok[(long)tok * p.H + h] = mine;
  }
  if (lane == 0) *ms = m;
}

template <typename T>
int run(const vlm_recurrence_args& a, int nseg, int ntok, hipStream_t st) {
  const int gated = a.gated == 1, rowgate = a.gated == 2;
  const int C = a.Dv + (gated ? 1 : 0);
  const int P = (a.D + DR - 1) / DR;
  if (P * CT > 1024) return VLM_ERR_SHAPE;
  int TB = 16;
  auto lds = [&](int tb) { return (size_t)tb * ((rowgate ? 3 : 2) * P * DR + CT + 4 + P * CT) * sizeof(float); };
  while (TB > 4 && lds(TB) > 48 * 1024) TB >>= 1;
  if (lds(TB) > 64 * 1024) return VLM_ERR_SHAPE;
  dim3 grid(nseg, a.H, (C + CT - 1) / CT), block(P * CT);
  if (gated) {
    // the per-token maxima first: the scan kernel overwrites the slot's running maximum
    hipLaunchKernelGGL(gate_max_kernel<T>, dim3(nseg * a.H), dim3(64), 0, st, a, nseg);
    VLM_CHECK_LAUNCH();
    hipLaunchKernelGGL((linear_recurrence_kernel<T, 1>), grid, block, lds(TB), st, a, P, TB);
  } else if (rowgate) {
    hipLaunchKernelGGL((linear_recurrence_kernel<T, 2>), grid, block, lds(TB), st, a, P, TB);
  } else {
    hipLaunchKernelGGL((linear_recurrence_kernel<T, 0>), grid, block, lds(TB), st, a, P, TB);
  }
  VLM_CHECK_LAUNCH();
  if (gated)
    hipLaunchKernelGGL((recurrence_finish_kernel<T, true>), dim3(ntok, a.H), dim3(64), 0, st, a.raw, a.H, a.Dv, a.mtok, a.eps,
                       (const T*)a.g, a.ldg, (const T*)a.normw, a.gate_act, (T*)a.out, a.ldo);
  else
    hipLaunchKernelGGL((recurrence_finish_kernel<T, false>), dim3(ntok, a.H), dim3(64), 0, st, a.raw, a.H, a.Dv, (const float*)nullptr,
                       a.eps, (const T*)a.g, a.ldg, (const T*)a.normw, a.gate_act, (T*)a.out, a.ldo);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

}  // namespace

extern "C" int vlm_linear_recurrence(const vlm_recurrence_args* a, int nseg, int ntok, int dtype, void* stream) {
  if (!a || nseg < 0 || ntok < 0) return VLM_ERR_ARG;
  if (a->gated < 0 || a->gated > 2 || a->gate_act < 0 || a->gate_act > 2 || (a->gated == 2 && a->rot_dims)) return VLM_ERR_ARG;
  if (!a->q || !a->k || !a->v || (!a->g && a->gate_act != 2) || !a->state || !a->raw || !a->out || !a->seg_start || !a->seg_slot || !a->seg_pos0)
    return VLM_ERR_ARG;
  if (a->H <= 0 || a->D <= 0 || a->Dv <= 0 || a->rot_dims < 0 || a->rot_dims > a->D || (a->rot_dims & 1)) return VLM_ERR_ARG;
  if (a->rot_dims && !a->inv_freq) return VLM_ERR_ARG;
  if (a->gated == 2 ? false : a->gated ? (!a->ipre || !a->fpre || !a->ib || !a->fb || !a->mstate || !a->mtok || !a->mprev || !(a->cap > 0.f)) : !a->decay) return VLM_ERR_ARG;
  if (a->ldq < (long)a->H * a->D || a->ldk < (long)a->H * a->D || a->ldv < (long)a->H * a->Dv || (a->g && a->ldg < (long)a->H * a->Dv) ||
      a->ldo < (long)a->H * a->Dv)
    return VLM_ERR_ARG;
  if (nseg == 0 || ntok == 0) return VLM_OK;
  if (nseg > 65535 * 16 || a->H > 65535) return VLM_ERR_SHAPE;
  return dtype ? run<float>(*a, nseg, ntok, (hipStream_t)stream) : run<bf16_t>(*a, nseg, ntok, (hipStream_t)stream);
}
