// The selective state-space scan: per sequence a state S [C][N] in fp32 (C channels, N states per channel),
//
//     dt_c = softplus(dt_pre_c + dt_bias_c)          A[c][n] = -exp(A_log[c][n])
//     S[c][n] <- exp(dt_c A[c][n]) S[c][n] + (dt_c x_c) B_n
//     y_c = sum_n S[c][n] C_n + D_c x_c              out_c = y_c * silu(z_c)
//
// x (after its short convolution and activation) and z are T-typed projection rows; dt_pre (or the low-rank rows dt_low it is
// projected from by W_dt), B and C are fp32 rows (everything
// that enters the recurrence after the projections is fp32: step sizes, decays, their exponentials, the state).  One kernel
// serves a prompt, a portion and a decoded token: a segment is a run of consecutive tokens of one sequence; the state is read
// from the sequence's slot (zero when the segment starts at position 0: a slot that is used again needs no clearing), advanced
// token by token with the same operations in the same order wherever the prompt was cut, and written back.
//
// Work split: workgroup of 256 lanes = 256 / P channels x P lanes per channel; lane p of a channel holds the states
// n = p, p + P, ... (NS of them) in registers, so one token costs a lane NS exponentials and 2 NS FMAs; the read-out is summed
// over the P lanes of a channel inside the wave (DPP quad swaps and row mirrors up to 16 lanes, lane exchanges above: no LDS
// traffic, the same tree whatever the cut).  Tokens are staged 16 at a time through LDS - softplus once per (token, channel) on
// the way in, optionally with the step-size projection itself (dt_pre = W_dt dt_low, a dot of dt_rank per (token, channel)
// against the staged low-rank rows) - and the 16 token updates are unrolled: only the state's FMA chain is sequential, the
// exponentials, products and sums of later tokens overlap it.  A block shorter than 16 tokens is padded with dt = x = B = C = 0
// (exp(0) * S + 0 leaves the state as it is).  The global loads of a stage are issued into registers one stage ahead, so they
// are in flight while the stage before is computed.  y is gated and written coalesced on the way out.
#include "common.hpp"
#include "../../include/vlm_hip.h"
#include "recurrence_finish.hpp"

namespace {

constexpr int TB = 16;

__device__ __forceinline__ float softplus_f(float v) { return v > 20.f ? v : log1pf(expf(v)); }

// sum over the P lanes of a channel (P a power of two, groups aligned to P): every lane of the group ends with the same bits
template <int P>
__device__ __forceinline__ float group_sum(float v) {
  if (P >= 2) v += vlm_dpp<0xB1, 0xf>(0.f, v);      // quad_perm [1,0,3,2]
  if (P >= 4) v += vlm_dpp<0x4E, 0xf>(0.f, v);      // quad_perm [2,3,0,1]
  if (P >= 8) v += vlm_dpp<0x141, 0xf>(0.f, v);     // row_half_mirror
  if (P >= 16) v += vlm_dpp<0x140, 0xf>(0.f, v);    // row_mirror
  if (P >= 32) v += __shfl_xor(v, 16);
  if (P >= 64) v += __shfl_xor(v, 32);
  return v;
}

constexpr int LMAX = 16;      // low-rank rows of a stage held in registers: 16 x 256 values = 16 tokens of dt_rank <= 256

template <typename T, int P, int NS>
__global__ __launch_bounds__(256) void selective_scan_kernel(vlm_selective_scan_args a, int wdt_lds) {
  extern __shared__ __align__(16) float smem[];
  constexpr int CH = 256 / P, NP = P * NS;
  constexpr int EX = (TB * CH + 255) / 256, EB = (TB * NP + 255) / 256;      // per-lane elements of a stage: channel rows, B / C rows
  float* dts = smem;                    // [TB][CH]
  float* xs = dts + TB * CH;            // [TB][CH]
  float* zs = xs + TB * CH;             // [TB][CH]
  float* ys = dts;                      // [TB][CH]: y takes the place of dt - a channel's lanes sit in ONE wave, which has read the
                                        // channel's dt (first pass) before its lane 0 writes y (last pass)
  float* Bs = zs + TB * CH;             // [TB][NP]
  float* Cs = Bs + TB * NP;             // [TB][NP]
  float* lows = Cs + TB * NP;           // [TB][R] (fused step-size projection)
  float* wdt = lows + TB * a.R;         // [CH][R + 1]: the block's rows of W_dt (when wdt_lds)
  const int seg = blockIdx.x, tid = threadIdx.x;
  const int ch = tid / P, p = tid % P, c0 = blockIdx.y * CH, c = c0 + ch;
  const int C = a.C, N = a.N, R = a.R;
  const int t_begin = a.seg_start[seg], t_end = a.seg_start[seg + 1];
  const int slot = a.seg_slot[seg], pos0 = a.seg_pos0[seg];
  const bool live = c < C, fused = a.dt_w != nullptr;
  float A[NS], s[NS];
  float* S = a.state + ((long)slot * C + (live ? c : 0)) * N;
#pragma unroll
  for (int j = 0; j < NS; ++j) {
    const int n = p + P * j;
    const bool on = live && n < N;
    A[j] = on ? -expf(ld_f((const T*)a.A_log + (long)c * N + n)) : 0.f;
    s[j] = (on && pos0 > 0) ? S[n] : 0.f;
  }
  const float Dc = live ? ld_f((const T*)a.D + c) : 0.f;
  if (fused && wdt_lds)
    for (int i = tid; i < CH * R; i += 256) wdt[(i / R) * (R + 1) + i % R] = c0 + i / R < C ? ld_f((const T*)a.dt_w + (long)(c0 + i / R) * R + i % R) : 0.f;
  float bias[EX];
#pragma unroll
  for (int e = 0; e < EX; ++e) {
    const int i = tid + 256 * e, cc = c0 + i % CH;
    bias[e] = (i < TB * CH && cc < C) ? ld_f((const T*)a.dt_bias + cc) : 0.f;
  }
  // the loads of a stage go to registers one stage ahead: they are in flight while the stage before is computed, so the only
  // exposed memory latency is the first stage's.  Elements past the segment's end are zeros (dt = x = B = C = 0 leave the state).
  float px[EX], pz[EX], pd[EX], pB[EB], pC[EB], pl[LMAX];
  auto prefetch = [&](int t0) {
    const int nb = min(TB, t_end - t0);
#pragma unroll
    for (int e = 0; e < EX; ++e) {
      const int i = tid + 256 * e, t = i / CH, cc = c0 + i % CH;
      const bool on = i < TB * CH && t < nb && cc < C;
      px[e] = on ? ld_f((const T*)a.x + (long)(t0 + t) * a.ldx + cc) : 0.f;
      pz[e] = on ? ld_f((const T*)a.z + (long)(t0 + t) * a.ldz + cc) : 0.f;
      pd[e] = (on && !fused) ? a.dt_pre[(long)(t0 + t) * a.lddt + cc] : 0.f;
    }
#pragma unroll
    for (int e = 0; e < EB; ++e) {
      const int i = tid + 256 * e, t = i / NP, n = i % NP;
      const bool on = i < TB * NP && t < nb && n < N;
      pB[e] = on ? a.B[(long)(t0 + t) * a.ldbc + n] : 0.f;
      pC[e] = on ? a.Cm[(long)(t0 + t) * a.ldbc + n] : 0.f;
    }
    if (fused) {
#pragma unroll
      for (int e = 0; e < LMAX; ++e) {
        const int i = tid + 256 * e;
        pl[e] = 0.f;
        if (i < nb * R) {                     // (a branch, not a select: the division stays out of the trips a short stage does not need)
          const int t = i / R;
          pl[e] = a.dt_low[(long)(t0 + t) * a.lddt + (i - t * R)];
        }
      }
    }
  };
  prefetch(t_begin);
  for (int t0 = t_begin; t0 < t_end; t0 += TB) {
    const int nb = min(TB, t_end - t0);
#pragma unroll
    for (int e = 0; e < EX; ++e) {
      const int i = tid + 256 * e;
      if (i < TB * CH) {
        xs[i] = px[e];
        zs[i] = pz[e];
      }
    }
#pragma unroll
    for (int e = 0; e < EB; ++e) {
      const int i = tid + 256 * e;
      if (i < TB * NP) {
        Bs[i] = pB[e];
        Cs[i] = pC[e];
      }
    }
    if (fused) {
#pragma unroll
      for (int e = 0; e < LMAX; ++e) {
        const int i = tid + 256 * e;
        if (i < nb * R) lows[i] = pl[e];
      }
    }
    float dpre[EX];
#pragma unroll
    for (int e = 0; e < EX; ++e) dpre[e] = pd[e];
    __syncthreads();
    if (t0 + TB < t_end) prefetch(t0 + TB);
    // step sizes: softplus once per (token, channel); with W_dt given, its dot with the staged low-rank row first
#pragma unroll
    for (int e = 0; e < EX; ++e) {
      const int i = tid + 256 * e, t = i / CH, cc = c0 + i % CH;
      if (i < TB * CH) {
        float dt = 0.f;
        if (t < nb && cc < C) {
          float pre = dpre[e];
          if (fused) {
            const float* lr = lows + t * R;
            pre = 0.f;
            if (wdt_lds) {
              const float* wl = wdt + (i % CH) * (R + 1);
#pragma unroll 8
              for (int r = 0; r < R; ++r) pre = fmaf(wl[r], lr[r], pre);      // (unrolled: eight pairs of LDS reads in flight per wait)
            } else {
              const T* wr = (const T*)a.dt_w + (long)cc * R;
#pragma unroll 8
              for (int r = 0; r < R; ++r) pre = fmaf(ld_f(wr + r), lr[r], pre);
            }
          }
          dt = softplus_f(pre + bias[e]);
        }
        dts[i] = dt;
      }
    }
    __syncthreads();
    {
    constexpr int tc = 0;
    // three passes over 16 staged tokens, so that only the FMA chain of the state is sequential: (1) decays and inputs of every
    // token, independent of the state; (2) the chain; (3) the sums over the channel's lanes, independent of each other
    float e[TB][NS], bx[TB][NS], part[TB];
#pragma unroll
    for (int t = 0; t < TB; ++t) {
      const float dt = dts[(tc + t) * CH + ch], dtx = dt * xs[(tc + t) * CH + ch];
#pragma unroll
      for (int j = 0; j < NS; ++j) {
        e[t][j] = expf(dt * A[j]);
        bx[t][j] = dtx * Bs[(tc + t) * NP + p + P * j];
      }
    }
#pragma unroll
    for (int t = 0; t < TB; ++t) {
      float acc = 0.f;
#pragma unroll
      for (int j = 0; j < NS; ++j) {
        s[j] = fmaf(e[t][j], s[j], bx[t][j]);
        acc = fmaf(s[j], Cs[(tc + t) * NP + p + P * j], acc);
      }
      part[t] = acc;
    }
#pragma unroll
    for (int t = 0; t < TB; ++t) part[t] = group_sum<P>(part[t]);
    if (p == 0) {
#pragma unroll
      for (int t = 0; t < TB; ++t) ys[(tc + t) * CH + ch] = fmaf(Dc, xs[(tc + t) * CH + ch], part[t]);
    }
    }
    __syncthreads();
    for (int i = tid; i < nb * CH; i += 256) {
      const int t = i / CH, cc = c0 + i % CH;
      if (cc < C) {
        const float zv = zs[i];
        st_f((T*)a.out + (long)(t0 + t) * a.ldo + cc, ys[i] * (zv / (1.f + expf(-zv))));
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int j = 0; j < NS; ++j) {
    const int n = p + P * j;
    if (live && n < N) S[n] = s[j];
  }
}

template <typename T, int P, int NS>
void launch(const vlm_selective_scan_args& a, int nseg, int maxlen, hipStream_t st) {
  constexpr int CH = 256 / P;
  const size_t per_tok = (size_t)(3 * CH + 2 * P * NS + (a.dt_w ? a.R : 0)) * sizeof(float);
  const size_t wl = a.dt_w ? (size_t)CH * (a.R + 1) * sizeof(float) : 0;
  const int wdt_lds = wl && TB * per_tok + wl <= 60 * 1024;          // (else the rows are read from memory in the staging loop)
  const size_t fixed = wdt_lds ? wl : 0;
  (void)maxlen;
  hipLaunchKernelGGL((selective_scan_kernel<T, P, NS>), dim3(nseg, (a.C + CH - 1) / CH), dim3(256), TB * per_tok + fixed, st, a, wdt_lds);
}

template <typename T>
int run(const vlm_selective_scan_args& a, int nseg, int maxlen, hipStream_t st) {
  const int NS = a.N <= 64 ? 1 : (a.N <= 128 ? 2 : 4);
  int P = 1;
  while (P * NS < a.N) P <<= 1;
  const int CH = 256 / P;
  if ((size_t)TB * (3 * CH + 2 * P * NS + (a.dt_w ? a.R : 0)) * sizeof(float) > 64 * 1024 || (a.dt_w && a.R > 16 * LMAX) || (a.C + CH - 1) / CH > 65535) return VLM_ERR_SHAPE;
  if (NS == 2) launch<T, 64, 2>(a, nseg, maxlen, st);
  else if (NS == 4) launch<T, 64, 4>(a, nseg, maxlen, st);
  else if (P == 1) launch<T, 1, 1>(a, nseg, maxlen, st);
  else if (P == 2) launch<T, 2, 1>(a, nseg, maxlen, st);
  else if (P == 4) launch<T, 4, 1>(a, nseg, maxlen, st);
  else if (P == 8) launch<T, 8, 1>(a, nseg, maxlen, st);
  else if (P == 16) launch<T, 16, 1>(a, nseg, maxlen, st);
  else if (P == 32) launch<T, 32, 1>(a, nseg, maxlen, st);
  else launch<T, 64, 1>(a, nseg, maxlen, st);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

}  // namespace

extern "C" int vlm_selective_scan(const vlm_selective_scan_args* a, int nseg, int ntok, int dtype, void* stream) {
  if (!a || nseg < 0 || ntok < 0) return VLM_ERR_ARG;
  if (!a->x || !a->z || !a->B || !a->Cm || !a->dt_bias || !a->A_log || !a->D || !a->seg_start || !a->seg_slot || !a->seg_pos0 ||
      !a->state || !a->out)
    return VLM_ERR_ARG;
  if (a->dt_w ? (!a->dt_low || a->R <= 0 || a->lddt < a->R) : (!a->dt_pre || a->lddt < a->C)) return VLM_ERR_ARG;
  if (a->C <= 0 || a->N <= 0 || a->ldx < a->C || a->ldz < a->C || a->ldbc < a->N || a->ldo < a->C) return VLM_ERR_ARG;
  if (nseg == 0 || ntok == 0) return VLM_OK;
  if (a->N > 256 || nseg > 65535 * 16) return VLM_ERR_SHAPE;
  return dtype ? run<float>(*a, nseg, ntok, (hipStream_t)stream) : run<bf16_t>(*a, nseg, ntok, (hipStream_t)stream);      // (ntok bounds a segment's length)
}
