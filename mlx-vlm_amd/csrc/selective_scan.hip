// The selective state-space scan: per sequence a state S [C][N] in fp32 (C channels, N states per channel),
//
//     dt_c = softplus(dt_pre_c + dt_bias_c)          A[c][n] = -exp(A_log[c][n])
//     S[c][n] <- exp(dt_c A[c][n]) S[c][n] + (dt_c x_c) B_n
//     y_c = sum_n S[c][n] C_n + D_c x_c              out_c = y_c * silu(z_c)
//
// x (after its short convolution and activation) and z are T-typed projection rows; dt_pre, B and C are fp32 rows (everything
// that enters the recurrence after the projections is fp32: step sizes, decays, their exponentials, the state).  One kernel
// serves a prompt, a portion and a decoded token: a segment is a run of consecutive tokens of one sequence; the state is read
// from the sequence's slot (zero when the segment starts at position 0: a slot that is used again needs no clearing), advanced
// token by token with the same operations in the same order wherever the prompt was cut, and written back.
//
// Work split: workgroup of 256 lanes = 256 / P channels x P lanes per channel; lane p of a channel holds the states
// n = p, p + P, ... (NS of them) in registers, so one token costs a lane NS exponentials and 2 NS FMAs; the read-out is summed
// over the P lanes of a channel by an xor tree inside the wave (P <= 64 divides the wave).  Tokens are staged 16 at a time
// through LDS: softplus is evaluated once per (token, channel) on the way in, y is gated and written coalesced on the way out.
#include "common.hpp"
#include "../../include/vlm_hip.h"
#include "recurrence_finish.hpp"

namespace {

__device__ __forceinline__ float softplus_f(float v) { return v > 20.f ? v : log1pf(expf(v)); }

template <typename T, int NS>
__global__ __launch_bounds__(256) void selective_scan_kernel(vlm_selective_scan_args a, int P, int TB) {
  extern __shared__ __align__(16) float smem[];
  const int CH = 256 / P, NP = P * NS;
  float* dts = smem;                    // [TB][CH]
  float* xs = dts + TB * CH;            // [TB][CH]
  float* ys = xs + TB * CH;             // [TB][CH]
  float* Bs = ys + TB * CH;             // [TB][NP]
  float* Cs = Bs + TB * NP;             // [TB][NP]
  const int seg = blockIdx.x, tid = threadIdx.x;
  const int ch = tid / P, p = tid % P, c0 = blockIdx.y * CH, c = c0 + ch;
  const int C = a.C, N = a.N;
  const int t_begin = a.seg_start[seg], t_end = a.seg_start[seg + 1];
  const int slot = a.seg_slot[seg], pos0 = a.seg_pos0[seg];
  const bool live = c < C;
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
  for (int t0 = t_begin; t0 < t_end; t0 += TB) {
    const int nb = min(TB, t_end - t0);
    for (int i = tid; i < nb * CH; i += 256) {
      const int t = i / CH, cc = c0 + i % CH;
      float dt = 0.f, xv = 0.f;
      if (cc < C) {
        dt = softplus_f(a.dt_pre[(long)(t0 + t) * a.lddt + cc] + ld_f((const T*)a.dt_bias + cc));
        xv = ld_f((const T*)a.x + (long)(t0 + t) * a.ldx + cc);
      }
      dts[i] = dt;
      xs[i] = xv;
    }
    for (int i = tid; i < nb * NP; i += 256) {
      const int t = i / NP, n = i % NP;
      Bs[i] = n < N ? a.B[(long)(t0 + t) * a.ldbc + n] : 0.f;
      Cs[i] = n < N ? a.Cm[(long)(t0 + t) * a.ldbc + n] : 0.f;
    }
    __syncthreads();
    for (int t = 0; t < nb; ++t) {
      const float dt = dts[t * CH + ch], xv = xs[t * CH + ch];
      const float dtx = dt * xv;
      float part = 0.f;
#pragma unroll
      for (int j = 0; j < NS; ++j) {
        const int n = p + P * j;
        s[j] = fmaf(expf(dt * A[j]), s[j], dtx * Bs[t * NP + n]);
        part = fmaf(s[j], Cs[t * NP + n], part);
      }
      for (int o = P >> 1; o > 0; o >>= 1) part += __shfl_xor(part, o);
      if (p == 0) ys[t * CH + ch] = fmaf(Dc, xv, part);
    }
    __syncthreads();
    for (int i = tid; i < nb * CH; i += 256) {
      const int t = i / CH, cc = c0 + i % CH;
      if (cc < C) {
        const float zv = ld_f((const T*)a.z + (long)(t0 + t) * a.ldz + cc);
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

}  // namespace

extern "C" int vlm_selective_scan(const vlm_selective_scan_args* a, int nseg, int ntok, int dtype, void* stream) {
  if (!a || nseg < 0 || ntok < 0) return VLM_ERR_ARG;
  if (!a->x || !a->z || !a->dt_pre || !a->B || !a->Cm || !a->dt_bias || !a->A_log || !a->D || !a->seg_start || !a->seg_slot ||
      !a->seg_pos0 || !a->state || !a->out)
    return VLM_ERR_ARG;
  if (a->C <= 0 || a->N <= 0 || a->ldx < a->C || a->ldz < a->C || a->lddt < a->C || a->ldbc < a->N || a->ldo < a->C) return VLM_ERR_ARG;
  if (nseg == 0 || ntok == 0) return VLM_OK;
  if (a->N > 256 || nseg > 65535 * 16) return VLM_ERR_SHAPE;
  const int NS = a->N <= 64 ? 1 : (a->N <= 128 ? 2 : 4);
  int P = 1;
  while (P * NS < a->N) P <<= 1;
  const int CH = 256 / P;
  int TB = 16;
  auto lds = [&](int tb) { return (size_t)tb * (3 * CH + 2 * P * NS) * sizeof(float); };
  if (lds(TB) > 48 * 1024) TB = 8;
  const unsigned nblk = (unsigned)((a->C + CH - 1) / CH);
  if (nblk > 65535) return VLM_ERR_SHAPE;
  dim3 grid(nseg, nblk);
  hipStream_t st = (hipStream_t)stream;
#define GO(T, K) hipLaunchKernelGGL((selective_scan_kernel<T, K>), grid, dim3(256), lds(TB), st, *a, P, TB)
  if (dtype) {
    if (NS == 1) GO(float, 1); else if (NS == 2) GO(float, 2); else GO(float, 4);
  } else {
    if (NS == 1) GO(bf16_t, 1); else if (NS == 2) GO(bf16_t, 2); else GO(bf16_t, 4);
  }
#undef GO
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}
