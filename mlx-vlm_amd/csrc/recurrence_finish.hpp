// Shared by the matrix-state recurrences (linear_recurrence.hip, delta_rule.hip): typed loads / stores and the finish pass
// that turns the raw read-out o [token][head][Dv (+ 1)] (fp32) into the mixer's output row:
//     o / denominator (gated form only)  ->  per-head unit RMS (eps)  ->  * normw[h][c] (optional)  ->  * silu or sigmoid of g (optional)
#pragma once
#include "common.hpp"

namespace {

template <typename T> __device__ __forceinline__ float ld_f(const T* p);
template <> __device__ __forceinline__ float ld_f<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ld_f<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void st_f(T* p, float v);
template <> __device__ __forceinline__ void st_f<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void st_f<bf16_t>(bf16_t* p, float v) { *p = f2bf(v); }

// grid (tokens, heads), one wave.  NORMALISER: column Dv of raw holds n . q, mtok the running maximum (exponential gating);
// gate_act: 0 = silu(g), 1 = sigmoid(g), 2 = no gate (g is not read)
template <typename T, bool NORMALISER>
__global__ __launch_bounds__(64) void recurrence_finish_kernel(const float* __restrict__ raw, int H, int Dv,
                                                               const float* __restrict__ mtok, float eps, const T* __restrict__ g,
                                                               long ldg, const T* __restrict__ normw, int gate_act,
                                                               T* __restrict__ out, long ldo) {
  const long tok = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const int C = Dv + (NORMALISER ? 1 : 0);
  const float* o = raw + (tok * H + h) * C;
  float inv = 1.f;
  if (NORMALISER) inv = 1.f / (fmaxf(fabsf(o[Dv]), expf(-mtok[tok * H + h])) + 1e-6f);
  float ss = 0.f;
  for (int c = lane; c < Dv; c += 64) {
    const float x = o[c] * inv;
    ss += x * x;
  }
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) ss += __shfl_xor(ss, d);
  const float r = 1.0f / sqrtf(ss / (float)Dv + eps);
  const T* gp = g + tok * ldg + (long)h * Dv;
  T* op = out + tok * ldo + (long)h * Dv;
  for (int c = lane; c < Dv; c += 64) {
    float x = o[c] * inv * r;
    if (normw) x *= ld_f(normw + (long)h * Dv + c);
    if (gate_act == 2) {
      st_f(op + c, x);
      continue;
    }
    const float gv = ld_f(gp + c), sg = 1.f / (1.f + expf(-gv));
    st_f(op + c, x * (gate_act == 0 ? gv * sg : sg));
  }
}

}  // namespace
