// Generic strided, batched linear layer for the shapes and number formats the MFMA GEMMs (gemm_bf16.hip) do not take:
//
//     C[b][m][n] (+)= sum_k A[b][m][k] * W[b][n][k]          b < batch, any M, N, K, any leading dimension
//
// A, W and C are each bf16 or fp32 (codes 0 / 1); products and sums are fp32 FMAs in ascending k, so a row of C depends on
// nothing but its own row of A: the result of a token is the same bits whatever else is in the batch and however a
// prompt was cut into steps.  With all three in fp32 this is the true 32-bit product of the float32 serving mode; with
// fp32 C and `accumulate` it adds a projection straight onto an fp32 residual stream.
//
// 64 x 64 output tile per workgroup of 256 lanes (4 waves), 16-deep k slabs staged through LDS as fp32, 4 x 4 outputs
// per lane.  Per-head projections of one tensor (latent attention's absorbed key / value maps) run as `batch` with
// element strides between heads.
#include "common.hpp"
#include "../../include/vlm_hip.h"

namespace {

template <typename T> __device__ __forceinline__ float ld_f(const T* p);
template <> __device__ __forceinline__ float ld_f<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ld_f<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void st_f(T* p, float v);
template <> __device__ __forceinline__ void st_f<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void st_f<bf16_t>(bf16_t* p, float v) { *p = f2bf(v); }

constexpr int BM = 64, BN = 64, BK = 16;

template <typename TA, typename TW, typename TC>
__global__ __launch_bounds__(256) void linear_any_kernel(const TA* __restrict__ A, const TW* __restrict__ W, TC* __restrict__ C,
                                                         int M, int N, int K, long lda, long ldw, long ldc, long sA, long sW,
                                                         long sC, int accumulate) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  const int b = blockIdx.z;
  A += (long)b * sA;
  W += (long)b * sW;
  C += (long)b * sC;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int tid = threadIdx.x;
  const int tm = (tid / 16) * 4, tn = (tid % 16) * 4;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += BK) {
    // 64 rows x 16 k of each operand: lane -> (row = tid / 4, 4 consecutive k)
    const int r = tid >> 2, kk = (tid & 3) * 4;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = k0 + kk + j;
      As[kk + j][r] = (m0 + r < M && k < K) ? ld_f(A + (long)(m0 + r) * lda + k) : 0.f;
      Ws[kk + j][r] = (n0 + r < N && k < K) ? ld_f(W + (long)(n0 + r) * ldw + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[k][tm + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[k][tn + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + tm + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tn + j;
      if (n >= N) continue;
      TC* c = C + (long)m * ldc + n;
      st_f(c, accumulate ? ld_f(c) + acc[i][j] : acc[i][j]);
    }
  }
}

// the same product on 16 x 64 output tiles (one row x four columns per lane) for shapes that give the 64 x 64 tiling too few
// workgroups to fill the chip: few rows, or few output columns (router logits, low-rank maps).  Every output is the same FMA
// chain over ascending k as in the 64 x 64 kernel - the same bits - so the choice between the two may depend on the row count.
constexpr int SM = 16;
template <typename TA, typename TW, typename TC>
__global__ __launch_bounds__(256) void linear_any_rows16_kernel(const TA* __restrict__ A, const TW* __restrict__ W, TC* __restrict__ C,
                                                                int M, int N, int K, long lda, long ldw, long ldc, long sA, long sW,
                                                                long sC, int accumulate) {
  __shared__ float As[BK][SM + 1];
  __shared__ float Ws[BK][BN + 4];
  const int b = blockIdx.z;
  A += (long)b * sA;
  W += (long)b * sW;
  C += (long)b * sC;
  const int m0 = blockIdx.y * SM, n0 = blockIdx.x * BN;
  const int tid = threadIdx.x;
  const int tm = tid / 16, tn = (tid % 16) * 4;
  float acc[4] = {};
  for (int k0 = 0; k0 < K; k0 += BK) {
    {
      const int r = tid >> 4, k = k0 + (tid & 15);           // 16 rows x 16 k of A: one element per lane
      As[tid & 15][r] = (m0 + r < M && k < K) ? ld_f(A + (long)(m0 + r) * lda + k) : 0.f;
    }
    const int r = tid >> 2, kk = (tid & 3) * 4;             // 64 rows x 16 k of W: lane -> (row, 4 consecutive k)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = k0 + kk + j;
      Ws[kk + j][r] = (n0 + r < N && k < K) ? ld_f(W + (long)(n0 + r) * ldw + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      const float a = As[k][tm];
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] = fmaf(a, Ws[k][tn + j], acc[j]);
    }
    __syncthreads();
  }
  const int m = m0 + tm;
  if (m >= M) return;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = n0 + tn + j;
    if (n >= N) continue;
    TC* c = C + (long)m * ldc + n;
    st_f(c, accumulate ? ld_f(c) + acc[j] : acc[j]);
  }
}

// few rows (decode steps): the weights are the traffic, so W is read ONCE for all rows.  One wave per output column, lanes
// across k (coalesced), up to 8 row accumulators per lane, xor-butterfly sum: a fixed order, so a row's result is still a
// function of that row alone.  Sum order differs from the tile kernel's (rounding only); not used when everything is fp32.
template <typename TA, typename TW, typename TC>
__global__ __launch_bounds__(256) void linear_rows_kernel(const TA* __restrict__ A, const TW* __restrict__ W, TC* __restrict__ C,
                                                          int M, int N, int K, long lda, long ldw, long ldc, long sA, long sW,
                                                          long sC, int accumulate) {
  const int b = blockIdx.z;
  A += (long)b * sA;
  W += (long)b * sW;
  C += (long)b * sC;
  const int n = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (n >= N) return;                                     // (whole waves leave together: n is uniform per wave)
  const TW* w = W + (long)n * ldw;
  float acc[8] = {};
  for (int k = lane; k < K; k += 64) {
    const float wv = ld_f(w + k);
#pragma unroll
    for (int m = 0; m < 8; ++m)
      if (m < M) acc[m] = fmaf(ld_f(A + (long)m * lda + k), wv, acc[m]);
  }
#pragma unroll
  for (int m = 0; m < 8; ++m) {
    if (m >= M) break;
    float v = acc[m];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    if (lane == 0) {
      TC* c = C + (long)m * ldc + n;
      st_f(c, accumulate ? ld_f(c) + v : v);
    }
  }
}

// the same for bf16 weights whose rows are 16-byte aligned with K a multiple of 8: every lane reads 8 weights per load
// (16 bytes, non-temporal: a decode step reads each weight once).  Two ways to skip weights that cannot matter, both exact:
//   * a lane whose 8 activations are zero in EVERY row does not load its 8 weights (the down projection of stacked experts:
//     the experts no row of the step chose are exact zeros in the activations);
//   * skip_gate != nullptr: output columns [skip_col0, skip_col0 + E * ff) belong to E stacked experts of ff columns each;
//     a column whose expert has a zero gate in every row is written as 0 without reading its weights (the up projection).
template <typename TA, typename TC>
__global__ __launch_bounds__(256) void linear_rows_vec_kernel(const TA* __restrict__ A, const bf16_t* __restrict__ W, TC* __restrict__ C,
                                                              int M, int N, int K, long lda, long ldw, long ldc, int accumulate,
                                                              const float* __restrict__ skip_gate, int skip_col0, int E, int ff) {
  const int n = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (n >= N) return;
  if (skip_gate && n >= skip_col0 && n < skip_col0 + E * ff) {
    const int e = (n - skip_col0) / ff;
    bool any = false;
    for (int m = 0; m < M; ++m) any |= skip_gate[(long)m * E + e] != 0.f;
    if (!any) {                                          // (wave-uniform)
      if (lane < M && !accumulate) st_f(C + (long)lane * ldc + n, 0.f);
      return;
    }
  }
  const bf16_t* w = W + (long)n * ldw;
  float acc[8] = {};
  for (int k = lane * 8; k < K; k += 512) {
    float a[8][8];
    bool nz = false;
#pragma unroll
    for (int m = 0; m < 8; ++m)
      if (m < M) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          a[m][j] = ld_f(A + (long)m * lda + k + j);
          nz |= a[m][j] != 0.f;
        }
      }
    if (!nz) continue;
    const uint4 wv = nt_load16(w + k);
    const float wf[8] = {bf_lo(wv.x), bf_hi(wv.x), bf_lo(wv.y), bf_hi(wv.y), bf_lo(wv.z), bf_hi(wv.z), bf_lo(wv.w), bf_hi(wv.w)};
#pragma unroll
    for (int m = 0; m < 8; ++m)
      if (m < M) {
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[m] = fmaf(a[m][j], wf[j], acc[m]);
      }
  }
#pragma unroll
  for (int m = 0; m < 8; ++m) {
    if (m >= M) break;
    float v = acc[m];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    if (lane == 0) {
      TC* c = C + (long)m * ldc + n;
      st_f(c, accumulate ? ld_f(c) + v : v);
    }
  }
}

template <typename TA, typename TW, typename TC>
int launch(const void* A, const void* W, void* C, int M, int N, int K, long lda, long ldw, long ldc, int batch, long sA, long sW,
           long sC, int accumulate, hipStream_t st) {
  // all-fp32 operands (the float32 serving mode) always take the tile kernel: one summation order for every row count, so a
  // token's result is the same bits in a prompt, in a portion and decoded alone
  constexpr bool all_f32 = sizeof(TA) == 4 && sizeof(TW) == 4 && sizeof(TC) == 4;
  if (M <= 8 && !all_f32) {
    dim3 grid((N + 3) / 4, 1, batch);
    hipLaunchKernelGGL((linear_rows_kernel<TA, TW, TC>), grid, dim3(256), 0, st, (const TA*)A, (const TW*)W, (TC*)C, M, N, K, lda,
                       ldw, ldc, sA, sW, sC, accumulate);
  } else if ((long)((N + BN - 1) / BN) * ((M + BM - 1) / BM) * batch < 256) {
    // fewer 64 x 64 tiles than compute units: 16-row tiles (the same bits per output)
    dim3 grid((N + BN - 1) / BN, (M + SM - 1) / SM, batch);
    hipLaunchKernelGGL((linear_any_rows16_kernel<TA, TW, TC>), grid, dim3(256), 0, st, (const TA*)A, (const TW*)W, (TC*)C, M, N, K, lda,
                       ldw, ldc, sA, sW, sC, accumulate);
  } else {
    dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM, batch);
    hipLaunchKernelGGL((linear_any_kernel<TA, TW, TC>), grid, dim3(256), 0, st, (const TA*)A, (const TW*)W, (TC*)C, M, N, K, lda,
                       ldw, ldc, sA, sW, sC, accumulate);
  }
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

}  // namespace

// decode-step form with the expert-column skip (see linear_rows_vec_kernel); M <= 8, bf16 weights, K % 8 == 0
extern "C" int vlm_linear_rows_bf16w(const void* A, const void* W, void* C, int M, int N, int K, long lda, long ldw, long ldc, int a_f32,
                                     int c_f32, int accumulate, const void* skip_gate, int skip_col0, int E, int ff, void* stream) {
  if (!A || !W || !C || M <= 0 || M > 8 || N <= 0 || K <= 0 || lda < K || ldw < K || ldc < N) return VLM_ERR_ARG;
  if (accumulate && !c_f32) return VLM_ERR_ARG;
  if (skip_gate && (E <= 0 || ff <= 0 || skip_col0 < 0 || skip_col0 + (long)E * ff > N)) return VLM_ERR_ARG;
  if (K % 8 || ldw % 8 || ((uintptr_t)W & 15)) return VLM_ERR_SHAPE;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((N + 3) / 4);
#define GO(TA, TC)                                                                                                              \
  hipLaunchKernelGGL((linear_rows_vec_kernel<TA, TC>), grid, dim3(256), 0, st, (const TA*)A, (const bf16_t*)W, (TC*)C, M, N, K, lda, \
                     ldw, ldc, accumulate, (const float*)skip_gate, skip_col0, E, ff)
  if (a_f32) {
    if (c_f32) GO(float, float); else GO(float, bf16_t);
  } else {
    if (c_f32) GO(bf16_t, float); else GO(bf16_t, bf16_t);
  }
#undef GO
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_linear_any(const void* A, const void* W, void* C, int M, int N, int K, long lda, long ldw, long ldc, int a_f32,
                              int w_f32, int c_f32, int batch, long strideA, long strideW, long strideC, int accumulate,
                              void* stream) {
  if (!A || !W || !C || M < 0 || N <= 0 || K <= 0 || batch <= 0 || lda < K || ldw < K || ldc < N) return VLM_ERR_ARG;
  if (accumulate && !c_f32) return VLM_ERR_ARG;
  if (M == 0) return VLM_OK;
  if (M > 65535 * 64 || batch > 65535) return VLM_ERR_SHAPE;
  hipStream_t st = (hipStream_t)stream;
  const int code = (a_f32 ? 4 : 0) | (w_f32 ? 2 : 0) | (c_f32 ? 1 : 0);
#define GO(TA, TW, TC) return launch<TA, TW, TC>(A, W, C, M, N, K, lda, ldw, ldc, batch, strideA, strideW, strideC, accumulate, st)
  switch (code) {
    case 0: GO(bf16_t, bf16_t, bf16_t);
    case 1: GO(bf16_t, bf16_t, float);
    case 2: GO(bf16_t, float, bf16_t);
    case 3: GO(bf16_t, float, float);
    case 4: GO(float, bf16_t, bf16_t);
    case 5: GO(float, bf16_t, float);
    case 6: GO(float, float, bf16_t);
    default: GO(float, float, float);
  }
#undef GO
}
