// Row operators of a decoder whose RESIDUAL STREAM is fp32 (the sum x <- x + f(x) never rounds to 16 bits) while
// projections run in the serving dtype T (bf16, or fp32 in the float32 mode).  Norm statistics, the sums and the
// activations are fp32; a T-typed output is rounded once.  dtype code: 0 = bf16, 1 = fp32 for every "T" pointer.
//
//   vlm_embed_scale_f32      x[t] = table[id[t]] * scale                              (scaled embedding lookup)
//   vlm_layernorm_nobias     out[t] = (x[t] - mean) * rsqrt(var + eps) * w            (two-pass variance: mean of squared deviations)
//   vlm_stream_add           x[t] += a[t] (+ b[t])                                    (parallel sublayers: one norm, two readers)
//   vlm_unit_rms_add         x[t] += y[t] * rsqrt(mean(y[t]^2) + eps) * w
//   vlm_gelu_tanh_gate_rows  out[t][j] = gelu_tanh(g[t][j]) * table[id[t]][col0 + j]  (per-layer token input: gated slice of a
//                                                                                      second embedding table)
//   vlm_stream_cast          h[t] = T(x[t])                                           (sublayers that read the stream un-normed)
//   vlm_rms_rows             out[t] = x[t] * rsqrt(mean(x[t]^2) + eps) * w            (RMS norm of the fp32 stream)
//   vlm_gated_rms_add        the residual step of a sublayer whose RESULT is gated and normed:
//                              y = a[t]                                               (one branch), or
//                              y = (rms(a[t]) * wa + rms(b[t]) * wb) / 2              (two branches side by side, each normed)
//                              x[t] += rms(y * sigmoid(gate[t] + gate_bias)) * w      and h[t] = T(x[t]) for the next reader
//   vlm_relu2_rows           out[t][j] = max(in[t][j], 0)^2
//   vlm_scaled_add_rms       the residual step of a pre-norm sublayer and the norm of the next reader in one pass:
//                              x[t] += mult * y[t] (+ mult2 * y2[t])                  (y may be NULL: norm only)
//                              h[t] = x[t] * rsqrt(mean(x[t]^2) + eps) * (w_offset + w)   (w may be NULL: add only; w_offset 1
//                                                                                      for weights kept as offsets from one)
#include "common.hpp"
#include "../../include/vlm_hip.h"

namespace {

template <typename T> __device__ __forceinline__ float ld_f(const T* p);
template <> __device__ __forceinline__ float ld_f<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ld_f<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void st_f(T* p, float v);
template <> __device__ __forceinline__ void st_f<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void st_f<bf16_t>(bf16_t* p, float v) { *p = f2bf(v); }

// sum over the 256 lanes of a workgroup, same value in every lane, fixed order
__device__ __forceinline__ float block_sum(float v, float* red) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  const int w = threadIdx.x >> 6;
  __syncthreads();                      // (red may still be read from a previous call)
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

template <typename T>
__global__ __launch_bounds__(256) void embed_scale_kernel(const int* __restrict__ ids, const T* __restrict__ table, float scale,
                                                          float* __restrict__ x, int D, int vocab) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  for (int d = threadIdx.x; d < D; d += 256) x[(long)t * D + d] = ld_f(table + (long)id * D + d) * scale;
}

template <typename T>
__global__ __launch_bounds__(256) void layernorm_nobias_kernel(const float* __restrict__ x, const T* __restrict__ w, T* __restrict__ out,
                                                               int D, long ldo, float eps) {
  __shared__ float red[4];
  const float* xr = x + (long)blockIdx.x * D;
  float s = 0.f;
  for (int d = threadIdx.x; d < D; d += 256) s += xr[d];
  const float mean = block_sum(s, red) / (float)D;
  float q = 0.f;
  for (int d = threadIdx.x; d < D; d += 256) {
    const float c = xr[d] - mean;
    q += c * c;
  }
  const float r = 1.0f / sqrtf(block_sum(q, red) / (float)D + eps);
  for (int d = threadIdx.x; d < D; d += 256) st_f(out + (long)blockIdx.x * ldo + d, (xr[d] - mean) * r * ld_f(w + d));
}

template <typename T>
__global__ __launch_bounds__(256) void stream_add_kernel(float* __restrict__ x, const T* __restrict__ a, long lda,
                                                         const T* __restrict__ b, long ldb, int D) {
  const long t = blockIdx.x;
  for (int d = threadIdx.x; d < D; d += 256) {
    float v = ld_f(a + t * lda + d);
    if (b) v += ld_f(b + t * ldb + d);
    x[t * D + d] += v;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void unit_rms_add_kernel(float* __restrict__ x, const T* __restrict__ y, long ldy,
                                                           const T* __restrict__ w, int D, float eps) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  float q = 0.f;
  for (int d = threadIdx.x; d < D; d += 256) {
    const float v = ld_f(y + t * ldy + d);
    q += v * v;
  }
  const float r = 1.0f / sqrtf(block_sum(q, red) / (float)D + eps);
  for (int d = threadIdx.x; d < D; d += 256) x[t * D + d] += ld_f(y + t * ldy + d) * r * (w ? ld_f(w + d) : 1.f);
}

__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <typename T>
__global__ __launch_bounds__(256) void gelu_gate_rows_kernel(const T* __restrict__ g, long ldg, const T* __restrict__ table, long ldt,
                                                             const int* __restrict__ ids, int col0, T* __restrict__ out, long ldo,
                                                             int rows, int dim, int vocab) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long)rows * dim) return;
  const long t = i / dim;
  const int j = (int)(i % dim);
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  st_f(out + t * ldo + j, gelu_tanh_f(ld_f(g + t * ldg + j)) * ld_f(table + (long)id * ldt + col0 + j));
}

template <typename T>
__global__ __launch_bounds__(256) void stream_cast_kernel(const float* __restrict__ x, T* __restrict__ h, long n) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) st_f(h + i, x[i]);
}

template <typename T>
__global__ __launch_bounds__(256) void rms_rows_kernel(const float* __restrict__ x, const T* __restrict__ w, T* __restrict__ out, int D,
                                                       long ldo, float eps) {
  __shared__ float red[4];
  const float* xr = x + (long)blockIdx.x * D;
  float q = 0.f;
  for (int d = threadIdx.x; d < D; d += 256) q += xr[d] * xr[d];
  const float r = 1.0f / sqrtf(block_sum(q, red) / (float)D + eps);
  for (int d = threadIdx.x; d < D; d += 256) st_f(out + (long)blockIdx.x * ldo + d, xr[d] * r * ld_f(w + d));
}

template <typename T>
__global__ __launch_bounds__(256) void gated_rms_add_kernel(float* __restrict__ x, const T* __restrict__ a, long lda,
                                                            const T* __restrict__ wa, const T* __restrict__ b, long ldb,
                                                            const T* __restrict__ wb, const T* __restrict__ gate, long ldg,
                                                            const T* __restrict__ gate_bias, const T* __restrict__ w,
                                                            T* __restrict__ h, int D, float eps) {
  extern __shared__ float y[];           // [D]
  __shared__ float red[4];
  const long t = blockIdx.x;
  if (b) {
    float qa = 0.f, qb = 0.f;
    for (int d = threadIdx.x; d < D; d += 256) {
      const float va = ld_f(a + t * lda + d), vb = ld_f(b + t * ldb + d);
      qa += va * va;
      qb += vb * vb;
    }
    const float ra = 1.0f / sqrtf(block_sum(qa, red) / (float)D + eps);
    const float rb = 1.0f / sqrtf(block_sum(qb, red) / (float)D + eps);
    for (int d = threadIdx.x; d < D; d += 256)
      y[d] = 0.5f * (ld_f(a + t * lda + d) * ra * ld_f(wa + d) + ld_f(b + t * ldb + d) * rb * ld_f(wb + d));
  } else {
    for (int d = threadIdx.x; d < D; d += 256) y[d] = ld_f(a + t * lda + d);
  }
  float q = 0.f;
  for (int d = threadIdx.x; d < D; d += 256) {          // (every lane re-reads only the entries it wrote)
    float v = y[d];
    if (gate) v *= 1.f / (1.f + expf(-(ld_f(gate + t * ldg + d) + (gate_bias ? ld_f(gate_bias + d) : 0.f))));
    y[d] = v;
    q += v * v;
  }
  const float r = 1.0f / sqrtf(block_sum(q, red) / (float)D + eps);
  for (int d = threadIdx.x; d < D; d += 256) {
    const float v = x[t * D + d] + y[d] * r * ld_f(w + d);
    x[t * D + d] = v;
    if (h) st_f(h + t * D + d, v);
  }
}

template <typename T, typename HT>
__global__ __launch_bounds__(256) void scaled_add_rms_kernel(float* __restrict__ x, const T* __restrict__ y, long ldy, float mult,
                                                             const T* __restrict__ y2, long ldy2, float mult2,
                                                             const T* __restrict__ w, float w_offset, HT* __restrict__ h, long ldh,
                                                             int D, float eps) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  float* xr = x + t * D;
  float q = 0.f;
  for (int d = threadIdx.x; d < D; d += 256) {          // (every lane re-reads only the entries it wrote)
    float v = xr[d];
    if (y) {
      v = fmaf(mult, ld_f(y + t * ldy + d), v);
      if (y2) v = fmaf(mult2, ld_f(y2 + t * ldy2 + d), v);
      xr[d] = v;
    }
    q += v * v;
  }
  if (!w) return;
  const float r = 1.0f / sqrtf(block_sum(q, red) / (float)D + eps);
  for (int d = threadIdx.x; d < D; d += 256) st_f(h + t * ldh + d, xr[d] * r * (w_offset + ld_f(w + d)));
}

template <typename T>
__global__ __launch_bounds__(256) void relu2_rows_kernel(const T* __restrict__ in, long ldi, T* __restrict__ out, long ldo, int rows,
                                                         int dim) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long)rows * dim) return;
  const long t = i / dim;
  const int j = (int)(i % dim);
  const float v = fmaxf(ld_f(in + t * ldi + j), 0.f);
  st_f(out + t * ldo + j, v * v);
}

}  // namespace

#define STREAM_ARGS_OK(rows, D) ((rows) >= 0 && (D) > 0)

extern "C" int vlm_embed_scale_f32(const void* ids, const void* table, float scale, void* x, int rows, int D, int vocab, int dtype,
                                   void* stream) {
  if (!ids || !table || !x || !STREAM_ARGS_OK(rows, D) || vocab <= 0) return VLM_ERR_ARG;
  if (rows == 0) return VLM_OK;
  hipStream_t st = (hipStream_t)stream;
  if (dtype) hipLaunchKernelGGL(embed_scale_kernel<float>, dim3(rows), dim3(256), 0, st, (const int*)ids, (const float*)table, scale, (float*)x, D, vocab);
  else hipLaunchKernelGGL(embed_scale_kernel<bf16_t>, dim3(rows), dim3(256), 0, st, (const int*)ids, (const bf16_t*)table, scale, (float*)x, D, vocab);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_layernorm_nobias(const void* x, const void* w, void* out, int rows, int D, long ldo, float eps, int dtype,
                                    void* stream) {
  if (!x || !w || !out || !STREAM_ARGS_OK(rows, D) || ldo < D) return VLM_ERR_ARG;
  if (rows == 0) return VLM_OK;
  hipStream_t st = (hipStream_t)stream;
  if (dtype) hipLaunchKernelGGL(layernorm_nobias_kernel<float>, dim3(rows), dim3(256), 0, st, (const float*)x, (const float*)w, (float*)out, D, ldo, eps);
  else hipLaunchKernelGGL(layernorm_nobias_kernel<bf16_t>, dim3(rows), dim3(256), 0, st, (const float*)x, (const bf16_t*)w, (bf16_t*)out, D, ldo, eps);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_stream_add(void* x, const void* a, long lda, const void* b, long ldb, int rows, int D, int dtype, void* stream) {
  if (!x || !a || !STREAM_ARGS_OK(rows, D) || lda < D || (b && ldb < D)) return VLM_ERR_ARG;
  if (rows == 0) return VLM_OK;
  hipStream_t st = (hipStream_t)stream;
  if (dtype) hipLaunchKernelGGL(stream_add_kernel<float>, dim3(rows), dim3(256), 0, st, (float*)x, (const float*)a, lda, (const float*)b, ldb, D);
  else hipLaunchKernelGGL(stream_add_kernel<bf16_t>, dim3(rows), dim3(256), 0, st, (float*)x, (const bf16_t*)a, lda, (const bf16_t*)b, ldb, D);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_unit_rms_add(void* x, const void* y, long ldy, const void* w, int rows, int D, float eps, int dtype, void* stream) {
  if (!x || !y || !STREAM_ARGS_OK(rows, D) || ldy < D) return VLM_ERR_ARG;
  if (rows == 0) return VLM_OK;
  hipStream_t st = (hipStream_t)stream;
  if (dtype) hipLaunchKernelGGL(unit_rms_add_kernel<float>, dim3(rows), dim3(256), 0, st, (float*)x, (const float*)y, ldy, (const float*)w, D, eps);
  else hipLaunchKernelGGL(unit_rms_add_kernel<bf16_t>, dim3(rows), dim3(256), 0, st, (float*)x, (const bf16_t*)y, ldy, (const bf16_t*)w, D, eps);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_gelu_tanh_gate_rows(const void* g, long ldg, const void* table, long ldt, const void* ids, int col0, void* out,
                                       long ldo, int rows, int dim, int vocab, int dtype, void* stream) {
  if (!g || !table || !ids || !out || rows < 0 || dim <= 0 || col0 < 0 || col0 + dim > ldt || ldg < dim || ldo < dim || vocab <= 0)
    return VLM_ERR_ARG;
  if (rows == 0) return VLM_OK;
  hipStream_t st = (hipStream_t)stream;
  const unsigned nb = (unsigned)(((long)rows * dim + 255) / 256);
  if (dtype) hipLaunchKernelGGL(gelu_gate_rows_kernel<float>, dim3(nb), dim3(256), 0, st, (const float*)g, ldg, (const float*)table, ldt, (const int*)ids, col0, (float*)out, ldo, rows, dim, vocab);
  else hipLaunchKernelGGL(gelu_gate_rows_kernel<bf16_t>, dim3(nb), dim3(256), 0, st, (const bf16_t*)g, ldg, (const bf16_t*)table, ldt, (const int*)ids, col0, (bf16_t*)out, ldo, rows, dim, vocab);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_stream_cast(const void* x, void* h, int rows, int D, int dtype, void* stream) {
  if (!x || !h || !STREAM_ARGS_OK(rows, D)) return VLM_ERR_ARG;
  if (rows == 0) return VLM_OK;
  hipStream_t st = (hipStream_t)stream;
  const long n = (long)rows * D;
  const unsigned nb = (unsigned)((n + 255) / 256);
  if (dtype) hipLaunchKernelGGL(stream_cast_kernel<float>, dim3(nb), dim3(256), 0, st, (const float*)x, (float*)h, n);
  else hipLaunchKernelGGL(stream_cast_kernel<bf16_t>, dim3(nb), dim3(256), 0, st, (const float*)x, (bf16_t*)h, n);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_rms_rows(const void* x, const void* w, void* out, int rows, int D, long ldo, float eps, int dtype, void* stream) {
  if (!x || !w || !out || !STREAM_ARGS_OK(rows, D) || ldo < D) return VLM_ERR_ARG;
  if (rows == 0) return VLM_OK;
  hipStream_t st = (hipStream_t)stream;
  if (dtype) hipLaunchKernelGGL(rms_rows_kernel<float>, dim3(rows), dim3(256), 0, st, (const float*)x, (const float*)w, (float*)out, D, ldo, eps);
  else hipLaunchKernelGGL(rms_rows_kernel<bf16_t>, dim3(rows), dim3(256), 0, st, (const float*)x, (const bf16_t*)w, (bf16_t*)out, D, ldo, eps);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_gated_rms_add(void* x, const void* a, long lda, const void* wa, const void* b, long ldb, const void* wb,
                                 const void* gate, long ldg, const void* gate_bias, const void* w, void* h, int rows, int D, float eps,
                                 int dtype, void* stream) {
  if (!x || !a || !w || !STREAM_ARGS_OK(rows, D) || lda < D || (b && (ldb < D || !wa || !wb)) || (gate && ldg < D)) return VLM_ERR_ARG;
  if (rows == 0) return VLM_OK;
  if ((size_t)D * sizeof(float) > 48 * 1024) return VLM_ERR_SHAPE;
  hipStream_t st = (hipStream_t)stream;
  const size_t lds = (size_t)D * sizeof(float);
  if (dtype)
    hipLaunchKernelGGL(gated_rms_add_kernel<float>, dim3(rows), dim3(256), lds, st, (float*)x, (const float*)a, lda, (const float*)wa,
                       (const float*)b, ldb, (const float*)wb, (const float*)gate, ldg, (const float*)gate_bias, (const float*)w,
                       (float*)h, D, eps);
  else
    hipLaunchKernelGGL(gated_rms_add_kernel<bf16_t>, dim3(rows), dim3(256), lds, st, (float*)x, (const bf16_t*)a, lda, (const bf16_t*)wa,
                       (const bf16_t*)b, ldb, (const bf16_t*)wb, (const bf16_t*)gate, ldg, (const bf16_t*)gate_bias, (const bf16_t*)w,
                       (bf16_t*)h, D, eps);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_relu2_rows(const void* in, long ldi, void* out, long ldo, int rows, int dim, int dtype, void* stream) {
  if (!in || !out || rows < 0 || dim <= 0 || ldi < dim || ldo < dim) return VLM_ERR_ARG;
  if (rows == 0) return VLM_OK;
  hipStream_t st = (hipStream_t)stream;
  const unsigned nb = (unsigned)(((long)rows * dim + 255) / 256);
  if (dtype) hipLaunchKernelGGL(relu2_rows_kernel<float>, dim3(nb), dim3(256), 0, st, (const float*)in, ldi, (float*)out, ldo, rows, dim);
  else hipLaunchKernelGGL(relu2_rows_kernel<bf16_t>, dim3(nb), dim3(256), 0, st, (const bf16_t*)in, ldi, (bf16_t*)out, ldo, rows, dim);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_scaled_add_rms(void* x, const void* y, long ldy, float mult, const void* y2, long ldy2, float mult2, const void* w,
                                  float w_offset, void* h, long ldh, int h_f32, int rows, int D, float eps, int dtype, void* stream) {
  if (!x || !STREAM_ARGS_OK(rows, D) || (y && ldy < D) || (y2 && (!y || ldy2 < D)) || (!y && !w) || (w && (!h || ldh < D))) return VLM_ERR_ARG;
  if (rows == 0) return VLM_OK;
  hipStream_t st = (hipStream_t)stream;
  if (dtype) hipLaunchKernelGGL((scaled_add_rms_kernel<float, float>), dim3(rows), dim3(256), 0, st, (float*)x, (const float*)y, ldy, mult, (const float*)y2, ldy2, mult2, (const float*)w, w_offset, (float*)h, ldh, D, eps);
  else if (h_f32) hipLaunchKernelGGL((scaled_add_rms_kernel<bf16_t, float>), dim3(rows), dim3(256), 0, st, (float*)x, (const bf16_t*)y, ldy, mult, (const bf16_t*)y2, ldy2, mult2, (const bf16_t*)w, w_offset, (float*)h, ldh, D, eps);
  else hipLaunchKernelGGL((scaled_add_rms_kernel<bf16_t, bf16_t>), dim3(rows), dim3(256), 0, st, (float*)x, (const bf16_t*)y, ldy, mult, (const bf16_t*)y2, ldy2, mult2, (const bf16_t*)w, w_offset, (bf16_t*)h, ldh, D, eps);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}
