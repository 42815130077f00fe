// Mixture-of-experts routing and the expert activation, for experts whose up / down projections are stacked into ONE matrix
// each (rows of W_up: expert 0's ff rows, expert 1's, ..., then the shared expert's; columns of W_down in the same order).
// A token's routed output is then   down( gate_e(t) * act(up_e h) for every expert e )   with gate_e(t) = 0 for the experts
// the token did not choose: one up GEMM, this activation pass, one down GEMM - the sum over experts is the k loop of the down
// projection, and the experts a token skipped contribute exact zeros.
//
//   vlm_moe_route        logits fp32 [T][E] -> the `top` largest per token (lowest index wins a tie), softmax over the chosen
//                        logits only; dense gate table fp32 [T][E] (0 where not chosen) + the chosen (index, weight) lists
//   vlm_moe_route_scored the same choice with the weights taken from the softmax over ALL experts, times `scale`, with no
//                        second normalisation over the chosen ones; and group-limited: consecutive experts are cut into
//                        `groups` blocks of one size, a block ranks by its best expert, and the choice is made among the
//                        experts of the `keep` top-ranked blocks (lowest index wins a tie).  groups = keep = 1: no limit.
//   vlm_moe_route_sigmoid  scores s = sigmoid(z) per expert; the choice is made on s + correction (a per-expert offset that enters
//                        nothing but the choice), limited to the `keep` best blocks of experts, a block ranking by the SUM of its
//                        `group_top` largest choice scores; the experts of the other blocks cannot be chosen whatever their
//                        scores (not even when the kept ones are negative); weights = the chosen s, divided by their sum + 1e-20
//                        (when normalise), times scale.  The sigmoid of `extra` further logit columns is handed out beside the
//                        table: the gate of an expert that every token uses.
//   vlm_glu_rows         out[t][c] = act(g[t][c]) * u[t][c]; act: 0 = tanh-form gelu, 1 = silu, 2 = sigmoid.  With a route table:
//                        E stacked experts of ff output columns, out[t][e ff + j] = act(g[t][e estride + j]) * u[t][e estride + j]
//                        * route[t][e] (estride: the distance of two experts' columns in g and u, e.g. 2 ff when every expert's
//                        gate and up rows lie side by side); T-typed in and out, fp32 inside
//   vlm_moe_relu2_gate   out[t][c] = relu(up[t][c])^2 * gate[t][c / ff]   for c < E * ff,   relu(up[t][c])^2 for the
//                        `shared` columns behind them (an expert every token uses); T-typed in and out, fp32 inside
#include "common.hpp"
#include "../../include/vlm_hip.h"

namespace {

template <typename T> __device__ __forceinline__ float ld_f(const T* p);
template <> __device__ __forceinline__ float ld_f<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ld_f<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void st_f(T* p, float v);
template <> __device__ __forceinline__ void st_f<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void st_f<bf16_t>(bf16_t* p, float v) { *p = f2bf(v); }

// one wave per token; lane l owns experts l, l + 64, ... (a bit per owned expert records what earlier rounds took)
// scored: weights = softmax over all experts * scale (else: softmax over the chosen logits); groups / keep: see the file head
__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ z, int T, int E, int top, int scored, int groups,
                                                        int keep, float scale, float* __restrict__ gate, int* __restrict__ idx,
                                                        float* __restrict__ wgt) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (t >= T) return;
  const float* zr = z + (long)t * E;
  for (int e = lane; e < E; e += 64) gate[(long)t * E + e] = 0.f;
  unsigned taken = 0u;                   // bit i: the lane's i-th expert is chosen, or (set before the choice) not eligible
  float all_max = 0.f, all_den = 1.f;
  if (scored) {                          // maximum and denominator over ALL experts, fixed order: lane-strided, then the xor tree
    float m = -INFINITY;
    for (int e = lane; e < E; e += 64) m = fmaxf(m, zr[e]);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
    float d = 0.f;
    for (int e = lane; e < E; e += 64) d += expf(zr[e] - m);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) d += __shfl_xor(d, o);
    all_max = m;
    all_den = d;
  }
  if (groups > 1 && keep < groups) {     // rank the blocks by their best expert, keep `keep` of them; the experts of every other block are marked
    const int gsz = E / groups;
    unsigned long long kept = 0ull;      // (groups <= 64)
    for (int k = 0; k < keep; ++k) {
      float best = -INFINITY;
      int bg = 0x7fffffff;
      for (int e = lane; e < E; e += 64) {
        const int g = e / gsz;
        const float v = zr[e];
        if (!((kept >> g) & 1ull) && (v > best || (v == best && g < bg))) {
          best = v;
          bg = g;
        }
      }
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        const float ob = __shfl_xor(best, o);
        const int og = __shfl_xor(bg, o);
        if (ob > best || (ob == best && og < bg)) {
          best = ob;
          bg = og;
        }
      }
      if (bg == 0x7fffffff) break;
      kept |= 1ull << bg;
    }
    for (int e = lane, i = 0; e < E; e += 64, ++i)
      if (!((kept >> (e / gsz)) & 1ull)) taken |= 1u << i;
  }
  float zmax = 0.f, denom = 0.f;
  float my_val = 0.f;                    // lane j < top keeps the j-th chosen logit
  int my_idx = -1;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane, i = 0; e < E; e += 64, ++i) {
      const float v = zr[e];
      if (!((taken >> i) & 1u) && (v > best || (v == best && e < bi))) {
        best = v;
        bi = e;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o);
      const int oi = __shfl_xor(bi, o);
      if (ob > best || (ob == best && oi < bi)) {
        best = ob;
        bi = oi;
      }
    }
    if (bi == 0x7fffffff) break;         // fewer comparable candidates than `top` (NaN logits): what was found is kept
    if (lane == (bi & 63)) taken |= 1u << (bi >> 6);
    if (j == 0) zmax = best;
    if (lane == j) {
      my_val = best;
      my_idx = bi;
    }
    denom += expf(best - zmax);
  }
  const float w = my_idx < 0 ? 0.f : (scored ? expf(my_val - all_max) / all_den * scale : expf(my_val - zmax) / denom);
  if (lane < top) {
    idx[(long)t * top + lane] = my_idx < 0 ? 0 : my_idx;
    wgt[(long)t * top + lane] = w;
  }
  for (int j = 0; j < top; ++j) {        // the owner of an expert writes its gate (it also wrote the zero)
    const int ej = __shfl(my_idx, j);
    const float wj = __shfl(w, j);
    if (ej >= 0 && lane == (ej & 63)) gate[(long)t * E + ej] = wj;
  }
}

// one wave per token; lane l owns experts l, l + 64, ... (bit i of `taken`: the lane's i-th expert is chosen or not eligible)
__global__ __launch_bounds__(256) void moe_route_sigmoid_kernel(const float* __restrict__ z, long ldz, int T, int E, int top, int groups,
                                                                int keep, int group_top, const float* __restrict__ corr, int normalise,
                                                                float scale, int extra, float* __restrict__ extra_out,
                                                                float* __restrict__ gate, int* __restrict__ idx, float* __restrict__ wgt) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (t >= T) return;
  const float* zr = z + (long)t * ldz;
  for (int e = lane; e < E; e += 64) gate[(long)t * E + e] = 0.f;
  for (int e = lane; e < extra; e += 64) extra_out[(long)t * extra + e] = 1.f / (1.f + expf(-zr[E + e]));
  auto choice = [&](int e) { return 1.f / (1.f + expf(-zr[e])) + (corr ? corr[e] : 0.f); };
  unsigned taken = 0u;
  if (groups > 1 && keep < groups) {
    const int gsz = E / groups;
    // lane g (groups <= 64): the sum of the group_top largest choice scores of block g, members taken in index order
    float gscore = -INFINITY;
    if (lane < groups) {
      float sum = 0.f;
      int last = -1;
      float lastv = INFINITY;
      for (int k = 0; k < group_top && k < gsz; ++k) {   // k-th largest: the largest value below (lastv, last) in (value desc, index asc) order
        float best = -INFINITY;
        int bi = -1;
        for (int j = 0; j < gsz; ++j) {
          const float v = choice(lane * gsz + j);
          const bool below = v < lastv || (v == lastv && j > last);
          if (below && (bi < 0 || v > best)) {
            best = v;
            bi = j;
          }
        }
        if (bi < 0) break;
        sum += best;
        lastv = best;
        last = bi;
      }
      gscore = sum;
    }
    unsigned long long kept = 0ull;
    for (int k = 0; k < keep; ++k) {
      float best = (lane < groups && !((kept >> lane) & 1ull)) ? gscore : -INFINITY;
      int bg = (lane < groups && !((kept >> lane) & 1ull)) ? lane : 0x7fffffff;
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        const float ob = __shfl_xor(best, o);
        const int og = __shfl_xor(bg, o);
        if (og != 0x7fffffff && (bg == 0x7fffffff || ob > best || (ob == best && og < bg))) {
          best = ob;
          bg = og;
        }
      }
      if (bg == 0x7fffffff) break;
      kept |= 1ull << bg;
    }
    for (int e = lane, i = 0; e < E; e += 64, ++i)
      if (!((kept >> (e / gsz)) & 1ull)) taken |= 1u << i;
  }
  float my_s = 0.f, denom = 0.f;
  int my_idx = -1;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane, i = 0; e < E; e += 64, ++i) {
      if ((taken >> i) & 1u) continue;
      const float v = choice(e);
      if (bi == 0x7fffffff || v > best || (v == best && e < bi)) {
        best = v;
        bi = e;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o);
      const int oi = __shfl_xor(bi, o);
      if (oi != 0x7fffffff && (bi == 0x7fffffff || ob > best || (ob == best && oi < bi))) {
        best = ob;
        bi = oi;
      }
    }
    if (bi == 0x7fffffff) break;
    if (lane == (bi & 63)) taken |= 1u << (bi >> 6);
    const float sj = 1.f / (1.f + expf(-zr[bi]));        // the weight uses the score WITHOUT the correction
    if (lane == j) {
      my_s = sj;
      my_idx = bi;
    }
    denom += sj;                                         // chosen order, the same in every lane
  }
  const float w = my_idx < 0 ? 0.f : (normalise ? my_s / (denom + 1e-20f) : my_s) * scale;
  if (lane < top) {
    idx[(long)t * top + lane] = my_idx < 0 ? 0 : my_idx;
    wgt[(long)t * top + lane] = w;
  }
  for (int j = 0; j < top; ++j) {
    const int ej = __shfl(my_idx, j);
    const float wj = __shfl(w, j);
    if (ej >= 0 && lane == (ej & 63)) gate[(long)t * E + ej] = wj;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_relu2_gate_kernel(const T* __restrict__ up, long ldu, const float* __restrict__ gate, int E,
                                                             int ff, int shared, T* __restrict__ out, long ldo, int rows) {
  const int cols = E * ff + shared;
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long)rows * cols) return;
  const long t = i / cols;
  const int c = (int)(i % cols);
  const float u = fmaxf(ld_f(up + t * ldu + c), 0.f);
  const float g = c < E * ff ? gate[t * E + c / ff] : 1.f;
  st_f(out + t * ldo + c, u * u * g);
}

__device__ __forceinline__ float glu_act(float z, int act) {
  if (act == 0) return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  const float sg = 1.f / (1.f + expf(-z));
  return act == 1 ? z * sg : sg;
}

template <typename T>
__global__ __launch_bounds__(256) void glu_rows_kernel(const T* __restrict__ g, long ldg, const T* __restrict__ u, long ldu,
                                                       const float* __restrict__ route, int E, int ff, int estride, int act,
                                                       T* __restrict__ out, long ldo, int rows, int dim) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long)rows * dim) return;
  const long t = i / dim;
  const int c = (int)(i % dim);
  float r = 1.f;
  long cs = c;                            // the column in g and u
  if (route) {
    const int e = c / ff;
    r = route[t * E + e];
    if (r == 0.f) {                       // an expert the token did not choose: an exact zero whatever its columns hold
      st_f(out + t * ldo + c, 0.f);
      return;
    }
    cs = (long)e * estride + (c - e * ff);
  }
  st_f(out + t * ldo + c, glu_act(ld_f(g + t * ldg + cs), act) * ld_f(u + t * ldu + cs) * r);
}

}  // namespace

extern "C" int vlm_moe_route(const void* logits, int T, int E, int top, void* gate, void* idx, void* wgt, void* stream) {
  if (!logits || !gate || !idx || !wgt || T < 0 || E <= 0 || top <= 0 || top > E) return VLM_ERR_ARG;
  if (top > 64 || E > 2048) return VLM_ERR_SHAPE;
  if (T == 0) return VLM_OK;
  hipLaunchKernelGGL(moe_route_kernel, dim3((T + 3) / 4), dim3(256), 0, (hipStream_t)stream, (const float*)logits, T, E, top, 0, 1, 1,
                     1.f, (float*)gate, (int*)idx, (float*)wgt);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_moe_route_scored(const void* logits, int T, int E, int top, int groups, int keep, float scale, void* gate, void* idx,
                                    void* wgt, void* stream) {
  if (!logits || !gate || !idx || !wgt || T < 0 || E <= 0 || top <= 0 || top > E || groups <= 0 || keep <= 0 || keep > groups ||
      E % groups || top > (long)keep * (E / groups))
    return VLM_ERR_ARG;
  if (top > 64 || E > 2048 || groups > 64) return VLM_ERR_SHAPE;
  if (T == 0) return VLM_OK;
  hipLaunchKernelGGL(moe_route_kernel, dim3((T + 3) / 4), dim3(256), 0, (hipStream_t)stream, (const float*)logits, T, E, top, 1, groups,
                     keep, scale, (float*)gate, (int*)idx, (float*)wgt);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_moe_route_sigmoid(const void* logits, long ldz, int T, int E, int top, int groups, int keep, int group_top,
                                     const void* correction, int normalise, float scale, int extra, void* extra_out, void* gate, void* idx,
                                     void* wgt, void* stream) {
  if (!logits || !gate || !idx || !wgt || T < 0 || E <= 0 || top <= 0 || top > E || groups <= 0 || keep <= 0 || keep > groups || E % groups ||
      top > (long)keep * (E / groups) || group_top < 1 || extra < 0 || (extra && !extra_out) || ldz < (long)E + extra)
    return VLM_ERR_ARG;
  if (top > 64 || E > 2048 || groups > 64) return VLM_ERR_SHAPE;
  if (T == 0) return VLM_OK;
  hipLaunchKernelGGL(moe_route_sigmoid_kernel, dim3((T + 3) / 4), dim3(256), 0, (hipStream_t)stream, (const float*)logits, ldz, T, E, top,
                     groups, keep, group_top, (const float*)correction, normalise, scale, extra, (float*)extra_out, (float*)gate, (int*)idx,
                     (float*)wgt);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_glu_rows(const void* g, long ldg, const void* u, long ldu, const void* route, int E, int ff, int estride, int act,
                            void* out, long ldo, int rows, int dim, int dtype, void* stream) {
  if (!g || !u || !out || rows < 0 || dim <= 0 || ldo < dim || act < 0 || act > 2) return VLM_ERR_ARG;
  if (route ? (E <= 0 || ff <= 0 || (long)E * ff != dim || estride < ff || ldg < (long)(E - 1) * estride + ff ||
               ldu < (long)(E - 1) * estride + ff)
            : (ldg < dim || ldu < dim))
    return VLM_ERR_ARG;
  if (rows == 0) return VLM_OK;
  const unsigned nb = (unsigned)(((long)rows * dim + 255) / 256);
  hipStream_t st = (hipStream_t)stream;
  if (dtype)
    hipLaunchKernelGGL(glu_rows_kernel<float>, dim3(nb), dim3(256), 0, st, (const float*)g, ldg, (const float*)u, ldu, (const float*)route,
                       E, ff, estride, act, (float*)out, ldo, rows, dim);
  else
    hipLaunchKernelGGL(glu_rows_kernel<bf16_t>, dim3(nb), dim3(256), 0, st, (const bf16_t*)g, ldg, (const bf16_t*)u, ldu,
                       (const float*)route, E, ff, estride, act, (bf16_t*)out, ldo, rows, dim);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_moe_relu2_gate(const void* up, long ldu, const void* gate, int E, int ff, int shared, void* out, long ldo, int rows,
                                  int dtype, void* stream) {
  if (!up || !out || rows < 0 || E < 0 || ff < 0 || shared < 0 || (E > 0 && !gate)) return VLM_ERR_ARG;
  const long cols = (long)E * ff + shared;
  if (cols <= 0 || ldu < cols || ldo < cols) return VLM_ERR_ARG;
  if (rows == 0) return VLM_OK;
  const unsigned nb = (unsigned)((rows * cols + 255) / 256);
  hipStream_t st = (hipStream_t)stream;
  if (dtype)
    hipLaunchKernelGGL(moe_relu2_gate_kernel<float>, dim3(nb), dim3(256), 0, st, (const float*)up, ldu, (const float*)gate, E, ff,
                       shared, (float*)out, ldo, rows);
  else
    hipLaunchKernelGGL(moe_relu2_gate_kernel<bf16_t>, dim3(nb), dim3(256), 0, st, (const bf16_t*)up, ldu, (const float*)gate, E, ff,
                       shared, (bf16_t*)out, ldo, rows);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}
