// Softmax attention over a paged per-token cache with grouped key / value heads, an optional sliding window, per-head
// RMS norm of q and k, interleaved-pair rotary positions on the first rot_dims dimensions, a per-head multiplier on the scores
// and an elementwise sigmoid gate on the output:
//
//     s_ij = (q_i . k_j) * scale * temp[h]        j visible from i  <=>  0 <= i - j < window  (window <= 0: every j <= i)
//     s_ij <- cap * tanh(s_ij / cap)              when a score cap is given (cap > 0)
//     o_i  = sum_j softmax_j(s_ij) v_j * sigmoid(gate_i)        gate_i: one number per value column, or one per head
//     sink: the softmax's denominator has one more term exp(0) that carries no value: p_ij = exp(s_ij) / (1 + sum_j exp(s_ij))
//
//   vlm_headnorm_rope_rows   x rows [T][heads][D] (T-typed) -> RMS norm per head (weight [D] shared by the heads, may be NULL)
//                            -> rotation of the pairs (2 i, 2 i + 1), i < rot_dims / 2, by pos * inv_freq[i] -> fp32, either
//                            dense [T][heads][D] (queries) or into the paged pool [page][64][heads * D] of the token's sequence
//                            (keys).  raw_pool (T-typed, same paging): the rows as they came, for designs whose values are the
//                            un-normed, un-rotated keys.
//   vlm_headnorm_rows        the same pass from an argument block, with what further designs need: a bias added to the rows
//                            first, an RMS norm WITHOUT a weight, a multiplier that grows with the logarithm of the position
//                            (1 + coef * ln(floor((pos + 1) / every) + 1), for queries), and separately projected value rows
//                            [T][heads][Dv] (+ bias) copied into their own paged pool in the same launch.
//   vlm_window_attn_blocks   prompt form: workgroup = (block of up to 16 consecutive queries of one sequence, head); tiles of 16
//                            keys at multiples of 16 counted from the sequence's first token go through LDS once per block, and
//                            every query runs the same per-tile update in the same order whatever block it sits in (a tile with
//                            no visible key leaves its running maximum, sum and accumulator untouched bit for bit): a token's
//                            result does not depend on how the prompt was cut or batched.
//   vlm_window_attn_rows     decode form: workgroup = (token, head); 16-byte loads of key and value rows when D % 4 == 0 and
//                            Dv % 8 == 0 (chunks of 1024 keys from the window's edge), else one key per lane in tiles of 256.
// Keys are cached in fp32 (norm and rotation are not rounded), values in T.  Scores, softmax and the weighted sum are fp32.
#include "common.hpp"
#include "../../include/vlm_hip.h"
#include "recurrence_finish.hpp"

namespace {

constexpr int PAGE = 64;
constexpr int QB = 16, KT = 16;

__device__ __forceinline__ float capped(float s, float cap) { return cap > 0.f ? cap * tanhf(s / cap) : s; }

// grid (tokens, heads), one wave.  norm: 0 = none, 1 = RMS norm (times w when given)
template <typename T>
__global__ __launch_bounds__(64) void headnorm_rope_kernel(const T* __restrict__ x, long ldx, int D, const T* __restrict__ bias,
                                                           const T* __restrict__ w, int norm, float eps, int rot_dims,
                                                           const float* __restrict__ inv_freq, float temp_coef, int temp_every,
                                                           const int* __restrict__ tok_pos, const int* __restrict__ tok_seq,
                                                           const int* __restrict__ block_table, int max_pages,
                                                           float* __restrict__ out, const T* __restrict__ raw, long ldraw, int Draw,
                                                           const T* __restrict__ raw_bias, T* __restrict__ raw_pool, int rot_half) {
  const long t = blockIdx.x;
  const int h = blockIdx.y, nh = gridDim.y, lane = threadIdx.x;
  const T* src = x + t * ldx + (long)h * D;
  const T* bs = bias ? bias + (long)h * D : nullptr;
  const int pos = tok_pos[t];
  long row = t;                                          // dense output row, or the token's place in the pool
  if (block_table) row = (long)block_table[(long)tok_seq[t] * max_pages + pos / PAGE] * PAGE + pos % PAGE;
  float* dst = out + (row * nh + h) * D;
  float ss = 0.f;
  for (int i = lane; i < D; i += 64) {
    const float v = ld_f(src + i) + (bs ? ld_f(bs + i) : 0.f);
    ss += v * v;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
  float r = norm ? 1.0f / sqrtf(ss / (float)D + eps) : 1.f;
  // (the multiplier is applied to the normed value as one more factor, so a design without it keeps its bits)
  const float mult = temp_every > 0 ? 1.f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.f) : 1.f;
  if (rot_half) {
    // pairs (i, i + rot_dims / 2), turned FIRST and normed after: every lane evaluates its own dimension from the two inputs of
    // its pair (the first half holds u, the second v: u' = u cos - v sin, v' = v cos + u sin), once for the sum of squares and
    // once more for the store
    const int half = rot_dims / 2;
    auto turned = [&](int i) {
      const float xi = ld_f(src + i) + (bs ? ld_f(bs + i) : 0.f);
      if (i >= rot_dims) return xi;
      const int j = i < half ? i + half : i - half;
      const float xj = ld_f(src + j) + (bs ? ld_f(bs + j) : 0.f);
      float sn, cs;
      sincosf((float)pos * inv_freq[i < half ? i : j], &sn, &cs);
      return i < half ? xi * cs - xj * sn : xi * cs + xj * sn;
    };
    float s2 = 0.f;
    for (int i = lane; i < D; i += 64) {
      const float v = turned(i);
      s2 += v * v;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) s2 += __shfl_xor(s2, o);
    r = norm ? 1.0f / sqrtf(s2 / (float)D + eps) : 1.f;
    for (int i = lane; i < D; i += 64) {
      float v = turned(i) * r * (w ? ld_f(w + i) : 1.f);
      if (temp_every > 0) v *= mult;
      dst[i] = v;
    }
  } else
  for (int i = lane; i < D / 2 + (D & 1); i += 64) {     // one pair per lane and trip (an odd last dimension passes alone)
    const int i0 = 2 * i, i1 = 2 * i + 1;
    float u = (ld_f(src + i0) + (bs ? ld_f(bs + i0) : 0.f)) * r * (w ? ld_f(w + i0) : 1.f);
    float v = i1 < D ? (ld_f(src + i1) + (bs ? ld_f(bs + i1) : 0.f)) * r * (w ? ld_f(w + i1) : 1.f) : 0.f;
    if (i1 < rot_dims) {
      float sn, cs;
      sincosf((float)pos * inv_freq[i], &sn, &cs);
      const float u2 = u * cs - v * sn;
      v = v * cs + u * sn;
      u = u2;
    }
    if (temp_every > 0) {
      u *= mult;
      v *= mult;
    }
    dst[i0] = u;
    if (i1 < D) dst[i1] = v;
  }
  if (raw_pool) {
    T* rd = raw_pool + (row * nh + h) * Draw;
    const T* rs = raw + t * ldraw + (long)h * Draw;
    if (raw_bias) {
      for (int i = lane; i < Draw; i += 64) st_f(rd + i, ld_f(rs + i) + ld_f(raw_bias + (long)h * Draw + i));
    } else {
      for (int i = lane; i < Draw; i += 64) rd[i] = rs[i];
    }
  }
}

// thread (r16, l16): score of (query r16, key l16) of the tile; then value dimensions l16 + 16 i of query r16
template <typename T, int NACC>
__global__ __launch_bounds__(256) void window_attn_block_kernel(const float* __restrict__ q, const float* __restrict__ kpool,
                                                                const T* __restrict__ vpool, const int* __restrict__ qb_start,
                                                                const int* __restrict__ qb_count, const int* __restrict__ tok_seq,
                                                                const int* __restrict__ tok_pos, const int* __restrict__ block_table,
                                                                int max_pages, int H, int KH, int D, int Dv, float scale,
                                                                const T* __restrict__ temp, int window, float cap, int sink, const T* __restrict__ gate,
                                                                long ldgate, int gate_head, T* __restrict__ out, long ldo) {
  extern __shared__ __align__(16) float smem[];
  const int DP = (D + 3) & ~3, KP = DP + 4, VP = NACC * 16;
  float* qs = smem;                         // [QB][DP]
  float* ks = qs + QB * DP;                 // [KT][KP]
  float* vs = ks + KT * KP;                 // [KT][VP]
  float* ps = vs + KT * VP;                 // [QB][KT + 1]
  float* mrun = ps + QB * (KT + 1);         // [QB]
  float* lrun = mrun + QB;                  // [QB]
  float* alph = lrun + QB;                  // [QB]
  const int t0 = qb_start[blockIdx.x], nq = qb_count[blockIdx.x];
  const int h = blockIdx.y, kh = h / (H / KH), tid = threadIdx.x;
  const int* bt = block_table + (long)tok_seq[t0] * max_pages;
  const int pos0 = tok_pos[t0];             // positions of the block's queries: pos0 .. pos0 + nq - 1
  const int r16 = tid >> 4, l16 = tid & 15;
  const float sc = scale * (temp ? ld_f(temp + h) : 1.f);
  for (int d = l16; d < DP; d += 16) qs[r16 * DP + d] = (r16 < nq && d < D) ? q[((long)(t0 + r16) * H + h) * D + d] : 0.f;
  if (tid < QB) {
    mrun[tid] = -INFINITY;
    lrun[tid] = 0.f;
  }
  float acc[NACC];
#pragma unroll
  for (int b = 0; b < NACC; ++b) acc[b] = 0.f;
  const int nkeys = pos0 + nq;
  const int first = window > 0 ? max(0, pos0 - window + 1) : 0;       // the first query's oldest visible key
  for (int j0 = (first / KT) * KT; j0 < nkeys; j0 += KT) {
    __syncthreads();
    {
      const int key = j0 + r16;
      float* kd = ks + r16 * KP;
      float* vd = vs + r16 * VP;
      if (key < nkeys) {
        const long rowk = (long)bt[key / PAGE] * PAGE + key % PAGE;
        const float* ksrc = kpool + (rowk * KH + kh) * D;
        const T* vsrc = vpool + (rowk * KH + kh) * Dv;
        for (int d = l16; d < DP; d += 16) kd[d] = d < D ? ksrc[d] : 0.f;
        for (int d = l16; d < VP; d += 16) vd[d] = d < Dv ? ld_f(vsrc + d) : 0.f;
      } else {
        for (int d = l16; d < DP; d += 16) kd[d] = 0.f;
        for (int d = l16; d < VP; d += 16) vd[d] = 0.f;
      }
    }
    __syncthreads();
    {
      const float4* qr = reinterpret_cast<const float4*>(qs + r16 * DP);
      const float4* kr = reinterpret_cast<const float4*>(ks + l16 * KP);
      float d = 0.f;
      for (int i = 0; i < DP / 4; ++i) {
        const float4 a = qr[i], b = kr[i];
        d = fmaf(a.x, b.x, d);
        d = fmaf(a.y, b.y, d);
        d = fmaf(a.z, b.z, d);
        d = fmaf(a.w, b.w, d);
      }
      const int dist = pos0 + r16 - (j0 + l16);
      const bool seen = r16 < nq && dist >= 0 && (window <= 0 || dist < window);
      ps[r16 * (KT + 1) + l16] = seen ? capped(d * sc, cap) : -INFINITY;
    }
    __syncthreads();
    if (tid < QB) {                         // per query: running maximum, tile weights, running sum (fixed order over the tile)
      float s[KT];
#pragma unroll
      for (int k = 0; k < KT; ++k) s[k] = ps[tid * (KT + 1) + k];
      float mt = s[0];
#pragma unroll
      for (int k = 1; k < KT; ++k) mt = fmaxf(mt, s[k]);
      const float m_old = mrun[tid], m_new = fmaxf(m_old, mt);
      float sum = 0.f;
#pragma unroll
      for (int k = 0; k < KT; ++k) {
        const float pv = s[k] == -INFINITY ? 0.f : expf(s[k] - m_new);
        ps[tid * (KT + 1) + k] = pv;
        sum += pv;
      }
      const float al = m_new == -INFINITY || m_old == m_new ? 1.f : expf(m_old - m_new);
      alph[tid] = al;
      lrun[tid] = lrun[tid] * al + sum;
      mrun[tid] = m_new;
    }
    __syncthreads();
    const float al = alph[r16];
#pragma unroll
    for (int b = 0; b < NACC; ++b) acc[b] *= al;
#pragma unroll 4
    for (int k = 0; k < KT; ++k) {
      const float pv = ps[r16 * (KT + 1) + k];
#pragma unroll
      for (int b = 0; b < NACC; ++b) acc[b] = fmaf(pv, vs[k * VP + l16 + 16 * b], acc[b]);
    }
  }
  __syncthreads();
  if (r16 < nq) {
    const long t = t0 + r16;
    const float inv = 1.f / (lrun[r16] + (sink ? expf(-mrun[r16]) : 0.f));
#pragma unroll
    for (int b = 0; b < NACC; ++b) {
      const int c = l16 + 16 * b;
      if (c < Dv) {
        float o = acc[b] * inv;
        if (gate) o *= 1.f / (1.f + expf(-ld_f(gate + t * ldgate + (gate_head ? (long)h : (long)h * Dv + c))));
        st_f(out + t * ldo + (long)h * Dv + c, o);
      }
    }
  }
}

// workgroup = (token, head): one key per lane and tile for the scores, one value dimension per lane for the weighted sum
template <typename T, int NACC>
__global__ __launch_bounds__(256) void window_attn_row_kernel(const float* __restrict__ q, const float* __restrict__ kpool,
                                                              const T* __restrict__ vpool, const int* __restrict__ tok_seq,
                                                              const int* __restrict__ tok_pos, const int* __restrict__ block_table,
                                                              int max_pages, int H, int KH, int D, int Dv, float scale,
                                                              const T* __restrict__ temp, int window, float cap, int sink, const T* __restrict__ gate,
                                                              long ldgate, int gate_head, T* __restrict__ out, long ldo) {
  extern __shared__ __align__(16) float smem[];
  float* qs = smem;              // [D]
  float* ps = qs + ((D + 3) & ~3);  // [256]
  float* red = ps + 256;         // [8]
  const long t = blockIdx.x;
  const int h = blockIdx.y, kh = h / (H / KH), tid = threadIdx.x;
  const int pos = tok_pos[t];
  const int* bt = block_table + (long)tok_seq[t] * max_pages;
  const float sc = scale * (temp ? ld_f(temp + h) : 1.f);
  for (int i = tid; i < D; i += 256) qs[i] = q[(t * H + h) * D + i];
  __syncthreads();
  float m_run = -INFINITY, l_run = 0.f;
  float acc[NACC];
#pragma unroll
  for (int a = 0; a < NACC; ++a) acc[a] = 0.f;
  const int nkeys = pos + 1;
  const int first = window > 0 ? max(0, pos - window + 1) : 0;
  for (int j0 = first; j0 < nkeys; j0 += 256) {
    const int j = j0 + tid;
    float s = -INFINITY;
    if (j < nkeys) {
      const float* kr = kpool + (((long)bt[j / PAGE] * PAGE + j % PAGE) * KH + kh) * D;
      float d = 0.f;
      for (int i = 0; i < D; ++i) d = fmaf(qs[i], kr[i], d);
      s = capped(d * sc, cap);
    }
    float mx = s;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    if ((tid & 63) == 0) red[tid >> 6] = mx;
    __syncthreads();
    const float m_new = fmaxf(m_run, fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3])));
    const float pj = j < nkeys ? expf(s - m_new) : 0.f;
    ps[tid] = pj;
    float sum = pj;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
    if ((tid & 63) == 0) red[4 + (tid >> 6)] = sum;
    __syncthreads();
    const float alpha = expf(m_run - m_new);           // (first tile: exp(-inf) = 0)
    l_run = l_run * alpha + ((red[4] + red[5]) + (red[6] + red[7]));
    m_run = m_new;
    const int nk = min(256, nkeys - j0);
#pragma unroll
    for (int a = 0; a < NACC; ++a) {
      const int dcol = tid + a * 256;
      if (dcol < Dv) {
        float v = acc[a] * alpha;
        for (int jj = 0; jj < nk; ++jj) {
          const int key = j0 + jj;
          v = fmaf(ps[jj], ld_f(vpool + (((long)bt[key / PAGE] * PAGE + key % PAGE) * KH + kh) * Dv + dcol), v);
        }
        acc[a] = v;
      }
    }
    __syncthreads();
  }
  const float inv = 1.f / (l_run + (sink ? expf(-m_run) : 0.f));
#pragma unroll
  for (int a = 0; a < NACC; ++a) {
    const int c = tid + a * 256;
    if (c < Dv) {
      float o = acc[a] * inv;
      if (gate) o *= 1.f / (1.f + expf(-ld_f(gate + t * ldgate + (gate_head ? (long)h : (long)h * Dv + c))));
      st_f(out + t * ldo + (long)h * Dv + c, o);
    }
  }
}

__device__ __forceinline__ void load8(const bf16_t* p, float* f) {
  const uint4 v = *reinterpret_cast<const uint4*>(p);
  f[0] = bf_lo(v.x); f[1] = bf_hi(v.x); f[2] = bf_lo(v.y); f[3] = bf_hi(v.y);
  f[4] = bf_lo(v.z); f[5] = bf_hi(v.z); f[6] = bf_lo(v.w); f[7] = bf_hi(v.w);
}
__device__ __forceinline__ void load8(const float* p, float* f) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
}

// Decode form for D % 4 == 0 and Dv % 8 == 0: workgroup = (token, head), the window in chunks of KC keys.
//   scores : thread (key, quarter): the four lanes of a DPP quad read one 64-byte piece of a key row per trip (16-byte loads)
//            and add their partial dot products; 64 keys per pass, no barrier between passes;
//   softmax: chunk maximum and sum over the scores in LDS (online across chunks);
//   values : thread (group of 8 value columns, key part): 16-byte loads of V rows, a wave covers whole rows; the key parts'
//            partial sums are added through LDS at the end.
constexpr int KC = 1024;
template <typename T>
__global__ __launch_bounds__(256) void window_attn_row_vec_kernel(const float* __restrict__ q, const float* __restrict__ kpool,
                                                                  const T* __restrict__ vpool, const int* __restrict__ tok_seq,
                                                                  const int* __restrict__ tok_pos, const int* __restrict__ block_table,
                                                                  int max_pages, int H, int KH, int D, int Dv, float scale,
                                                                  const T* __restrict__ temp, int window, float cap, int sink, const T* __restrict__ gate,
                                                                  long ldgate, int gate_head, T* __restrict__ out, long ldo) {
  extern __shared__ __align__(16) float smem[];
  float* qs = smem;                  // [D]
  float* sc = qs + D;                // [KC] scores, then weights
  float* part = sc + KC;             // [256 * 8] partial weighted sums
  int* rowi = reinterpret_cast<int*>(part + 2048);   // [KC] the chunk's keys as pool rows (page * 64 + place): one table lookup per key
  __shared__ float red[8];
  const long t = blockIdx.x;
  const int h = blockIdx.y, kh = h / (H / KH), tid = threadIdx.x, wave = tid >> 6;
  const int pos = tok_pos[t];
  const int* bt = block_table + (long)tok_seq[t] * max_pages;
  const float scl = scale * (temp ? ld_f(temp + h) : 1.f);
  for (int i = tid; i < D; i += 256) qs[i] = q[(t * H + h) * D + i];
  const int ngroups = Dv / 8, nparts = 256 / ngroups;          // value-column groups, key parts
  const int dg = tid % ngroups, kp = tid / ngroups;
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  const int nkeys = pos + 1;
  const int first = window > 0 ? max(0, pos - window + 1) : 0;
  const int D4 = D / 4;
  __syncthreads();
  for (int k0 = first; k0 < nkeys; k0 += KC) {
    const int nk = min(KC, nkeys - k0);
    for (int j = tid; j < nk; j += 256) rowi[j] = bt[(k0 + j) / PAGE] * PAGE + (k0 + j) % PAGE;
    __syncthreads();
#pragma unroll 2
    for (int jb = 0; jb < nk; jb += 64) {
      const int j = jb + (tid >> 2), qp = tid & 3;
      float d = 0.f;
      if (j < nk) {
        const float4* kr = reinterpret_cast<const float4*>(kpool + ((long)rowi[j] * KH + kh) * D);
        const float4* qr = reinterpret_cast<const float4*>(qs);
        for (int c = qp; c < D4; c += 4) {
          const float4 a = qr[c], b = kr[c];
          d = fmaf(a.x, b.x, d);
          d = fmaf(a.y, b.y, d);
          d = fmaf(a.z, b.z, d);
          d = fmaf(a.w, b.w, d);
        }
      }
      d += vlm_dpp<0xB1, 0xf>(0.f, d);     // quad_perm [1,0,3,2]
      d += vlm_dpp<0x4E, 0xf>(0.f, d);     // quad_perm [2,3,0,1]
      if (qp == 0 && j < nk) sc[j] = capped(d * scl, cap);
    }
    __syncthreads();
    float mx = -INFINITY;
    for (int j = tid; j < nk; j += 256) mx = fmaxf(mx, sc[j]);
    mx = wave_max(mx);
    if ((tid & 63) == 0) red[wave] = mx;
    __syncthreads();
    const float m_new = fmaxf(m_run, fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3])));
    float sum = 0.f;
    for (int j = tid; j < nk; j += 256) {
      const float pj = expf(sc[j] - m_new);
      sc[j] = pj;
      sum += pj;
    }
    sum = wave_sum(sum);
    if ((tid & 63) == 0) red[4 + wave] = sum;
    __syncthreads();
    const float alpha = expf(m_run - m_new);           // (first chunk: exp(-inf) = 0)
    l_run = l_run * alpha + ((red[4] + red[5]) + (red[6] + red[7]));
    m_run = m_new;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] *= alpha;
    if (kp < nparts) {
#pragma unroll 4
      for (int j = kp; j < nk; j += nparts) {
        float f[8];
        load8(vpool + ((long)rowi[j] * KH + kh) * Dv + dg * 8, f);
        const float pj = sc[j];
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = fmaf(pj, f[i], acc[i]);
      }
    }
    __syncthreads();                                    // (the next chunk overwrites sc and red)
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) part[tid * 8 + i] = acc[i];
  __syncthreads();
  const float inv = 1.f / (l_run + (sink ? expf(-m_run) : 0.f));
  for (int c = tid; c < Dv; c += 256) {
    float o = 0.f;
    for (int pp = 0; pp < nparts; ++pp) o += part[(pp * ngroups + c / 8) * 8 + (c & 7)];
    o *= inv;
    if (gate) o *= 1.f / (1.f + expf(-ld_f(gate + t * ldgate + (gate_head ? (long)h : (long)h * Dv + c))));
    st_f(out + t * ldo + (long)h * Dv + c, o);
  }
}

}  // namespace

static int headnorm_launch(const vlm_headnorm_args* a, int rows, int dtype, void* stream) {
  if (!a || !a->x || !a->tok_pos || !a->out || a->heads <= 0 || a->D <= 0 || a->rot_dims < 0 || a->rot_dims > a->D || (a->rot_dims & 1) ||
      (a->rot_dims && !a->inv_freq) || a->ldx < (long)a->heads * a->D || rows < 0 || (a->block_table && (!a->tok_seq || a->max_pages <= 0)) ||
      (a->raw_pool && (!a->block_table || !a->raw || a->Draw <= 0 || a->ldraw < (long)a->heads * a->Draw)) || (a->raw_bias && !a->raw_pool))
    return VLM_ERR_ARG;
  if (rows == 0) return VLM_OK;
  if (a->heads > 65535) return VLM_ERR_SHAPE;
  hipStream_t st = (hipStream_t)stream;
  if (dtype)
    hipLaunchKernelGGL(headnorm_rope_kernel<float>, dim3(rows, a->heads), dim3(64), 0, st, (const float*)a->x, a->ldx, a->D,
                       (const float*)a->bias, (const float*)a->w, a->norm, a->eps, a->rot_dims, a->inv_freq, a->temp_coef, a->temp_every,
                       a->tok_pos, a->tok_seq, a->block_table, a->max_pages, a->out, (const float*)a->raw, a->ldraw, a->Draw,
                       (const float*)a->raw_bias, (float*)a->raw_pool, a->rot_half);
  else
    hipLaunchKernelGGL(headnorm_rope_kernel<bf16_t>, dim3(rows, a->heads), dim3(64), 0, st, (const bf16_t*)a->x, a->ldx, a->D,
                       (const bf16_t*)a->bias, (const bf16_t*)a->w, a->norm, a->eps, a->rot_dims, a->inv_freq, a->temp_coef, a->temp_every,
                       a->tok_pos, a->tok_seq, a->block_table, a->max_pages, a->out, (const bf16_t*)a->raw, a->ldraw, a->Draw,
                       (const bf16_t*)a->raw_bias, (bf16_t*)a->raw_pool, a->rot_half);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_headnorm_rows(const vlm_headnorm_args* a, int rows, int dtype, void* stream) {
  return headnorm_launch(a, rows, dtype, stream);
}

extern "C" int vlm_headnorm_rope_rows(const void* x, long ldx, int heads, int D, const void* w, float eps, int rot_dims,
                                      const void* inv_freq, const void* tok_pos, const void* tok_seq, const void* block_table,
                                      int max_pages, void* out, void* raw_pool, int rows, int dtype, void* stream) {
  vlm_headnorm_args a = {};
  a.x = x; a.ldx = ldx; a.heads = heads; a.D = D; a.w = w; a.norm = w != nullptr; a.eps = eps; a.rot_dims = rot_dims;
  a.inv_freq = (const float*)inv_freq; a.tok_pos = (const int*)tok_pos; a.tok_seq = (const int*)tok_seq;
  a.block_table = (const int*)block_table; a.max_pages = max_pages; a.out = (float*)out;
  if (raw_pool) { a.raw = x; a.ldraw = ldx; a.Draw = D; a.raw_pool = raw_pool; }       // the rows as they came
  return headnorm_launch(&a, rows, dtype, stream);
}

#define WINDOW_ARGS_BAD                                                                                                             \
  (!q || !kpool || !vpool || !tok_seq || !tok_pos || !block_table || !out || H <= 0 || KH <= 0 || H % KH || D <= 0 || Dv <= 0 ||      \
   max_pages <= 0 || (gate && ldgate < (gate_head ? (long)H : (long)H * Dv)) || ldo < (long)H * Dv || !(cap >= 0.f))

extern "C" int vlm_window_attn_blocks(const void* q, const void* kpool, const void* vpool, const void* qb_start, const void* qb_count,
                                      int nblocks, const void* tok_seq, const void* tok_pos, const void* block_table, int max_pages,
                                      int H, int KH, int D, int Dv, float scale, const void* temp, int window, float cap, int sink,
                                      const void* gate, long ldgate, int gate_head, void* out, long ldo, int dtype, void* stream) {
  if (WINDOW_ARGS_BAD || !qb_start || !qb_count || nblocks < 0) return VLM_ERR_ARG;
  if (nblocks == 0) return VLM_OK;
  const int nacc = (Dv + 15) / 16 <= 4 ? 4 : ((Dv + 15) / 16 <= 8 ? 8 : 16);
  const int DP = (D + 3) & ~3;
  const size_t lds = ((size_t)QB * DP + (size_t)KT * (DP + 4) + (size_t)KT * nacc * 16 + QB * (KT + 1) + 3 * QB) * sizeof(float);
  if (Dv > 256 || H > 65535 || lds > 48 * 1024) return VLM_ERR_SHAPE;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid(nblocks, H);
#define GO(T, N)                                                                                                                    \
  hipLaunchKernelGGL((window_attn_block_kernel<T, N>), grid, dim3(256), lds, st, (const float*)q, (const float*)kpool, (const T*)vpool, \
                     (const int*)qb_start, (const int*)qb_count, (const int*)tok_seq, (const int*)tok_pos, (const int*)block_table,  \
                     max_pages, H, KH, D, Dv, scale, (const T*)temp, window, cap, sink, (const T*)gate, ldgate, gate_head, (T*)out, ldo)
  if (dtype) {
    if (nacc == 4) GO(float, 4); else if (nacc == 8) GO(float, 8); else GO(float, 16);
  } else {
    if (nacc == 4) GO(bf16_t, 4); else if (nacc == 8) GO(bf16_t, 8); else GO(bf16_t, 16);
  }
#undef GO
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_window_attn_rows(const void* q, const void* kpool, const void* vpool, const void* tok_seq, const void* tok_pos,
                                    const void* block_table, int max_pages, int H, int KH, int D, int Dv, float scale,
                                    const void* temp, int window, float cap, int sink, const void* gate, long ldgate, int gate_head,
                                    void* out, long ldo, int rows, int dtype, void* stream) {
  if (WINDOW_ARGS_BAD || rows < 0) return VLM_ERR_ARG;
  if (rows == 0) return VLM_OK;
  if (Dv > 1024 || D > 8192 || H > 65535) return VLM_ERR_SHAPE;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid(rows, H);
  if (D % 4 == 0 && Dv % 8 == 0 && Dv <= 2048 && (size_t)(D + 2 * KC + 2048) * sizeof(float) <= 48 * 1024) {
    const size_t ldsv = (size_t)(D + 2 * KC + 2048) * sizeof(float);
    if (dtype)
      hipLaunchKernelGGL(window_attn_row_vec_kernel<float>, grid, dim3(256), ldsv, st, (const float*)q, (const float*)kpool,
                         (const float*)vpool, (const int*)tok_seq, (const int*)tok_pos, (const int*)block_table, max_pages, H, KH, D, Dv,
                         scale, (const float*)temp, window, cap, sink, (const float*)gate, ldgate, gate_head, (float*)out, ldo);
    else
      hipLaunchKernelGGL(window_attn_row_vec_kernel<bf16_t>, grid, dim3(256), ldsv, st, (const float*)q, (const float*)kpool,
                         (const bf16_t*)vpool, (const int*)tok_seq, (const int*)tok_pos, (const int*)block_table, max_pages, H, KH, D,
                         Dv, scale, (const bf16_t*)temp, window, cap, sink, (const bf16_t*)gate, ldgate, gate_head, (bf16_t*)out, ldo);
    VLM_CHECK_LAUNCH();
    return VLM_OK;
  }
  const size_t lds = (size_t)(((D + 3) & ~3) + 256 + 8) * sizeof(float);
#define GO(T, N)                                                                                                                    \
  hipLaunchKernelGGL((window_attn_row_kernel<T, N>), grid, dim3(256), lds, st, (const float*)q, (const float*)kpool, (const T*)vpool, \
                     (const int*)tok_seq, (const int*)tok_pos, (const int*)block_table, max_pages, H, KH, D, Dv, scale,              \
                     (const T*)temp, window, cap, sink, (const T*)gate, ldgate, gate_head, (T*)out, ldo)
  const int nacc = (Dv + 255) / 256;
  if (dtype) {
    if (nacc == 1) GO(float, 1); else if (nacc == 2) GO(float, 2); else GO(float, 4);
  } else {
    if (nacc == 1) GO(bf16_t, 1); else if (nacc == 2) GO(bf16_t, 2); else GO(bf16_t, 4);
  }
#undef GO
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}
