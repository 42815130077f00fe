// Latent attention: every head reads ONE cached row per token - a low-rank latent c [R] (RMS-normed with a weight) and one
// rotated key part kr [Dr] shared by all heads.  Per-head keys and values are linear maps of c (k_h = U_k,h c, v_h = U_v,h c),
// so the maps are moved to the query and output side ("absorbed"): with q'_h = U_k,h^T q_h the score of key j is
//
//     s_hj = scale * (q'_h . c_j + rope(q_rot,h) . kr_j)          o_h = U_v,h sum_j softmax(s_h)_j c_j
//
// and attention runs straight over the cached rows [c | kr] with "head dim" R + Dr for scores and R for values; nothing
// per head is ever cached or materialised per key.  A layer may read ANOTHER layer's cache (same R, Dr, rotation).
//
//   vlm_latent_kv_write      d = W_dkv h rows -> c = d[:R] * rsqrt(mean(d[:R]^2) + eps) * w, kr = rope(d[R:], pos) into the
//                            paged pool [page][64][R + Dr] (T-typed) of the token's sequence
//   vlm_rope_pairs_rows      rotate the Dr-wide rotary part of every head's query into the fp32 query buffer behind the
//                            absorbed part
//                            (both: pairs (2 i, 2 i + 1), or with rot_half the pairs (i, i + Dr / 2))
//   vlm_latent_attn          causal softmax attention of fp32 queries [T][H][R + Dr] over the pool, one workgroup per (token,
//                            head); output fp32 [T][H][R], times sigmoid(gate[t][h]) when a gate is given.  Rows of whole
//                            16-byte pieces ((R + Dr) % 8 == 0, R % 8 == 0) are read with 16-byte loads, four lanes to a key;
//                            other shapes take one key per lane in tiles of 256 keys at multiples of 256 counted from the
//                            sequence's first token
// A sliding window (window > 0) limits query i to the keys j with 0 <= i - j < window; tiles still sit at multiples of their
// size counted from the sequence's first token and start at the tile that holds the window's edge.
// Scores, softmax and the weighted sum are fp32.  dtype: 0 = bf16, 1 = fp32 for the T-typed pointers.
#include "common.hpp"
#include "../../include/vlm_hip.h"

namespace {

template <typename T> __device__ __forceinline__ float ld_f(const T* p);
template <> __device__ __forceinline__ float ld_f<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ld_f<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void st_f(T* p, float v);
template <> __device__ __forceinline__ void st_f<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void st_f<bf16_t>(bf16_t* p, float v) { *p = f2bf(v); }

constexpr int PAGE = 64;

template <typename T>
__global__ __launch_bounds__(256) void latent_kv_write_kernel(const T* __restrict__ d, long ldd, const T* __restrict__ w, int R, int Dr,
                                                              const float* __restrict__ inv_freq, const int* __restrict__ tok_seq,
                                                              const int* __restrict__ tok_pos, const int* __restrict__ block_table,
                                                              int max_pages, T* __restrict__ pool, float eps, int rot_half) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  const T* row = d + t * ldd;
  const int pos = tok_pos[t];
  const int page = block_table[(long)tok_seq[t] * max_pages + pos / PAGE];
  T* dst = pool + ((long)page * PAGE + pos % PAGE) * (R + Dr);
  float q = 0.f;
  for (int i = threadIdx.x; i < R; i += 256) {
    const float v = ld_f(row + i);
    q += v * v;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) q += __shfl_xor(q, o);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = q;
  __syncthreads();
  const float r = 1.0f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)R + eps);
  for (int i = threadIdx.x; i < R; i += 256) st_f(dst + i, ld_f(row + i) * r * ld_f(w + i));
  for (int i = threadIdx.x; i < Dr / 2; i += 256) {
    const int i0 = rot_half ? i : 2 * i, i1 = rot_half ? i + Dr / 2 : 2 * i + 1;
    const float u = ld_f(row + R + i0), v = ld_f(row + R + i1);
    float sn, cs;
    sincosf((float)pos * inv_freq[i], &sn, &cs);
    st_f(dst + R + i0, u * cs - v * sn);
    st_f(dst + R + i1, v * cs + u * sn);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void rope_pairs_rows_kernel(const T* __restrict__ q, long ldq, long head_stride, int H, int Dr,
                                                              const float* __restrict__ inv_freq, const int* __restrict__ tok_pos,
                                                              float* __restrict__ out, long ldo, long out_head_stride, int rows,
                                                              int rot_half) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  const int hp = Dr / 2;
  if (i >= (long)rows * H * hp) return;
  const int pi = (int)(i % hp), h = (int)((i / hp) % H);
  const long t = i / ((long)hp * H);
  const T* src = q + t * ldq + (long)h * head_stride;
  const int i0 = rot_half ? pi : 2 * pi, i1 = rot_half ? pi + hp : 2 * pi + 1;
  const float u = ld_f(src + i0), v = ld_f(src + i1);
  float sn, cs;
  sincosf((float)tok_pos[t] * inv_freq[pi], &sn, &cs);
  float* dst = out + t * ldo + (long)h * out_head_stride;
  dst[i0] = u * cs - v * sn;
  dst[i1] = v * cs + u * sn;
}

// workgroup = (token, head): one key per lane and tile for the scores, one value dimension per lane for the weighted sum
template <typename T, int NACC>
__global__ __launch_bounds__(256) void latent_attn_kernel(const float* __restrict__ q, const T* __restrict__ pool,
                                                          const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
                                                          const int* __restrict__ block_table, int max_pages, int H, int R, int Dr,
                                                          float scale, int window, const T* __restrict__ gate, long ldgate,
                                                          float* __restrict__ out) {
  extern __shared__ float smem[];
  const int Dk = R + Dr;
  float* qs = smem;              // [Dk]
  float* ps = qs + Dk;           // [256]
  float* red = ps + 256;         // [8]
  const long t = blockIdx.x;
  const int h = blockIdx.y, tid = threadIdx.x;
  const int pos = tok_pos[t];
  const int* bt = block_table + (long)tok_seq[t] * max_pages;
  for (int i = tid; i < Dk; i += 256) qs[i] = q[(t * H + h) * Dk + i];
  __syncthreads();
  float m_run = -INFINITY, l_run = 0.f;
  float acc[NACC];
#pragma unroll
  for (int a = 0; a < NACC; ++a) acc[a] = 0.f;
  const int nkeys = pos + 1;
  const int first = window > 0 ? max(0, pos - window + 1) : 0;          // the oldest visible key
  for (int j0 = (first / 256) * 256; j0 < nkeys; j0 += 256) {
    const int j = j0 + tid;
    float s = -INFINITY;
    if (j < nkeys && j >= first) {
      const T* kr = pool + ((long)bt[j / PAGE] * PAGE + j % PAGE) * Dk;
      float d = 0.f;
      for (int i = 0; i < Dk; ++i) d = fmaf(qs[i], ld_f(kr + i), d);
      s = d * scale;
    }
    float mx = s;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    if ((tid & 63) == 0) red[tid >> 6] = mx;
    __syncthreads();
    const float m_new = fmaxf(m_run, fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3])));
    const float pj = (j < nkeys && j >= first) ? expf(s - m_new) : 0.f;
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
      if (dcol < R) {
        float v = acc[a] * alpha;
        for (int jj = max(0, first - j0); jj < nk; ++jj) {
          const int key = j0 + jj;
          v = fmaf(ps[jj], ld_f(pool + ((long)bt[key / PAGE] * PAGE + key % PAGE) * Dk + dcol), v);
        }
        acc[a] = v;
      }
    }
    __syncthreads();
  }
  float gsc = 1.f / l_run;
  if (gate) gsc *= 1.f / (1.f + expf(-ld_f(gate + t * ldgate + h)));
#pragma unroll
  for (int a = 0; a < NACC; ++a) {
    const int dcol = tid + a * 256;
    if (dcol < R) out[(t * H + h) * R + dcol] = acc[a] * gsc;
  }
}

// Prompt form: workgroup = (block of up to QB consecutive query tokens of one sequence, head).  Key tiles of KT cached rows are
// staged through LDS once for all queries of the block; tile j covers keys [KT j, KT j + KT) counted from the sequence's first
// token, and every query runs the same per-tile update in the same order whatever block it sits in (a tile that holds no
// visible key for a query leaves its running maximum, sum and accumulator untouched bit for bit), so a token's result does
// not depend on how the prompt was cut or batched.
constexpr int QB = 16, KT = 16;

__device__ __forceinline__ void load8(const bf16_t* p, float* f) {
  const uint4 v = *reinterpret_cast<const uint4*>(p);
  f[0] = bf_lo(v.x); f[1] = bf_hi(v.x); f[2] = bf_lo(v.y); f[3] = bf_hi(v.y);
  f[4] = bf_lo(v.z); f[5] = bf_hi(v.z); f[6] = bf_lo(v.w); f[7] = bf_hi(v.w);
}
__device__ __forceinline__ void load8(const float* p, float* f) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
}

// DP: the row pitch of q and k in LDS, Dk rounded up to 8 (+ 4 for the key rows: 16-byte aligned rows whose 16 starts
// spread over the banks); the pad columns hold zeros, so the 4-wide dot product runs over them
template <typename T, int NACC>
__global__ __launch_bounds__(256) void latent_attn_block_kernel(const float* __restrict__ q, const T* __restrict__ pool,
                                                                const int* __restrict__ qb_start, const int* __restrict__ qb_count,
                                                                const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
                                                                const int* __restrict__ block_table, int max_pages, int H, int R,
                                                                int Dr, float scale, int window, const T* __restrict__ gate,
                                                                long ldgate, float* __restrict__ out) {
  extern __shared__ float smem[];
  const int Dk = R + Dr, DP = (Dk + 7) & ~7, KP = DP + 4;
  float* qs = smem;                         // [QB][DP]
  float* ks = qs + QB * DP;                 // [KT][KP]
  float* ps = ks + KT * KP;                 // [KT][QB]   (key-major: the weighted sum reads the 16 weights of a key as 4 x float4)
  float* mrun = ps + QB * KT;               // [QB]
  float* lrun = mrun + QB;                  // [QB]
  float* alph = lrun + QB;                  // [QB]
  const int t0 = qb_start[blockIdx.x], nq = qb_count[blockIdx.x];
  const int h = blockIdx.y, tid = threadIdx.x;
  const int* bt = block_table + (long)tok_seq[t0] * max_pages;
  const int pos0 = tok_pos[t0];             // positions of the block's queries: pos0 .. pos0 + nq - 1
  const int r16 = tid >> 4, l16 = tid & 15; // (row of a 16-row tile, lane within the row's 16 lanes)
  for (int d = l16; d < DP; d += 16) qs[r16 * DP + d] = (r16 < nq && d < Dk) ? q[((long)(t0 + r16) * H + h) * Dk + d] : 0.f;
  if (tid < QB) {
    mrun[tid] = -INFINITY;
    lrun[tid] = 0.f;
  }
  float acc[QB][NACC];
#pragma unroll
  for (int a = 0; a < QB; ++a)
#pragma unroll
    for (int b = 0; b < NACC; ++b) acc[a][b] = 0.f;
  const int nkeys = pos0 + nq;              // the last query sees keys 0 .. pos0 + nq - 1
  const bool vec = (Dk & 7) == 0;           // rows of the pool are 16-byte aligned and a whole number of 8-element groups
  const int first = window > 0 ? max(0, pos0 - window + 1) : 0;        // the first query's oldest visible key
  for (int j0 = (first / KT) * KT; j0 < nkeys; j0 += KT) {
    __syncthreads();                        // (qs / state initialised; the previous tile's ks and ps are no longer read)
    {
      const int key = j0 + r16;
      float* dst = ks + r16 * KP;
      if (key < nkeys) {
        const T* src = pool + ((long)bt[key / PAGE] * PAGE + key % PAGE) * Dk;
        if (vec) {
          for (int d = l16 * 8; d < Dk; d += 128) {
            float f[8];
            load8(src + d, f);
            *reinterpret_cast<float4*>(dst + d) = make_float4(f[0], f[1], f[2], f[3]);
            *reinterpret_cast<float4*>(dst + d + 4) = make_float4(f[4], f[5], f[6], f[7]);
          }
        } else {
          for (int d = l16; d < DP; d += 16) dst[d] = d < Dk ? ld_f(src + d) : 0.f;
        }
      } else {
        for (int d = l16; d < DP; d += 16) dst[d] = 0.f;
      }
    }
    __syncthreads();
    {
      // one (query r16, key l16) pair per lane, four dimensions per LDS read, ascending - a fixed order per pair
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
      ps[l16 * QB + r16] = seen ? d * scale : -INFINITY;
    }
    __syncthreads();
    if (tid < QB) {                         // per query: running maximum, tile weights, running sum (fixed order over the tile)
      float sc[KT];
#pragma unroll
      for (int k = 0; k < KT; ++k) sc[k] = ps[k * QB + tid];
      float mt = sc[0];
#pragma unroll
      for (int k = 1; k < KT; ++k) mt = fmaxf(mt, sc[k]);
      const float m_old = mrun[tid], m_new = fmaxf(m_old, mt);
      float sum = 0.f;
#pragma unroll
      for (int k = 0; k < KT; ++k) {
        const float pv = sc[k] == -INFINITY ? 0.f : expf(sc[k] - m_new);
        ps[k * QB + tid] = pv;
        sum += pv;
      }
      const float al = m_new == -INFINITY || m_old == m_new ? 1.f : expf(m_old - m_new);
      alph[tid] = al;
      lrun[tid] = lrun[tid] * al + sum;
      mrun[tid] = m_new;
    }
    __syncthreads();
#pragma unroll
    for (int a = 0; a < QB; ++a) {
      const float al = alph[a];
#pragma unroll
      for (int b = 0; b < NACC; ++b) acc[a][b] *= al;
    }
#pragma unroll 2
    for (int k = 0; k < KT; ++k) {
      float c[NACC];
#pragma unroll
      for (int b = 0; b < NACC; ++b) c[b] = tid + 256 * b < R ? ks[k * KP + tid + 256 * b] : 0.f;
      const float4* pk = reinterpret_cast<const float4*>(ps + k * QB);
#pragma unroll
      for (int a4 = 0; a4 < QB / 4; ++a4) {
        const float4 pv = pk[a4];
#pragma unroll
        for (int b = 0; b < NACC; ++b) {
          acc[4 * a4 + 0][b] = fmaf(pv.x, c[b], acc[4 * a4 + 0][b]);
          acc[4 * a4 + 1][b] = fmaf(pv.y, c[b], acc[4 * a4 + 1][b]);
          acc[4 * a4 + 2][b] = fmaf(pv.z, c[b], acc[4 * a4 + 2][b]);
          acc[4 * a4 + 3][b] = fmaf(pv.w, c[b], acc[4 * a4 + 3][b]);
        }
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int a = 0; a < QB; ++a) {
    if (a >= nq) break;
    float gsc = 1.f / lrun[a];
    if (gate) gsc *= 1.f / (1.f + expf(-ld_f(gate + (long)(t0 + a) * ldgate + h)));
#pragma unroll
    for (int b = 0; b < NACC; ++b)
      if (tid + 256 * b < R) out[((long)(t0 + a) * H + h) * R + tid + 256 * b] = acc[a][b] * gsc;
  }
}

// Decode form for (R + Dr) % 8 == 0 and R % 8 == 0: workgroup = (token, head), the visible keys in chunks of KC rows from the
// window's edge (or the sequence's first token).
//   scores : thread (key, quarter): the four lanes of a DPP quad read one cached row in 16-byte pieces (lane q takes pieces q,
//            q + 4, ...) and add their partial dot products; 64 keys per pass, no barrier between passes;
//   softmax: chunk maximum and sum over the scores in LDS (online across chunks);
//   values : thread (group of 8 latent columns, key part): 16-byte loads of the rows' first R columns, a wave covers whole
//            rows; the key parts' partial sums are added through LDS at the end.
constexpr int KC = 1024;
template <typename T>
__global__ __launch_bounds__(256) void latent_attn_row_vec_kernel(const float* __restrict__ q, const T* __restrict__ pool,
                                                                  const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
                                                                  const int* __restrict__ block_table, int max_pages, int H, int R,
                                                                  int Dr, float scale, int window, const T* __restrict__ gate,
                                                                  long ldgate, float* __restrict__ out) {
  extern __shared__ __align__(16) float smem[];
  const int Dk = R + Dr;
  float* qs = smem;                  // [Dk]
  float* sc = qs + Dk;               // [KC] scores, then weights
  float* part = sc + KC;             // [256 * 8] partial weighted sums
  int* rowi = reinterpret_cast<int*>(part + 2048);   // [KC] the chunk's keys as pool rows (page * 64 + place): one table lookup per key
  __shared__ float red[8];
  const long t = blockIdx.x;
  const int h = blockIdx.y, tid = threadIdx.x, wave = tid >> 6;
  const int pos = tok_pos[t];
  const int* bt = block_table + (long)tok_seq[t] * max_pages;
  for (int i = tid; i < Dk; i += 256) qs[i] = q[(t * H + h) * Dk + i];
  const int ngroups = R / 8, nparts = 256 / ngroups;           // latent-column groups, key parts
  const int dg = tid % ngroups, kp = tid / ngroups;
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  const int nkeys = pos + 1;
  const int first = window > 0 ? max(0, pos - window + 1) : 0;
  const int D8 = Dk / 8;
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
        const T* kr = pool + (long)rowi[j] * Dk;
        for (int c = qp; c < D8; c += 4) {
          float f[8];
          load8(kr + c * 8, f);
          const float4 a = *reinterpret_cast<const float4*>(qs + c * 8), b = *reinterpret_cast<const float4*>(qs + c * 8 + 4);
          d = fmaf(a.x, f[0], d);
          d = fmaf(a.y, f[1], d);
          d = fmaf(a.z, f[2], d);
          d = fmaf(a.w, f[3], d);
          d = fmaf(b.x, f[4], d);
          d = fmaf(b.y, f[5], d);
          d = fmaf(b.z, f[6], d);
          d = fmaf(b.w, f[7], d);
        }
      }
      d += vlm_dpp<0xB1, 0xf>(0.f, d);     // quad_perm [1,0,3,2]
      d += vlm_dpp<0x4E, 0xf>(0.f, d);     // quad_perm [2,3,0,1]
      if (qp == 0 && j < nk) sc[j] = d * scale;
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
        load8(pool + (long)rowi[j] * Dk + dg * 8, f);
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
  float gsc = 1.f / l_run;
  if (gate) gsc *= 1.f / (1.f + expf(-ld_f(gate + t * ldgate + h)));
  for (int c = tid; c < R; c += 256) {
    float o = 0.f;
    for (int pp = 0; pp < nparts; ++pp) o += part[(pp * ngroups + c / 8) * 8 + (c & 7)];
    out[(t * H + h) * R + c] = o * gsc;
  }
}

}  // namespace

extern "C" int vlm_latent_kv_write(const void* d, long ldd, const void* w, int R, int Dr, const void* inv_freq, const void* tok_seq,
                                   const void* tok_pos, const void* block_table, int max_pages, void* pool, float eps, int rot_half,
                                   int rows, int dtype, void* stream) {
  if (!d || !w || !tok_seq || !tok_pos || !block_table || !pool || R <= 0 || Dr < 0 || (Dr & 1) || (Dr && !inv_freq) ||
      ldd < R + Dr || max_pages <= 0 || rows < 0)
    return VLM_ERR_ARG;
  if (rows == 0) return VLM_OK;
  hipStream_t st = (hipStream_t)stream;
  if (dtype)
    hipLaunchKernelGGL(latent_kv_write_kernel<float>, dim3(rows), dim3(256), 0, st, (const float*)d, ldd, (const float*)w, R, Dr,
                       (const float*)inv_freq, (const int*)tok_seq, (const int*)tok_pos, (const int*)block_table, max_pages,
                       (float*)pool, eps, rot_half);
  else
    hipLaunchKernelGGL(latent_kv_write_kernel<bf16_t>, dim3(rows), dim3(256), 0, st, (const bf16_t*)d, ldd, (const bf16_t*)w, R, Dr,
                       (const float*)inv_freq, (const int*)tok_seq, (const int*)tok_pos, (const int*)block_table, max_pages,
                       (bf16_t*)pool, eps, rot_half);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_rope_pairs_rows(const void* q, long ldq, long head_stride, int H, int Dr, const void* inv_freq, const void* tok_pos,
                                   void* out, long ldo, long out_head_stride, int rot_half, int rows, int dtype, void* stream) {
  if (!q || !tok_pos || !out || H <= 0 || Dr < 0 || (Dr & 1) || (Dr && !inv_freq) || rows < 0) return VLM_ERR_ARG;
  if (rows == 0 || Dr == 0) return VLM_OK;
  hipStream_t st = (hipStream_t)stream;
  const unsigned nb = (unsigned)(((long)rows * H * (Dr / 2) + 255) / 256);
  if (dtype)
    hipLaunchKernelGGL(rope_pairs_rows_kernel<float>, dim3(nb), dim3(256), 0, st, (const float*)q, ldq, head_stride, H, Dr,
                       (const float*)inv_freq, (const int*)tok_pos, (float*)out, ldo, out_head_stride, rows, rot_half);
  else
    hipLaunchKernelGGL(rope_pairs_rows_kernel<bf16_t>, dim3(nb), dim3(256), 0, st, (const bf16_t*)q, ldq, head_stride, H, Dr,
                       (const float*)inv_freq, (const int*)tok_pos, (float*)out, ldo, out_head_stride, rows, rot_half);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_latent_attn(const void* q, const void* pool, const void* tok_seq, const void* tok_pos, const void* block_table,
                               int max_pages, int H, int R, int Dr, float scale, int window, const void* gate, long ldgate, void* out,
                               int rows, int dtype, void* stream) {
  if (!q || !pool || !tok_seq || !tok_pos || !block_table || !out || H <= 0 || R <= 0 || Dr < 0 || max_pages <= 0 || rows < 0 ||
      (gate && ldgate < H))
    return VLM_ERR_ARG;
  if (rows == 0) return VLM_OK;
  if (R > 1024 || H > 65535) return VLM_ERR_SHAPE;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid(rows, H);
  if ((R + Dr) % 8 == 0 && R % 8 == 0 && R / 8 <= 256) {
    const size_t ldsv = (size_t)(R + Dr + 2 * KC + 2048) * sizeof(float);
    if (dtype)
      hipLaunchKernelGGL(latent_attn_row_vec_kernel<float>, grid, dim3(256), ldsv, st, (const float*)q, (const float*)pool,
                         (const int*)tok_seq, (const int*)tok_pos, (const int*)block_table, max_pages, H, R, Dr, scale, window,
                         (const float*)gate, ldgate, (float*)out);
    else
      hipLaunchKernelGGL(latent_attn_row_vec_kernel<bf16_t>, grid, dim3(256), ldsv, st, (const float*)q, (const bf16_t*)pool,
                         (const int*)tok_seq, (const int*)tok_pos, (const int*)block_table, max_pages, H, R, Dr, scale, window,
                         (const bf16_t*)gate, ldgate, (float*)out);
    VLM_CHECK_LAUNCH();
    return VLM_OK;
  }
  const size_t lds = (size_t)(R + Dr + 256 + 8) * sizeof(float);
#define GO(T, N)                                                                                                                  \
  hipLaunchKernelGGL((latent_attn_kernel<T, N>), grid, dim3(256), lds, st, (const float*)q, (const T*)pool, (const int*)tok_seq,  \
                     (const int*)tok_pos, (const int*)block_table, max_pages, H, R, Dr, scale, window, (const T*)gate, ldgate, (float*)out)
  const int nacc = (R + 255) / 256;
  if (dtype) {
    if (nacc == 1) GO(float, 1); else if (nacc == 2) GO(float, 2); else GO(float, 4);
  } else {
    if (nacc == 1) GO(bf16_t, 1); else if (nacc == 2) GO(bf16_t, 2); else GO(bf16_t, 4);
  }
#undef GO
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_latent_attn_blocks(const void* q, const void* pool, const void* qb_start, const void* qb_count, int nblocks,
                                      const void* tok_seq, const void* tok_pos, const void* block_table, int max_pages, int H, int R,
                                      int Dr, float scale, int window, const void* gate, long ldgate, void* out, int dtype,
                                      void* stream) {
  if (!q || !pool || !qb_start || !qb_count || !tok_seq || !tok_pos || !block_table || !out || H <= 0 || R <= 0 || Dr < 0 ||
      max_pages <= 0 || nblocks < 0 || (gate && ldgate < H))
    return VLM_ERR_ARG;
  if (nblocks == 0) return VLM_OK;
  const int Dk = R + Dr;
  const int DP = (Dk + 7) & ~7;
  const size_t lds = ((size_t)QB * DP + (size_t)KT * (DP + 4) + QB * KT + 3 * QB) * sizeof(float);
  if (R > 512 || H > 65535 || lds > 150 * 1024) return VLM_ERR_SHAPE;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid(nblocks, H);
#define GO(T, N)                                                                                                                   \
  do {                                                                                                                             \
    if (lds > 48 * 1024) {                                                                                                         \
      hipError_t e = hipFuncSetAttribute((const void*)latent_attn_block_kernel<T, N>, hipFuncAttributeMaxDynamicSharedMemorySize,  \
                                         (int)lds);                                                                                \
      if (e != hipSuccess) return VLM_ERR_HIP + (int)e;                                                                            \
    }                                                                                                                              \
    hipLaunchKernelGGL((latent_attn_block_kernel<T, N>), grid, dim3(256), lds, st, (const float*)q, (const T*)pool,                \
                       (const int*)qb_start, (const int*)qb_count, (const int*)tok_seq, (const int*)tok_pos,                       \
                       (const int*)block_table, max_pages, H, R, Dr, scale, window, (const T*)gate, ldgate, (float*)out);          \
  } while (0)
  const int nacc = (R + 255) / 256;
  if (dtype) {
    if (nacc == 1) GO(float, 1); else GO(float, 2);
  } else {
    if (nacc == 1) GO(bf16_t, 1); else GO(bf16_t, 2);
  }
#undef GO
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}
