// Short causal convolutions over time, one filter per channel, on the rows of a ragged step:
//
//     out[t][c] = (residual ? in[t][c] : 0) + bias[c] + sum_(j < taps) w[c][j] * in(t - taps + 1 + j)[c]        (then silu, act = 1)
//
// in(.) before the sequence's first token is zero.  A step brings any run of consecutive tokens of a sequence (a prompt, a
// portion, one decoded token): the taps - 1 inputs before the run live in the sequence's CARRY, fp32 [slots][taps - 1][C],
// oldest first, indexed by the same slot as the sequence's recurrent state.  A run that starts at position 0 never reads the
// carry (positions below 0 are zero by the position test), so a slot that is used again needs no clearing.
//
//   vlm_short_conv_rows    one thread per (token, channel); taps are summed oldest first with fp32 FMAs whatever the cut, so
//                          the bits of a token do not depend on how its prompt was cut
//   vlm_short_conv_carry   one thread per (segment, channel), launched after every token has read the old carry: the carry
//                          becomes the last taps - 1 inputs at the segment's end (kept entries of the old carry shift down)
// Input and output rows may each be fp32 or T: a convolution over normed fp32 rows that feeds a bf16 projection, or one over a
// projection's rows that feeds a recurrence.
#include "common.hpp"
#include "../../include/vlm_hip.h"
#include "recurrence_finish.hpp"

namespace {

constexpr int MAX_TAPS = 16;

template <typename T, typename TI, typename TO>
__global__ __launch_bounds__(256) void short_conv_rows_kernel(vlm_short_conv_args p, int ntok) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  const long t = blockIdx.y;
  if (c >= p.C) return;
  const int slot = p.tok_seq[t], pos = p.tok_pos[t], taps = p.taps;
  // how many of the taps - 1 tokens before t are rows of this step (segments are runs of consecutive tokens of one sequence)
  int nin = 0;
  while (nin < taps - 1 && t - nin - 1 >= 0 && p.tok_seq[t - nin - 1] == slot) ++nin;
  const TI* in = (const TI*)p.in;
  const T* w = (const T*)p.w + (long)c * taps;
  const float* carry = p.carry + (long)slot * (taps - 1) * p.C;
  const float cur = ld_f(in + t * p.ldin + c);
  float acc = p.bias ? ld_f((const T*)p.bias + c) : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int back = taps - 1 - j;                       // oldest first
    float v = 0.f;
    if (back == 0) v = cur;
    else if (pos - back >= 0) v = back <= nin ? ld_f(in + (t - back) * p.ldin + c) : carry[(long)(taps - 1 - (back - nin)) * p.C + c];
    acc = fmaf(ld_f(w + j), v, acc);
  }
  if (p.residual) acc += cur;
  if (p.act == 1) acc = acc / (1.f + expf(-acc));
  st_f((TO*)p.out + t * p.ldo + c, acc);
}

template <typename TI>
__global__ __launch_bounds__(256) void short_conv_carry_kernel(vlm_short_conv_args p, int nseg) {
  const int c = blockIdx.x * 256 + threadIdx.x, seg = blockIdx.y;
  if (c >= p.C) return;
  const int t0 = p.seg_start[seg], len = p.seg_start[seg + 1] - t0, pos0 = p.seg_pos0[seg], keep = p.taps - 1;
  float* carry = p.carry + (long)p.seg_slot[seg] * keep * p.C;
  const TI* in = (const TI*)p.in;
  float v[MAX_TAPS - 1];
#pragma unroll
  for (int i = 0; i < MAX_TAPS - 1; ++i) {
    if (i < keep) {
      const int r = len - keep + i;                      // the row of the segment that lands in entry i (negative: before the segment)
      const int pos = pos0 + r;
      v[i] = pos < 0 ? 0.f : (r >= 0 ? ld_f(in + (long)(t0 + r) * p.ldin + c) : carry[(long)(keep + r) * p.C + c]);
    }
  }
#pragma unroll
  for (int i = 0; i < MAX_TAPS - 1; ++i)
    if (i < keep) carry[(long)i * p.C + c] = v[i];
}

bool bad(const vlm_short_conv_args* a) {
  return !a || !a->in || !a->w || a->C <= 0 || a->taps < 1 || a->ldin < a->C || (a->taps > 1 && !a->carry) || a->act < 0 || a->act > 1;
}

}  // namespace

extern "C" int vlm_short_conv_rows(const vlm_short_conv_args* a, int ntok, int dtype, void* stream) {
  if (bad(a) || !a->out || a->ldo < a->C || !a->tok_seq || !a->tok_pos || ntok < 0) return VLM_ERR_ARG;
  if (a->taps > MAX_TAPS || ntok > 65535 * 16) return VLM_ERR_SHAPE;
  if (ntok == 0) return VLM_OK;
  dim3 grid((a->C + 255) / 256, ntok);
  hipStream_t st = (hipStream_t)stream;
#define GO(T, TI, TO) hipLaunchKernelGGL((short_conv_rows_kernel<T, TI, TO>), grid, dim3(256), 0, st, *a, ntok)
  if (dtype) GO(float, float, float);
  else if (a->in_f32 && a->out_f32) GO(bf16_t, float, float);
  else if (a->in_f32) GO(bf16_t, float, bf16_t);
  else if (a->out_f32) GO(bf16_t, bf16_t, float);
  else GO(bf16_t, bf16_t, bf16_t);
#undef GO
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}

extern "C" int vlm_short_conv_carry(const vlm_short_conv_args* a, int nseg, int dtype, void* stream) {
  if (bad(a) || !a->seg_start || !a->seg_slot || !a->seg_pos0 || nseg < 0) return VLM_ERR_ARG;
  if (a->taps > MAX_TAPS || nseg > 65535) return VLM_ERR_SHAPE;
  if (nseg == 0 || a->taps == 1) return VLM_OK;
  dim3 grid((a->C + 255) / 256, nseg);
  hipStream_t st = (hipStream_t)stream;
  if (dtype || a->in_f32) hipLaunchKernelGGL(short_conv_carry_kernel<float>, grid, dim3(256), 0, st, *a, nseg);
  else hipLaunchKernelGGL(short_conv_carry_kernel<bf16_t>, grid, dim3(256), 0, st, *a, nseg);
  VLM_CHECK_LAUNCH();
  return VLM_OK;
}
