// dgi/csrc/mix/causal_conv.hip — per-channel causal convolution over time on packed rows, with the
// inputs older than the step kept per sequence in a state slot.
//
//   out[t][c] = f( bias[c] + sum_j w[c][j] * x[pos(t) - taps + 1 + j][c] )  (+ x[t][c] with `residual`)
//
// f = identity or SiLU; inputs at negative positions are zero.  A row's older inputs are either
// rows of the same step (same sequence, found through seq_row0) or, for positions before the
// portion, entries of tail[slot] = the sequence's last taps - 1 inputs (fp32).  The tail is brought
// up to date by a second kernel after every row has read the old one: a thread owns one channel,
// loads the taps - 1 new entries (from rows or from the old tail) into registers, then writes them.
// Position 0 is "no state yet": a portion that starts there never reads the slot, so slots need no
// clearing when they change hands.
//
// x may be a column slice of a wider row (its own row stride); math in fp32; out in fp32 or bf16.
#include "../common.h"

using namespace dgi;

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf16_to_f32(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<uint16_t>(uint16_t* p, float v) { *p = f32_to_bf16(v); }

constexpr int MAXTAPS = 8;

template <typename TI, typename TO>
__global__ __launch_bounds__(256) void causal_conv_kernel(
    TO* __restrict__ out, const TI* __restrict__ x, int x_stride, int C, int taps, const float* __restrict__ w,
    const float* __restrict__ bias, const float* __restrict__ tail, const int* __restrict__ positions,
    const int* __restrict__ row_seq, const int* __restrict__ seq_row0, const int* __restrict__ seq_slots, int act,
    int residual) {
  const int row = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int seq = row_seq[row];
  const int r0 = seq_row0[seq];
  const int pos = positions[row], p0 = positions[r0];
  const float* tl = tail ? tail + (size_t)seq_slots[seq] * (taps - 1) * C : nullptr;
  float acc = bias ? bias[c] : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int pp = pos - (taps - 1) + j;
    if (pp < 0) continue;
    float v;
    if (pp >= p0) v = ldf<TI>(x + (size_t)(r0 + pp - p0) * x_stride + c);
    else v = tl[(size_t)(pp - (p0 - (taps - 1))) * C + c];
    acc += w[(size_t)c * taps + j] * v;
  }
  if (act == 1) acc = acc / (1.f + expf(-acc));
  if (residual) acc += ldf<TI>(x + (size_t)row * x_stride + c);
  stf<TO>(out + (size_t)row * C + c, acc);
}

template <typename TI>
__global__ __launch_bounds__(256) void conv_tail_kernel(
    float* __restrict__ tail, const TI* __restrict__ x, int x_stride, int C, int taps, const int* __restrict__ positions,
    const int* __restrict__ seq_row0, const int* __restrict__ seq_slots) {
  const int seq = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int r0 = seq_row0[seq], n = seq_row0[seq + 1] - r0;
  if (n <= 0) return;
  const int p0 = positions[r0];
  float* tl = tail + (size_t)seq_slots[seq] * (taps - 1) * C;
  float nv[MAXTAPS];
#pragma unroll
  for (int k = 0; k < MAXTAPS; ++k) {
    nv[k] = 0.f;
    if (k < taps - 1) {
      const int pn = p0 + n - (taps - 1) + k;         // position held by entry k afterwards
      if (pn >= p0) nv[k] = ldf<TI>(x + (size_t)(r0 + pn - p0) * x_stride + c);
      else if (pn >= 0) nv[k] = tl[(size_t)(pn - (p0 - (taps - 1))) * C + c];
    }
  }
#pragma unroll
  for (int k = 0; k < MAXTAPS; ++k)
    if (k < taps - 1) tl[(size_t)k * C + c] = nv[k];
}

}  // namespace

extern "C" int dgi_causal_conv(void* out, int out_f32, const void* x, int x_f32, int x_stride, int T, int C, int taps,
                               const float* w, const float* bias, float* tail, const int* positions,
                               const int* row_seq, const int* seq_row0, const int* seq_slots, int n_seq, int act,
                               int residual, hipStream_t s) {
  if (T == 0) return 0;
  if (taps < 1 || taps > MAXTAPS) return -2;
  if (taps > 1 && !tail) return -3;
  const dim3 grid(T, (C + 255) / 256);
  if (grid.y > 65535) return -4;
#define DGI_CONV(TI, TO)                                                                                           \
  causal_conv_kernel<TI, TO><<<grid, 256, 0, s>>>((TO*)out, (const TI*)x, x_stride, C, taps, w, bias, tail, positions, \
                                                  row_seq, seq_row0, seq_slots, act, residual)
  if (x_f32 && out_f32) DGI_CONV(float, float);
  else if (x_f32) DGI_CONV(float, uint16_t);
  else if (out_f32) DGI_CONV(uint16_t, float);
  else DGI_CONV(uint16_t, uint16_t);
#undef DGI_CONV
  DGI_CHECK_LAUNCH();
  if (taps > 1) {
    const dim3 g2(n_seq, (C + 255) / 256);
    if (x_f32) conv_tail_kernel<float><<<g2, 256, 0, s>>>(tail, (const float*)x, x_stride, C, taps, positions, seq_row0, seq_slots);
    else conv_tail_kernel<uint16_t><<<g2, 256, 0, s>>>(tail, (const uint16_t*)x, x_stride, C, taps, positions, seq_row0, seq_slots);
    DGI_CHECK_LAUNCH();
  }
  return 0;
}
