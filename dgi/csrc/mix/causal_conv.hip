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

// Four channels per thread: 16-byte (fp32) / 8-byte (bf16) row accesses and the thread's 4 x taps
// weights as contiguous 16-byte loads.  Same arithmetic per channel.
template <typename T> __device__ __forceinline__ void ld4(const T* p, float* f);
template <> __device__ __forceinline__ void ld4<float>(const float* p, float* f) {
  const float4 v = *reinterpret_cast<const float4*>(p);
  f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
}
template <> __device__ __forceinline__ void ld4<uint16_t>(const uint16_t* p, float* f) {
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
  f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
}
template <typename T> __device__ __forceinline__ void st4(T* p, const float* f);
template <> __device__ __forceinline__ void st4<float>(float* p, const float* f) {
  *reinterpret_cast<float4*>(p) = make_float4(f[0], f[1], f[2], f[3]);
}
template <> __device__ __forceinline__ void st4<uint16_t>(uint16_t* p, const float* f) {
  *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]));
}

// A thread walks `rpw` consecutive rows with the last TAPS - 1 inputs of its channels in registers: inside a
// sequence's portion every input is read once (rows of a portion are consecutive positions); at the first row of
// the walk and wherever a new sequence starts the window is loaded afresh (rows of the step or the slot's tail).
template <typename TI, typename TO, int TAPS>
__global__ __launch_bounds__(256) void causal_conv_vec_kernel(
    TO* __restrict__ out, const TI* __restrict__ x, int x_stride, int T, int C, const float* __restrict__ w,
    const float* __restrict__ bias, const float* __restrict__ tail, const int* __restrict__ positions,
    const int* __restrict__ row_seq, const int* __restrict__ seq_row0, const int* __restrict__ seq_slots, int act,
    int residual, int rpw) {
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * 4;
  if (c >= C) return;
  float wv[4 * TAPS];
#pragma unroll
  for (int i = 0; i < TAPS; ++i) ld4<float>(w + (size_t)c * TAPS + 4 * i, wv + 4 * i);     // wv[ch * TAPS + j]
  float bv[4] = {0.f, 0.f, 0.f, 0.f};
  if (bias) ld4<float>(bias + c, bv);
  float win[TAPS][4];                                  // win[j]: input at position pos - (TAPS - 1) + j
  const int row_begin = blockIdx.x * rpw, row_end = min(T, row_begin + rpw);
  for (int row = row_begin; row < row_end; ++row) {
    const int seq = row_seq[row];
    const int r0 = seq_row0[seq];
    if (row == row_begin || row == r0) {               // load the older inputs
      const int pos = positions[row], p0 = positions[r0];
      const float* tl = tail ? tail + (size_t)seq_slots[seq] * (TAPS - 1) * C : nullptr;
#pragma unroll
      for (int j = 0; j < TAPS - 1; ++j) {
        const int pp = pos - (TAPS - 1) + j;
#pragma unroll
        for (int ch = 0; ch < 4; ++ch) win[j][ch] = 0.f;
        if (pp >= p0) ld4<TI>(x + (size_t)(r0 + pp - p0) * x_stride + c, win[j]);
        else if (pp >= 0) ld4<float>(tl + (size_t)(pp - (p0 - (TAPS - 1))) * C + c, win[j]);
      }
    } else {
#pragma unroll
      for (int j = 0; j < TAPS - 1; ++j)
#pragma unroll
        for (int ch = 0; ch < 4; ++ch) win[j][ch] = win[j + 1][ch];
    }
    ld4<TI>(x + (size_t)row * x_stride + c, win[TAPS - 1]);
    float acc[4];
#pragma unroll
    for (int ch = 0; ch < 4; ++ch) {
      float a = bv[ch];
#pragma unroll
      for (int j = 0; j < TAPS; ++j) a += wv[ch * TAPS + j] * win[j][ch];
      if (act == 1) a = a / (1.f + expf(-a));
      if (residual) a += win[TAPS - 1][ch];
      acc[ch] = a;
    }
    st4<TO>(out + (size_t)row * C + c, acc);
  }
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
  // vector path: channels in fours, rows and tables 16-byte aligned
  const bool vec = C % 4 == 0 && x_stride % 4 == 0 && taps >= 2 && taps <= 4 &&
                   (((uintptr_t)x | (uintptr_t)out | (uintptr_t)w | (uintptr_t)bias | (uintptr_t)tail) & 15) == 0;
  if (vec) {
    const int rpw = T >= 2048 ? 8 : 1;                 // rows per thread walk: large steps only (small ones need the workgroups)
    const dim3 vgrid((T + rpw - 1) / rpw, (C / 4 + 255) / 256);
#define DGI_CONVV(TI, TO, TP)                                                                                      \
  causal_conv_vec_kernel<TI, TO, TP><<<vgrid, 256, 0, s>>>((TO*)out, (const TI*)x, x_stride, T, C, w, bias, tail,  \
                                                          positions, row_seq, seq_row0, seq_slots, act, residual, rpw)
#define DGI_CONVT(TI, TO) \
  do { if (taps == 2) DGI_CONVV(TI, TO, 2); else if (taps == 3) DGI_CONVV(TI, TO, 3); else DGI_CONVV(TI, TO, 4); } while (0)
    if (x_f32 && out_f32) DGI_CONVT(float, float);
    else if (x_f32) DGI_CONVT(float, uint16_t);
    else if (out_f32) DGI_CONVT(uint16_t, float);
    else DGI_CONVT(uint16_t, uint16_t);
#undef DGI_CONVT
#undef DGI_CONVV
  } else {
#define DGI_CONV(TI, TO)                                                                                           \
  causal_conv_kernel<TI, TO><<<grid, 256, 0, s>>>((TO*)out, (const TI*)x, x_stride, C, taps, w, bias, tail, positions, \
                                                  row_seq, seq_row0, seq_slots, act, residual)
  if (x_f32 && out_f32) DGI_CONV(float, float);
  else if (x_f32) DGI_CONV(float, uint16_t);
  else if (out_f32) DGI_CONV(uint16_t, float);
  else DGI_CONV(uint16_t, uint16_t);
#undef DGI_CONV
  }
  DGI_CHECK_LAUNCH();
  if (taps > 1) {
    const dim3 g2(n_seq, (C + 255) / 256);
    if (x_f32) conv_tail_kernel<float><<<g2, 256, 0, s>>>(tail, (const float*)x, x_stride, C, taps, positions, seq_row0, seq_slots);
    else conv_tail_kernel<uint16_t><<<g2, 256, 0, s>>>(tail, (const uint16_t*)x, x_stride, C, taps, positions, seq_row0, seq_slots);
    DGI_CHECK_LAUNCH();
  }
  return 0;
}
