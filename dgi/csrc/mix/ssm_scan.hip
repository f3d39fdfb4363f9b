// dgi/csrc/mix/ssm_scan.hip — Mamba-2 selective scan over packed rows with the state in a slot, and
// the gated group RMS norm that follows it.
//
// Per sequence of the step and head h (group g = h / (heads / G)), for its rows in order:
//
//     dt  = softplus(dt_raw[t][h] + dt_bias[h])             a = exp(-exp(a_log[h]) * dt)
//     S  <- a * S + dt * B_t x_t^T                          S: [N, dv] fp32
//     y_t = S^T C_t + d_skip[h] * x_t
//
// S starts as state[slot][h] (zero when the portion starts at position 0) and goes back there after
// the last row; decode rows (one token) and prompt portions run the same code, so the result does
// not depend on how a prompt was cut.  x | B | C come as one fp32 row (the convolution's output).
//
// Work split: a workgroup owns (sequence, head, 16 value columns); thread (column v, n-lane l) keeps
// S[n][v] for n = l + 16 i in registers, so the y reduction over n is four shuffles inside a 16-lane
// group.  Everything is fp32 (softplus in its overflow-free form max(z, 0) + log1p(exp(-|z|))).
//
// gated_group_norm: g = y * silu(z), each of `groups` equal parts of a row divided by its own root
// mean square (eps inside the root), times w.
#include "../common.h"

using namespace dgi;

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf16_to_f32(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<uint16_t>(uint16_t* p, float v) { *p = f32_to_bf16(v); }

constexpr int COLS = 16;     // value columns per workgroup
constexpr int NL = 16;       // n-lanes per column

template <typename TD, int NPT>
__global__ __launch_bounds__(COLS * NL) void ssm_scan_kernel(
    float* __restrict__ y, const float* __restrict__ xbc, int xbc_stride, const TD* __restrict__ dt_raw, int dt_stride,
    const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ d_skip,
    float* __restrict__ state, const int* __restrict__ positions, const int* __restrict__ seq_row0,
    const int* __restrict__ seq_slots, int heads, int dv, int N, int G) {
  const int seq = blockIdx.x, h = blockIdx.y;
  const int l = threadIdx.x & (NL - 1);
  const int v = blockIdx.z * COLS + (threadIdx.x >> 4);
  const int r0 = seq_row0[seq], r1 = seq_row0[seq + 1];
  if (r1 <= r0) return;
  const bool vok = v < dv;
  const int g = h / (heads / G);
  const int inner = heads * dv;
  const float* bp = xbc + inner + (size_t)g * N;
  const float* cp = bp + (size_t)G * N;
  float* sp = state + (((size_t)seq_slots[seq] * heads + h) * N) * dv + v;
  float S[NPT];
  const bool fresh = positions[r0] == 0;
#pragma unroll
  for (int i = 0; i < NPT; ++i) {
    const int n = l + NL * i;
    S[i] = (!fresh && vok && n < N) ? sp[(size_t)n * dv] : 0.f;
  }
  const float na = -expf(a_log[h]), bias = dt_bias[h], dsk = d_skip[h];
  for (int t = r0; t < r1; ++t) {
    const float z = ldf<TD>(dt_raw + (size_t)t * dt_stride + h) + bias;
    const float dt = fmaxf(z, 0.f) + log1pf(expf(-fabsf(z)));
    const float a = expf(na * dt);
    const float* row = xbc + (size_t)t * xbc_stride;
    const float xv = vok ? row[(size_t)h * dv + v] : 0.f;
    const float dx = dt * xv;
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
      const int n = l + NL * i;
      if (n < N) {
        const float bn = bp[(size_t)t * xbc_stride + n], cn = cp[(size_t)t * xbc_stride + n];
        S[i] = a * S[i] + bn * dx;
        acc += S[i] * cn;
      }
    }
#pragma unroll
    for (int o = NL / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
    if (l == 0 && vok) y[(size_t)t * inner + (size_t)h * dv + v] = acc + dsk * xv;
  }
  if (vok) {
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
      const int n = l + NL * i;
      if (n < N) sp[(size_t)n * dv] = S[i];
    }
  }
}

template <typename TZ, typename TO>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(
    TO* __restrict__ out, const float* __restrict__ y, const TZ* __restrict__ z, int z_stride,
    const float* __restrict__ w, int C, int groups, float eps) {
  __shared__ float red[4];
  const int row = blockIdx.x, grp = blockIdx.y;
  const int gs = C / groups;
  const float* yp = y + (size_t)row * C + (size_t)grp * gs;
  const TZ* zp = z + (size_t)row * z_stride + (size_t)grp * gs;
  float ss = 0.f;
  for (int i = threadIdx.x; i < gs; i += 256) {
    const float zz = ldf<TZ>(zp + i);
    const float gv = yp[i] * zz / (1.f + expf(-zz));
    ss += gv * gv;
  }
  ss = wave_sum(ss);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float r = 1.f / sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)gs + eps);
  for (int i = threadIdx.x; i < gs; i += 256) {
    const float zz = ldf<TZ>(zp + i);
    const float gv = yp[i] * zz / (1.f + expf(-zz));
    stf<TO>(out + (size_t)row * C + (size_t)grp * gs + i, gv * r * w[(size_t)grp * gs + i]);
  }
}

}  // namespace

extern "C" int dgi_ssm_scan(float* y, const float* xbc, int xbc_stride, const void* dt_raw, int dt_f32, int dt_stride,
                            const float* dt_bias, const float* a_log, const float* d_skip, float* state,
                            const int* positions, const int* seq_row0, const int* seq_slots, int n_seq, int heads,
                            int dv, int N, int G, hipStream_t s) {
  if (n_seq == 0) return 0;
  if (G <= 0 || heads % G) return -2;
  if (N > NL * 16 || N <= 0 || dv <= 0) return -3;
  const dim3 grid(n_seq, heads, (dv + COLS - 1) / COLS);
  if (heads > 65535 || grid.z > 65535) return -4;
#define DGI_SCAN(TD, NPT)                                                                                            \
  ssm_scan_kernel<TD, NPT><<<grid, COLS * NL, 0, s>>>(y, xbc, xbc_stride, (const TD*)dt_raw, dt_stride, dt_bias, a_log, \
                                                      d_skip, state, positions, seq_row0, seq_slots, heads, dv, N, G)
  const int npt = (N + NL - 1) / NL;
  if (dt_f32) {
    if (npt <= 4) DGI_SCAN(float, 4); else if (npt <= 8) DGI_SCAN(float, 8); else DGI_SCAN(float, 16);
  } else {
    if (npt <= 4) DGI_SCAN(uint16_t, 4); else if (npt <= 8) DGI_SCAN(uint16_t, 8); else DGI_SCAN(uint16_t, 16);
  }
#undef DGI_SCAN
  DGI_CHECK_LAUNCH();
  return 0;
}

extern "C" int dgi_gated_group_norm(void* out, int out_f32, const float* y, const void* z, int z_f32, int z_stride,
                                    const float* w, int T, int C, int groups, float eps, hipStream_t s) {
  if (T == 0) return 0;
  if (groups <= 0 || C % groups || groups > 65535) return -2;
  const dim3 grid(T, groups);
  if (z_f32 && out_f32)
    gated_group_norm_kernel<float, float><<<grid, 256, 0, s>>>((float*)out, y, (const float*)z, z_stride, w, C, groups, eps);
  else if (!z_f32 && !out_f32)
    gated_group_norm_kernel<uint16_t, uint16_t><<<grid, 256, 0, s>>>((uint16_t*)out, y, (const uint16_t*)z, z_stride, w, C, groups, eps);
  else
    return -3;
  DGI_CHECK_LAUNCH();
  return 0;
}
