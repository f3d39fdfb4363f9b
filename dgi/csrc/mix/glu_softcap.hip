// dgi/csrc/mix/glu_softcap.hip — clamped sigmoid-GLU activation and logit scaling with a soft cap.
//
//   glu_clamped   act = g * sigmoid(alpha * g) * (u + 1),  g = min(gate, limit),
//                 u = clamp(up, -limit, limit), over the fused gate|up GEMM output [T, 2 I]
//                 (activation.hip's silu_mul for feed-forwards that bound both branches).
//   scale_softcap out = cap * tanh(logits * scale / cap) in fp32 (cap <= 0: out = logits * scale).
//
// Elementwise, one workgroup per row; fp32 math, one rounding on the way out.
#include "../common.h"

using namespace dgi;

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf16_to_f32(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<uint16_t>(uint16_t* p, float v) { *p = f32_to_bf16(v); }

template <typename T>
__global__ __launch_bounds__(256) void glu_clamped_kernel(const T* __restrict__ gu, int gu_stride, T* __restrict__ out,
                                                          int I, float limit, float alpha) {
  const T* g = gu + (size_t)blockIdx.y * gu_stride;
  T* o = out + (size_t)blockIdx.y * I;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= I) return;
  const float gv = fminf(ldf<T>(g + c), limit);
  const float uv = fminf(fmaxf(ldf<T>(g + I + c), -limit), limit);
  stf<T>(o + c, gv * (1.f / (1.f + expf(-alpha * gv))) * (uv + 1.f));
}

// CPT 16-byte chunks of gate and of up per thread, all loads issued before any math (memory-bound:
// bytes in flight per CU set the bandwidth); sigmoid through the hardware exp / rcp (absolute
// error below 2e-7).  I a multiple of 8 bf16 / 4 fp32, rows 16-byte aligned.
constexpr int CPT = 4;

template <typename T>
__global__ __launch_bounds__(256) void glu_clamped_vec_kernel(const T* __restrict__ gu, int gu_stride,
                                                              T* __restrict__ out, int I, float limit, float alpha) {
  constexpr int E = 16 / sizeof(T);
  const T* g = gu + (size_t)blockIdx.y * gu_stride;
  T* o = out + (size_t)blockIdx.y * I;
  const int c0 = (blockIdx.x * (256 * CPT) + threadIdx.x) * E;
  u32x4 a[CPT], b[CPT];
#pragma unroll
  for (int k = 0; k < CPT; ++k) {
    const int c = c0 + k * 256 * E;
    if (c < I) {
      a[k] = *reinterpret_cast<const u32x4*>(g + c);
      b[k] = *reinterpret_cast<const u32x4*>(g + I + c);
    }
  }
#pragma unroll
  for (int k = 0; k < CPT; ++k) {
    const int c = c0 + k * 256 * E;
    if (c >= I) continue;
    float gv[8], uv[8], ov[8];
    if constexpr (sizeof(T) == 2) {
      unpack8(a[k], gv);
      unpack8(b[k], uv);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        gv[j] = __uint_as_float(a[k][j]);
        uv[j] = __uint_as_float(b[k][j]);
      }
    }
#pragma unroll
    for (int j = 0; j < E; ++j) {
      const float x = fminf(gv[j], limit);
      const float u = fminf(fmaxf(uv[j], -limit), limit);
      ov[j] = x * __builtin_amdgcn_rcpf(1.f + __expf(-alpha * x)) * (u + 1.f);
    }
    u32x4 r;
    if constexpr (sizeof(T) == 2) {
      r = pack8(ov);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) r[j] = __float_as_uint(ov[j]);
    }
    *reinterpret_cast<u32x4*>(o + c) = r;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void scale_softcap_kernel(const T* __restrict__ x, int x_stride, float* __restrict__ out,
                                                            int V, float scale, float cap) {
  const T* r = x + (size_t)blockIdx.y * x_stride;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= V) return;
  const float v = ldf<T>(r + c) * scale;
  out[(size_t)blockIdx.y * V + c] = cap > 0.f ? cap * tanhf(v / cap) : v;
}

}  // namespace

extern "C" int dgi_glu_clamped(const void* gu, int gu_stride, void* out, int is_f32, int T, int I, float limit,
                               float alpha, hipStream_t s) {
  if (T == 0) return 0;
  if (T > 65535) return -3;
  const int E = is_f32 ? 4 : 8;
  if (I % E == 0 && gu_stride % E == 0 && ((uintptr_t)gu | (uintptr_t)out) % 16 == 0) {
    const dim3 vgrid((I / E + 256 * CPT - 1) / (256 * CPT), T);
    if (is_f32)
      glu_clamped_vec_kernel<float><<<vgrid, 256, 0, s>>>((const float*)gu, gu_stride, (float*)out, I, limit, alpha);
    else
      glu_clamped_vec_kernel<uint16_t><<<vgrid, 256, 0, s>>>((const uint16_t*)gu, gu_stride, (uint16_t*)out, I, limit, alpha);
    DGI_CHECK_LAUNCH();
    return 0;
  }
  const dim3 grid((I + 255) / 256, T);
  if (is_f32) glu_clamped_kernel<float><<<grid, 256, 0, s>>>((const float*)gu, gu_stride, (float*)out, I, limit, alpha);
  else glu_clamped_kernel<uint16_t><<<grid, 256, 0, s>>>((const uint16_t*)gu, gu_stride, (uint16_t*)out, I, limit, alpha);
  DGI_CHECK_LAUNCH();
  return 0;
}

extern "C" int dgi_scale_softcap(const void* x, int x_stride, float* out, int is_f32, int T, int V, float scale,
                                 float cap, hipStream_t s) {
  if (T == 0) return 0;
  if (T > 65535) return -3;
  const dim3 grid((V + 255) / 256, T);
  if (is_f32) scale_softcap_kernel<float><<<grid, 256, 0, s>>>((const float*)x, x_stride, out, V, scale, cap);
  else scale_softcap_kernel<uint16_t><<<grid, 256, 0, s>>>((const uint16_t*)x, x_stride, out, V, scale, cap);
  DGI_CHECK_LAUNCH();
  return 0;
}
