// dgi/csrc/mix/dyt_norm.hip — Dynamic-Tanh normalisation of an fp32 residual stream.
//
// A Dynamic-Tanh norm computes no row statistics: y = tanh(alpha * x) * w + b with a learned
// scalar alpha and per-channel w, b.  The kernels here are the DyT counterparts of
// rmsnorm.hip's rmsnorm / fused_add_rmsnorm, for models that keep the residual stream in fp32:
//
//   dyt            y   = dyt_n(x)                                   (x fp32 -> y in the GEMM dtype)
//   dyt_add        res += dyt_a(h) * ls ;  y = dyt_n(res)            (sublayer output norm + layer
//                                                                    scale + residual add, fused
//                                                                    with the next sublayer's input
//                                                                    norm: one pass over the row)
//   embed_dyt      res = dyt_a(table[id] * scale)                    (token gather + embedding norm)
//
// Elementwise and memory-bound: one workgroup per row, fp32 math (the
// stream and every norm are kept in 32-bit also when the projections run in bf16).  Norm
// parameters are fp32; TA is the activation dtype (bf16 bit patterns or float).
#include "../common.h"

using namespace dgi;

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf16_to_f32(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<uint16_t>(uint16_t* p, float v) { *p = f32_to_bf16(v); }

// tanh(x) = sign(x) (1 - e) / (1 + e), e = exp(-2 |x|) in (0, 1]: the hardware exponential and
// reciprocal (absolute error below 2e-7, no overflow), a quarter of the instructions of the
// library tanhf — these kernels evaluate two tanh per element and were ALU-bound on it.
__device__ __forceinline__ float tanh_fast(float x) {
  const float e = __expf(-2.f * fabsf(x));
  return copysignf((1.f - e) * __builtin_amdgcn_rcpf(1.f + e), x);
}

struct DytParams {
  const float* alpha;   // [1]
  const float* w;       // [W]
  const float* b;       // [W]
};

// four consecutive elements per thread (W % 4 == 0: 16-byte fp32 / 8-byte bf16 accesses)
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
  uint2 v;
  v.x = pack_bf16x2(f[0], f[1]);
  v.y = pack_bf16x2(f[2], f[3]);
  *reinterpret_cast<uint2*>(p) = v;
}

template <typename TA, bool VEC>
__global__ __launch_bounds__(256) void dyt_kernel(const float* __restrict__ x, DytParams n, TA* __restrict__ y,
                                                  int W) {
  const size_t row = (size_t)blockIdx.x * W;
  const float a = n.alpha[0];
  if (VEC) {
    for (int c = threadIdx.x * 4; c < W; c += 1024) {
      float v[4], w[4], b[4], o[4];
      ld4<float>(x + row + c, v); ld4<float>(n.w + c, w); ld4<float>(n.b + c, b);
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = tanh_fast(a * v[j]) * w[j] + b[j];
      st4<TA>(y + row + c, o);
    }
  } else {
    for (int c = threadIdx.x; c < W; c += 256) stf<TA>(y + row + c, tanh_fast(a * x[row + c]) * n.w[c] + n.b[c]);
  }
}

// res += (tanh(a1 * h) * w1 + b1) * ls;  y = tanh(a2 * res) * w2 + b2 (when y != nullptr)
template <typename TA, bool VEC>
__global__ __launch_bounds__(256) void dyt_add_kernel(const TA* __restrict__ h, int h_stride, DytParams post,
                                                      const float* __restrict__ ls, float* __restrict__ res,
                                                      DytParams next, TA* __restrict__ y, int W) {
  const size_t row = (size_t)blockIdx.x * W;
  const TA* hr = h + (size_t)blockIdx.x * h_stride;
  const float a1 = post.alpha[0];
  const float a2 = y ? next.alpha[0] : 0.f;
  if (VEC) {
    for (int c = threadIdx.x * 4; c < W; c += 1024) {
      float hv[4], r[4], w[4], b[4], l[4];
      ld4<TA>(hr + c, hv); ld4<float>(res + row + c, r);
      ld4<float>(post.w + c, w); ld4<float>(post.b + c, b); ld4<float>(ls + c, l);
#pragma unroll
      for (int j = 0; j < 4; ++j) r[j] += (tanh_fast(a1 * hv[j]) * w[j] + b[j]) * l[j];
      st4<float>(res + row + c, r);
      if (y) {
        float o[4];
        ld4<float>(next.w + c, w); ld4<float>(next.b + c, b);
#pragma unroll
        for (int j = 0; j < 4; ++j) o[j] = tanh_fast(a2 * r[j]) * w[j] + b[j];
        st4<TA>(y + row + c, o);
      }
    }
  } else {
    for (int c = threadIdx.x; c < W; c += 256) {
      const float v = res[row + c] + (tanh_fast(a1 * ldf<TA>(hr + c)) * post.w[c] + post.b[c]) * ls[c];
      res[row + c] = v;
      if (y) stf<TA>(y + row + c, tanh_fast(a2 * v) * next.w[c] + next.b[c]);
    }
  }
}

// Tiled form of dyt_add for 16-byte-aligned rows: a thread owns four columns, loads their norm
// parameters once and walks RPB rows, so the five fp32 parameter vectors (20 bytes per column,
// more than the 12 bytes per element of data) are read once per RPB rows instead of once per row.
constexpr int RPB = 8;

template <typename TA>
__global__ __launch_bounds__(256) void dyt_add_tile_kernel(const TA* __restrict__ h, int h_stride, DytParams post,
                                                           const float* __restrict__ ls, float* __restrict__ res,
                                                           DytParams next, TA* __restrict__ y, int T, int W) {
  const int c = (blockIdx.x * 256 + threadIdx.x) * 4;
  if (c >= W) return;
  const int r0 = blockIdx.y * RPB, r1 = min(T, r0 + RPB);
  const float a1 = post.alpha[0];
  const float a2 = y ? next.alpha[0] : 0.f;
  float w1[4], b1[4], l[4], w2[4], b2[4];
  ld4<float>(post.w + c, w1); ld4<float>(post.b + c, b1); ld4<float>(ls + c, l);
  if (y) { ld4<float>(next.w + c, w2); ld4<float>(next.b + c, b2); }
  float hv[RPB][4], rv[RPB][4];
#pragma unroll
  for (int i = 0; i < RPB; ++i)
    if (r0 + i < r1) {
      ld4<TA>(h + (size_t)(r0 + i) * h_stride + c, hv[i]);
      ld4<float>(res + (size_t)(r0 + i) * W + c, rv[i]);
    }
#pragma unroll
  for (int i = 0; i < RPB; ++i)
    if (r0 + i < r1) {
#pragma unroll
      for (int j = 0; j < 4; ++j) rv[i][j] += (tanh_fast(a1 * hv[i][j]) * w1[j] + b1[j]) * l[j];
      st4<float>(res + (size_t)(r0 + i) * W + c, rv[i]);
      if (y) {
        float o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) o[j] = tanh_fast(a2 * rv[i][j]) * w2[j] + b2[j];
        st4<TA>(y + (size_t)(r0 + i) * W + c, o);
      }
    }
}

template <typename TA, bool VEC>
__global__ __launch_bounds__(256) void embed_dyt_kernel(const long long* __restrict__ ids, const TA* __restrict__ table,
                                                        int vocab, float scale, DytParams n, float* __restrict__ res,
                                                        int W) {
  const size_t row = (size_t)blockIdx.x * W;
  long long id = ids[blockIdx.x];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const TA* e = table + (size_t)id * W;
  const float a = n.alpha[0];
  if (VEC) {
    for (int c = threadIdx.x * 4; c < W; c += 1024) {
      float v[4], w[4], b[4], o[4];
      ld4<TA>(e + c, v); ld4<float>(n.w + c, w); ld4<float>(n.b + c, b);
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = tanh_fast(a * (v[j] * scale)) * w[j] + b[j];
      st4<float>(res + row + c, o);
    }
  } else {
    for (int c = threadIdx.x; c < W; c += 256) res[row + c] = tanh_fast(a * (ldf<TA>(e + c) * scale)) * n.w[c] + n.b[c];
  }
}

}  // namespace

extern "C" int dgi_dyt(const float* x, const float* alpha, const float* w, const float* b, void* y, int is_f32,
                       int T, int W, hipStream_t s) {
  if (T == 0) return 0;
  const DytParams n{alpha, w, b};
  const bool vec = W % 4 == 0 && ((uintptr_t)x | (uintptr_t)w | (uintptr_t)b | (uintptr_t)y) % 16 == 0;
  if (is_f32) {
    if (vec) dyt_kernel<float, true><<<T, 256, 0, s>>>(x, n, (float*)y, W);
    else dyt_kernel<float, false><<<T, 256, 0, s>>>(x, n, (float*)y, W);
  } else {
    if (vec) dyt_kernel<uint16_t, true><<<T, 256, 0, s>>>(x, n, (uint16_t*)y, W);
    else dyt_kernel<uint16_t, false><<<T, 256, 0, s>>>(x, n, (uint16_t*)y, W);
  }
  DGI_CHECK_LAUNCH();
  return 0;
}

extern "C" int dgi_dyt_add(const void* h, int h_stride, const float* alpha1, const float* w1, const float* b1,
                           const float* ls, float* res, const float* alpha2, const float* w2, const float* b2,
                           void* y, int is_f32, int T, int W, hipStream_t s) {
  if (T == 0) return 0;
  const DytParams post{alpha1, w1, b1}, next{alpha2, w2, b2};
  const bool vec = W % 4 == 0 && h_stride % 4 == 0 &&
                   ((uintptr_t)h | (uintptr_t)w1 | (uintptr_t)b1 | (uintptr_t)ls | (uintptr_t)res | (uintptr_t)w2 |
                    (uintptr_t)b2 | (uintptr_t)y) % 16 == 0;
  if (vec && T >= 2 * RPB && (T + RPB - 1) / RPB <= 65535) {
    const dim3 grid((W / 4 + 255) / 256, (T + RPB - 1) / RPB);
    if (is_f32)
      dyt_add_tile_kernel<float><<<grid, 256, 0, s>>>((const float*)h, h_stride, post, ls, res, next, (float*)y, T, W);
    else
      dyt_add_tile_kernel<uint16_t><<<grid, 256, 0, s>>>((const uint16_t*)h, h_stride, post, ls, res, next, (uint16_t*)y, T, W);
    DGI_CHECK_LAUNCH();
    return 0;
  }
  if (is_f32) {
    if (vec) dyt_add_kernel<float, true><<<T, 256, 0, s>>>((const float*)h, h_stride, post, ls, res, next, (float*)y, W);
    else dyt_add_kernel<float, false><<<T, 256, 0, s>>>((const float*)h, h_stride, post, ls, res, next, (float*)y, W);
  } else {
    if (vec) dyt_add_kernel<uint16_t, true><<<T, 256, 0, s>>>((const uint16_t*)h, h_stride, post, ls, res, next, (uint16_t*)y, W);
    else dyt_add_kernel<uint16_t, false><<<T, 256, 0, s>>>((const uint16_t*)h, h_stride, post, ls, res, next, (uint16_t*)y, W);
  }
  DGI_CHECK_LAUNCH();
  return 0;
}

extern "C" int dgi_embed_dyt(const long long* ids, const void* table, int vocab, float scale, const float* alpha,
                             const float* w, const float* b, float* res, int is_f32, int T, int W, hipStream_t s) {
  if (T == 0) return 0;
  const DytParams n{alpha, w, b};
  const bool vec = W % 4 == 0 && ((uintptr_t)table | (uintptr_t)w | (uintptr_t)b | (uintptr_t)res) % 16 == 0;
  if (is_f32) {
    if (vec) embed_dyt_kernel<float, true><<<T, 256, 0, s>>>(ids, (const float*)table, vocab, scale, n, res, W);
    else embed_dyt_kernel<float, false><<<T, 256, 0, s>>>(ids, (const float*)table, vocab, scale, n, res, W);
  } else {
    if (vec) embed_dyt_kernel<uint16_t, true><<<T, 256, 0, s>>>(ids, (const uint16_t*)table, vocab, scale, n, res, W);
    else embed_dyt_kernel<uint16_t, false><<<T, 256, 0, s>>>(ids, (const uint16_t*)table, vocab, scale, n, res, W);
  }
  DGI_CHECK_LAUNCH();
  return 0;
}
