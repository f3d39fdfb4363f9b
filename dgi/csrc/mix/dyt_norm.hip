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
// Elementwise and memory-bound: one workgroup per row, fp32 math with the accurate tanhf (the
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

struct DytParams {
  const float* alpha;   // [1]
  const float* w;       // [W]
  const float* b;       // [W]
};

template <typename TA>
__global__ __launch_bounds__(256) void dyt_kernel(const float* __restrict__ x, DytParams n, TA* __restrict__ y,
                                                  int W) {
  const size_t row = (size_t)blockIdx.x * W;
  const float a = n.alpha[0];
  for (int c = threadIdx.x; c < W; c += 256) stf<TA>(y + row + c, tanhf(a * x[row + c]) * n.w[c] + n.b[c]);
}

// res += (tanh(a1 * h) * w1 + b1) * ls;  y = tanh(a2 * res) * w2 + b2 (when y != nullptr)
template <typename TA>
__global__ __launch_bounds__(256) void dyt_add_kernel(const TA* __restrict__ h, int h_stride, DytParams post,
                                                      const float* __restrict__ ls, float* __restrict__ res,
                                                      DytParams next, TA* __restrict__ y, int W) {
  const size_t row = (size_t)blockIdx.x * W;
  const TA* hr = h + (size_t)blockIdx.x * h_stride;
  const float a1 = post.alpha[0];
  const float a2 = y ? next.alpha[0] : 0.f;
  for (int c = threadIdx.x; c < W; c += 256) {
    const float v = res[row + c] + (tanhf(a1 * ldf<TA>(hr + c)) * post.w[c] + post.b[c]) * ls[c];
    res[row + c] = v;
    if (y) stf<TA>(y + row + c, tanhf(a2 * v) * next.w[c] + next.b[c]);
  }
}

template <typename TA>
__global__ __launch_bounds__(256) void embed_dyt_kernel(const long long* __restrict__ ids, const TA* __restrict__ table,
                                                        int vocab, float scale, DytParams n, float* __restrict__ res,
                                                        int W) {
  const size_t row = (size_t)blockIdx.x * W;
  long long id = ids[blockIdx.x];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const TA* e = table + (size_t)id * W;
  const float a = n.alpha[0];
  for (int c = threadIdx.x; c < W; c += 256) res[row + c] = tanhf(a * (ldf<TA>(e + c) * scale)) * n.w[c] + n.b[c];
}

}  // namespace

extern "C" int dgi_dyt(const float* x, const float* alpha, const float* w, const float* b, void* y, int is_f32,
                       int T, int W, hipStream_t s) {
  if (T == 0) return 0;
  const DytParams n{alpha, w, b};
  if (is_f32) dyt_kernel<float><<<T, 256, 0, s>>>(x, n, (float*)y, W);
  else dyt_kernel<uint16_t><<<T, 256, 0, s>>>(x, n, (uint16_t*)y, W);
  DGI_CHECK_LAUNCH();
  return 0;
}

extern "C" int dgi_dyt_add(const void* h, int h_stride, const float* alpha1, const float* w1, const float* b1,
                           const float* ls, float* res, const float* alpha2, const float* w2, const float* b2,
                           void* y, int is_f32, int T, int W, hipStream_t s) {
  if (T == 0) return 0;
  const DytParams post{alpha1, w1, b1}, next{alpha2, w2, b2};
  if (is_f32)
    dyt_add_kernel<float><<<T, 256, 0, s>>>((const float*)h, h_stride, post, ls, res, next, (float*)y, W);
  else
    dyt_add_kernel<uint16_t><<<T, 256, 0, s>>>((const uint16_t*)h, h_stride, post, ls, res, next, (uint16_t*)y, W);
  DGI_CHECK_LAUNCH();
  return 0;
}

extern "C" int dgi_embed_dyt(const long long* ids, const void* table, int vocab, float scale, const float* alpha,
                             const float* w, const float* b, float* res, int is_f32, int T, int W, hipStream_t s) {
  if (T == 0) return 0;
  const DytParams n{alpha, w, b};
  if (is_f32) embed_dyt_kernel<float><<<T, 256, 0, s>>>(ids, (const float*)table, vocab, scale, n, res, W);
  else embed_dyt_kernel<uint16_t><<<T, 256, 0, s>>>(ids, (const uint16_t*)table, vocab, scale, n, res, W);
  DGI_CHECK_LAUNCH();
  return 0;
}
