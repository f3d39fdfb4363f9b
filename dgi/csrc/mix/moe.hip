// dgi/csrc/mix/moe.hip — mixture-of-experts feed-forward: routing, per-pair expert evaluation for
// small steps, and the combine of sorted-segment expert outputs for large ones.
//
//   moe_route         one wave per token: s = softmax(logits) over all R routes (fp32), the `top` routes
//                     with the largest s + correction (ties: lowest index), weights = s of those routes
//   silu_mul          silu(g) * u over fused [gate | up] rows
//   moe_pair_gate_up  grid (token * top + k, ff tiles): mid[pair][f] = silu(Wg[e] h)[f] * (Wu[e] h)[f],
//                     straight from the stacked expert weights [E, 2 ff, W]; identity routes (e >= E) skip
//   moe_pair_down     grid (token, W tiles): out[t][w] = sum_k wt_k * (Wd[e_k] mid_k)[w]  (identity: wt_k * h[t][w])
//                     + shared[t][w]; the routes are added in their fixed order k = 0..top-1
//   moe_combine       the same sum when the expert outputs sit in a buffer sorted by expert
//                     (ys[where[pair]]), as the segment GEMMs of a large step leave them
//
// Dot products run one output per wave with lanes striding the reduction dim, fp32 accumulation.
#include "../common.h"

using namespace dgi;

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf16_to_f32(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<uint16_t>(uint16_t* p, float v) { *p = f32_to_bf16(v); }

constexpr int MAXR = 8;      // routes per lane: R <= 512

__global__ __launch_bounds__(64) void moe_route_kernel(int* __restrict__ idx, float* __restrict__ wts,
                                                       const float* __restrict__ logits, int l_stride,
                                                       const float* __restrict__ corr, int R, int top) {
  const int t = blockIdx.x, lane = threadIdx.x;
  const float* lp = logits + (size_t)t * l_stride;
  float s[MAXR], c[MAXR];
  float m = -__builtin_inff();
#pragma unroll
  for (int i = 0; i < MAXR; ++i) {
    const int r = lane + 64 * i;
    s[i] = r < R ? lp[r] : -__builtin_inff();
    m = fmaxf(m, s[i]);
  }
  m = wave_max(m);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < MAXR; ++i) {
    const int r = lane + 64 * i;
    s[i] = r < R ? expf(s[i] - m) : 0.f;
    sum += s[i];
  }
  const float inv = 1.f / wave_sum(sum);
#pragma unroll
  for (int i = 0; i < MAXR; ++i) {
    const int r = lane + 64 * i;
    s[i] *= inv;
    c[i] = r < R ? s[i] + corr[r] : -__builtin_inff();
  }
  for (int k = 0; k < top; ++k) {
    float bv = -__builtin_inff();
    int bi = 1 << 30;
#pragma unroll
    for (int i = 0; i < MAXR; ++i) {
      const int r = lane + 64 * i;
      if (c[i] > bv) { bv = c[i]; bi = r; }          // ascending r within a lane: the lowest index wins ties
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
#pragma unroll
    for (int i = 0; i < MAXR; ++i) {
      if (lane + 64 * i == bi) {
        idx[(size_t)t * top + k] = bi;
        wts[(size_t)t * top + k] = s[i];
        c[i] = -__builtin_inff();
      }
    }
  }
}

template <typename T>
__global__ void silu_mul_kernel(T* __restrict__ out, const T* __restrict__ gu, int gu_stride, int rows, int I) {
  const size_t n = (size_t)rows * I;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const size_t r = i / I, c = i - r * I;
    const float g = ldf<T>(gu + r * gu_stride + c), u = ldf<T>(gu + r * gu_stride + I + c);
    stf<T>(out + i, g / (1.f + expf(-g)) * u);
  }
}

constexpr int OPW = 4;       // outputs per wave

template <typename T>
__global__ __launch_bounds__(256) void moe_pair_gate_up_kernel(
    float* __restrict__ mid, const T* __restrict__ h, int h_stride, const int* __restrict__ idx,
    const T* __restrict__ gate_up, int E, int top, int ff, int W) {
  extern __shared__ float hs[];            // [W] the token's input
  const int pair = blockIdx.x;
  const int e = idx[pair];
  if (e >= E || e < 0) return;             // identity route: nothing to project
  const int t = pair / top;
  for (int w = threadIdx.x; w < W; w += 256) hs[w] = ldf<T>(h + (size_t)t * h_stride + w);
  __syncthreads();
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const T* wg = gate_up + (size_t)e * 2 * ff * W;
  for (int j = 0; j < OPW; ++j) {
    const int f = (blockIdx.y * 4 + wave) * OPW + j;
    if (f >= ff) break;
    const T* gp = wg + (size_t)f * W;
    const T* up = wg + (size_t)(ff + f) * W;
    float ag = 0.f, au = 0.f;
    for (int w = lane; w < W; w += 64) {
      const float x = hs[w];
      ag += ldf<T>(gp + w) * x;
      au += ldf<T>(up + w) * x;
    }
    ag = wave_sum(ag);
    au = wave_sum(au);
    if (lane == 0) mid[(size_t)pair * ff + f] = ag / (1.f + expf(-ag)) * au;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_pair_down_kernel(
    T* __restrict__ out, const float* __restrict__ mid, const T* __restrict__ h, int h_stride,
    const int* __restrict__ idx, const float* __restrict__ wts, const T* __restrict__ down, const T* __restrict__ shared,
    int shared_stride, int E, int top, int ff, int W) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  for (int j = 0; j < OPW; ++j) {
    const int w = (blockIdx.y * 4 + wave) * OPW + j;
    if (w >= W) break;
    float acc = shared ? ldf<T>(shared + (size_t)t * shared_stride + w) : 0.f;
    for (int k = 0; k < top; ++k) {
      const int e = idx[(size_t)t * top + k];
      const float wt = wts[(size_t)t * top + k];
      if (e >= E || e < 0) {
        acc += wt * ldf<T>(h + (size_t)t * h_stride + w);
      } else {
        const T* dp = down + ((size_t)e * W + w) * ff;
        const float* mp = mid + ((size_t)t * top + k) * ff;
        float d = 0.f;
        for (int f = lane; f < ff; f += 64) d += ldf<T>(dp + f) * mp[f];
        acc += wt * wave_sum(d);
      }
    }
    if (lane == 0) stf<T>(out + (size_t)t * W + w, acc);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_combine_kernel(
    T* __restrict__ out, const T* __restrict__ ys, const int* __restrict__ where, const T* __restrict__ h, int h_stride,
    const int* __restrict__ idx, const float* __restrict__ wts, const T* __restrict__ shared, int shared_stride, int E,
    int top, int W) {
  const int t = blockIdx.x;
  const int w = blockIdx.y * 256 + threadIdx.x;
  if (w >= W) return;
  float acc = shared ? ldf<T>(shared + (size_t)t * shared_stride + w) : 0.f;
  for (int k = 0; k < top; ++k) {
    const int e = idx[(size_t)t * top + k];
    const float wt = wts[(size_t)t * top + k];
    if (e >= E || e < 0) acc += wt * ldf<T>(h + (size_t)t * h_stride + w);
    else acc += wt * ldf<T>(ys + (size_t)where[(size_t)t * top + k] * W + w);
  }
  stf<T>(out + (size_t)t * W + w, acc);
}

}  // namespace

extern "C" int dgi_moe_route(int* idx, float* wts, const float* logits, int l_stride, const float* corr, int T, int R,
                             int top, hipStream_t s) {
  if (T == 0) return 0;
  if (R > 64 * MAXR || top > R || top < 1) return -2;
  moe_route_kernel<<<T, 64, 0, s>>>(idx, wts, logits, l_stride, corr, R, top);
  DGI_CHECK_LAUNCH();
  return 0;
}

extern "C" int dgi_glu_silu(void* out, const void* gu, int gu_stride, int rows, int I, int is_f32, hipStream_t s) {
  if (rows == 0 || I == 0) return 0;
  const size_t n = (size_t)rows * I;
  const int blocks = (int)((n + 255) / 256 > 65535 ? 65535 : (n + 255) / 256);
  if (is_f32) silu_mul_kernel<float><<<blocks, 256, 0, s>>>((float*)out, (const float*)gu, gu_stride, rows, I);
  else silu_mul_kernel<uint16_t><<<blocks, 256, 0, s>>>((uint16_t*)out, (const uint16_t*)gu, gu_stride, rows, I);
  DGI_CHECK_LAUNCH();
  return 0;
}

extern "C" int dgi_moe_pair_gate_up(float* mid, const void* h, int h_stride, const int* idx, const void* gate_up,
                                    int T, int E, int top, int ff, int W, int is_f32, hipStream_t s) {
  if (T == 0) return 0;
  if (W > 16384) return -2;
  const dim3 grid(T * top, (ff + 4 * OPW - 1) / (4 * OPW));
  if (grid.y > 65535) return -3;
  if (is_f32)
    moe_pair_gate_up_kernel<float><<<grid, 256, (size_t)W * 4, s>>>(mid, (const float*)h, h_stride, idx,
                                                                    (const float*)gate_up, E, top, ff, W);
  else
    moe_pair_gate_up_kernel<uint16_t><<<grid, 256, (size_t)W * 4, s>>>(mid, (const uint16_t*)h, h_stride, idx,
                                                                       (const uint16_t*)gate_up, E, top, ff, W);
  DGI_CHECK_LAUNCH();
  return 0;
}

extern "C" int dgi_moe_pair_down(void* out, const float* mid, const void* h, int h_stride, const int* idx,
                                 const float* wts, const void* down, const void* shared, int shared_stride, int T,
                                 int E, int top, int ff, int W, int is_f32, hipStream_t s) {
  if (T == 0) return 0;
  const dim3 grid(T, (W + 4 * OPW - 1) / (4 * OPW));
  if (grid.y > 65535) return -3;
  if (is_f32)
    moe_pair_down_kernel<float><<<grid, 256, 0, s>>>((float*)out, mid, (const float*)h, h_stride, idx, wts,
                                                     (const float*)down, (const float*)shared, shared_stride, E, top, ff, W);
  else
    moe_pair_down_kernel<uint16_t><<<grid, 256, 0, s>>>((uint16_t*)out, mid, (const uint16_t*)h, h_stride, idx, wts,
                                                        (const uint16_t*)down, (const uint16_t*)shared, shared_stride, E,
                                                        top, ff, W);
  DGI_CHECK_LAUNCH();
  return 0;
}

extern "C" int dgi_moe_combine(void* out, const void* ys, const int* where, const void* h, int h_stride, const int* idx,
                               const float* wts, const void* shared, int shared_stride, int T, int E, int top, int W,
                               int is_f32, hipStream_t s) {
  if (T == 0) return 0;
  const dim3 grid(T, (W + 255) / 256);
  if (grid.y > 65535) return -3;
  if (is_f32)
    moe_combine_kernel<float><<<grid, 256, 0, s>>>((float*)out, (const float*)ys, where, (const float*)h, h_stride, idx, wts,
                                                   (const float*)shared, shared_stride, E, top, W);
  else
    moe_combine_kernel<uint16_t><<<grid, 256, 0, s>>>((uint16_t*)out, (const uint16_t*)ys, where, (const uint16_t*)h,
                                                      h_stride, idx, wts, (const uint16_t*)shared, shared_stride, E, top, W);
  DGI_CHECK_LAUNCH();
  return 0;
}
