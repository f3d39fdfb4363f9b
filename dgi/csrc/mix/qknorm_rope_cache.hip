// dgi/csrc/mix/qknorm_rope_cache.hip — per-head RMS norm of q and k, rotary positions, paged KV write.
//
// rope_cache.hip's job for mixers that normalise queries and keys per head before rotating
// them, whose key and value heads may differ in size, and whose projections may run in fp32:
// one kernel reads a token's fused projection row [q: H*dk | k: G*dk | v: G*dv | ...] once and
//   * replaces each q head by  rot(q / sqrt(mean(q^2) + eps) * wq)   in place,
//   * writes  rot(k / sqrt(mean(k^2) + eps) * wk)  and v into the paged cache at the row's slot.
// rot() turns the interleaved pairs (2i, 2i+1) of the first rd dims by the row's position; the
// other dims pass through.  cos_sin is the fp32 table [max_pos, rd] (rd/2 cos | rd/2 sin) that
// rope_cache.hip reads too (frequency scaling is folded into the table); rd = 0: no rotation.
// The norm, its weight and the rotation are computed in fp32 whatever the activation dtype.
//
// Cache layout per layer: k [num_blocks, G, block_size, dk], v [num_blocks, G, block_size, dv].
// One workgroup per token; a wave owns one head at a time (sum of squares by wave reduction).
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
__global__ __launch_bounds__(256) void qknorm_rope_cache_kernel(
    T* __restrict__ qkv, int stride, const int* __restrict__ positions, const int* __restrict__ slots,
    const float* __restrict__ qw, const float* __restrict__ kw, float eps, const float* __restrict__ cos_sin,
    int rd, int H, int G, int dk, int dv, T* __restrict__ k_cache, T* __restrict__ v_cache, int block_size) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  T* row = qkv + (size_t)t * stride;
  const int slot = slots ? slots[t] : -1;
  const int blk = slot >= 0 ? slot / block_size : 0;
  const int off = slot >= 0 ? slot - blk * block_size : 0;
  const float* cs = rd > 0 ? cos_sin + (size_t)positions[t] * rd : nullptr;
  const int rh = rd >> 1;
  const float inv_dk = 1.f / (float)dk;

  for (int head = wave; head < H + G; head += 4) {
    T* hp = row + (size_t)head * dk;                      // q heads, then k heads
    const float* nw = head < H ? qw : kw;
    float ss = 0.f;
    for (int e = lane; e < dk; e += 64) {
      const float x = ldf<T>(hp + e);
      ss += x * x;
    }
    ss = wave_sum(ss);
    const float r = 1.f / sqrtf(ss * inv_dk + eps);
    T* dst = nullptr;
    if (head >= H) {
      if (slot < 0) continue;
      dst = k_cache + (((size_t)blk * G + (head - H)) * block_size + off) * dk;
    }
    // the pair partner e ^ 1 lives in the same pass (neighbouring lane): both values are read
    // before either lane stores
    for (int e0 = 0; e0 < dk; e0 += 64) {
      const int e = e0 + lane;
      float o = 0.f;
      if (e < dk) {
        const float x = ldf<T>(hp + e) * r * nw[e];
        if (e < rd) {
          const float y = ldf<T>(hp + (e ^ 1)) * r * nw[e ^ 1];
          const float c = cs[e >> 1], s = cs[rh + (e >> 1)];
          o = (e & 1) ? x * c + y * s : x * c - y * s;
        } else {
          o = x;
        }
      }
      __builtin_amdgcn_wave_barrier();
      if (e < dk) stf<T>((dst ? dst : hp) + e, o);
    }
  }
  if (slot >= 0) {
    const T* vsrc = row + (size_t)(H + G) * dk;
    for (int i = threadIdx.x; i < G * dv; i += 256) {
      const int vh = i / dv, d = i - vh * dv;
      v_cache[(((size_t)blk * G + vh) * block_size + off) * dv + d] = vsrc[i];
    }
  }
}

}  // namespace

extern "C" int dgi_qknorm_rope_cache(void* qkv, int is_f32, int T, int stride, const int* positions,
                                     const int* slots, const float* qw, const float* kw, float eps,
                                     const float* cos_sin, int rd, int H, int G, int dk, int dv, void* k_cache,
                                     void* v_cache, int block_size, hipStream_t s) {
  if (T == 0) return 0;
  if (rd < 0 || rd > dk || (rd & 1)) return -2;
  if (is_f32)
    qknorm_rope_cache_kernel<float><<<T, 256, 0, s>>>((float*)qkv, stride, positions, slots, qw, kw, eps, cos_sin,
                                                      rd, H, G, dk, dv, (float*)k_cache, (float*)v_cache, block_size);
  else
    qknorm_rope_cache_kernel<uint16_t><<<T, 256, 0, s>>>((uint16_t*)qkv, stride, positions, slots, qw, kw, eps,
                                                         cos_sin, rd, H, G, dk, dv, (uint16_t*)k_cache,
                                                         (uint16_t*)v_cache, block_size);
  DGI_CHECK_LAUNCH();
  return 0;
}
