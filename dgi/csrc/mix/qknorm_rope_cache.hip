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
// Optional query temperature (qt_every > 0): a row at position p has its normalised q multiplied
// by 1 + qt_coef * ln(floor((p + 1) / qt_every) + 1) — attention that sharpens as the context grows.
// The norm, its weight, the temperature and the rotation are computed in fp32 whatever the activation dtype.
//
// Cache layout per layer: k [num_blocks, G, block_size, dk], v [num_blocks, G, block_size, dv].
// One workgroup per token; a wave owns one head at a time (sum of squares by wave reduction),
// a lane its rotation pairs; v rows are copied in 16-byte chunks where the sizes allow.
#include <cstdlib>
#include "../common.h"

using namespace dgi;

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf16_to_f32(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<uint16_t>(uint16_t* p, float v) { *p = f32_to_bf16(v); }

template <typename T> __device__ __forceinline__ void ld2(const T* p, float* f);
template <> __device__ __forceinline__ void ld2<float>(const float* p, float* f) {
  const float2 v = *reinterpret_cast<const float2*>(p);
  f[0] = v.x; f[1] = v.y;
}
template <> __device__ __forceinline__ void ld2<uint16_t>(const uint16_t* p, float* f) {
  const uint32_t v = *reinterpret_cast<const uint32_t*>(p);
  f[0] = __uint_as_float(v << 16); f[1] = __uint_as_float(v & 0xffff0000u);
}
template <typename T> __device__ __forceinline__ void st2(T* p, const float* f);
template <> __device__ __forceinline__ void st2<float>(float* p, const float* f) {
  *reinterpret_cast<float2*>(p) = make_float2(f[0], f[1]);
}
template <> __device__ __forceinline__ void st2<uint16_t>(uint16_t* p, const float* f) {
  *reinterpret_cast<uint32_t*>(p) = pack_bf16x2(f[0], f[1]);
}

template <typename T>
__global__ __launch_bounds__(256) void qknorm_rope_cache_kernel(
    T* __restrict__ qkv, int stride, const int* __restrict__ positions, const int* __restrict__ slots,
    const float* __restrict__ qw, const float* __restrict__ kw, float eps, const float* __restrict__ cos_sin,
    int rd, int H, int G, int dk, int dv, T* __restrict__ k_cache, T* __restrict__ v_cache, int block_size,
    float qt_coef, int qt_every) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float qtemp = qt_every > 0 ? 1.f + qt_coef * logf((float)((positions[t] + 1) / qt_every + 1)) : 1.f;
  T* row = qkv + (size_t)t * stride;
  const int slot = slots ? slots[t] : -1;
  const int blk = slot >= 0 ? slot / block_size : 0;
  const int off = slot >= 0 ? slot - blk * block_size : 0;
  const float* cs = rd > 0 ? cos_sin + (size_t)positions[t] * rd : nullptr;
  const int rh = rd >> 1;
  const float inv_dk = 1.f / (float)dk;

  // a lane owns the rotation pairs (2i, 2i+1), i = lane + 64 j: one 4-byte (bf16) or 8-byte
  // (fp32) access per pair when rows and heads start on even elements, values stay in registers
  // between the sum of squares and the store (dk <= 512)
  const bool pairvec = ((dk | stride) & 1) == 0;
  for (int head = wave; head < H + G; head += 4) {
    T* hp = row + (size_t)head * dk;                      // q heads, then k heads
    const float* nw = head < H ? qw : kw;
    T* dst = hp;
    if (head >= H) {
      if (slot < 0) continue;
      dst = k_cache + (((size_t)blk * G + (head - H)) * block_size + off) * dk;
    }
    float xv[4][2];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int e = 2 * (lane + 64 * j);
      xv[j][0] = xv[j][1] = 0.f;
      if (e + 1 < dk && pairvec) {
        ld2<T>(hp + e, xv[j]);
      } else if (e < dk) {
        xv[j][0] = ldf<T>(hp + e);
        if (e + 1 < dk) xv[j][1] = ldf<T>(hp + e + 1);
      }
      ss += xv[j][0] * xv[j][0] + xv[j][1] * xv[j][1];
    }
    ss = wave_sum(ss);
    const float r = 1.f / sqrtf(ss * inv_dk + eps) * (head < H ? qtemp : 1.f);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int e = 2 * (lane + 64 * j);
      if (e >= dk) continue;
      const float x = xv[j][0] * r * nw[e];
      const float y = e + 1 < dk ? xv[j][1] * r * nw[e + 1] : 0.f;
      float o[2] = {x, y};
      if (e + 1 < rd) {
        const float c = cs[e >> 1], sn = cs[rh + (e >> 1)];
        o[0] = x * c - y * sn;
        o[1] = y * c + x * sn;
      }
      if (e + 1 < dk && pairvec) {
        st2<T>(dst + e, o);
      } else {
        stf<T>(dst + e, o[0]);
        if (e + 1 < dk) stf<T>(dst + e + 1, o[1]);
      }
    }
  }
  if (slot >= 0) {
    const T* vsrc = row + (size_t)(H + G) * dk;
    constexpr int EPV = 16 / sizeof(T);
    if (dv % EPV == 0 && stride % EPV == 0 && ((H + G) * dk) % EPV == 0 && ((uintptr_t)qkv & 15) == 0) {
      const int cpv = dv / EPV;
      for (int i = threadIdx.x; i < G * cpv; i += 256) {
        const int vh = i / cpv, c = i - vh * cpv;
        *reinterpret_cast<u32x4*>(v_cache + (((size_t)blk * G + vh) * block_size + off) * dv + c * EPV) =
            *reinterpret_cast<const u32x4*>(vsrc + (size_t)vh * dv + c * EPV);
      }
    } else {
      for (int i = threadIdx.x; i < G * dv; i += 256) {
        const int vh = i / dv, d = i - vh * dv;
        v_cache[(((size_t)blk * G + vh) * block_size + off) * dv + d] = vsrc[i];
      }
    }
  }
}

// Sixteen lanes per head, 16-byte chunks (dk a multiple of 8 bf16 / 4 fp32): a workgroup
// normalises sixteen heads of one token at once (grid.y walks the heads), each lane keeps up to
// MAXCH chunks in registers between the sum of squares (four shuffles inside the 16-lane
// group) and the store; norm weights and cos / sin come in as 16-byte loads.
template <typename T, int MAXCH>
__global__ __launch_bounds__(1024) void qknorm_rope_cache_vec_kernel(
    T* __restrict__ qkv, int stride, const int* __restrict__ positions, const int* __restrict__ slots,
    const float* __restrict__ qw, const float* __restrict__ kw, float eps, const float* __restrict__ cos_sin,
    int rd, int H, int G, int dk, int dv, T* __restrict__ k_cache, T* __restrict__ v_cache, int block_size,
    float qt_coef, int qt_every) {
  constexpr int E = 16 / sizeof(T);
  const int t = blockIdx.x;
  const float qtemp = qt_every > 0 ? 1.f + qt_coef * logf((float)((positions[t] + 1) / qt_every + 1)) : 1.f;
  const int grp = threadIdx.x >> 4, l = threadIdx.x & 15;
  T* row = qkv + (size_t)t * stride;
  const int slot = slots ? slots[t] : -1;
  const int blk = slot >= 0 ? slot / block_size : 0;
  const int off = slot >= 0 ? slot - blk * block_size : 0;
  const float* cs = rd > 0 ? cos_sin + (size_t)positions[t] * rd : nullptr;
  const int rh = rd >> 1;
  const float inv_dk = 1.f / (float)dk;
  const int nch = dk / E;

  const int head = blockIdx.y * (blockDim.x >> 4) + grp;  // blockDim / 16 heads per workgroup, grid.y for the rest
  if (head < H + G && !(head >= H && slot < 0)) {
    T* hp = row + (size_t)head * dk;
    const float* nw = head < H ? qw : kw;
    T* dst = hp;
    if (head >= H) dst = k_cache + (((size_t)blk * G + (head - H)) * block_size + off) * dk;
    const bool csvec = (rd & 7) == 0 && E == 8;         // four cos + four sin of a chunk as two float4
    float x[MAXCH][E];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < MAXCH; ++j) {
      const int c = l + 16 * j;
      if (c < nch) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(hp + c * E);
        if constexpr (sizeof(T) == 2) {
          unpack8(v, x[j]);
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i) x[j][i] = __uint_as_float(v[i]);
        }
#pragma unroll
        for (int i = 0; i < E; ++i) ss += x[j][i] * x[j][i];
      }
    }
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
    const float r = 1.f / sqrtf(ss * inv_dk + eps) * (head < H ? qtemp : 1.f);
#pragma unroll
    for (int j = 0; j < MAXCH; ++j) {
      const int c = l + 16 * j;
      if (c >= nch) continue;
      const int e0 = c * E;
      float o[E], wv[E], cv[E / 2], sv[E / 2];
#pragma unroll
      for (int i = 0; i < E; i += 4) *reinterpret_cast<float4*>(wv + i) = *reinterpret_cast<const float4*>(nw + e0 + i);
      if (csvec && e0 + E <= rd) {
        *reinterpret_cast<float4*>(cv) = *reinterpret_cast<const float4*>(cs + (e0 >> 1));
        *reinterpret_cast<float4*>(sv) = *reinterpret_cast<const float4*>(cs + rh + (e0 >> 1));
      } else {
#pragma unroll
        for (int i = 0; i < E / 2; ++i) {
          const bool rot = e0 + 2 * i + 1 < rd;
          cv[i] = rot ? cs[(e0 >> 1) + i] : 1.f;
          sv[i] = rot ? cs[rh + (e0 >> 1) + i] : 0.f;
        }
      }
#pragma unroll
      for (int i = 0; i < E; i += 2) {
        const float a = x[j][i] * r * wv[i], b = x[j][i + 1] * r * wv[i + 1];
        o[i] = a * cv[i >> 1] - b * sv[i >> 1];
        o[i + 1] = b * cv[i >> 1] + a * sv[i >> 1];
      }
      u32x4 w;
      if constexpr (sizeof(T) == 2) {
        w = pack8(o);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = __float_as_uint(o[i]);
      }
      *reinterpret_cast<u32x4*>(dst + e0) = w;
    }
  }
  if (slot >= 0 && blockIdx.y == 0) {
    const T* vsrc = row + (size_t)(H + G) * dk;
    if (dv % E == 0) {
      const int cpv = dv / E;
      for (int i = threadIdx.x; i < G * cpv; i += blockDim.x) {
        const int vh = i / cpv, c = i - vh * cpv;
        *reinterpret_cast<u32x4*>(v_cache + (((size_t)blk * G + vh) * block_size + off) * dv + c * E) =
            *reinterpret_cast<const u32x4*>(vsrc + (size_t)vh * dv + c * E);
      }
    } else {
      for (int i = threadIdx.x; i < G * dv; i += blockDim.x) {
        const int vh = i / dv, d = i - vh * dv;
        v_cache[(((size_t)blk * G + vh) * block_size + off) * dv + d] = vsrc[i];
      }
    }
  }
}

}  // namespace

extern "C" int dgi_qknorm_rope_cache(void* qkv, int is_f32, int T, int stride, const int* positions,
                                     const int* slots, const float* qw, const float* kw, float eps,
                                     const float* cos_sin, int rd, int H, int G, int dk, int dv, void* k_cache,
                                     void* v_cache, int block_size, float qt_coef, int qt_every, hipStream_t s) {
  if (T == 0) return 0;
  if (rd < 0 || rd > dk || (rd & 1)) return -2;
  if (dk > 512) return -3;
  const int E = is_f32 ? 4 : 8;
  if (dk % E == 0 && stride % E == 0 && dk <= 64 * E && ((uintptr_t)qkv | (uintptr_t)k_cache | (uintptr_t)v_cache) % 16 == 0) {
    // heads per workgroup (16 lanes each): 4 to 16 measured alike on 8B-class rows (36-39 us for
    // 8192 tokens), 32 and more slower (bigger workgroups hide less latency); DGI_QKNORM_HPB for sweeps
    static const int hpb_env = [] { const char* e = getenv("DGI_QKNORM_HPB"); return e ? atoi(e) : 0; }();
    int hpb = hpb_env > 0 ? (hpb_env > 64 ? 64 : hpb_env) : 8;
    if (hpb > H + G) hpb = H + G;
    const int vthreads = (hpb * 16 + 63) / 64 * 64;
    if ((H + G + hpb - 1) / hpb > 65535) return -4;
    const dim3 vgrid(T, (H + G + hpb - 1) / hpb);
    if (is_f32)
      qknorm_rope_cache_vec_kernel<float, 4><<<vgrid, vthreads, 0, s>>>((float*)qkv, stride, positions, slots, qw, kw, eps, cos_sin,
                                                               rd, H, G, dk, dv, (float*)k_cache, (float*)v_cache, block_size, qt_coef, qt_every);
    else
      qknorm_rope_cache_vec_kernel<uint16_t, 4><<<vgrid, vthreads, 0, s>>>((uint16_t*)qkv, stride, positions, slots, qw, kw, eps,
                                                                  cos_sin, rd, H, G, dk, dv, (uint16_t*)k_cache,
                                                                  (uint16_t*)v_cache, block_size, qt_coef, qt_every);
    DGI_CHECK_LAUNCH();
    return 0;
  }
  if (is_f32)
    qknorm_rope_cache_kernel<float><<<T, 256, 0, s>>>((float*)qkv, stride, positions, slots, qw, kw, eps, cos_sin,
                                                      rd, H, G, dk, dv, (float*)k_cache, (float*)v_cache, block_size, qt_coef, qt_every);
  else
    qknorm_rope_cache_kernel<uint16_t><<<T, 256, 0, s>>>((uint16_t*)qkv, stride, positions, slots, qw, kw, eps,
                                                         cos_sin, rd, H, G, dk, dv, (uint16_t*)k_cache,
                                                         (uint16_t*)v_cache, block_size, qt_coef, qt_every);
  DGI_CHECK_LAUNCH();
  return 0;
}
