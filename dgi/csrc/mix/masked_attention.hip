// dgi/csrc/mix/masked_attention.hip — row-wise softmax attention over the paged KV pool for any
// head geometry, in bf16 or fp32, with a block ("chunk") mask and an output gate.
//
// decode_attention.hip and prefill_attention.hip are MFMA kernels for bf16 heads of 64 / 128
// dims whose keys and values share one size.  This kernel is the general form the other
// geometries run on (key size != value size, sizes that are no multiple of 16, fp32 caches)
// and the one both step phases share: every query row — a decode row or one row of a prompt
// portion — is one wave that walks its own visible keys
//
//     [first(p), p],   first(p) = floor(p / mask) * mask   (mask > 0: keys of the row's own block
//                                                            of `mask` positions, counted from
//                                                            position 0 of the sequence)
//                      first(p) = 0                          (mask == 0: plain causal)
//
// straight from the cache (this step's keys are written before it runs), so the result does
// not depend on how the prompt was cut into steps or on what else is in the batch.
// Scores, the online softmax and the output accumulation are fp32; exp is the accurate expf.
// Optional epilogue: out *= sigmoid(gate) element by element (the mixer's output gate, read
// from the same fused projection row as q).
//
// Wave layout: lane j scores key first + 64 i + j (a contiguous dk-vector per lane, 16-byte
// loads where dk allows); the 64 probabilities go through LDS and every lane accumulates the
// value dims d = lane + 64 c, so the V reads of one key are one coalesced row.
// grid = (rows, H), 64 threads.
#include "../common.h"

using namespace dgi;

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf16_to_f32(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<uint16_t>(uint16_t* p, float v) { *p = f32_to_bf16(v); }

constexpr int MAXC = 8;       // value dims per lane: dv <= 64 * MAXC
constexpr int MAXDK = 512;    // query vector staged in LDS

__device__ __forceinline__ float dot_row(const float* __restrict__ qs, const float* __restrict__ k, int dk) {
  float acc = 0.f;
  if ((dk & 3) == 0) {
    for (int e = 0; e < dk; e += 4) {
      const float4 v = *reinterpret_cast<const float4*>(k + e);
      acc += qs[e] * v.x + qs[e + 1] * v.y + qs[e + 2] * v.z + qs[e + 3] * v.w;
    }
  } else {
    for (int e = 0; e < dk; ++e) acc += qs[e] * k[e];
  }
  return acc;
}

__device__ __forceinline__ float dot_row(const float* __restrict__ qs, const uint16_t* __restrict__ k, int dk) {
  float acc = 0.f;
  if ((dk & 7) == 0) {
    for (int e = 0; e < dk; e += 8) {
      float f[8];
      unpack8(*reinterpret_cast<const u32x4*>(k + e), f);
#pragma unroll
      for (int j = 0; j < 8; ++j) acc += qs[e + j] * f[j];
    }
  } else {
    for (int e = 0; e < dk; ++e) acc += qs[e] * bf16_to_f32(k[e]);
  }
  return acc;
}

template <typename T>
__global__ __launch_bounds__(64) void masked_attn_rows_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ cu_seqlens, int n_seqs,
    const int* __restrict__ positions, int G, int dk, int dv, int bs, float scale, int mask,
    const T* __restrict__ gate, int gate_stride, T* __restrict__ out, int out_stride) {
  __shared__ float qs[MAXDK];
  __shared__ float ps[64];
  __shared__ long long vo[64];

  const int row = blockIdx.x, head = blockIdx.y, H = gridDim.y;
  const int lane = threadIdx.x;
  const int kvh = head / (H / G);
  // the row's sequence: row index itself (decode rows), or the portion holding it (cu_seqlens)
  int seq = row;
  if (cu_seqlens) {
    int lo = 0, hi = n_seqs - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (cu_seqlens[mid] <= row) lo = mid; else hi = mid - 1;
    }
    seq = lo;
  }
  const int* bt = block_tables + (size_t)seq * bt_stride;
  const int pos = positions[row];
  const int first = mask > 0 ? (pos / mask) * mask : 0;

  const T* qp = q + (size_t)row * q_stride + (size_t)head * dk;
  for (int e = lane; e < dk; e += 64) qs[e] = ldf<T>(qp + e);
  __syncthreads();

  float m_run = -__builtin_inff(), l_run = 0.f;
  float o[MAXC];
#pragma unroll
  for (int c = 0; c < MAXC; ++c) o[c] = 0.f;
  const int nc = (dv + 63) >> 6;

  for (int k0 = first; k0 <= pos; k0 += 64) {
    const int key = k0 + lane;
    const bool ok = key <= pos;
    float s = -__builtin_inff();
    long long vbase = 0;
    if (ok) {
      const int blk = bt[key / bs];
      const long long slot = ((long long)blk * G + kvh) * bs + (key % bs);
      s = dot_row(qs, k_cache + slot * dk, dk) * scale;
      vbase = slot * dv;
    }
    const float m_new = fmaxf(m_run, wave_max(s));     // lane 0's key k0 is always visible: finite
    const float p = ok ? expf(s - m_new) : 0.f;
    const float corr = expf(m_run - m_new);            // first tile: exp(-inf) = 0
    l_run = l_run * corr + wave_sum(p);
    m_run = m_new;
    __syncthreads();                                   // previous tile's ps / vo fully read
    ps[lane] = p;
    vo[lane] = vbase;
    __syncthreads();
    const int n = min(64, pos - k0 + 1);
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
      if (c < nc) {
        const int d = lane + 64 * c;
        float acc = o[c] * corr;
        if (d < dv)
          for (int j = 0; j < n; ++j) acc += ps[j] * ldf<T>(v_cache + vo[j] + d);
        o[c] = acc;
      }
    }
  }
  const float inv = 1.f / l_run;
  T* op = out + (size_t)row * out_stride + (size_t)head * dv;
  const T* gp = gate ? gate + (size_t)row * gate_stride + (size_t)head * dv : nullptr;
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int d = lane + 64 * c;
    if (c < nc && d < dv) {
      float v = o[c] * inv;
      if (gp) v *= 1.f / (1.f + expf(-ldf<T>(gp + d)));
      stf<T>(op + d, v);
    }
  }
}

}  // namespace

// q / gate / out: row-major with their own row strides (elements); cu_seqlens (n_seqs + 1 row
// offsets) maps rows to block-table rows, nullptr: row i uses block-table row i.
extern "C" int dgi_masked_attn_rows(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                                    const int* block_tables, int bt_stride, const int* cu_seqlens, int n_seqs,
                                    const int* positions, int rows, int H, int G, int dk, int dv, int block_size,
                                    float scale, int mask, const void* gate, int gate_stride, void* out,
                                    int out_stride, int is_f32, hipStream_t s) {
  if (rows == 0) return 0;
  if (G <= 0 || H % G) return -2;
  if (dk > MAXDK || dv > 64 * MAXC || dk <= 0 || dv <= 0) return -3;
  if (H > 65535 || mask < 0) return -4;
  const dim3 grid(rows, H);
  if (is_f32)
    masked_attn_rows_kernel<float><<<grid, 64, 0, s>>>(
        (const float*)q, q_stride, (const float*)k_cache, (const float*)v_cache, block_tables, bt_stride, cu_seqlens,
        n_seqs, positions, G, dk, dv, block_size, scale, mask, (const float*)gate, gate_stride, (float*)out, out_stride);
  else
    masked_attn_rows_kernel<uint16_t><<<grid, 64, 0, s>>>(
        (const uint16_t*)q, q_stride, (const uint16_t*)k_cache, (const uint16_t*)v_cache, block_tables, bt_stride,
        cu_seqlens, n_seqs, positions, G, dk, dv, block_size, scale, mask, (const uint16_t*)gate, gate_stride,
        (uint16_t*)out, out_stride);
  DGI_CHECK_LAUNCH();
  return 0;
}
