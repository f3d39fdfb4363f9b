// dgi/csrc/mix/streams.hip — several fp32 residual streams per token ("hyper-connections") and the
// embedding that starts them.
//
//   embed_streams   x_s[t] = E[tok] + Bg[(prev * a + tok * b) mod n] + P[pos]  for every stream s
//                   (a sequence's first token takes bigram row n; the token before a portion's first
//                   row comes from the sequence's state slot, which then receives the portion's last
//                   token in a second, tiny kernel — a portion's first and last rows are different
//                   workgroups, so the slot is not rewritten while it may still be read)
//   hc_mix_norm     one pass over a token's S streams that (a) applies the update of the sublayer
//                   that just ran, x_t <- sum_s mix[s][t] x_s + out[t] * y * sigmoid(gate + gate_b),
//                   all streams from the old values, and (b) reads the next sublayer's input out of the
//                   new values, u = sum_s in[s] x_s, h = (u - mean) / sqrt(var + eps) * w, written in
//                   fp32 and, for bf16 models, also in bf16 (the GEMM input).  Either half may be absent.
//
// All arithmetic is fp32; the variance is the mean of squared deviations (two passes over the row,
// which sits in LDS).  One workgroup per token row.
#include "../common.h"

using namespace dgi;

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf16_to_f32(*p); }

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

constexpr int MAXS = 8;      // streams

__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int w = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  float r = 0.f;
  for (int i = 0; i < nw; ++i) r += red[i];
  return r;
}

template <typename T>
__global__ __launch_bounds__(256) void embed_streams_kernel(
    float* __restrict__ xs, int S, int NT, int W, const int* __restrict__ ids, const int* __restrict__ positions,
    const int* __restrict__ row_seq, const int* __restrict__ seq_row0, const int* __restrict__ seq_slots,
    const int* __restrict__ prev_tok, const T* __restrict__ embed, int vocab, const T* __restrict__ bigram,
    int buckets, long long mul_prev, long long mul_cur, const T* __restrict__ pos_table, int max_pos) {
  const int row = blockIdx.x;
  int tok = ids[row];
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  const int pos = positions[row];
  const T* e = embed + (size_t)tok * W;
  const T* b = nullptr;
  if (bigram) {
    long long br = buckets;
    if (pos > 0) {
      const int seq = row_seq[row];
      const long long prev = row == seq_row0[seq] ? prev_tok[seq_slots[seq]] : ids[row - 1];
      br = (prev * mul_prev + (long long)ids[row] * mul_cur) % buckets;
      if (br < 0) br += buckets;
    }
    b = bigram + (size_t)br * W;
  }
  const T* p = nullptr;
  if (pos_table) p = pos_table + (size_t)(pos < 0 ? 0 : (pos >= max_pos ? max_pos - 1 : pos)) * W;
  for (int w = threadIdx.x; w < W; w += blockDim.x) {
    float v = ldf<T>(e + w);
    if (b) v += ldf<T>(b + w);
    if (p) v += ldf<T>(p + w);
    for (int s = 0; s < S; ++s) xs[((size_t)s * NT + row) * W + w] = v;
  }
}

__global__ void store_last_token_kernel(int* __restrict__ prev_tok, const int* __restrict__ ids,
                                        const int* __restrict__ seq_row0, const int* __restrict__ seq_slots, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int r0 = seq_row0[i], r1 = seq_row0[i + 1];
  if (r1 > r0) prev_tok[seq_slots[i]] = ids[r1 - 1];
}

// V = 4: four consecutive columns per thread (16-byte stream accesses; W, strides and pointers allow it),
// V = 1: any width.  The arithmetic per column is the same.
template <typename T, int V>
__global__ __launch_bounds__(256) void hc_mix_norm_kernel(
    float* __restrict__ xs, int S, int NT, int W, const T* __restrict__ y, int y_stride, const T* __restrict__ gate,
    int gate_stride, const float* __restrict__ gate_b, const float* __restrict__ mixm, const float* __restrict__ outc,
    const float* __restrict__ in_next, const float* __restrict__ norm_w, float eps, float* __restrict__ h32,
    T* __restrict__ hd) {
  extern __shared__ float us[];          // [W] the read-out row
  __shared__ float red[8];
  __shared__ float cm[MAXS * MAXS], co[MAXS], ci[MAXS];
  const int row = blockIdx.x;
  if (threadIdx.x < S * S && y) cm[threadIdx.x] = mixm[threadIdx.x];
  if (threadIdx.x < S) {
    if (y) co[threadIdx.x] = outc[threadIdx.x];
    if (in_next) ci[threadIdx.x] = in_next[threadIdx.x];
  }
  __syncthreads();
  float sum = 0.f;
  for (int w = threadIdx.x * V; w < W; w += blockDim.x * V) {
    float x[MAXS][V];
#pragma unroll
    for (int s = 0; s < MAXS; ++s) {
      if (s < S) {
        if constexpr (V == 4) ld4<float>(xs + ((size_t)s * NT + row) * W + w, x[s]);
        else x[s][0] = xs[((size_t)s * NT + row) * W + w];
      } else {
#pragma unroll
        for (int k = 0; k < V; ++k) x[s][k] = 0.f;
      }
    }
    if (y) {
      float yy[V], gg[V], gb[V];
      if constexpr (V == 4) {
        ld4<T>(y + (size_t)row * y_stride + w, yy);
        if (gate) { ld4<T>(gate + (size_t)row * gate_stride + w, gg); ld4<float>(gate_b + w, gb); }
      } else {
        yy[0] = ldf<T>(y + (size_t)row * y_stride + w);
        if (gate) { gg[0] = ldf<T>(gate + (size_t)row * gate_stride + w); gb[0] = gate_b[w]; }
      }
      if (gate) {
#pragma unroll
        for (int k = 0; k < V; ++k) yy[k] *= 1.f / (1.f + expf(-(gg[k] + gb[k])));
      }
      float nx[MAXS][V];
#pragma unroll
      for (int t = 0; t < MAXS; ++t) {
#pragma unroll
        for (int k = 0; k < V; ++k) {
          float a = 0.f;
          if (t < S) {
#pragma unroll
            for (int s = 0; s < MAXS; ++s)
              if (s < S) a += cm[s * S + t] * x[s][k];
            a += co[t] * yy[k];
          }
          nx[t][k] = a;
        }
        if (t < S) {
          if constexpr (V == 4)
            *reinterpret_cast<float4*>(xs + ((size_t)t * NT + row) * W + w) = make_float4(nx[t][0], nx[t][1], nx[t][2], nx[t][3]);
          else xs[((size_t)t * NT + row) * W + w] = nx[t][0];
        }
      }
#pragma unroll
      for (int t = 0; t < MAXS; ++t)
#pragma unroll
        for (int k = 0; k < V; ++k) x[t][k] = nx[t][k];
    }
    if (in_next) {
#pragma unroll
      for (int k = 0; k < V; ++k) {
        float u = 0.f;
#pragma unroll
        for (int s = 0; s < MAXS; ++s)
          if (s < S) u += ci[s] * x[s][k];
        us[w + k] = u;
        sum += u;
      }
    }
  }
  if (!in_next) return;
  const float mean = block_sum(sum, red) / (float)W;
  float sq = 0.f;
  for (int w = threadIdx.x; w < W; w += blockDim.x) {
    const float d = us[w] - mean;
    sq += d * d;
  }
  const float rstd = 1.f / sqrtf(block_sum(sq, red) / (float)W + eps);
  for (int w = threadIdx.x; w < W; w += blockDim.x) {
    const float h = (us[w] - mean) * rstd * norm_w[w];
    h32[(size_t)row * W + w] = h;
    if constexpr (sizeof(T) == 2) {
      if (hd) hd[(size_t)row * W + w] = f32_to_bf16(h);
    }
  }
}

}  // namespace

extern "C" int dgi_embed_streams(float* xs, int S, int T, int W, const int* ids, const int* positions,
                                 const int* row_seq, const int* seq_row0, const int* seq_slots, int n_seq,
                                 int* prev_tok, const void* embed, int vocab, const void* bigram, int buckets,
                                 long long mul_prev, long long mul_cur, const void* pos_table, int max_pos, int is_f32,
                                 hipStream_t s) {
  if (T == 0) return 0;
  if (S < 1 || S > MAXS) return -2;
  if (bigram && buckets <= 0) return -3;
  if (is_f32)
    embed_streams_kernel<float><<<T, 256, 0, s>>>(xs, S, T, W, ids, positions, row_seq, seq_row0, seq_slots, prev_tok,
                                                  (const float*)embed, vocab, (const float*)bigram, buckets, mul_prev,
                                                  mul_cur, (const float*)pos_table, max_pos);
  else
    embed_streams_kernel<uint16_t><<<T, 256, 0, s>>>(xs, S, T, W, ids, positions, row_seq, seq_row0, seq_slots,
                                                     prev_tok, (const uint16_t*)embed, vocab, (const uint16_t*)bigram,
                                                     buckets, mul_prev, mul_cur, (const uint16_t*)pos_table, max_pos);
  DGI_CHECK_LAUNCH();
  store_last_token_kernel<<<(n_seq + 255) / 256, 256, 0, s>>>(prev_tok, ids, seq_row0, seq_slots, n_seq);
  DGI_CHECK_LAUNCH();
  return 0;
}

// y / gate: bf16 (is_f32 0) or fp32 rows with their own strides, or null; hd: bf16 copy of h (bf16 models)
extern "C" int dgi_hc_mix_norm(float* xs, int S, int T, int W, const void* y, int y_stride, const void* gate,
                               int gate_stride, const float* gate_b, const float* mixm, const float* outc,
                               const float* in_next, const float* norm_w, float eps, float* h32, void* hd, int is_f32,
                               hipStream_t s) {
  if (T == 0) return 0;
  if (S < 1 || S > MAXS) return -2;
  if (W > 16384) return -3;
  const size_t lds = in_next ? (size_t)W * 4 : 0;
  const bool vec = W % 4 == 0 && y_stride % 4 == 0 && gate_stride % 4 == 0 &&
                   (((uintptr_t)xs | (uintptr_t)y | (uintptr_t)gate | (uintptr_t)gate_b) & 15) == 0;
  if (is_f32) {
    if (hd) return -4;
    if (vec)
      hc_mix_norm_kernel<float, 4><<<T, 256, lds, s>>>(xs, S, T, W, (const float*)y, y_stride, (const float*)gate,
                                                       gate_stride, gate_b, mixm, outc, in_next, norm_w, eps, h32, nullptr);
    else
      hc_mix_norm_kernel<float, 1><<<T, 256, lds, s>>>(xs, S, T, W, (const float*)y, y_stride, (const float*)gate,
                                                       gate_stride, gate_b, mixm, outc, in_next, norm_w, eps, h32, nullptr);
  } else {
    if (vec)
      hc_mix_norm_kernel<uint16_t, 4><<<T, 256, lds, s>>>(xs, S, T, W, (const uint16_t*)y, y_stride, (const uint16_t*)gate,
                                                          gate_stride, gate_b, mixm, outc, in_next, norm_w, eps, h32,
                                                          (uint16_t*)hd);
    else
      hc_mix_norm_kernel<uint16_t, 1><<<T, 256, lds, s>>>(xs, S, T, W, (const uint16_t*)y, y_stride, (const uint16_t*)gate,
                                                          gate_stride, gate_b, mixm, outc, in_next, norm_w, eps, h32,
                                                          (uint16_t*)hd);
  }
  DGI_CHECK_LAUNCH();
  return 0;
}
