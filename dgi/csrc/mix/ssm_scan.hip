// dgi/csrc/mix/ssm_scan.hip — Mamba-2 selective scan over packed rows with the state in a slot, and
// the gated group RMS norm that follows it.
//
// Per sequence of the step and head h (group g = h / (heads / G)), for its rows in order:
//
//     dt  = softplus(dt_raw[t][h] + dt_bias[h])             a = exp(-exp(a_log[h]) * dt)
//     S  <- a * S + dt * B_t x_t^T                          S: [N, dv] fp32
//     y_t = S^T C_t + d_skip[h] * x_t
//
// S starts as state[slot][h] (stored transposed, [dv][N]; zero when the portion starts at position 0) and goes back there after
// the last row; decode rows (one token) and prompt portions run the same code, so the result does
// not depend on how a prompt was cut.  x | B | C come as one fp32 row (the convolution's output).
//
// Work split: a workgroup owns (sequence, head, 16 value columns); thread (column v, n-lane l) keeps
// S[n][v] for n = 4 l + 64 q + j in registers, so the y reduction over n is four DPP rotate-adds inside a
// 16-lane row.  The serial loop over tokens never waits for global memory: B, C, x and the step
// sizes of 16 tokens are staged in LDS (the next tile's loads are in flight, in registers, while the
// current one is consumed; softplus and the decay are computed once per token while staging), and a
// token costs two 16-byte LDS reads per four state values.  The state is stored value-major,
// [slot][head][v][n], so a thread's values are contiguous.  Everything is fp32 (softplus in its
// overflow-free form max(z, 0) + log1p(exp(-|z|))).
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

// Sum over the 16 lanes of a DPP row (lanes 16 r .. 16 r + 15), result in every lane: four rotate-and-add
// steps in the VALU (row_ror 8, 4, 2, 1) — no trip through the LDS permute unit, which a per-token
// reduction inside a serial loop would otherwise wait for four times.
__device__ __forceinline__ float row16_sum(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x122, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x121, 0xf, 0xf, false));
  return v;
}

constexpr int COLS = 16;     // value columns per workgroup
constexpr int NL = 16;       // n-lanes per column
constexpr int TT = 16;       // tokens per staged tile

// NQ: float4 groups of state per thread (N <= 64 * NQ); thread (column v, n-lane l) owns
// n = 4 l + 64 q + j, j < 4.  LDS tile: B [TT][NP], C [TT][NP] (NP = 64 NQ, zero beyond N), x [TT][COLS],
// dt [TT], decay [TT].
template <typename TD, int NQ>
__global__ __launch_bounds__(COLS * NL) void ssm_scan_kernel(
    float* __restrict__ y, const float* __restrict__ xbc, int xbc_stride, const TD* __restrict__ dt_raw, int dt_stride,
    const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ d_skip,
    float* __restrict__ state, const int* __restrict__ positions, const int* __restrict__ seq_row0,
    const int* __restrict__ seq_slots, int heads, int dv, int N, int G, int mode, int L, int nchunks,
    float* __restrict__ ws, float* __restrict__ wsd) {
  constexpr int NP = 64 * NQ;
  constexpr int PB = (TT * NP) / (COLS * NL);          // B (and C) values a thread stages per tile
  extern __shared__ __attribute__((aligned(16))) float sm[];
  float* sB = sm;
  float* sC = sB + TT * NP;
  float* sX = sC + TT * NP;
  float* sDt = sX + TT * COLS;
  float* sDa = sDt + TT;
  // mode 0: a workgroup runs a sequence's whole portion from its state slot and back.  Modes 1 and 3
  // run one chunk of L rows (blockIdx.x = sequence * nchunks + chunk): 1 from a zero state into the
  // workspace (no outputs; also the chunk's summed log decay), 3 from the workspace state into y.
  const int seq = mode ? blockIdx.x / nchunks : blockIdx.x, h = blockIdx.y;
  const int chunk = mode ? blockIdx.x - seq * nchunks : 0;
  const int tid = threadIdx.x;
  const int l = tid & (NL - 1), col = tid >> 4;
  const int v = blockIdx.z * COLS + col;
  const int s0 = seq_row0[seq], s1 = seq_row0[seq + 1];
  const int r0 = s0 + chunk * L, r1 = mode ? min(s1, r0 + L) : s1;
  if (r1 <= r0) return;
  const bool vok = v < dv;
  const int g = h / (heads / G);
  const int inner = heads * dv;
  const float* bp = xbc + inner + (size_t)g * N;
  const float* cp = bp + (size_t)G * N;
  float* sp = mode ? ws + (((size_t)blockIdx.x * heads + h) * dv + v) * N
                   : state + (((size_t)seq_slots[seq] * heads + h) * dv + v) * N;     // [..][head][v][n]
  const bool fresh = mode == 1 || (mode == 0 && positions[s0] == 0);
  float ldec = 0.f;                                    // mode 1: sum of log decays (threads < TT)
  float S[NQ][4];
#pragma unroll
  for (int q = 0; q < NQ; ++q)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = 4 * l + 64 * q + j;
      S[q][j] = (!fresh && vok && n < N) ? sp[n] : 0.f;
    }
  const float na = -expf(a_log[h]), bias = dt_bias[h], dsk = d_skip[h];

  float rb[PB], rc[PB], rx = 0.f, rdt = 0.f;
  auto prefetch = [&](int t0) {
#pragma unroll
    for (int i = 0; i < PB; ++i) {
      const int idx = tid + i * (COLS * NL);
      const int tok = idx / NP, n = idx - tok * NP;
      const bool ok = t0 + tok < r1 && n < N;
      rb[i] = ok ? bp[(size_t)(t0 + tok) * xbc_stride + n] : 0.f;
      rc[i] = ok ? cp[(size_t)(t0 + tok) * xbc_stride + n] : 0.f;
    }
    {
      const int tok = tid / COLS, c = tid - tok * COLS;            // TT * COLS == blockDim
      const int vv = blockIdx.z * COLS + c;
      rx = (t0 + tok < r1 && vv < dv) ? xbc[(size_t)(t0 + tok) * xbc_stride + (size_t)h * dv + vv] : 0.f;
    }
    if (tid < TT) rdt = t0 + tid < r1 ? ldf<TD>(dt_raw + (size_t)(t0 + tid) * dt_stride + h) : 0.f;
  };
  prefetch(r0);
  for (int t0 = r0; t0 < r1; t0 += TT) {
    __syncthreads();                                     // the previous tile is fully consumed
#pragma unroll
    for (int i = 0; i < PB; ++i) {
      sB[tid + i * (COLS * NL)] = rb[i];
      sC[tid + i * (COLS * NL)] = rc[i];
    }
    sX[tid] = rx;
    if (tid < TT) {
      const float z = rdt + bias;
      const float dt = fmaxf(z, 0.f) + log1pf(expf(-fabsf(z)));
      sDt[tid] = dt;
      sDa[tid] = expf(na * dt);
      if (t0 + tid < r1) ldec += na * dt;
    }
    __syncthreads();
    if (t0 + TT < r1) prefetch(t0 + TT);                 // in flight while this tile is consumed
    const int cnt = min(TT, r1 - t0);
    for (int k = 0; k < cnt; ++k) {
      const float a = sDa[k], xv = sX[k * COLS + col];
      const float dx = sDt[k] * xv;
      float acc = 0.f;
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        const float4 b4 = *reinterpret_cast<const float4*>(sB + k * NP + 4 * l + 64 * q);
        const float4 c4 = *reinterpret_cast<const float4*>(sC + k * NP + 4 * l + 64 * q);
        S[q][0] = a * S[q][0] + b4.x * dx;
        S[q][1] = a * S[q][1] + b4.y * dx;
        S[q][2] = a * S[q][2] + b4.z * dx;
        S[q][3] = a * S[q][3] + b4.w * dx;
        acc += S[q][0] * c4.x + S[q][1] * c4.y + S[q][2] * c4.z + S[q][3] * c4.w;
      }
      if (mode != 1) {                                   // mode 1: chunk states only, no outputs
        acc = row16_sum(acc);
        if (l == 0 && vok) y[(size_t)(t0 + k) * inner + (size_t)h * dv + v] = acc + dsk * xv;
      }
    }
  }
  if (mode == 1 && blockIdx.z == 0 && tid < TT) {      // TT lanes of wave 0
#pragma unroll
    for (int o = TT / 2; o > 0; o >>= 1) ldec += __shfl_xor(ldec, o, 64);
    if (tid == 0) wsd[(size_t)blockIdx.x * heads + h] = ldec;
  }
  if (vok && mode != 3) {
#pragma unroll
    for (int q = 0; q < NQ; ++q)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int n = 4 * l + 64 * q + j;
        if (n < N) sp[n] = S[q][j];
      }
  }
}

// Between the two chunk passes: per (sequence, head, state element) walk the chunks in order,
// S_in[c] <- S;  S <- exp(logdecay[c]) * S + S_local[c], starting from the state slot (zero at
// position 0); the workspace then holds every chunk's incoming state and the slot the final one.
__global__ __launch_bounds__(256) void ssm_chunk_states_kernel(
    float* __restrict__ ws, const float* __restrict__ wsd, float* __restrict__ state, const int* __restrict__ positions,
    const int* __restrict__ seq_row0, const int* __restrict__ seq_slots, int heads, int per_head, int L, int nchunks) {
  const int seq = blockIdx.x, h = blockIdx.y;
  const int e = blockIdx.z * 256 + threadIdx.x;
  if (e >= per_head) return;
  const int s0 = seq_row0[seq], n = seq_row0[seq + 1] - s0;
  if (n <= 0) return;
  float* sp = state + ((size_t)seq_slots[seq] * heads + h) * per_head + e;
  float S = positions[s0] == 0 ? 0.f : *sp;
  const int nc = (n + L - 1) / L;
  for (int c = 0; c < nc; ++c) {
    float* wp = ws + (((size_t)seq * nchunks + c) * heads + h) * per_head + e;
    const float loc = *wp;
    *wp = S;
    S = expf(wsd[((size_t)seq * nchunks + c) * heads + h]) * S + loc;
  }
  *sp = S;
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

// One pass: a group of up to 256 * 4 * VPT values stays in registers between the sum of squares and the
// store (y and z are read once); groups in fours of columns, 16-byte accesses.
template <typename TZ, typename TO, int VPT>
__global__ __launch_bounds__(256) void gated_group_norm_reg_kernel(
    TO* __restrict__ out, const float* __restrict__ y, const TZ* __restrict__ z, int z_stride,
    const float* __restrict__ w, int C, int groups, float eps) {
  __shared__ float red[4];
  const int row = blockIdx.x, grp = blockIdx.y;
  const int gs = C / groups;
  const float* yp = y + (size_t)row * C + (size_t)grp * gs;
  const TZ* zp = z + (size_t)row * z_stride + (size_t)grp * gs;
  float gv[VPT][4];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int c = (threadIdx.x + 256 * i) * 4;
    if (c < gs) {
      float yy[4], zz[4];
      ld4<float>(yp + c, yy);
      ld4<TZ>(zp + c, zz);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        gv[i][k] = yy[k] * zz[k] / (1.f + expf(-zz[k]));
        ss += gv[i][k] * gv[i][k];
      }
    }
  }
  ss = wave_sum(ss);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float r = 1.f / sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)gs + eps);
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int c = (threadIdx.x + 256 * i) * 4;
    if (c < gs) {
      float ww[4], o[4];
      ld4<float>(w + (size_t)grp * gs + c, ww);
#pragma unroll
      for (int k = 0; k < 4; ++k) o[k] = gv[i][k] * r * ww[k];
      st4<TO>(out + (size_t)row * C + (size_t)grp * gs + c, o);
    }
  }
}

}  // namespace

// ws / wsd: workspace for the chunked form ([n_seq * nchunks][heads][dv][N] states and [n_seq * nchunks][heads]
// log decays) or null: one pass, sequence by sequence.  The chunked form splits every portion into chunks
// of L rows that run in parallel (local states from zero, a short serial pass over the chunk states, then
// the outputs from each chunk's incoming state): twice the recurrence work, nchunks times the workgroups.
// It reassociates the fp32 sums, so fp32 models keep the one-pass form.
extern "C" int dgi_ssm_scan(float* y, const float* xbc, int xbc_stride, const void* dt_raw, int dt_f32, int dt_stride,
                            const float* dt_bias, const float* a_log, const float* d_skip, float* state,
                            const int* positions, const int* seq_row0, const int* seq_slots, int n_seq, int heads,
                            int dv, int N, int G, float* ws, float* wsd, int L, int nchunks, hipStream_t s) {
  if (n_seq == 0) return 0;
  if (G <= 0 || heads % G) return -2;
  if (N > 256 || N <= 0 || dv <= 0) return -3;
  if (ws && (L < 1 || nchunks < 1 || !wsd)) return -5;
  if (heads > 65535 || (dv + COLS - 1) / COLS > 65535) return -4;
  const int nq = (N + 63) / 64;
  auto launch = [&](int mode) {
    const dim3 grid(mode ? n_seq * nchunks : n_seq, heads, (dv + COLS - 1) / COLS);
#define DGI_SCAN(TD, NQ)                                                                                                \
  ssm_scan_kernel<TD, NQ><<<grid, COLS * NL, (size_t)(2 * TT * 64 * NQ + TT * COLS + 2 * TT) * 4, s>>>(             \
      y, xbc, xbc_stride, (const TD*)dt_raw, dt_stride, dt_bias, a_log, d_skip, state, positions, seq_row0, seq_slots, \
      heads, dv, N, G, mode, L, nchunks, ws, wsd)
    if (dt_f32) {
      if (nq <= 1) DGI_SCAN(float, 1); else if (nq <= 2) DGI_SCAN(float, 2); else DGI_SCAN(float, 4);
    } else {
      if (nq <= 1) DGI_SCAN(uint16_t, 1); else if (nq <= 2) DGI_SCAN(uint16_t, 2); else DGI_SCAN(uint16_t, 4);
    }
#undef DGI_SCAN
  };
  if (!ws) {
    launch(0);
    DGI_CHECK_LAUNCH();
    return 0;
  }
  launch(1);
  DGI_CHECK_LAUNCH();
  const int per_head = dv * N;
  ssm_chunk_states_kernel<<<dim3(n_seq, heads, (per_head + 255) / 256), 256, 0, s>>>(ws, wsd, state, positions, seq_row0,
                                                                                      seq_slots, heads, per_head, L, nchunks);
  DGI_CHECK_LAUNCH();
  launch(3);
  DGI_CHECK_LAUNCH();
  return 0;
}

extern "C" int dgi_gated_group_norm(void* out, int out_f32, const float* y, const void* z, int z_f32, int z_stride,
                                    const float* w, int T, int C, int groups, float eps, hipStream_t s) {
  if (T == 0) return 0;
  if (groups <= 0 || C % groups || groups > 65535) return -2;
  const dim3 grid(T, groups);
  const int gs = C / groups;
  if (gs % 4 == 0 && gs <= 256 * 4 * 8 && z_stride % 4 == 0 &&
      (((uintptr_t)out | (uintptr_t)y | (uintptr_t)z | (uintptr_t)w) & 15) == 0 && z_f32 == out_f32) {
    if (z_f32) {
      if (gs <= 256 * 4 * 2)
        gated_group_norm_reg_kernel<float, float, 2><<<grid, 256, 0, s>>>((float*)out, y, (const float*)z, z_stride, w, C, groups, eps);
      else
        gated_group_norm_reg_kernel<float, float, 8><<<grid, 256, 0, s>>>((float*)out, y, (const float*)z, z_stride, w, C, groups, eps);
    } else {
      if (gs <= 256 * 4 * 2)
        gated_group_norm_reg_kernel<uint16_t, uint16_t, 2><<<grid, 256, 0, s>>>((uint16_t*)out, y, (const uint16_t*)z, z_stride, w, C, groups, eps);
      else
        gated_group_norm_reg_kernel<uint16_t, uint16_t, 8><<<grid, 256, 0, s>>>((uint16_t*)out, y, (const uint16_t*)z, z_stride, w, C, groups, eps);
    }
    DGI_CHECK_LAUNCH();
    return 0;
  }
  if (z_f32 && out_f32)
    gated_group_norm_kernel<float, float><<<grid, 256, 0, s>>>((float*)out, y, (const float*)z, z_stride, w, C, groups, eps);
  else if (!z_f32 && !out_f32)
    gated_group_norm_kernel<uint16_t, uint16_t><<<grid, 256, 0, s>>>((uint16_t*)out, y, (const uint16_t*)z, z_stride, w, C, groups, eps);
  else
    return -3;
  DGI_CHECK_LAUNCH();
  return 0;
}
