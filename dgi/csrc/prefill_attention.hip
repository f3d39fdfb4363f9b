// dgi/csrc/prefill_attention.hip — varlen causal flash attention over the paged
// KV pool (prefill, chunked prefill, prefix-cache hits, EAGLE tree
// verification).
//
// The reference runs prefill inside HF `generate` / `ModelShard.forward`
// (worker/engines/llm.py:61-69, worker/distributed/model_shard.py:173-228)
// and has no prefix-aware attention.  Here new queries attend over
// [cached prefix | freshly written KV] straight from the block pool.
//
// CDNA4 structure:
//   grid = (q_tiles, n_heads), 256 threads = 4 waves x 32 query rows.
//   K/V tiles of 64 keys are staged through LDS by the whole workgroup:
//     * K image: 256-byte rows, 16-byte chunk XOR-swizzled by (row & 15) so the
//       32-row ds_read_b128 fragment reads are conflict free (guide T2);
//     * V image: chunk XOR (row & 3) << 2 so ds_read_b64_tr_b16 transposed
//       reads (guide T10) are conflict free.
//   Scores are computed swapped, S^T = K Q^T with mfma_f32_32x32x16_bf16, so a
//   lane owns one query: the softmax row reduction is lane-local plus one
//   xor-32 shuffle, and the probabilities are consumed from the accumulator
//   registers as the B operand of O^T += V^T P^T (guide §3 "accumulator tile
//   as the next MFMA's operand").
//   Optional tree mask: for EAGLE verification the last `tree_n` queries of a
//   sequence see the cached prefix plus their ancestors, given as one 64-bit
//   ancestor mask per query (built by tree.hip).
#include "prefill_attention_kernel.h"

using namespace dgi;
using namespace dgi::prefill;

// tiles: int32 [n_tiles, 2] = (sequence index, first query row of the tile_rows-row tile)
extern "C" int dgi_paged_prefill(const void* q, int q_stride, const void* k_cache,
                                 const void* v_cache, const int* block_tables, int bt_stride,
                                 const int* cu_seqlens_q, const int* context_lens, const int* tiles,
                                 int n_tiles, void* out, int out_stride, int nh, int nkv, int hd,
                                 int block_size, float scale, const unsigned long long* tree_mask,
                                 int tree_n, int tile_rows, hipStream_t s) {
  if (n_tiles == 0) return 0;
  if (hd != 128 && hd != 64) return -5;
  if (nh % nkv) return -2;
  if (tree_n > 64) return -6;
  int bs_log2 = 0;
  while ((1 << bs_log2) < block_size) ++bs_log2;
  if ((1 << bs_log2) != block_size) return -4;
  const float scale_log2 = scale * 1.4426950408889634f;
  const int db = (tile_rows >> 16) & 1;          // bit 16: two LDS stages (prefill_attn_kernel DB)
  tile_rows &= 0xffff;
  if (tile_rows != 128 && tile_rows != 256) return -7;
#define DGI_PREFILL(HDV, NWV, DBV)                                                                     \
  prefill_attn_kernel<HDV, NWV, DBV><<<dim3(n_tiles, nh), NWV * 64, 0, s>>>(                           \
      (const uint16_t*)q, q_stride, (const uint16_t*)k_cache, (const uint16_t*)v_cache, block_tables,     \
      bt_stride, cu_seqlens_q, context_lens, tiles, (uint16_t*)out, out_stride, nh, nkv, bs_log2,         \
      scale_log2, tree_mask, tree_n)
  if (hd == 128) {
    if (tile_rows == 256) { if (db) DGI_PREFILL(128, 8, 1); else DGI_PREFILL(128, 8, 0); }
    else { if (db) DGI_PREFILL(128, 4, 1); else DGI_PREFILL(128, 4, 0); }
  } else {
    if (tile_rows == 256) { if (db) DGI_PREFILL(64, 8, 1); else DGI_PREFILL(64, 8, 0); }
    else { if (db) DGI_PREFILL(64, 4, 1); else DGI_PREFILL(64, 4, 0); }
  }
#undef DGI_PREFILL
  DGI_CHECK_LAUNCH();
  return 0;
}
