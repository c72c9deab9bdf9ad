// Tiled paged attention for prompt portions on the matrix cores (bfloat16).
//
// One block per (tile of 32 QW queries of one request, head), QW = 2, 1 or 4.  Its QW KS waves
// are arranged as QW x KS: a wave owns 32 consecutive queries and, of every tile of keys, KR
// runs of 32 keys, with an online-softmax state of its own; the KS states of a query are merged
// through LDS at the end.  (Tiles of 32 queries are for steps whose tiles of 64 would leave
// half of the compute units without a block: a prompt portion beside decoded tokens.  Tiles of
// 128 queries, four waves that each take all 64 keys of a tile, are for long prompts: what
// bounds the tiles of 64 there is what a compute unit takes in, 16 KB of keys and values per
// 4,096 scores, and what a wave does per tile beside the scores; both are halved.)
// A request's longest tile decides how long the launch takes, and splitting its keys over
// waves shortens exactly that.  Keys and values are visited 32 KS at a time through the
// request's block table, from the first key any query of the tile may see to the tile's last
// position (the portion's own keys are already in the pages, so a whole prompt, a later
// portion and a portion that starts in the middle of a page are one case).
//
// Loads.  The rows of the block table that the tile needs are copied into LDS once.  K and V
// tiles then go from the pages straight into LDS (global_load_lds_dwordx4), several tiles
// ahead of the one being multiplied, into a ring of stages; a tile lies there as in the
// pages, [64 keys][head_dim], with the 16-byte pieces of a row rotated by the key's number
// so that the operand reads below spread over the LDS banks.  Per tile there is one wait
// (own loads of that tile have landed) and one barrier.
//
// Per key tile and wave:
//   * S^T = K Q^T with v_mfma_f32_32x32x16_bf16: keys are the rows, queries the columns, so
//     a lane holds 16 keys of its own query per block of 32 keys;
//   * scale, causal/window mask (skipped where the whole tile is visible), online softmax in
//     float per query (running max and sum, as src/kernels/triton_paged_attention.py:275-331)
//     in units of log 2, probabilities rounded to bfloat16;
//   * O^T += V^T P^T with the same instruction: head dimensions are the rows.  The row operand
//     needs, per lane, consecutive keys of one head dimension, which ds_read_b64_tr_b16
//     delivers from the row-major tile: within 16 lanes, lane r points at 4 dimensions of key
//     r / 4 and receives dimension r of four keys.
//
// head_dim is any multiple of 16 up to 256; other sizes, and block tables wider than
// AP_TABLE_MAX pages, run on the row-wise kernel.
#include <math.h>

#include "common.h"
#include "pagedserve_hip.h"

#include "attention_prefill_block.h"

// What the host has to know of this file's constants to list a step's tiles.
extern "C" int ps_attention_prefill_query_tile(void) { return AP_QUERIES; }
extern "C" int ps_attention_prefill_small_tile(void) { return AP_QUERIES / 2; }
extern "C" int ps_attention_prefill_large_tile(void) { return AP_QUERIES * 2; }
extern "C" int ps_attention_prefill_large_tile_head_dim(void) { return AP_LARGE_HEAD_DIM; }
extern "C" int ps_attention_prefill_table_max(void) { return AP_TABLE_MAX; }

extern "C" int ps_attention_prefill(const void* q, int64_t q_stride, const void* k_pool,
                                    const void* v_pool, void* out, int64_t out_stride,
                                    const int* tile_item, const int* tile_q0, int tiles,
                                    const int* cu_tokens, const int* kv_lens, const int* tables,
                                    int table_width, int heads, int kv_heads, int head_dim,
                                    int page_size, int num_pages, float scale, int window,
                                    int max_kv_len, int query_tile, int dtype, void* stream) {
  PS_REQUIRE(tiles >= 0 && heads > 0 && kv_heads > 0 && page_size > 0 && num_pages > 0 &&
                 table_width > 0,
             "ps_attention_prefill: bad sizes");
  PS_REQUIRE(dtype == PS_BF16, "ps_attention_prefill: bfloat16 only (dtype %d)", dtype);
  PS_REQUIRE(heads % kv_heads == 0,
             "ps_attention_prefill: heads (%d) must be a multiple of kv_heads (%d)", heads, kv_heads);
  PS_REQUIRE(head_dim > 0 && head_dim % 16 == 0 && head_dim <= 256,
             "ps_attention_prefill: head_dim %d must be a multiple of 16 up to 256", head_dim);
  PS_REQUIRE(window >= 0 && tiles <= 65535, "ps_attention_prefill: bad window or too many tiles (%d)", tiles);
  PS_REQUIRE(query_tile == AP_QUERIES || (query_tile == AP_QUERIES / 2 && head_dim <= 128) ||
                 (query_tile == AP_QUERIES * 2 && head_dim <= AP_LARGE_HEAD_DIM),
             "ps_attention_prefill: tiles of %d, (head sizes up to 128) %d or (head sizes up to %d) %d "
             "queries, not %d", AP_QUERIES, AP_QUERIES / 2, AP_LARGE_HEAD_DIM, AP_QUERIES * 2, query_tile);
  PS_REQUIRE((int64_t)num_pages * kv_heads * page_size < ((int64_t)1 << 32),
             "ps_attention_prefill: a pool of %d pages x %d heads x %d keys has 2^32 key rows or more",
             num_pages, kv_heads, page_size);
  PS_REQUIRE(scale > 0.f, "ps_attention_prefill: the score scale must be positive, got %g", scale);
  PS_REQUIRE(table_width <= AP_TABLE_MAX,
             "ps_attention_prefill: block tables of %d pages exceed the %d that a tile keeps",
             table_width, AP_TABLE_MAX);
  PS_REQUIRE((q_stride % 8) == 0 && ((uintptr_t)q % 16) == 0 && (out_stride % 4) == 0 &&
                 ((uintptr_t)out % 8) == 0,
             "ps_attention_prefill: q and out rows must allow 16- and 8-byte accesses");
  if (tiles == 0) return 0;
  int page_shift = -1;
  if ((page_size & (page_size - 1)) == 0) {
    page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
  }
  hipStream_t s = (hipStream_t)stream;
  dim3 grid(heads, tiles);
  // With few blocks, up to two per compute unit, which hold them all at once (128 registers and
  // 72 KB of LDS each), four waves along the keys shorten the longest block (2 x 1,024 tokens of
  // 12 heads, 384 blocks: 16.6 against 18.6 us; of 16 heads, 512 blocks: 17.3 against 18.7; 3 x
  // 1,024 of 12 heads, 576 blocks: level; 768 blocks: 24.5 against 20.6).  If the caller knows of
  // no long context that does not pay; with many, smaller blocks balance better.
  const bool wide = (int64_t)tiles * heads <= ps_compute_units() * 2 &&
                    (max_kv_len <= 0 || max_kv_len >= 512);
  // tiles of 32 queries: one wave along the queries, four along the keys (two such blocks
  // share a compute unit)
#define PS_LAUNCH_AP_SMALL(NDB)                                                                 \
  hipLaunchKernelGGL((attention_prefill_kernel<NDB, 4, 1>), grid, dim3(256), 0, s,              \
                     (const bf16_t*)q, q_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool,  \
                     (bf16_t*)out, out_stride, tile_item, tile_q0, cu_tokens, kv_lens, tables,  \
                     table_width, heads, kv_heads, page_size, page_shift, num_pages, scale, window)
  // tiles of 128 queries: four waves along the queries, each with all 64 keys of a tile: a
  // block takes in half as many keys and values per score, and a wave's work per tile that
  // does not depend on the scores (addresses, waits, checks) is spread over twice as many
#define PS_LAUNCH_AP_LARGE_TILE(NDB)                                                            \
  hipLaunchKernelGGL((attention_prefill_kernel<NDB, 1, 4, 2>), grid, dim3(256), 0, s,           \
                     (const bf16_t*)q, q_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool,  \
                     (bf16_t*)out, out_stride, tile_item, tile_q0, cu_tokens, kv_lens, tables,  \
                     table_width, heads, kv_heads, page_size, page_shift, num_pages, scale, window)
  if (query_tile == AP_QUERIES * 2) {
    static_assert(AP_LARGE_HEAD_DIM == 64, "the cases below");
    switch (head_dim / 16) {
      case 1: PS_LAUNCH_AP_LARGE_TILE(1); break;
      case 2: PS_LAUNCH_AP_LARGE_TILE(2); break;
      case 3: PS_LAUNCH_AP_LARGE_TILE(3); break;
      default: PS_LAUNCH_AP_LARGE_TILE(4); break;
    }
    PS_CHECK_LAUNCH("ps_attention_prefill");
    return 0;
  }
#undef PS_LAUNCH_AP_LARGE_TILE
  if (query_tile != AP_QUERIES) {
    switch (head_dim / 16) {
      case 1: PS_LAUNCH_AP_SMALL(1); break;
      case 2: PS_LAUNCH_AP_SMALL(2); break;
      case 3: PS_LAUNCH_AP_SMALL(3); break;
      case 4: PS_LAUNCH_AP_SMALL(4); break;
      case 5: PS_LAUNCH_AP_SMALL(5); break;
      case 6: PS_LAUNCH_AP_SMALL(6); break;
      case 7: PS_LAUNCH_AP_SMALL(7); break;
      default: PS_LAUNCH_AP_SMALL(8); break;
    }
    PS_CHECK_LAUNCH("ps_attention_prefill");
    return 0;
  }
#undef PS_LAUNCH_AP_SMALL
#define PS_LAUNCH_AP(NDB)                                                                       \
  do {                                                                                          \
    if (wide)                                                                                   \
      hipLaunchKernelGGL((attention_prefill_kernel<NDB, 4>), grid, dim3(512), 0, s,             \
                         (const bf16_t*)q, q_stride, (const bf16_t*)k_pool,                     \
                         (const bf16_t*)v_pool, (bf16_t*)out, out_stride, tile_item, tile_q0,   \
                         cu_tokens, kv_lens, tables, table_width, heads, kv_heads, page_size,   \
                         page_shift, num_pages, scale, window);                                 \
    else                                                                                        \
      hipLaunchKernelGGL((attention_prefill_kernel<NDB, 2>), grid, dim3(256), 0, s,             \
                         (const bf16_t*)q, q_stride, (const bf16_t*)k_pool,                     \
                         (const bf16_t*)v_pool, (bf16_t*)out, out_stride, tile_item, tile_q0,   \
                         cu_tokens, kv_lens, tables, table_width, heads, kv_heads, page_size,   \
                         page_shift, num_pages, scale, window);                                 \
  } while (0)
  switch (head_dim / 16) {
    case 1: PS_LAUNCH_AP(1); break;
    case 2: PS_LAUNCH_AP(2); break;
    case 3: PS_LAUNCH_AP(3); break;
    case 4: PS_LAUNCH_AP(4); break;
    case 5: PS_LAUNCH_AP(5); break;
    case 6: PS_LAUNCH_AP(6); break;
    case 7: PS_LAUNCH_AP(7); break;
    case 8: PS_LAUNCH_AP(8); break;
    // head sizes beyond 128: blocks of four waves only, each wave with the whole register
    // file of its SIMD (accumulators and operands of 256 dimensions take 450 registers)
#define PS_LAUNCH_AP_LARGE(NDB)                                                                 \
  hipLaunchKernelGGL((attention_prefill_kernel<NDB, 2>), grid, dim3(256), 0, s,                 \
                     (const bf16_t*)q, q_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool,  \
                     (bf16_t*)out, out_stride, tile_item, tile_q0, cu_tokens, kv_lens, tables,  \
                     table_width, heads, kv_heads, page_size, page_shift, num_pages, scale, window)
    case 9: PS_LAUNCH_AP_LARGE(9); break;
    case 10: PS_LAUNCH_AP_LARGE(10); break;
    case 11: PS_LAUNCH_AP_LARGE(11); break;
    case 12: PS_LAUNCH_AP_LARGE(12); break;
    case 13: PS_LAUNCH_AP_LARGE(13); break;
    case 14: PS_LAUNCH_AP_LARGE(14); break;
    case 15: PS_LAUNCH_AP_LARGE(15); break;
    default: PS_LAUNCH_AP_LARGE(16); break;
#undef PS_LAUNCH_AP_LARGE
  }
#undef PS_LAUNCH_AP
  PS_CHECK_LAUNCH("ps_attention_prefill");
  return 0;
}
