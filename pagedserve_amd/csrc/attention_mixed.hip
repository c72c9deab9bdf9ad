// The two attention launches of a step that mixes decoded tokens with prompt portions, as one.
//
// Such a step has items of one token, which the split-KV decode kernel takes (a block per
// token and head, bound by the latency of its few rounds of loads), and items of several,
// which the tiled kernel takes (a block per tile of queries and head, bound by its matrix and
// vector instructions).  Launched one after the other, each leaves most of the chip waiting:
// 32 decoded tokens of 12 heads over 500 keys take 15.6 us, a portion of 512 tokens 8.9 us.
// Here both kinds of block run in one grid: the first `decode_blocks` blocks do the work of
// attention_decode_block (four waves, one range of keys, the output written directly), the
// others that of attention_prefill_block (tiles of 64 queries, four waves as 2 x 2, a ring of
// two stages: 40 KB of LDS, so that four blocks of either kind share a compute unit).  A block
// takes the LDS of the larger kind; the two kinds read disjoint rows of `q` and write disjoint
// rows of `out`.  Streams of different priorities or two streams joined by events are the
// alternatives; the second was measured and costs more than it saves (the dependency across
// queues), and a launch "in any order" on one queue is not offered for this hardware.
//
// bfloat16, head sizes of 16 to 64 in steps of 16; other shapes keep the two launches.
#include "attention_decode_block.h"
#include "attention_prefill_block.h"
#include "pagedserve_hip.h"

#define AM_WAVES 4
#define AM_UNROLL 4

template <int NDB, int LPK, bool NT>
__global__ __launch_bounds__(64 * AM_WAVES) void attention_mixed_kernel(
    const bf16_t* __restrict__ q, int64_t q_stride, const bf16_t* __restrict__ k_pool,
    const bf16_t* __restrict__ v_pool, bf16_t* __restrict__ out, int64_t out_stride,
    // the items of one token
    int decode_blocks, const int* __restrict__ tok_list, const int* __restrict__ tok_item,
    const int* __restrict__ tok_pos,
    // the items of several
    const int* __restrict__ tile_item, const int* __restrict__ tile_q0,
    const int* __restrict__ cu_tokens, const int* __restrict__ kv_lens,
    // both
    const int* __restrict__ tables, int table_width, int heads, int kv_heads, int page_size,
    int page_shift, int num_pages, float scale, int window) {
  typedef PrefillLds<NDB, 2, 2, 1> TileLds;
  union Lds {
    TileLds tiles;
    DecodeLds<AM_WAVES> decode;
  };
  __shared__ Lds lds;
  const int block = blockIdx.x;
  if (block < decode_blocks) {
    // tokens fastest, as in the decode kernel's own grid
    const int count = decode_blocks / heads;
    const int head = block / count;
    const int n = block - head * count;
    attention_decode_block<bf16_t, LPK, AM_WAVES, AM_UNROLL, NT>(
        lds.decode, n, head, 0, q, q_stride, k_pool, v_pool, out, out_stride, nullptr, tok_list,
        tok_item, tok_pos, tables, table_width, heads, kv_heads, NDB * 16, page_size, page_shift,
        num_pages, scale * 1.4426950408889634f, window, 1);
  } else {
    // heads fastest, as in the tiled kernel's own grid: the tiles that see the most keys first
    const int rest = block - decode_blocks;
    const int tile_index = rest / heads;
    const int head = rest - tile_index * heads;
    attention_prefill_block<NDB, 2, 2, 1>(lds.tiles, head, tile_index, q, q_stride, k_pool, v_pool, out,
                                          out_stride, tile_item, tile_q0, cu_tokens, kv_lens, tables,
                                          table_width, heads, kv_heads, page_size, page_shift,
                                          num_pages, scale, window);
  }
}

extern "C" int ps_attention_mixed_supported(int dtype, int head_dim, int table_width) {
  return dtype == PS_BF16 && head_dim >= 16 && head_dim <= 64 && head_dim % 16 == 0 &&
         table_width <= AP_TABLE_MAX;
}

extern "C" int ps_attention_mixed(const void* q, int64_t q_stride, const void* k_pool,
                                  const void* v_pool, void* out, int64_t out_stride,
                                  const int* tok_list, int singles, const int* tok_item,
                                  const int* tok_pos, const int* tile_item, const int* tile_q0,
                                  int tiles, const int* cu_tokens, const int* kv_lens,
                                  const int* tables, int table_width, int heads, int kv_heads,
                                  int head_dim, int page_size, int num_pages, float scale,
                                  int window, int dtype, void* stream) {
  PS_REQUIRE(singles >= 0 && tiles >= 0 && heads > 0 && kv_heads > 0 && page_size > 0 &&
                 num_pages > 0 && table_width > 0,
             "ps_attention_mixed: bad sizes");
  PS_REQUIRE(ps_attention_mixed_supported(dtype, head_dim, table_width),
             "ps_attention_mixed: bfloat16, head sizes of 16 to 64 in steps of 16 and block tables of up "
             "to %d pages (dtype %d, head_dim %d, %d pages): launch the two kernels instead",
             AP_TABLE_MAX, dtype, head_dim, table_width);
  PS_REQUIRE(heads % kv_heads == 0, "ps_attention_mixed: heads (%d) must be a multiple of kv_heads (%d)",
             heads, kv_heads);
  PS_REQUIRE(window >= 0 && scale > 0.f, "ps_attention_mixed: bad window or scale");
  PS_REQUIRE(tok_list != nullptr && tok_item != nullptr,
             "ps_attention_mixed: the one-token items are given by their list and the tokens' items");
  PS_REQUIRE((int64_t)num_pages * kv_heads * page_size < ((int64_t)1 << 32),
             "ps_attention_mixed: a pool of %d pages x %d heads x %d keys has 2^32 key rows or more",
             num_pages, kv_heads, page_size);
  PS_REQUIRE((q_stride % 8) == 0 && ((uintptr_t)q % 16) == 0 && (out_stride % 4) == 0 &&
                 ((uintptr_t)out % 8) == 0,
             "ps_attention_mixed: q and out rows must allow 16- and 8-byte accesses");
  const int64_t blocks = (int64_t)singles * heads + (int64_t)tiles * heads;
  PS_REQUIRE(blocks < ((int64_t)1 << 31), "ps_attention_mixed: too many blocks");
  if (blocks == 0) return 0;
  int page_shift = -1;
  if ((page_size & (page_size - 1)) == 0) {
    page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
  }
  hipStream_t s = (hipStream_t)stream;
  const int decode_blocks = singles * heads;
  // as the decode kernel chooses: more blocks of its kind than compute units read their keys
  // without leaving lines in the caches
  const bool streaming = decode_blocks > ps_compute_units();
#define PS_LAUNCH_AM(NDB, LPK, NT)                                                              \
  hipLaunchKernelGGL((attention_mixed_kernel<NDB, LPK, NT>), dim3((unsigned)blocks),            \
                     dim3(64 * AM_WAVES), 0, s, (const bf16_t*)q, q_stride,                     \
                     (const bf16_t*)k_pool, (const bf16_t*)v_pool, (bf16_t*)out, out_stride,    \
                     decode_blocks, tok_list, tok_item, tok_pos, tile_item, tile_q0, cu_tokens, \
                     kv_lens, tables, table_width, heads, kv_heads, page_size, page_shift,      \
                     num_pages, scale, window)
#define PS_LAUNCH_AM_NT(NDB, LPK)     \
  do {                                \
    if (streaming) {                  \
      PS_LAUNCH_AM(NDB, LPK, true);   \
    } else {                          \
      PS_LAUNCH_AM(NDB, LPK, false);  \
    }                                 \
  } while (0)
  switch (head_dim / 16) {
    case 1: PS_LAUNCH_AM_NT(1, 2); break;
    case 2: PS_LAUNCH_AM_NT(2, 4); break;
    case 3: PS_LAUNCH_AM_NT(3, 8); break;
    default: PS_LAUNCH_AM_NT(4, 8); break;
  }
#undef PS_LAUNCH_AM_NT
#undef PS_LAUNCH_AM
  PS_CHECK_LAUNCH("ps_attention_mixed");
  return 0;
}
