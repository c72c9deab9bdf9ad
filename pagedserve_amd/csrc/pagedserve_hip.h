// C interface of libpagedserve_hip.so: the gfx950 kernels of the engine.
//
// Conventions
//   * every function returns 0 on success; otherwise ps_last_error() names the fault
//     (a rejected size, an alignment that a kernel needs, a failed launch);
//   * pointers are device pointers; `stream` is a hipStream_t;
//   * `dtype` is PS_F32 (0) or PS_BF16 (1) and names the storage type of activations,
//     matrices and the cache; norm scales, biases, the residual stream and logits are
//     always float;
//   * matrices are stored [out, in] (row n holds the weights of output n), so a product
//     is C[m, n] = sum_k A[m, k] * W[n, k].
#pragma once

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* ps_last_error(void);
int ps_device_info(int* compute_units, int* lds_bytes, char* arch, int arch_len);

// out[t, :] = scale * table[id(t), :] + (pos_table ? pos_table[positions[t], :] : 0), in float,
// where id(t) = ids[t], or carried[src[t]] if src is given and src[t] >= 0.
int ps_embed(const void* table, const void* pos_table, const int* ids, const int* src,
             const int* carried, const int* positions, float* out, int tokens, int width,
             int vocab, int max_positions, float scale, int dtype, void* stream);

// out[r, :] = norm(x[rows ? rows[r] : r, :]) * gamma (+ beta).  rms != 0: no mean, no beta.
int ps_norm(const float* x, const int* rows, const float* gamma, const float* beta, void* out,
            int n_rows, int width, float eps, int rms, int out_dtype, void* stream);

// C[m, n] = epilogue(sum_k A[m, k] W[n, k] + bias[n]).
//   c_dtype is the storage type of C; PS_EPI_RESIDUAL needs float C and adds into it.
int ps_gemm_nt(const void* a, const void* w, const float* bias, void* c, int m, int n, int k,
               int lda, int ldc, int dtype, int c_dtype, int epilogue, void* stream);

// A linear layer with what may be fused around it.
//   * norm_h != null: the input rows are norm(norm_h[norm_rows ? norm_rows[r] : r]) * gamma
//     (+ beta) instead of `a`; `norm_out` ([m, k] of `dtype`) is scratch for when the norm
//     cannot be fused into the product (it is fused for bfloat16, m <= 16, k <= 1024);
//   * k_pool != null: the output is [q | k | v] columns (q_cols, then kv_cols twice); besides
//     being written to c, the k and v columns of row t are stored in the cache at the page
//     slot of position tok_pos[t] of item tok_item[t] (what ps_kv_write does).
//   * w_packed != null (bfloat16, k a multiple of 64): a second copy of w for the products of
//     few rows, which stream the weights once and are bound by how they read them.  Rows are
//     padded to a multiple of 16; the 16 x 64 tile of rows 16 t .. 16 t + 15 and columns
//     64 s .. 64 s + 63 lies at element ((t * (k / 64) + s) * 1024 as two runs of 512: run h
//     holds, for lane = g * 16 + r (g = 0..3, r = 0..15), the 8 values w[16 t + r][64 s + 16 g +
//     8 h ..]: the order in which a wave's lanes hold the operand of v_mfma_f32_16x16x32_bf16,
//     so that one load of a wave is 1 KB of consecutive memory.
//   * packed activations: between two products of 17 to 64 rows (a decode step of a larger
//     batch) the rows may be kept in the order in which the second product's lanes hold their
//     operand, rows in blocks of 16 and tiles of 16 x 64 as for w_packed; it is bound by the
//     loads of its activations as much as of its weights.  The norm in front of a product is
//     written that way by ps_linear itself; for c the caller asks (c_packed_request, bfloat16
//     output, n a multiple of 64, no residual epilogue, no scatter), is told through c_layout,
//     and passes a_packed to the call that reads the buffer.
typedef struct PsLinearArgs {
  const void* a;
  const void* w;
  const float* bias;
  void* c;
  int m, n, k, lda, ldc;
  int dtype, c_dtype, epilogue;
  const float* norm_h;
  const int* norm_rows;
  const float* gamma;
  const float* beta;
  void* norm_out;
  float eps;
  int rms;
  int ldh;
  void* k_pool;
  void* v_pool;
  const int* tok_item;
  const int* tok_pos;
  const int* tables;
  int table_width, q_cols, kv_cols, head_dim, kv_heads, page_size, num_pages;
  const void* w_packed;   // null, or the copy of w described above
  int a_packed;           // the rows of a lie in the packed activation order (see below)
  int c_packed_request;   // c may be written in that order if the kernel chosen can
  int c_rows;             // rows that c has room for (the packed order rounds m up to 16)
  int norm_out_rows;      // rows that norm_out has room for
  int* c_layout;          // null, or where ps_linear says how it wrote c: 0 rows, 1 packed
  // Null, or: the caller also wants tokens[r] = the column of the largest value of row r of c
  // (the lowest such column on ties), as ps_sample gives it without a temperature.  Float
  // output and the plain epilogue only.  The kernels for few bfloat16 rows do it in their
  // epilogue and *top_done becomes 1; otherwise it becomes 0, nothing is written to tokens,
  // and the caller runs ps_sample.  top_keys: m * 16 * 32 64-bit words, top_ticket: 17 * 64 ints; both
  // zero before the first call and left at zero by every call, and not shared by launches
  // that may overlap.
  int* top_tokens;
  void* top_keys;
  int* top_ticket;
  int* top_done;
  // With a scatter: nobody reads the key and value columns of c (attention takes them from
  // the pages), so a kernel may leave them unwritten; they are unspecified afterwards.  The
  // tiled kernel for many rows does, which takes 40 % off what a prompt's QKV product writes.
  int scatter_only;
} PsLinearArgs;

int ps_linear(const PsLinearArgs* args, void* stream);
int ps_linear_args_size(void);   // sizeof(PsLinearArgs) as this library was built

// Store keys and values of the step's tokens into their pages.
//   k, v: [tokens, kv_heads * head_dim] with row stride `stride`;
//   pools: [pages, kv_heads, page_size, head_dim].
int ps_kv_write(const void* k, const void* v, int64_t stride, void* k_pool, void* v_pool,
                const int* tok_item, const int* tok_pos, const int* tables, int table_width,
                int tokens, int kv_heads, int head_dim, int page_size, int num_pages, int dtype,
                void* stream);

// Attention of `tokens` tokens of the step (those listed in tok_list, or all when it is
// null) over their requests' cached keys 0..position (or the last `window` of them), one
// wave per (token, head).  Any head_dim from 1 to 256; heads must be a multiple of kv_heads.
int ps_attention_rowwise(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                         void* out, int64_t out_stride, const int* tok_list, const int* tok_item,
                         const int* tok_pos, const int* tables, int table_width, int tokens,
                         int heads, int kv_heads, int head_dim, int page_size, int num_pages,
                         float scale, int window, int dtype, void* stream);

// The same result in true 32-bit for the items of several tokens (prompt portions), a block
// of four waves per (tile of ps_attention_tiled_f32_tile() queries, head): float pools, float
// q and out, keys and values through LDS, scores by plain fused multiply-adds.  The tiles are
// listed as for ps_attention_prefill (item and first query of each, cut at the tile size).
// head_dim a multiple of 4 up to 128 (ps_attention_tiled_f32_supported); 16-byte aligned rows.
int ps_attention_tiled_f32_supported(int head_dim);
int ps_attention_tiled_f32_tile();
int ps_attention_tiled_f32(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                           void* out, int64_t out_stride, const int* tile_item, const int* tile_q0,
                           int tiles, const int* cu_tokens, const int* kv_lens, const int* tables,
                           int table_width, int heads, int kv_heads, int head_dim, int page_size,
                           int num_pages, float scale, int window, void* stream);

// The same result for single queries, with each token's keys cut into `splits` ranges that
// run as separate blocks of `waves` (4 or 16) waves; `partial` is scratch of
// count * heads * splits * (head_dim + 2) floats (unused when splits == 1).  head_dim is a
// multiple of 8 up to 256.  tok_item may be null (here and in the two variants below): token t
// is then item t, row t of `tables`, as in a step of single tokens, and the kernel asks for its
// block table beside the position instead of behind the item index.
int ps_attention_decode(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                        void* out, int64_t out_stride, float* partial, int64_t partial_floats,
                        const int* tok_list, const int* tok_item, const int* tok_pos,
                        const int* tables, int table_width, int count, int heads, int kv_heads,
                        int head_dim, int page_size, int num_pages, float scale, int window,
                        int splits, int waves, int dtype, void* stream);

// Only the records of ps_attention_decode: (unnormalised sum of values [head_dim], maximum in
// units of log 2, sum) per (token, head, range) at partial[((n * heads + head) * splits + s) *
// (head_dim + 2)], also with one range; nothing is merged and no output rows are written.
int ps_attention_decode_partial(const void* q, int64_t q_stride, const void* k_pool,
                                const void* v_pool, float* partial, int64_t partial_floats,
                                const int* tok_list, const int* tok_item, const int* tok_pos,
                                const int* tables, int table_width, int count, int heads,
                                int kv_heads, int head_dim, int page_size, int num_pages,
                                float scale, int window, int splits, int waves, int dtype,
                                void* stream);

// The merge of those records inside the output projection, for up to 16 tokens and head sizes
// that are multiples of 64 (bfloat16 weights in their packed copy, n output columns,
// k = heads * head_dim):  residual[t(r), :] += merged context of row r  W^T + bias, where
// t(r) = tok_list ? tok_list[r] : r.  One wave per (tile of 16 columns, head), up to four heads
// to a block, whose sum is added with float atomics.  tiles_per_block: 0 (the library chooses),
// or the heads per block: 1, 2 or 4.
int ps_attention_merge_linear(const float* partial, int64_t partial_floats, const int* tok_list,
                              int count, int heads, int head_dim, int splits,
                              const void* w_packed, const float* bias, float* residual,
                              int64_t ld_res, int n, int tiles_per_block, void* stream);

// ps_attention_decode for callers that cannot allocate device memory: code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
// reference.  The partial results of the key ranges go into a device array that is part of the
// library (PS_DECODE_STATIC_SCRATCH_FLOATS floats = 8 MiB, held by every GPU the library runs
// on until the process ends) instead of a buffer of the caller; the call allocates and frees
// nothing.  count * heads * splits * (head_dim + 2) beyond that size is refused with an error.
// All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (different
// streams, or threads) race on it and give wrong results; calls on one stream are ordered and
// safe.  Nothing in the array has to be cleared between calls.
#define PS_DECODE_STATIC_SCRATCH_FLOATS (2 * 1024 * 1024)
int ps_attention_decode_static(const void* q, int64_t q_stride, const void* k_pool,
                               const void* v_pool, void* out, int64_t out_stride,
                               const int* tok_list, const int* tok_item, const int* tok_pos,
                               const int* tables, int table_width, int count, int heads,
                               int kv_heads, int head_dim, int page_size, int num_pages,
                               float scale, int window, int splits, int waves, int dtype,
                               void* stream);

// Tiled attention on the matrix cores for items that bring several tokens (bfloat16, head_dim a
// multiple of 16 up to 256).  Tile i covers queries tile_q0[i] .. tile_q0[i] + 63 of item
// tile_item[i]; cu_tokens and kv_lens describe the step's items.  Blocks start in the order of
// the list (all heads of tile 0, then of tile 1, ...): list the tiles that see the most keys first.
// max_kv_len: no query sees more keys than that (0: unknown); it only steers the launch shape.
// query_tile: the queries per tile that the list was cut for: ps_attention_prefill_query_tile(),
// or, for head sizes up to 128, ps_attention_prefill_small_tile() (steps with so few tiles that
// the larger ones would leave compute units without a block), or, for head sizes up to
// ps_attention_prefill_large_tile_head_dim(), ps_attention_prefill_large_tile() (long prompts:
// a block then takes in half as many keys and values per score).
int ps_attention_prefill(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                         void* out, int64_t out_stride, const int* tile_item, const int* tile_q0,
                         int tiles, const int* cu_tokens, const int* kv_lens, const int* tables,
                         int table_width, int heads, int kv_heads, int head_dim, int page_size,
                         int num_pages, float scale, int window, int max_kv_len, int query_tile,
                         int dtype, void* stream);

// Both of the above in one launch, for a step that has items of one token (tok_list lists the
// `singles` tokens; tok_item and tok_pos are indexed by token as in ps_attention_decode, which
// this computes with one range of keys) and items of several (tiles of
// ps_attention_prefill_query_tile() queries as in ps_attention_prefill): blocks of both kinds
// share the compute units, where two launches would leave most of them waiting twice.
// bfloat16 and head sizes of 16 to 64 in steps of 16 (ps_attention_mixed_supported).
int ps_attention_mixed_supported(int dtype, int head_dim, int table_width);
int ps_attention_mixed(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                       void* out, int64_t out_stride, const int* tok_list, int singles,
                       const int* tok_item, const int* tok_pos, const int* tile_item,
                       const int* tile_q0, int tiles, const int* cu_tokens, const int* kv_lens,
                       const int* tables, int table_width, int heads, int kv_heads, int head_dim,
                       int page_size, int num_pages, float scale, int window, int dtype,
                       void* stream);

// The constants of that kernel that a caller builds its index arrays by: queries per tile (of
// the two sizes), and the widest block table (entries per item) that it takes.
int ps_attention_prefill_query_tile(void);
int ps_attention_prefill_small_tile(void);
int ps_attention_prefill_large_tile(void);
int ps_attention_prefill_large_tile_head_dim(void);
int ps_attention_prefill_table_max(void);

// tokens[r] = argmax (inv_temperature[r] == 0) or a draw from softmax(logits * inv_temperature[r])
// by inverse CDF at uniform[r] in [0, 1).
int ps_sample(const float* logits, int64_t ld, const float* inv_temperature, const float* uniform,
              int* tokens, int rows, int vocab, void* stream);

// Record the launches issued on `stream` between begin and end into an executable graph.
int ps_graph_begin(void* stream);
int ps_graph_end(void* stream, void** exec_out, int* node_count);
int ps_graph_abort(void* stream);
int ps_graph_launch(void* exec, void* stream);
int ps_graph_destroy(void* exec);

#ifdef __cplusplus
}
#endif
