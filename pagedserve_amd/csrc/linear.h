// What the matrix-product kernels may fuse around the product: a norm in front of it and the
// scatter of key/value columns into cache pages behind it.
#pragma once

#include "common.h"

struct KvScatter {
  void* k_pool;          // null: no scatter
  void* v_pool;
  const int* tok_item;
  const int* tok_pos;
  const int* tables;
  int table_width, q_cols, kv_cols, head_dim, kv_heads, page_size, page_shift, num_pages;
  int cache_only;        // the key and value columns need not be written to the output as well
};

// The product of the output head may also choose each row's token (the column of its largest
// value, the lowest one on ties) instead of leaving that to a kernel of its own.  Blocks
// raise 64-bit keys (value in an order that integers keep, then the column counted from
// above) with atomic maxima, spread over PS_TOP_SLOTS keys per row, 256 bytes apart, so that
// few blocks meet at one address and the keys lie on many memory channels (atomics on one
// address, and on one channel, are performed one after the other: 1,571 blocks drawing from
// one ticket added 27 us to the kernel, 12,568 maxima within one kilobyte 10 us).  The block
// that draws the last ticket reads the keys, writes the tokens, and leaves keys and tickets
// at zero for the next launch.  Launches that share keys must not overlap.
#define PS_TOP_SLOTS 16
#define PS_TOP_STRIDE 32      // 64-bit words from one key to the next, and 2 ints from ticket to ticket: 256 bytes,
                              // so that keys and tickets spread over the memory channels
struct TopChoice {
  unsigned long long* keys;   // null: no choice; else [rows * PS_TOP_SLOTS] keys, zero between launches
  int* ticket;                // 1 + PS_TOP_SLOTS counters, zero between launches
  int* tokens;                // [rows]
};
__device__ inline unsigned long long* top_choice_slot(const TopChoice& top, int row, int slot) {
  return top.keys + ((int64_t)row * PS_TOP_SLOTS + slot) * PS_TOP_STRIDE;
}
__device__ inline int* top_choice_ticket(const TopChoice& top, int index) {
  return top.ticket + index * 2 * PS_TOP_STRIDE;
}

__device__ inline unsigned long long top_choice_key(float v, int col) {
  if (v == 0.f) v = 0.f;   // one zero
  const unsigned int bits = __float_as_uint(v);
  const unsigned int ordered = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
  return ((unsigned long long)ordered << 32) | (unsigned long long)(0xFFFFFFFFu - (unsigned int)col);
}

// Activations of a decode step (17 to 64 rows) may lie in the order in which the lanes of the
// skinny product hold their operand, like the packed weight copies: rows in blocks of 16, the
// 16 x 64 tile of row block t and columns 64 s .. 64 s + 63 at element (t * (cols / 64) + s) *
// 1024 as two runs of 512, run h holding for lane = g * 16 + r the 8 values of row 16 t + r,
// columns 64 s + 16 g + 8 h ...  A producer writes element (row, col) at this offset.
__host__ __device__ inline int64_t packed_offset(int row, int col, int cols) {
  return ((((int64_t)(row >> 4) * (cols >> 6) + (col >> 6)) * 2 + ((col >> 3) & 1)) * 64 +
          (((col >> 4) & 3) * 16 + (row & 15))) * 8 + (col & 7);
}

struct NormPrologue {
  const float* h;        // null: no norm
  const int* rows;
  const float* gamma;
  const float* beta;
  float eps;
  int rms;
  int ldh;
};

// The two halves of that address, for kernels that finish many elements of one row or one
// column: kv_scatter_row gives the element offset of (page, slot) of a token, or -1;
// kv_scatter_col gives the pool and the offset of (head, dim) inside a page, or null for a
// query column.
__device__ inline int64_t kv_scatter_row(const KvScatter& s, int row) {
  const int pos = s.tok_pos[row];
  const int logical = s.page_shift >= 0 ? (pos >> s.page_shift) : pos / s.page_size;
  if (logical >= s.table_width) return -1;
  const int page = s.tables[(int64_t)s.tok_item[row] * s.table_width + logical];
  if (page < 0 || page >= s.num_pages) return -1;
  return ((int64_t)page * s.kv_heads * s.page_size + (pos - logical * s.page_size)) * s.head_dim;
}

template <typename T>
__device__ inline T* kv_scatter_col(const KvScatter& s, int col, int64_t* offset) {
  if (s.k_pool == nullptr || col < s.q_cols) return nullptr;
  int within = col - s.q_cols;
  T* pool = reinterpret_cast<T*>(s.k_pool);
  if (within >= s.kv_cols) {
    within -= s.kv_cols;
    pool = reinterpret_cast<T*>(s.v_pool);
  }
  const int head = within / s.head_dim;
  *offset = (int64_t)head * s.page_size * s.head_dim + (within - head * s.head_dim);
  return pool;
}

// Column `col` of output row `row` also goes into the cache when it is a key or value column:
// token at position p of item r lands at (page = table[r][p / page], offset = p % page)
// (reference: src/model/kv_manager.py:303-308,403-404).
template <typename T>
__device__ inline void kv_scatter_store(const KvScatter& s, int row, int col, float v) {
  if (s.k_pool == nullptr || col < s.q_cols) return;
  int within = col - s.q_cols;
  T* pool = reinterpret_cast<T*>(s.k_pool);
  if (within >= s.kv_cols) {
    within -= s.kv_cols;
    pool = reinterpret_cast<T*>(s.v_pool);
  }
  const int head = within / s.head_dim;
  const int dim = within - head * s.head_dim;
  const int pos = s.tok_pos[row];
  const int logical = s.page_shift >= 0 ? (pos >> s.page_shift) : pos / s.page_size;
  if (logical >= s.table_width) return;
  const int page = s.tables[(int64_t)s.tok_item[row] * s.table_width + logical];
  if (page < 0 || page >= s.num_pages) return;
  pool[(((int64_t)page * s.kv_heads + head) * s.page_size + (pos - logical * s.page_size)) *
           s.head_dim + dim] = from_float<T>(v);
}
