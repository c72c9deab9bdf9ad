// What the skinny matrix products (gemm_mfma.hip, gemm_skinny_norm.hip) share: the shape of a
// block and the epilogue that sums the waves' partial tiles.
#pragma once

#include "common.h"
#include "linear.h"
#include "pagedserve_hip.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

#define SK_WAVES 4
#define SK_UNROLL 4   // 64-k steps whose loads are issued together

// Sum the four waves' partial tiles and finish the block's 16 columns of MB x 16 rows.
// Element i of lane l of an accumulator is column (l / 16) * 4 + i of row l % 16; thread t
// finishes column t % 16 of row t / 16 of each accumulator, so that 16 consecutive threads
// store one run of 16 columns.
template <typename TOut, int EPI, int MB>
__device__ inline void skinny_epilogue(float (*partial)[MB][4][64], const float* bias, TOut* c,
                                       int m, int n, int ldc, int n0, int row0, int split,
                                       int k_splits, const KvScatter& scatter, int c_packed = 0) {
  const int col_in = threadIdx.x & 15;
  const int row_in = threadIdx.x >> 4;
  const int col = n0 + col_in;
  if (col >= n) return;
  const int i = col_in & 3;
  const int lane = (col_in >> 2) * 16 + row_in;
  const float bias_here = (bias != nullptr && split == 0) ? bias[col] : 0.f;
#pragma unroll
  for (int b = 0; b < MB; ++b) {
    const int row = row0 + b * 16 + row_in;
    if (row >= m) continue;
    float v = partial[0][b][i][lane] + partial[1][b][i][lane] + partial[2][b][i][lane] +
              partial[3][b][i][lane] + bias_here;
    // (c_packed: the output is the operand of another skinny product and is written in the
    // order in which that one reads it)
    TOut* dst = c_packed ? c + packed_offset(row, col, n) : c + (int64_t)row * ldc + col;
    if (EPI == PS_EPI_RESIDUAL) {
      if (k_splits > 1) {
        unsafeAtomicAdd(reinterpret_cast<float*>(dst), v);
      } else {
        *dst = from_float<TOut>(v + to_float<TOut>(*dst));
      }
    } else {
      v = apply_activation<EPI>(v);
      *dst = from_float<TOut>(v);
      if (EPI == PS_EPI_NONE) kv_scatter_store<TOut>(scatter, row, col, v);
    }
  }
}
