// What the tiled bfloat16 products share: vector types, the fast GELU of a bfloat16 result, and
// the epilogue that takes a wave's 32 x 32 accumulators to memory.
#pragma once

#include "common.h"
#include "linear.h"
#include "pagedserve_hip.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;

#define TB_BK 64     // values of k per stage
#define TB_ROW 128   // bytes per row and stage

typedef const __attribute__((address_space(1))) void* global_ptr_t;
typedef __attribute__((address_space(3))) void* lds_ptr_t;

// gelu_tanh(u) = u * sigmoid(2 z), z = sqrt(2/pi) (u + 0.044715 u^3), with the hardware
// exponential and reciprocal: its error (about 1e-6 relative) is far below the rounding of a
// bfloat16 result, which is the only place where it is used.
__device__ inline float gelu_tanh_fast(float u) {
  const float z2 = 1.5957691216057308f * (u + 0.044715f * u * u * u);
  return u * __frcp_rn(1.0f + __expf(-z2));
}

template <int EPI, typename TOut>
__device__ inline float finish_value(float v) {
  if (EPI == PS_EPI_GELU_TANH && sizeof(TOut) == 2) return gelu_tanh_fast(v);
  return apply_activation<EPI>(v);
}

// Eight finished values to eight consecutive outputs (16-byte aligned).
__device__ inline void store8(float* out, const float* v) {
  *reinterpret_cast<float4*>(out) = make_float4(v[0], v[1], v[2], v[3]);
  *reinterpret_cast<float4*>(out + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
__device__ inline void store8(bf16_t* out, const float* v) {
  uint4 packed;
  packed.x = pack2_bf16(v[0], v[1]);
  packed.y = pack2_bf16(v[2], v[3]);
  packed.z = pack2_bf16(v[4], v[5]);
  packed.w = pack2_bf16(v[6], v[7]);
  *reinterpret_cast<uint4*>(out) = packed;
}

// The accumulators acc[WM][WN] of one wave (32 x 32 each, rows row_base + 32 i ..., columns
// col_base + 32 j ...) to C, through `region`, an area of LDS of 32 x (32 WN + 8) floats that
// belongs to this wave alone: bias, activation, residual add into the float stream, key/value
// columns into cache pages.  `split` / `k_splits`: partial sums of a k range are added with
// atomics, the bias by split 0 only.
template <int WM, int WN, typename TOut, int EPI>
__device__ inline void store_wave_tile(f32x16 (&acc)[WM][WN], float* region, int lane, int row_base,
                                       int col_base, int m, int n, int ldc, TOut* __restrict__ c,
                                       const float* __restrict__ bias, int split, int k_splits,
                                       const KvScatter& scatter) {
  // ---- epilogue.  Element e of a 32 x 32 accumulator is row (e / 4) * 8 + (lane / 32) * 4 +
  // e % 4, column lane % 32: a lane holds one column.  Each wave turns 32 rows at a time
  // through a region of LDS of its own, after which a lane holds eight consecutive columns of
  // one row: bias and activation are applied there and rows leave in pieces of 16 or 32
  // bytes, eight (or more) lanes to a row.
  constexpr int EP_STRIDE = WN * 32 + 8;          // floats; 4 rows further is 32 banks further
  constexpr int EP_CHUNKS = WN * 4;               // pieces of eight columns per row
  constexpr int EP_ROWS = 64 / EP_CHUNKS;         // rows per pass of the wave
  const int chunk = lane % EP_CHUNKS;
  const int row_in_pass = lane / EP_CHUNKS;
  const int col0 = col_base + chunk * 8;
  const bool full = col0 + 8 <= n;
  const bool vec_c = ldc % (16 / (int)sizeof(TOut)) == 0 && (reinterpret_cast<uintptr_t>(c) & 15u) == 0;
  const bool by_column = !vec_c || k_splits > 1;
  float b[8];
#pragma unroll
  for (int q = 0; q < 8; ++q) b[q] = (bias && split == 0 && col0 + q < n) ? bias[col0 + q] : 0.f;
  // key and value columns also go into cache pages: eight consecutive columns lie in one head
  const bool scatters = EPI == PS_EPI_NONE && scatter.k_pool != nullptr && col0 < n &&
                        col0 + 8 > scatter.q_cols;
  const bool vec_kv = full && col0 >= scatter.q_cols && scatter.head_dim % 8 == 0 &&
                      scatter.q_cols % 8 == 0 && scatter.kv_cols % 8 == 0;
  TOut* pool = nullptr;
  int64_t pool_offset = 0;
  if (scatters && vec_kv) pool = kv_scatter_col<TOut>(scatter, col0, &pool_offset);

#pragma unroll
  for (int i = 0; i < WM; ++i) {
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e)
        region[((e >> 2) * 8 + (lane >> 5) * 4 + (e & 3)) * EP_STRIDE + j * 32 + (lane & 31)] =
            acc[i][j][e];
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (by_column) {
      // rows that cannot leave in aligned pieces, and partial sums of a split k: a wave's
      // lanes take consecutive columns of one row
#pragma unroll 8
      for (int r = 0; r < 32; ++r) {
        const int row = row_base + i * 32 + r;
        if (row >= m) continue;
#pragma unroll
        for (int half = 0; half < (WN + 1) / 2; ++half) {
          const int within = half * 64 + lane;
          const int col = col_base + within;
          if (within >= WN * 32 || col >= n) continue;
          const float bias_here = (bias && split == 0) ? bias[col] : 0.f;
          const float v = finish_value<EPI, TOut>(region[r * EP_STRIDE + within] + bias_here);
          TOut* out = c + (int64_t)row * ldc + col;
          if (EPI == PS_EPI_RESIDUAL) {
            float* sum = reinterpret_cast<float*>(out);
            if (k_splits > 1) unsafeAtomicAdd(sum, v);
            else *sum += v;
          } else {
            *out = from_float<TOut>(v);
            if (EPI == PS_EPI_NONE) kv_scatter_store<TOut>(scatter, row, col, v);
          }
        }
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      continue;
    }
#pragma unroll 2
    for (int pass = 0; pass < 32 / EP_ROWS; ++pass) {
      const int r = pass * EP_ROWS + row_in_pass;
      const int row = row_base + i * 32 + r;
      const float4 lo = *reinterpret_cast<const float4*>(region + r * EP_STRIDE + chunk * 8);
      const float4 hi = *reinterpret_cast<const float4*>(region + r * EP_STRIDE + chunk * 8 + 4);
      if (row >= m || col0 >= n) continue;
      float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
      for (int q = 0; q < 8; ++q) v[q] = finish_value<EPI, TOut>(v[q] + b[q]);
      TOut* out = c + (int64_t)row * ldc + col0;
      if (EPI == PS_EPI_RESIDUAL) {
        float* sum = reinterpret_cast<float*>(out);
        if (full) {
          float4 o0 = *reinterpret_cast<const float4*>(sum);
          float4 o1 = *reinterpret_cast<const float4*>(sum + 4);
          o0.x += v[0]; o0.y += v[1]; o0.z += v[2]; o0.w += v[3];
          o1.x += v[4]; o1.y += v[5]; o1.z += v[6]; o1.w += v[7];
          *reinterpret_cast<float4*>(sum) = o0;
          *reinterpret_cast<float4*>(sum + 4) = o1;
        } else {
          for (int q = 0; q < 8; ++q)
            if (col0 + q < n) sum[q] += v[q];
        }
        continue;
      }
      if (full) {
        // (eight key or value columns that go to their page and that nobody reads from c)
        if (!(scatters && pool != nullptr && scatter.cache_only)) store8(out, v);
      } else {
        for (int q = 0; q < 8; ++q)
          if (col0 + q < n) out[q] = from_float<TOut>(v[q]);
      }
      if (scatters) {
        if (pool != nullptr) {
          const int64_t slot = kv_scatter_row(scatter, row);
          if (slot >= 0) store8(pool + slot + pool_offset, v);
        } else if (!vec_kv) {
          for (int q = 0; q < 8; ++q)
            if (col0 + q < n) kv_scatter_store<TOut>(scatter, row, col0 + q, v[q]);
        }
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
}
