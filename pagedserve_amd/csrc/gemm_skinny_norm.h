// The skinny matrix product for up to 16 rows with the norm of its input fused in front
// (C[m, n] = epi(sum_k norm(h)[m, k] W[n, k] + b[n]), bfloat16 weights, float rows):
// while the block's weight loads are in flight, each wave normalises up to four of the float
// input rows in registers (statistics by lane exchanges, as the norm kernel) and leaves them in
// LDS as bfloat16; the product then reads its column operand from LDS.  One launch and one trip
// to memory instead of two launches.
//
// The kernel and its launcher are a header because two sources instantiate them, one for k up
// to 1024 and one beyond (gemm_skinny_norm.hip, gemm_skinny_norm_long.hip): together they are
// most of the library's compile time, and sources compile side by side.
#pragma once

#include "gemm_skinny.h"

// ---------------------------------------------------------------- skinny with fused norm
#define SN_MAX_K 1792              // one round of loads covers it: 4 waves x 7 steps x 64
// LDS row stride in elements (16-byte aligned, skewed by four banks a row); 16 rows of the
// longest k with the partial sums stay under the 64 KB that a block may declare
#define SN_STRIDE(UNROLL) (((UNROLL) <= 4 ? 1024 : (UNROLL) * SK_WAVES * 64) + 8)

// NR: rows that a wave normalises (rows wave, wave + 4, ...: 4 NR >= m).  Rows of LDS beyond
// them stay as they are: they only feed outputs that are never stored.
// NT: accumulator tiles of 16 columns per block.  A block owns `cols` consecutive columns
// (16 with one tile; 17 to 32 with two, the second tile partly empty): with more tiles of 16
// than compute units the columns are dealt out evenly instead, one block to a unit, because a
// unit that gets a second block takes twice as long as the others (1600 k, 1 row: 4,096
// columns 5.7 us, 4,800 columns as 300 tiles 9.0 us).
template <typename TOut, int EPI, int NR, int UNROLL, int NT>
__global__ __launch_bounds__(64 * SK_WAVES) void gemm_nt_skinny_norm_kernel(
    NormPrologue norm, const bf16_t* __restrict__ w, const float* __restrict__ bias,
    TOut* __restrict__ c, int m, int n, int k, int ldc, KvScatter scatter,
    const bf16_t* __restrict__ wp, int cols) {
  constexpr int STRIDE = SN_STRIDE(UNROLL);
  // with two tiles the partial sums take the place of the rows once these have been used:
  // both together would pass the 64 KB that a block may declare
  constexpr int OWN_PARTIAL = NT == 1 ? SK_WAVES * 4 * 64 : 1;
  __shared__ float partial_own[OWN_PARTIAL];
  __shared__ __attribute__((aligned(16))) bf16_t xs[16 * STRIDE];
  static_assert(NT <= 2 && NT * SK_WAVES * 4 * 64 * sizeof(float) <= 16 * STRIDE * sizeof(bf16_t), "partial sums fit");
  float (*partial)[SK_WAVES][1][4][64] = reinterpret_cast<float (*)[SK_WAVES][1][4][64]>(
      NT == 1 ? partial_own : reinterpret_cast<float*>(xs));
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  // (one tile: always 16 columns from a multiple of 16, and the addresses are as simple as that)
  const int n0 = NT == 1 ? blockIdx.x * 16 : blockIdx.x * cols;
  const int n1 = NT == 1 ? n : (n0 + cols < n ? n0 + cols : n);
  const int sub = lane & 15;
  const int group = lane >> 4;
  const bf16_t* w_ptr[NT];
  if (NT == 1) {
    const int w_row = n0 + sub < n ? n0 + sub : n - 1;
    w_ptr[0] = w + (int64_t)w_row * k + group * 16;
    if (wp != nullptr) w_ptr[0] = wp + (int64_t)(n0 / 16) * (k / 64) * 1024 + lane * 8;   // packed copy
  } else {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int w_row = n0 + t * 16 + sub < n1 ? n0 + t * 16 + sub : n1 - 1;
      w_ptr[t] = w + (int64_t)w_row * k + group * 16;
      // packed copy: row r is lane group * 16 + r % 16 of tile r / 16
      if (wp != nullptr)
        w_ptr[t] = wp + (int64_t)(w_row >> 4) * (k / 64) * 1024 + (group * 16 + (w_row & 15)) * 8;
    }
  }
  const uint4 zero = {0u, 0u, 0u, 0u};

  uint4 wf[UNROLL][NT][2];
  bool first[UNROLL], second[UNROLL];
  // 1. rows wave, wave + 4, wave + 8, wave + 12: statistics and normalisation in registers
  //    (mean, centred values, biased variance, rsqrt(var + eps), scale, shift; reference:
  //    src/kernels/triton_residual_layernorm.py:25-39), result to LDS as bfloat16.  A lane
  //    owns columns 4 * lane + 256 * i (one 16-byte load each); all loads of the four rows and
  //    of the scale and shift leave together.
  {
    constexpr int V4 = UNROLL * SK_WAVES / 4;   // 256 columns each: what the rounds of k cover
    const float4 zero4 = {0.f, 0.f, 0.f, 0.f};
    float4 g[V4], bt[V4], v[NR][V4];
    bool in_row[V4];
    const float* src[NR];
#pragma unroll
    for (int j = 0; j < NR; ++j) {
      const int token = wave + j * SK_WAVES;
      const int t = token < m ? token : m - 1;
      src[j] = norm.h + (int64_t)(norm.rows ? norm.rows[t] : t) * norm.ldh;
    }
    int safe[V4];
#pragma unroll
    for (int i = 0; i < V4; ++i) {
      const int col = 4 * lane + 256 * i;
      in_row[i] = col < k;
      safe[i] = in_row[i] ? col : 0;
    }
    // row by row, the scale and shift behind them: the sums of a row start when the row is there
#pragma unroll
    for (int j = 0; j < NR; ++j)
#pragma unroll
      for (int i = 0; i < V4; ++i) v[j][i] = *reinterpret_cast<const float4*>(src[j] + safe[i]);
#pragma unroll
    for (int i = 0; i < V4; ++i) {
      g[i] = *reinterpret_cast<const float4*>(norm.gamma + safe[i]);
      bt[i] = (!norm.rms && norm.beta != nullptr)
                  ? *reinterpret_cast<const float4*>(norm.beta + safe[i])
                  : zero4;
    }
    // 2. this wave's weights.  A wave's loads come back in the order in which they left, so
    //    these leave after the loads of the rows (which come from the L2 and are there first)
    //    and travel while the rows are normalised; issued before them they would hold the
    //    rows back for the whole trip to memory.
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int ku = wave * 64 + u * SK_WAVES * 64;
      const int kk = ku + group * 16;
      first[u] = kk < k;
      second[u] = kk + 8 < k;
      const int p0 = wp != nullptr ? (first[u] ? (ku / 64) * 1024 : 0) : (first[u] ? ku : -group * 16);
      const int p1 = wp != nullptr ? p0 + 512 : (second[u] ? ku + 8 : -group * 16);
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        wf[u][t][0] = *reinterpret_cast<const uint4*>(w_ptr[t] + p0);
        wf[u][t][1] = *reinterpret_cast<const uint4*>(w_ptr[t] + p1);
      }
    }
    // The rows of a wave go through every stage together (the sums of all, the means of all,
    // ...), so that the lane exchanges and the square root of one row run behind those of
    // the others instead of one after the other.  A wave whose last rows lie beyond m works
    // on copies of row m - 1 and writes zeros for them.
    float sum[NR], sq[NR], mean[NR], inv_std[NR];
#pragma unroll
    for (int j = 0; j < NR; ++j) {
      sum[j] = 0.f;
#pragma unroll
      for (int i = 0; i < V4; ++i) {
        if (!in_row[i]) v[j][i] = zero4;
        sum[j] += (v[j][i].x + v[j][i].y) + (v[j][i].z + v[j][i].w);
      }
    }
#pragma unroll
    for (int j = 0; j < NR; ++j) mean[j] = norm.rms ? 0.f : wave_sum(sum[j]) / (float)k;
#pragma unroll
    for (int j = 0; j < NR; ++j) {
      sq[j] = 0.f;
#pragma unroll
      for (int i = 0; i < V4; ++i) {
        if (in_row[i]) {
          v[j][i].x -= mean[j];
          v[j][i].y -= mean[j];
          v[j][i].z -= mean[j];
          v[j][i].w -= mean[j];
        }
        sq[j] += (v[j][i].x * v[j][i].x + v[j][i].y * v[j][i].y) +
                 (v[j][i].z * v[j][i].z + v[j][i].w * v[j][i].w);
      }
    }
#pragma unroll
    for (int j = 0; j < NR; ++j) inv_std[j] = 1.0f / sqrtf(wave_sum(sq[j]) / (float)k + norm.eps);
#pragma unroll
    for (int j = 0; j < NR; ++j) {
      const int token = wave + j * SK_WAVES;
      const bool live = token < m;     // the same for the whole wave
#pragma unroll
      for (int i = 0; i < V4; ++i) {
        if (!in_row[i]) continue;
        uint2 packed = {0u, 0u};
        if (live) {
          const float y0 = v[j][i].x * inv_std[j] * g[i].x + bt[i].x;
          const float y1 = v[j][i].y * inv_std[j] * g[i].y + bt[i].y;
          const float y2 = v[j][i].z * inv_std[j] * g[i].z + bt[i].z;
          const float y3 = v[j][i].w * inv_std[j] * g[i].w + bt[i].w;
          packed.x = pack2_bf16(y0, y1);
          packed.y = pack2_bf16(y2, y3);
        }
        *reinterpret_cast<uint2*>(&xs[token * STRIDE + 4 * lane + 256 * i]) = packed;
      }
    }
  }
  __syncthreads();

  // 3. the product: column operand from LDS
  f32x4 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const int ku = wave * 64 + u * SK_WAVES * 64;
    const int kk = ku + group * 16;
    uint4 x0 = zero, x1 = zero;
    if (first[u]) x0 = *reinterpret_cast<const uint4*>(&xs[sub * STRIDE + kk]);
    if (second[u]) x1 = *reinterpret_cast<const uint4*>(&xs[sub * STRIDE + kk + 8]);
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const uint4 w0 = first[u] ? wf[u][t][0] : zero;
      const uint4 w1 = second[u] ? wf[u][t][1] : zero;
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(&w0),
                                                       *reinterpret_cast<const bf16x8*>(&x0), acc[t], 0, 0, 0);
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(&w1),
                                                       *reinterpret_cast<const bf16x8*>(&x1), acc[t], 0, 0, 0);
    }
  }
  if (NT > 1) __syncthreads();   // every wave has read its rows: their place is free
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) partial[t][wave][0][i][lane] = acc[t][i];
  __syncthreads();
#pragma unroll
  for (int t = 0; t < NT; ++t)
    if (n0 + t * 16 < n1)
      skinny_epilogue<TOut, EPI, 1>(partial[t], bias, c, m, n1, ldc, n0 + t * 16, 0, 0, 1, scatter);
}

// --------------------------------------------------------------------------------- host
// SHORT, LONG: steps of 64 k per wave of the two instantiations that a source holds; a k of up
// to 256 SHORT takes the first.
template <typename TOut, int SHORT, int LONG>
static int launch_skinny_norm(const NormPrologue& norm, const void* w, const float* bias, void* c,
                              int m, int n, int k, int ldc, int epilogue, const KvScatter& scatter,
                              const bf16_t* wp, hipStream_t s) {
  if (k % 64 != 0) wp = nullptr;
  // More tiles of 16 columns than compute units (up to twice as many): the columns are dealt
  // out evenly, one block to a unit, each with a whole tile and a partly empty one.
  const int tiles = (n + 15) / 16;
  const int units = ps_compute_units();
  const bool even = tiles > units && tiles <= 2 * units;
  const int cols = even ? (n + units - 1) / units : 16;
  // (read from the matrix itself: in the packed copy a line of 128 bytes holds rows of two
  // blocks, which would fetch it twice; 1600 k, 4,800 columns, 1 row: 7.7 against 8.5 us)
  if (even && cols % 16 != 0) wp = nullptr;
  dim3 grid((n + cols - 1) / cols);
  dim3 block(64 * SK_WAVES);
#define PS_NORM_TILES(EPI, NR, STEPS, NT)                                                     \
  hipLaunchKernelGGL((gemm_nt_skinny_norm_kernel<TOut, EPI, NR, STEPS, NT>), grid, block, 0,  \
                     s, norm, (const bf16_t*)w, bias, (TOut*)c, m, n, k, ldc, scatter, wp, cols)
#define PS_NORM_STEPS(EPI, NR, STEPS)                                                         \
  do {                                                                                        \
    if (even) PS_NORM_TILES(EPI, NR, STEPS, 2);                                               \
    else PS_NORM_TILES(EPI, NR, STEPS, 1);                                                    \
  } while (0)
#define PS_NORM_LAUNCH(EPI, NR)                                                               \
  do {                                                                                        \
    if (k <= SK_WAVES * SHORT * 64) PS_NORM_STEPS(EPI, NR, SHORT);                            \
    else PS_NORM_STEPS(EPI, NR, LONG);                                                        \
  } while (0)
#define PS_NORM_CASE(EPI)                                                                     \
  case EPI:                                                                                   \
    if (m <= 4) PS_NORM_LAUNCH(EPI, 1);                                                       \
    else if (m <= 8) PS_NORM_LAUNCH(EPI, 2);                                                  \
    else if (m <= 12) PS_NORM_LAUNCH(EPI, 3);                                                 \
    else PS_NORM_LAUNCH(EPI, 4);                                                              \
    break
  switch (epilogue) {
    PS_NORM_CASE(PS_EPI_NONE);
    PS_NORM_CASE(PS_EPI_GELU_TANH);
    PS_NORM_CASE(PS_EPI_GELU_ERF);
    PS_NORM_CASE(PS_EPI_RESIDUAL);
    default: ps_set_error("ps_linear: unknown epilogue %d", epilogue); return 1;
  }
#undef PS_NORM_CASE
#undef PS_NORM_LAUNCH
#undef PS_NORM_STEPS
#undef PS_NORM_TILES
  PS_CHECK_LAUNCH("ps_linear(skinny, fused norm)");
  return 0;
}

template <int SHORT, int LONG>
static int skinny_norm_by_type(const NormPrologue& norm, const void* w, const float* bias, void* c,
                               int m, int n, int k, int ldc, int c_dtype, int epilogue,
                               const KvScatter& scatter, const void* w_packed, hipStream_t s) {
  const bf16_t* wp = (const bf16_t*)w_packed;
  if (c_dtype == PS_F32)
    return launch_skinny_norm<float, SHORT, LONG>(norm, w, bias, c, m, n, k, ldc, epilogue, scatter, wp, s);
  return launch_skinny_norm<bf16_t, SHORT, LONG>(norm, w, bias, c, m, n, k, ldc, epilogue, scatter, wp, s);
}
