// The merge of decode attention's key ranges inside the output projection, for steps of up
// to 16 single-token items (bfloat16, head sizes that are multiples of 64):
//
//   residual[t, :] += concat_h(softmax-merged context of head h of token t) W^T + bias
//
// attention_decode_kernel leaves, per (token, head, range), the unnormalised sum of values
// `acc`, the maximum `m` (in units of log 2) and the sum `l` of its range.  Merging them is
// out = sum_s acc_s 2^(m_s - M) / sum_s l_s 2^(m_s - M).  A kernel of its own for that costs a
// launch and a trip to memory per layer, as much as the attention of a small batch itself;
// doing it in front of an output projection whose every block needs every head costs the same
// again, since each block then pulls every record through its one compute unit (measured both
// ways: blocks of 16 columns with the heads spread over their waves are slower than the merge
// kernel they replace).  Here the projection is split over the heads instead: block (c, h) is
// one wave that merges head h of all rows (each lane the 16 values of its own row that it
// needs as matrix-core operand; with fewer than 9 rows the lanes of the free operand columns
// take a share of the ranges each and exchange their sums), multiplies them with the piece of W that belongs to its columns and to
// head h (out of the packed copy of W, pagedserve_hip.h); the waves of a block (up to four
// heads) sum their results through LDS and the first adds them into the float residual rows
// with atomic adds; the blocks of the first heads add the bias.  The sum over heads is
// therefore made by the adds, in an order that differs from run to run within float rounding,
// as for every product here whose k range is split over blocks.
#include "gemm_bf16_common.h"

typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;

// STEPS: head_dim / 64; PARTS: lanes that share the ranges of a row; GROUP: heads per block, one
// wave each, whose results are summed through LDS before they are added to the residual rows.
// (The adds of the blocks of one column tile meet at that tile's addresses, other tiles are
// elsewhere: spread like that, float atomic adds run at 75 to 90 per nanosecond, and the 74,000
// of 12 heads at 8 rows of 768 take under a microsecond.  Four heads to a block are chosen by
// what was measured, below.)
template <int STEPS, int PARTS, int GROUP>
__global__ __launch_bounds__(64 * GROUP) void attention_merge_linear_kernel(
    const float* __restrict__ partial, const int* __restrict__ tok_list, int count, int heads,
    int splits, const bf16_t* __restrict__ wp, const float* __restrict__ bias,
    float* __restrict__ residual, int64_t ld_res, int n) {
  constexpr int TILES = 1;             // tiles of 16 columns per block (two measured slower)
  constexpr int rows_pow2 = 16 / PARTS;
  constexpr int parts = PARTS;
  constexpr int HEAD_DIM = STEPS * 64;
  constexpr int STRIDE = HEAD_DIM + 2;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // the same in every lane: scalar
  const int column = lane & 15;        // column of the matrix-core operand: a row of the step
  const int group = lane >> 4;         // which 16 of every 64 head dimensions
  // (a wave beyond the last head works on a copy of the last head and adds nothing)
  const bool real_head = blockIdx.y * GROUP + wave < heads;
  const int head = real_head ? blockIdx.y * GROUP + wave : heads - 1;
  // Fewer rows than 16 leave operand columns free: they take a share of the ranges of the rows
  // that are there (row = column mod rows_pow2, the smallest power of two that holds the
  // rows; the column's other bits pick every parts-th range), and the shares are merged by
  // lane exchanges afterwards.  One row with 64 ranges then costs four records per lane
  // instead of 64.
  const int row = column & (rows_pow2 - 1);
  const int part = column / rows_pow2;
  const bool has_row = column < count;       // this lane's results are stored
  const bool merges = row < count;
  const int safe_row = merges ? row : 0;
  const float* records = partial + ((int64_t)safe_row * heads + head) * splits * STRIDE;

  // the pieces of W: tiles of 16 columns, k steps head * STEPS ..., element
  // ((tile * k_steps + step) * 2 + h) * 512 + lane * 8 of the packed copy; asked for first,
  // they travel while the records are merged
  const int k_steps = heads * STEPS;
  const int tiles_n = (n + 15) / 16;
  uint4 w_raw[TILES][STEPS][2];
#pragma unroll
  for (int c = 0; c < TILES; ++c) {
    int tile = blockIdx.x * TILES + c;
    if (tile >= tiles_n) tile = tiles_n - 1;     // beyond n: never stored
    const bf16_t* w_tile = wp + ((int64_t)tile * k_steps + (int64_t)head * STEPS) * 1024 + lane * 8;
#pragma unroll
    for (int st = 0; st < STEPS; ++st)
#pragma unroll
      for (int h = 0; h < 2; ++h)
        w_raw[c][st][h] = *reinterpret_cast<const uint4*>(w_tile + (st * 2 + h) * 512);
  }

  // Merge as the ranges come (a running maximum, earlier sums rescaled when it moves), so that
  // no load waits for a result.
  float total_m = -INFINITY;
  float total_l = 0.f;
  float value[STEPS][2][8];
#pragma unroll
  for (int st = 0; st < STEPS; ++st)
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int e = 0; e < 8; ++e) value[st][h][e] = 0.f;
#pragma unroll 4
  for (int s = part; s < splits; s += parts) {
    const float* record = records + s * STRIDE;
    const float m_s = record[HEAD_DIM];
    const float l_s = record[HEAD_DIM + 1];
    float2 piece[STEPS][2][4];
#pragma unroll
    for (int st = 0; st < STEPS; ++st)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          // the k values that lane group `group` holds in product h of step st (the order of
          // the packed copy): 64 st + 16 group + 8 h ...; records start at multiples of 8 bytes
          piece[st][h][q] = *reinterpret_cast<const float2*>(record + st * 64 + group * 16 + h * 8 + 2 * q);
    const float new_m = fmaxf(total_m, m_s);
    // an empty range has m = -inf and sums of zero: it changes nothing
    const float keep = (total_m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(total_m - new_m);
    const float weight = (m_s == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_s - new_m);
    total_l = total_l * keep + l_s * weight;
#pragma unroll
    for (int st = 0; st < STEPS; ++st)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          value[st][h][2 * q] = fmaf(piece[st][h][q].x, weight, value[st][h][2 * q] * keep);
          value[st][h][2 * q + 1] = fmaf(piece[st][h][q].y, weight, value[st][h][2 * q + 1] * keep);
        }
    total_m = new_m;
  }
  // the shares of a row: lanes whose column differs in the bits above the row's
#pragma unroll
  for (int offset = rows_pow2; offset < 16; offset <<= 1) {
    const float other_m = __shfl_xor(total_m, offset, 64);
    const float other_l = __shfl_xor(total_l, offset, 64);
    const float new_m = fmaxf(total_m, other_m);
    const float keep = (total_m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(total_m - new_m);
    const float weight = (other_m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(other_m - new_m);
    total_l = total_l * keep + other_l * weight;
#pragma unroll
    for (int st = 0; st < STEPS; ++st)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int e = 0; e < 8; ++e)
          value[st][h][e] = fmaf(__shfl_xor(value[st][h][e], offset, 64), weight, value[st][h][e] * keep);
    total_m = new_m;
  }
  const float inverse = (merges && total_l > 0.f) ? 1.f / total_l : 0.f;

  f32x4_t acc[TILES];
#pragma unroll
  for (int c = 0; c < TILES; ++c) acc[c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int st = 0; st < STEPS; ++st)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      uint4 x_raw;
      x_raw.x = pack2_bf16(value[st][h][0] * inverse, value[st][h][1] * inverse);
      x_raw.y = pack2_bf16(value[st][h][2] * inverse, value[st][h][3] * inverse);
      x_raw.z = pack2_bf16(value[st][h][4] * inverse, value[st][h][5] * inverse);
      x_raw.w = pack2_bf16(value[st][h][6] * inverse, value[st][h][7] * inverse);
#pragma unroll
      for (int c = 0; c < TILES; ++c)
        acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(&w_raw[c][st][h]),
                                                         *reinterpret_cast<const bf16x8*>(&x_raw), acc[c], 0, 0, 0);
    }
  // element i of lane l: column (l / 16) * 4 + i of the tile, row l % 16
  if (GROUP > 1) {
    // the heads of this block are summed by its first wave
    __shared__ f32x4_t sums[GROUP > 1 ? GROUP - 1 : 1][TILES][64];
    if (wave > 0)
#pragma unroll
      for (int c = 0; c < TILES; ++c)
        sums[wave - 1][c][lane] = real_head ? acc[c] : f32x4_t{0.f, 0.f, 0.f, 0.f};
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w = 0; w < GROUP - 1; ++w)
#pragma unroll
      for (int c = 0; c < TILES; ++c) acc[c] += sums[w][c][lane];
  }
  if (!has_row) return;
  const int t = tok_list ? tok_list[column] : column;
#pragma unroll
  for (int c = 0; c < TILES; ++c)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int col = (blockIdx.x * TILES + c) * 16 + group * 4 + i;
      if (col >= n) continue;
      float v = acc[c][i];
      if (blockIdx.y == 0 && bias != nullptr) v += bias[col];
      unsafeAtomicAdd(residual + (int64_t)t * ld_res + col, v);
    }
}

bool ps_attention_merge_linear_supported(int count, int head_dim, int dtype) {
  return dtype == PS_BF16 && count >= 1 && count <= 16 && head_dim % 64 == 0 && head_dim <= 256;
}

// tiles_per_block: 0, or how many heads a block takes (1, 2 or 4 waves whose results are summed
// before they are added to the residual rows); 0 leaves the choice to this file.
extern "C" int ps_attention_merge_linear(const float* partial, int64_t partial_floats,
                                         const int* tok_list, int count, int heads, int head_dim,
                                         int splits, const void* w_packed, const float* bias,
                                         float* residual, int64_t ld_res, int n,
                                         int tiles_per_block, void* stream) {
  PS_REQUIRE(count >= 0 && heads > 0 && heads <= 65535 && splits >= 1 && splits <= 64 && n > 0 &&
                 ld_res >= n,
             "ps_attention_merge_linear: bad sizes (count %d, heads %d, splits %d, n %d)", count,
             heads, splits, n);
  PS_REQUIRE(ps_attention_merge_linear_supported(count > 0 ? count : 1, head_dim, PS_BF16),
             "ps_attention_merge_linear: up to 16 rows and head sizes of 64, 128, 192 or 256, not "
             "%d rows of head size %d", count, head_dim);
  PS_REQUIRE(partial != nullptr && partial_floats >= (int64_t)count * heads * splits * (head_dim + 2),
             "ps_attention_merge_linear: the records need %lld floats",
             (long long)count * heads * splits * (head_dim + 2));
  PS_REQUIRE(w_packed != nullptr && residual != nullptr &&
                 (reinterpret_cast<uintptr_t>(w_packed) & 15u) == 0 &&
                 (reinterpret_cast<uintptr_t>(partial) & 7u) == 0,
             "ps_attention_merge_linear: null or unaligned operand");
  PS_REQUIRE(tiles_per_block == 0 || tiles_per_block == 1 || tiles_per_block == 2 || tiles_per_block == 4,
             "ps_attention_merge_linear: 1, 2 or 4 heads per block, not %d", tiles_per_block);
  if (count == 0) return 0;
  const int tiles_n = (n + 15) / 16;
  // Four heads to a block save three quarters of the atomic adds, but a block then pulls four
  // waves' records through one compute unit, and fewer blocks than units leave units idle.
  // Measured (8 rows x 8 ranges, 12 heads of 64: 5.9 us with one head per block, 6.4 with four;
  // 16 rows x 2 ranges: 5.9 and 4.4; one row x 8 ranges: 5.4 and 4.8; 16 heads and more: four
  // heads ahead or level throughout): four where the records are few or the blocks still fill
  // the chip, else one.
  int group_heads = tiles_per_block;
  if (group_heads == 0) {
    const int wanted = heads >= 4 ? 4 : (heads >= 2 ? 2 : 1);
    const bool light = splits <= 2 || count * splits <= 16;
    const bool fills = tiles_n * ((heads + wanted - 1) / wanted) >= ps_compute_units();
    group_heads = (light || fills) ? wanted : 1;
  }
  dim3 grid(tiles_n, (heads + group_heads - 1) / group_heads);
  hipStream_t s = (hipStream_t)stream;
  // shares of the ranges for the free operand columns where there are many ranges (up to 8
  // ranges a lane has them all in flight at once, and shares measured no faster)
  int rows_pow2 = 1;
  while (rows_pow2 < count) rows_pow2 <<= 1;
  if (splits <= 8) rows_pow2 = 16;
  const int parts = 16 / rows_pow2;
#define PS_LAUNCH_AMLG(STEPS, PARTS, GROUP)                                                     \
  hipLaunchKernelGGL((attention_merge_linear_kernel<STEPS, PARTS, GROUP>), grid, dim3(64 * GROUP), \
                     0, s, partial, tok_list, count, heads, splits, (const bf16_t*)w_packed, bias, \
                     residual, ld_res, n)
#define PS_LAUNCH_AML(STEPS, PARTS)                        \
  do {                                                     \
    if (group_heads == 4) PS_LAUNCH_AMLG(STEPS, PARTS, 4); \
    else if (group_heads == 2) PS_LAUNCH_AMLG(STEPS, PARTS, 2); \
    else PS_LAUNCH_AMLG(STEPS, PARTS, 1);                  \
  } while (0)
#define PS_LAUNCH_AMLP(STEPS)                     \
  do {                                            \
    if (parts == 1) PS_LAUNCH_AML(STEPS, 1);      \
    else if (parts == 2) PS_LAUNCH_AML(STEPS, 2); \
    else if (parts == 4) PS_LAUNCH_AML(STEPS, 4); \
    else if (parts == 8) PS_LAUNCH_AML(STEPS, 8); \
    else PS_LAUNCH_AML(STEPS, 16);                \
  } while (0)
  switch (head_dim / 64) {
    case 1: PS_LAUNCH_AMLP(1); break;
    case 2: PS_LAUNCH_AMLP(2); break;
    case 3: PS_LAUNCH_AMLP(3); break;
    default: PS_LAUNCH_AMLP(4); break;
  }
#undef PS_LAUNCH_AMLP
#undef PS_LAUNCH_AML
#undef PS_LAUNCH_AMLG
  PS_CHECK_LAUNCH("ps_attention_merge_linear");
  return 0;
}
