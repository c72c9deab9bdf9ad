// Tiled bfloat16 matrix product for many rows (prompt portions) on gfx950:
//   C[m, n] = epi(sum_k A[m, k] W[n, k] + b[n]),   k a multiple of 64.
//
// Operand tiles go from global memory straight into LDS (global_load_lds_dwordx4: no trip
// through registers), several k tiles ahead of the one being multiplied.  A stage holds 64
// values of k (128 bytes) of every row of the block's A and W tiles.  One load instruction of
// a wave fills 1024 contiguous bytes of LDS, eight rows; which 16-byte piece of its row a
// lane fetches is chosen so that piece c of row r lands in slot c ^ ((r >> 1) & 7) of the
// row.  With that, the 16 lanes that read one k piece of 16 consecutive rows for an MFMA
// operand touch every LDS bank once.
//
// Four waves in a 2 x 2 arrangement; a wave owns WM x WN accumulators of 32 x 32
// (v_mfma_f32_32x32x16_bf16, float accumulation), so a block makes 64 WM x 64 WN outputs.
// With KW = 2 the two waves of a row of the arrangement share one accumulator of 32 columns
// instead and take every other k tile each; the block meets once per pair of tiles, and the
// two sums meet in LDS at the end.  A block then makes 64 x 32 outputs: twice as many blocks
// for a product of up to 64 rows whose tiles of 64 columns would leave most compute units
// without one, and half as many meetings along k, which is what such a lone block waits for.
// Per k tile there is one wait (own loads of the next tile have landed; later tiles stay in
// flight) and one barrier, placed before the tile's last k step so that three steps' products
// are queued in the matrix core meanwhile; after it the stage that was multiplied before is
// refilled and the next tile's first operands are fetched.
//
// Rows beyond m or n are fetched from the last valid row instead (they only feed outputs that
// are never stored).  The epilogue is the one of the other products: bias, GELU, residual
// add into the float stream, key/value columns into cache pages.
#include "common.h"
#include "linear.h"
#include "pagedserve_hip.h"

#include "gemm_bf16_common.h"

// Wait until at most `pending` of this wave's loads are in flight, then meet the other waves.
// The asm statements are compiler barriers for memory as well: LDS reads stay behind them.
template <int PENDING>
__device__ inline void wait_loads_and_sync() {
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(PENDING) : "memory");
}

// The same with `ahead` tiles (known only at run time) of LOADS loads each left in flight.
template <int LOADS, int MOST>
__device__ inline void wait_ahead_and_sync(int ahead) {
  if (ahead <= 0) wait_loads_and_sync<0>();
  else if (ahead == 1 || MOST == 1) wait_loads_and_sync<LOADS>();
  else if (ahead == 2 || MOST == 2) wait_loads_and_sync<2 * LOADS>();
  else if (ahead == 3 || MOST == 3) wait_loads_and_sync<(MOST >= 3 ? 3 : 0) * LOADS>();
  else if (ahead == 4 || MOST == 4) wait_loads_and_sync<(MOST >= 4 ? 4 : 0) * LOADS>();
  else if (ahead == 5 || MOST == 5) wait_loads_and_sync<(MOST >= 5 ? 5 : 0) * LOADS>();
  else wait_loads_and_sync<(MOST >= 6 ? 6 : 0) * LOADS>();
}

template <int WM, int WN, int STAGES, typename TOut, int EPI, int KW = 1>
__global__ __launch_bounds__(256) void gemm_nt_bf16_tiled_kernel(
    const bf16_t* __restrict__ a, const bf16_t* __restrict__ w, const float* __restrict__ bias,
    TOut* __restrict__ c, int m, int n, int k, int lda, int ldc, int tiles_m, int tiles_n,
    int row_major, int k_splits, int k_chunk, KvScatter scatter) {
  static_assert(KW == 1 || (KW == 2 && WM == 1 && WN == 1), "k halves go with one accumulator per wave");
  constexpr int BM = 64 * WM, BN = 64 * WN / KW;
  constexpr int STAGE_BYTES = (BM + BN) * TB_ROW;
  constexpr int LOADS_A = BM / 32;   // load instructions per wave and stage (8 rows each)
  constexpr int LOADS_W = BN / 32;
  constexpr int LOADS = LOADS_A + LOADS_W;
  static_assert(STAGES >= 2 && STAGES <= 8, "two to eight stages");
  static_assert(LOADS * (STAGES - 1) < 64, "the load counter has six bits");
  __shared__ __attribute__((aligned(1024))) unsigned char lds[STAGES * STAGE_BYTES];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // the same in every lane: scalar
  const int wave_m = wave >> 1;
  const int wave_n = KW == 1 ? wave & 1 : 0;
  const int wave_k = KW == 1 ? 0 : wave & 1;     // which tile of a pair of k tiles
  // Consecutive block ids run on different XCDs, each with an L2 of its own: blocks are
  // renumbered so that every XCD works on a contiguous run of tiles.  A run walked along the
  // rows of C reads few rows of A and all of W, one walked down the columns few rows of W and
  // all of A: the host picks the cheaper one.
  const int blocks = gridDim.x;
  const int per_xcd = blocks / 8;
  int logical = blockIdx.x;
  if (blockIdx.x < per_xcd * 8) logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  const int tiles = tiles_m * tiles_n;
  const int split = logical / tiles;
  const int tile = logical - split * tiles;
  const int tile_n = row_major ? tile % tiles_n : tile / tiles_m;
  const int tile_m = row_major ? tile / tiles_n : tile % tiles_m;
  const int m0 = tile_m * BM;
  const int n0 = tile_n * BN;
  const int k_begin = split * k_chunk;
  const int k_tiles = ((k_begin + k_chunk < k ? k_begin + k_chunk : k) - k_begin) / TB_BK;

  // ---- loads: lane l of a load instruction fills slot l % 8 of row l / 8 of its eight rows
  const bf16_t* src[LOADS];
  int dst[LOADS];
#pragma unroll
  for (int j = 0; j < LOADS; ++j) {
    const bool is_a = j < LOADS_A;
    const int group = is_a ? wave * LOADS_A + j : wave * LOADS_W + (j - LOADS_A);
    const int tile_row = group * 8 + (lane >> 3);
    const int piece = (lane & 7) ^ ((tile_row >> 1) & 7);
    if (is_a) {
      const int row = m0 + tile_row < m ? m0 + tile_row : m - 1;
      src[j] = a + (int64_t)row * lda + k_begin + piece * 8;
      dst[j] = group * 8 * TB_ROW;
    } else {
      const int row = n0 + tile_row < n ? n0 + tile_row : n - 1;
      src[j] = w + (int64_t)row * k + k_begin + piece * 8;
      dst[j] = (BM + group * 8) * TB_ROW;
    }
  }
  auto issue = [&](int kt) {
    unsigned char* stage = lds + (kt % STAGES) * STAGE_BYTES;
#pragma unroll
    for (int j = 0; j < LOADS; ++j)
      __builtin_amdgcn_global_load_lds((global_ptr_t)(src[j] + (int64_t)kt * TB_BK),
                                       (lds_ptr_t)(stage + dst[j]), 16, 0, 0);
  };

  f32x16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // ---- operands: lane l reads the 16 bytes of k piece 2 s + l / 32 of row l % 32
  const int key = (lane >> 1) & 7;   // ((row >> 1) & 7) of every row this lane reads
  const int a_row = (wave_m * WM * 32 + (lane & 31)) * TB_ROW;
  const int w_row = (BM + wave_n * WN * 32 + (lane & 31)) * TB_ROW;
  // The operands of k step s + 1 are fetched before the products of step s are issued, also
  // across tiles: before the last step of a tile the wave waits for the next tile's loads
  // and meets the other waves, with three steps' products already queued in the matrix core,
  // then fetches the next tile's first operands.
  //
  // The reads are written as assembly with counted waits.  Left to itself the compiler waits
  // for every LDS read in flight (lgkmcnt(0)) before each product, the ones it has just issued
  // for the next step included, so that every step paid a whole trip to LDS and a k tile of a
  // lone block took 800 cycles, of which the matrix instructions are 128.  LDS reads come back
  // in the order of issue: waiting until READS are left in flight leaves exactly the next
  // step's.
  typedef unsigned int tb_u32x4 __attribute__((ext_vector_type(4)));
  constexpr int READS = WM + WN;    // LDS reads of one k step
  tb_u32x4 fa[2][WM], fw[2][WN];
  const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
  auto fetch = [&](int kt, int s, tb_u32x4* da, tb_u32x4* dw) {
    const uint32_t stage = lds_base + (uint32_t)((kt % STAGES) * STAGE_BYTES);
    const uint32_t slot = (uint32_t)(((2 * s + (lane >> 5)) ^ key) << 4);
#pragma unroll
    for (int i = 0; i < WM; ++i)
      asm volatile("ds_read_b128 %0, %1"
                   : "=v"(da[i])
                   : "v"(stage + (uint32_t)(a_row + i * 32 * TB_ROW) + slot)
                   : "memory");
#pragma unroll
    for (int j = 0; j < WN; ++j)
      asm volatile("ds_read_b128 %0, %1"
                   : "=v"(dw[j])
                   : "v"(stage + (uint32_t)(w_row + j * 32 * TB_ROW) + slot)
                   : "memory");
  };
  constexpr int STEPS = TB_BK / 16;
  static_assert(STEPS % 2 == 0, "the operand buffers alternate per step");

  if constexpr (KW == 2) {
    // Tiles in pairs: tile 2 p belongs to the first wave of a row, tile 2 p + 1 to the second.
    // The ring holds STAGES / 2 pairs.  Per pair: wait until its two tiles have landed (later
    // ones stay in flight), meet the other waves (which are then past the pair before, so
    // that pair's stages can be refilled), multiply the own tile's four steps.
    static_assert(STAGES % 2 == 0 && STAGES >= 4, "the ring holds whole pairs");
    constexpr int HELD = STAGES / 2;
    const int pairs = (k_tiles + 1) / 2;
#pragma unroll
    for (int d = 0; d < 2 * (HELD - 1); ++d)
      if (d < k_tiles) issue(d);
    for (int p = 0; p < pairs; ++p) {
      const int issued = k_tiles < 2 * (p + HELD - 1) ? k_tiles : 2 * (p + HELD - 1);
      wait_ahead_and_sync<LOADS, STAGES - 4>(issued - (2 * p + 2));
#pragma unroll
      for (int d = 0; d < 2; ++d)
        if (2 * (p + HELD - 1) + d < k_tiles) issue(2 * (p + HELD - 1) + d);
      const int kt = 2 * p + wave_k;
      if (kt < k_tiles) {
        // all four steps' operands are asked for at once and used as they arrive (reads come
        // back in the order of issue): one trip to LDS per tile stands open, not one per step
        tb_u32x4 ga[STEPS], gw[STEPS];
#pragma unroll
        for (int s = 0; s < STEPS; ++s) fetch(kt, s, &ga[s], &gw[s]);
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
          if (s == 0) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(READS * (STEPS - 1)) : "memory");
          else if (s == 1) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(READS * (STEPS - 2)) : "memory");
          else if (s == 2) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(READS * (STEPS - 3)) : "memory");
          else asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
          asm volatile("" : "+v"(ga[s]));
          asm volatile("" : "+v"(gw[s]));
          acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
              *reinterpret_cast<const bf16x8*>(&ga[s]), *reinterpret_cast<const bf16x8*>(&gw[s]),
              acc[0][0], 0, 0, 0);
        }
      }
    }
  } else {
  #pragma unroll
    for (int d = 0; d < STAGES - 1; ++d)
      if (d < k_tiles) issue(d);
    {
      // tile 0 has landed; tiles 1 .. STAGES - 2 may stay in flight, as far as they exist
      const int ahead = k_tiles - 1 < STAGES - 2 ? k_tiles - 1 : STAGES - 2;
      wait_ahead_and_sync<LOADS, STAGES - 2>(ahead);
    }
    fetch(0, 0, fa[0], fw[0]);
    for (int kt = 0; kt < k_tiles; ++kt) {
      // the stage of tile kt - 1 is free: every wave met the others after its last read of it
      if (kt + STAGES - 1 < k_tiles) issue(kt + STAGES - 1);
  #pragma unroll
      for (int s = 0; s < STEPS; ++s) {
        if (s + 1 < STEPS) {
          fetch(kt, s + 1, fa[(s + 1) & 1], fw[(s + 1) & 1]);
          asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(READS) : "memory");   // step s has arrived
        } else {
          // own reads of this tile are complete before the others may overwrite its stage
          // (one wait for both cases, ahead of the branch: the last step's operands are then
          // complete on every path that leads to their product)
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
          if (kt + 1 < k_tiles) {
            // tiles kt + 2 .. kt + STAGES - 1 may stay in flight, as far as they exist
            const int last = k_tiles - 1 < kt + STAGES - 1 ? k_tiles - 1 : kt + STAGES - 1;
            wait_ahead_and_sync<LOADS, STAGES - 2>(last - (kt + 1));
            fetch(kt + 1, 0, fa[0], fw[0]);
          }
        }
        // the registers are used only behind the wait (the compiler does not know that the
        // assembly above left them on their way)
  #pragma unroll
        for (int i = 0; i < WM; ++i) asm volatile("" : "+v"(fa[s & 1][i]));
  #pragma unroll
        for (int j = 0; j < WN; ++j) asm volatile("" : "+v"(fw[s & 1][j]));
  #pragma unroll
        for (int i = 0; i < WM; ++i)
  #pragma unroll
          for (int j = 0; j < WN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                *reinterpret_cast<const bf16x8*>(&fa[s & 1][i]),
                *reinterpret_cast<const bf16x8*>(&fw[s & 1][j]), acc[i][j], 0, 0, 0);
      }
    }
  }

  // ---- epilogue (gemm_bf16_common.h): each wave turns its accumulators through a region of
  // LDS of its own and stores rows in aligned pieces
  static_assert(4 * 32 * (WN * 32 + 8) * 4 + (KW - 1) * 2 * 16 * 64 * 4 <= STAGES * STAGE_BYTES,
                "the epilogue reuses the stages");
  // every wave is past its last operand reads (and no assembly read is on its way any more,
  // whichever way the loop was left)
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  if (KW == 2) {
    // the wave of the odd k tiles hands its sums to the wave of the even ones, behind the
    // regions that the epilogue uses
    float* meet = reinterpret_cast<float*>(lds) + 4 * 32 * (WN * 32 + 8) + wave_m * 16 * 64;
    if (wave_k == 1) {
#pragma unroll
      for (int e = 0; e < 16; ++e) meet[e * 64 + lane] = acc[0][0][e];
    }
    __syncthreads();
    if (wave_k == 1) return;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[0][0][e] += meet[e * 64 + lane];
  }
  store_wave_tile<WM, WN, TOut, EPI>(acc, reinterpret_cast<float*>(lds) + wave * 32 * (WN * 32 + 8),
                                     lane, m0 + wave_m * WM * 32, n0 + wave_n * WN * 32, m, n, ldc,
                                     c, bias, split, k_splits, scatter);
}

// --------------------------------------------------------------------------------- host
bool ps_gemm_nt_bf16_tiled_supported(const void* a, const void* w, int m, int k, int lda) {
  return m > 32 && k % TB_BK == 0 && lda % 8 == 0 &&
         (reinterpret_cast<uintptr_t>(a) & 15u) == 0 && (reinterpret_cast<uintptr_t>(w) & 15u) == 0;
}

template <int WM, int WN, int STAGES, typename TOut, int KW = 1>
static int launch_variant(const void* a, const void* w, const float* bias, void* c, int m, int n,
                          int k, int lda, int ldc, int epilogue, const KvScatter& scatter,
                          hipStream_t s) {
  constexpr int BM = 64 * WM, BN = 64 * WN / KW;
  const int tiles_m = (m + BM - 1) / BM;
  const int tiles_n = (n + BN - 1) / BN;
  // what one XCD's run of tiles fetches into its L2, in rows of k values
  const int run = (tiles_m * tiles_n + 7) / 8;
  const int64_t rows_along = (int64_t)((run + tiles_n - 1) / tiles_n) * BM + n;   // along rows of C
  const int64_t rows_down = (int64_t)((run + tiles_m - 1) / tiles_m) * BN + m;    // down columns
  const int row_major = rows_along < rows_down ? 1 : 0;
  // Few tiles with a long k leave most of the chip idle: where partial sums can be added in
  // place (residual epilogue) k is split over blocks.  Float atomics are slow, so this pays
  // only while the output is small.
  int k_splits = 1;
  if (epilogue == PS_EPI_RESIDUAL && tiles_m * tiles_n <= ps_compute_units() / 4 && k >= 2048) {
    k_splits = ps_compute_units() / (tiles_m * tiles_n);
    if (k_splits > k / 256) k_splits = k / 256;
  }
  int k_chunk = (k / TB_BK + k_splits - 1) / k_splits * TB_BK;
  k_splits = (k + k_chunk - 1) / k_chunk;
  dim3 grid(tiles_m * tiles_n * k_splits);
#define PS_LAUNCH_TB(EPI)                                                                     \
  hipLaunchKernelGGL((gemm_nt_bf16_tiled_kernel<WM, WN, STAGES, TOut, EPI, KW>), grid, dim3(256), 0, \
                     s, (const bf16_t*)a, (const bf16_t*)w, bias, (TOut*)c, m, n, k, lda, ldc, \
                     tiles_m, tiles_n, row_major, k_splits, k_chunk, scatter)
  switch (epilogue) {
    case PS_EPI_NONE: PS_LAUNCH_TB(PS_EPI_NONE); break;
    case PS_EPI_GELU_TANH: PS_LAUNCH_TB(PS_EPI_GELU_TANH); break;
    case PS_EPI_GELU_ERF: PS_LAUNCH_TB(PS_EPI_GELU_ERF); break;
    case PS_EPI_RESIDUAL: PS_LAUNCH_TB(PS_EPI_RESIDUAL); break;
    default: ps_set_error("ps_linear: unknown epilogue %d", epilogue); return 1;
  }
#undef PS_LAUNCH_TB
  PS_CHECK_LAUNCH("ps_linear(tiled, bfloat16)");
  return 0;
}

// Tile shapes by the number of blocks they give against the chip's compute units: a product
// of this size is over in a few microseconds, so filling them counts for more than the reuse
// inside a large tile.
template <typename TOut>
static int launch_tiled_bf16(const void* a, const void* w, const float* bias, void* c, int m,
                             int n, int k, int lda, int ldc, int epilogue,
                             const KvScatter& scatter, hipStream_t s) {
  const int64_t tiles_128 = (int64_t)((m + 127) / 128) * ((n + 127) / 128);
  const int64_t tiles_128_64 = (int64_t)((m + 127) / 128) * ((n + 63) / 64);
  const int units = ps_compute_units();
  if (m > 64 && tiles_128 >= 3 * units)
    return launch_variant<2, 2, 2, TOut>(a, w, bias, c, m, n, k, lda, ldc, epilogue, scatter, s);
  // 128 x 64: three stages while two blocks per unit hold them all (1100 x 3072 x 1024 with
  // weights from memory: 16.1 against 17.7 us), two stages, which let a third block in, beyond
  if (m > 64 && tiles_128_64 >= units + units / 2 && tiles_128_64 <= 2 * units)
    return launch_variant<2, 1, 3, TOut>(a, w, bias, c, m, n, k, lda, ldc, epilogue, scatter, s);
  if (m > 64 && tiles_128_64 >= units + units / 2)
    return launch_variant<2, 1, 2, TOut>(a, w, bias, c, m, n, k, lda, ldc, epilogue, scatter, s);
  // a long k with a block per compute unit: four stages of 128 x 64 (2048 x 1024 x 4096 with
  // weights from memory: 34.7 us against 37.8 for 64 x 64 tiles)
  if (m > 64 && k >= 2048 && tiles_128_64 >= units)
    return launch_variant<2, 1, 4, TOut>(a, w, bias, c, m, n, k, lda, ldc, epilogue, scatter, s);
  // 64 x 64 tiles.  What a compute unit has in flight decides how long a k tile takes to
  // arrive from memory.  Many blocks fill a unit by their number and keep two stages, which
  // lets five of them in; up to two blocks per unit get four stages each.  That also holds for
  // a single row of tiles over a long k (a decode step of a wide model), which leaves most
  // units empty and the others with one block: a ring of eight stages, as deep as LDS allows,
  // measured behind four there once the weights came from memory and not from the caches
  // (64 x 4800 x 1600: 13.8 against 11.9 us; 3 % of the decode step at that width).
  const int64_t tiles_64 = (int64_t)((m + 63) / 64) * ((n + 63) / 64);
  const int k_tiles = k / TB_BK;
  // So few tiles of 64 x 64 that half of the units would be without a block (the QKV and first
  // feed-forward products of a wide model's decode step; the products with few columns of a
  // step that mixes a prompt portion with decoded tokens): tiles of 32 columns, twice the
  // blocks, each fetching the rows and half as much of the matrix, and the two waves of a row
  // taking every other k tile (64 x 4800 x 1600 with weights from memory: 9.9 against 11.4 us;
  // 64 x 5120 x 1280: 8.9 against 10.4; 544 x 768 x 3072: 14.7 against 17.1; 544 x 768 x 768: 6.2
  // against 7.0; 544 x 1024 x 4096, 288 blocks: 20.7 against 22.0; with a short k more blocks than
  // units lose instead: 200 x 2304 x 768 on 288 blocks 7.2 against 6.8).  Six stages: two pairs of
  // tiles in flight while one is multiplied (four stages 13.5 us, eight 9.8).  What remains is
  // what a compute unit takes in: 307 KB per block at 55 KB/us beside 4.4 us that do not depend
  // on k (the time hardly depends on the columns: 8,192 take 10.4 us); asking for a tile's four
  // steps of operands at once instead of one step ahead changes nothing, and eight waves on a
  // tile of 64 x 64, four for the even and four for the odd k tiles, gain a third of this.
  if ((2 * tiles_64 <= units || (k >= 2048 && 16 * tiles_64 <= 9 * units)) && k_tiles > 2)
    return launch_variant<1, 1, 6, TOut, 2>(a, w, bias, c, m, n, k, lda, ldc, epilogue, scatter, s);
  if ((tiles_64 <= 2 * units && k_tiles > 2) || k >= 2048)
    return launch_variant<1, 1, 4, TOut>(a, w, bias, c, m, n, k, lda, ldc, epilogue, scatter, s);
  // up to three blocks per unit: three stages each (544 x 4096 x 1024: 15.9 against 18.2 us)
  if (tiles_64 <= 3 * units && k_tiles > 2)
    return launch_variant<1, 1, 3, TOut>(a, w, bias, c, m, n, k, lda, ldc, epilogue, scatter, s);
  return launch_variant<1, 1, 2, TOut>(a, w, bias, c, m, n, k, lda, ldc, epilogue, scatter, s);
}

int ps_gemm_nt_bf16_tiled(const void* a, const void* w, const float* bias, void* c, int m, int n,
                          int k, int lda, int ldc, int c_dtype, int epilogue,
                          const KvScatter& scatter, hipStream_t s) {
  if (c_dtype == PS_F32)
    return launch_tiled_bf16<float>(a, w, bias, c, m, n, k, lda, ldc, epilogue, scatter, s);
  return launch_tiled_bf16<bf16_t>(a, w, bias, c, m, n, k, lda, ldc, epilogue, scatter, s);
}
