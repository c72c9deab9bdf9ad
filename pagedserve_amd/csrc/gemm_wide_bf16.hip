// Tiled bfloat16 matrix product for many rows whose weight operand never passes through LDS:
//   C[m, n] = epi(sum_k A[m, k] W[n, k] + b[n]),   k a multiple of 64, W given in its packed copy.
//
// At the rate of the matrix cores a compute unit has to feed them 2 KB of operands per 32 x 32
// x 16 product; LDS delivers 128 bytes per cycle and the vector cache 64.  The kernel in
// gemm_tiled_bf16.hip brings both operands through LDS and reuses each fragment twice, which
// fills the LDS path at half the matrix cores' rate.  Here a block is four waves side by side
// along n: a wave owns 32 WM rows x 64 columns, the block 32 WM x 256.  The rows of A are
// shared by the four waves and go through LDS (straight from global memory, three k tiles in
// a ring, the rotation of pieces against bank conflicts as in the other kernel); the weights
// of a wave's 64 columns belong to it alone and come from global memory into registers, two
// k tiles ahead, out of the packed copy that the products of few rows use (pagedserve_hip.h:
// every 16 x 64 tile in the lanes' operand order), in which the lanes of one load read four
// runs of 256 consecutive bytes and four loads cover 4 KB without a gap.  With WM = 4 a
// fragment from LDS feeds two products and a fragment from memory four: LDS carries half of
// what it can, the vector cache likewise.
//
// Per k tile: the loads of the tile after next are issued (A into the LDS stage that was
// multiplied last, W into the register set that was multiplied last), four k steps of WM x 2
// products each run with the next step's A fragments fetched ahead, and before the last step
// the wave waits for its loads of the next tile and meets the other waves.  A wave's loads
// return in the order of issue, so that wait leaves exactly the loads issued in this tile in
// flight.
#include <type_traits>

#include "gemm_bf16_common.h"

typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;

#define GW_WN 2          // 32-column fragments per wave
#define GW_BN 256        // columns per block

template <int PENDING>
__device__ inline void gw_wait_loads_and_sync() {
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(PENDING) : "memory");
}

// The same with `tiles` tiles (known only at run time, at most MOST) of LOADS loads each left
// in flight.
template <int LOADS, int MOST>
__device__ inline void gw_wait_tiles_and_sync(int tiles) {
  if (tiles <= 0 || MOST == 0) gw_wait_loads_and_sync<0>();
  else if (tiles == 1 || MOST == 1) gw_wait_loads_and_sync<LOADS>();
  else if (tiles == 2 || MOST == 2) gw_wait_loads_and_sync<(MOST >= 2 ? 2 : 0) * LOADS>();
  else gw_wait_loads_and_sync<(MOST >= 3 ? 3 : 0) * LOADS>();
}

template <int WM, int GW_STAGES, typename TOut, int EPI>
__global__ __launch_bounds__(256) void gemm_nt_bf16_wide_kernel(
    const bf16_t* __restrict__ a, const bf16_t* __restrict__ wp, const float* __restrict__ bias,
    TOut* __restrict__ c, int m, int n, int k, int lda, int ldc, int tiles_m, int tiles_n,
    int row_major, int w_tiles16, KvScatter scatter) {
  constexpr int BM = 32 * WM;
  constexpr int STAGE_BYTES = BM * TB_ROW;
  constexpr int LOADS_A = WM;                     // BM / 8 loads of eight rows, four waves
  constexpr int LOADS_W = GW_WN * 4;              // per k tile: four k steps of each fragment
  constexpr int EP_BYTES = 4 * 32 * (GW_WN * 32 + 8) * 4;
  constexpr int LDS_BYTES = GW_STAGES * STAGE_BYTES > EP_BYTES ? GW_STAGES * STAGE_BYTES : EP_BYTES;
  __shared__ __attribute__((aligned(1024))) unsigned char lds[LDS_BYTES];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // the same in every lane: scalar
  // every XCD works on a contiguous run of tiles (see gemm_tiled_bf16.hip)
  const int blocks = gridDim.x;
  const int per_xcd = blocks / 8;
  int tile = blockIdx.x;
  if (blockIdx.x < per_xcd * 8) tile = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  const int tile_n = row_major ? tile % tiles_n : tile / tiles_m;
  const int tile_m = row_major ? tile / tiles_n : tile % tiles_m;
  const int m0 = tile_m * BM;
  const int n0 = tile_n * GW_BN;
  const int k_tiles = k / TB_BK;

  // ---- A: lane l of a load instruction fills slot l % 8 of row l / 8 of its eight rows
  const bf16_t* a_src[LOADS_A];
  int a_dst[LOADS_A];
#pragma unroll
  for (int j = 0; j < LOADS_A; ++j) {
    const int group = wave * LOADS_A + j;
    const int tile_row = group * 8 + (lane >> 3);
    const int piece = (lane & 7) ^ ((tile_row >> 1) & 7);
    const int row = m0 + tile_row < m ? m0 + tile_row : m - 1;
    a_src[j] = a + (int64_t)row * lda + piece * 8;
    a_dst[j] = group * 8 * TB_ROW;
  }
  // ---- W: lane l holds row l % 32 of a fragment and k piece l / 32; rows 0..15 of the
  // fragment lie in one 16-row tile of the packed copy, rows 16..31 in the next.  Element
  // (tile T, k tile s, k piece h, k step g, row r) of the copy is at
  // ((T * k_tiles + s) * 2 + h) * 512 + (g * 16 + r) * 8.
  const bf16_t* w_src[GW_WN];
#pragma unroll
  for (int j = 0; j < GW_WN; ++j) {
    int tile16 = (n0 + wave * (GW_WN * 32) + j * 32) / 16 + ((lane >> 4) & 1);
    if (tile16 >= w_tiles16) tile16 = w_tiles16 - 1;   // columns beyond n: never stored
    w_src[j] = wp + ((int64_t)tile16 * k_tiles * 2 + (lane >> 5)) * 512 + (lane & 15) * 8;
  }

  f32x16 acc[WM][GW_WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < GW_WN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // Weight fragments are loaded by assembly as well: the compiler then inserts no waits of its
  // own (at the head of the loop it would wait for every load in flight), and the one wait per
  // tile below covers them, since a wave's loads return in the order of issue.
  u32x4_t wreg[GW_STAGES][GW_WN][4];
  auto load_w = [&](int set, int tile_index) {
#pragma unroll
    for (int j = 0; j < GW_WN; ++j) {
      const bf16_t* source = w_src[j] + (int64_t)tile_index * 1024;
#pragma unroll
      for (int g = 0; g < 4; ++g)
        asm volatile("global_load_dwordx4 %0, %1, off offset:%2"
                     : "=v"(wreg[set][j][g])
                     : "v"(source), "n"(g * 256)
                     : "memory");
    }
  };
  u32x4_t fa[2][WM];
  const int key = (lane >> 1) & 7;
  const int a_row = (lane & 31) * TB_ROW;

  auto issue_a = [&](int kt, int stage_index) {
    unsigned char* stage = lds + stage_index * STAGE_BYTES;
#pragma unroll
    for (int j = 0; j < LOADS_A; ++j)
      __builtin_amdgcn_global_load_lds((global_ptr_t)(a_src[j] + (int64_t)kt * TB_BK),
                                       (lds_ptr_t)(stage + a_dst[j]), 16, 0, 0);
  };
  // the A fragments of k step `step` of the tile in LDS stage `stage_index`, by assembly: the
  // compiler does not see these as LDS reads and so does not wait for the loads in flight
  auto fetch_a = [&](int stage_index, int step, u32x4_t* dst) {
    const unsigned address = (unsigned)(uintptr_t)(lds_ptr_t)(lds + stage_index * STAGE_BYTES) +
                             a_row + (((2 * step + (lane >> 5)) ^ key) << 4);
#pragma unroll
    for (int i = 0; i < WM; ++i)
      asm volatile("ds_read_b128 %0, %1" : "=v"(dst[i]) : "v"(address + i * 32 * TB_ROW) : "memory");
  };

  // One k tile whose operands lie in LDS stage / register set B (a constant: the three sets
  // are three groups of registers).  `inner` says that two further tiles follow: the body then
  // has no branch, and the compiler, which counts the loads in flight along every path, leaves
  // the loads of the tiles ahead in flight (a path that skips loads makes it wait for all).
  auto run_tile = [&](int kt, auto set, auto inner) {
    constexpr int B = decltype(set)::value;
    constexpr int AHEAD = GW_STAGES - 1;
    constexpr int B2 = (B + AHEAD) % GW_STAGES;
    constexpr bool INNER = decltype(inner)::value;
    const bool more = INNER || kt + AHEAD < k_tiles;
    if (more) {
      // stage B2 held tile kt - 1: every wave met the others after its last read of it
      issue_a(kt + AHEAD, B2);
      load_w(B2, kt + AHEAD);
    }
#pragma unroll
    for (int step = 0; step < 4; ++step) {
      if (step < 3) {
        fetch_a(B, step + 1, fa[(step + 1) & 1]);
        // the fragments of this step were asked for before those: they have arrived when at
        // most WM reads are still on their way
        asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(WM) : "memory");
      } else {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (INNER || kt + 1 < k_tiles) {
          // own loads of tile kt + 1 have landed; the tiles asked for after it may stay in flight
          if (INNER) gw_wait_loads_and_sync<(GW_STAGES - 2) * (LOADS_A + LOADS_W)>();
          else gw_wait_tiles_and_sync<LOADS_A + LOADS_W, GW_STAGES - 2>(
                   (k_tiles - 1 < kt + AHEAD ? k_tiles - 1 : kt + AHEAD) - (kt + 1));
          fetch_a((B + 1) % GW_STAGES, 0, fa[0]);
        }
      }
#pragma unroll
      for (int i = 0; i < WM; ++i) {
        asm volatile("" : "+v"(fa[step & 1][i]));   // used only behind the wait
#pragma unroll
        for (int j = 0; j < GW_WN; ++j) {
          asm volatile("" : "+v"(wreg[B][j][step]));
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
              *reinterpret_cast<const bf16x8*>(&fa[step & 1][i]),
              *reinterpret_cast<const bf16x8*>(&wreg[B][j][step]), acc[i][j], 0, 0, 0);
        }
      }
      // the products of this step are issued before the next step's reads and waits
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // ---- the first tiles of the ring are asked for (without a branch, see above: beyond the
  // last k tile the last one is asked for again); tile 0 has landed when only the others'
  // loads are in flight
  static_assert(GW_STAGES >= 3 && GW_STAGES <= 5, "three to five sets of operands");
  static_assert((GW_STAGES - 1) * (LOADS_A + LOADS_W) < 64, "the load counter has six bits");
#pragma unroll
  for (int d = 0; d < GW_STAGES - 1; ++d) {
    const int tile_d = d < k_tiles ? d : k_tiles - 1;
    issue_a(tile_d, d);
    load_w(d, tile_d);
  }
  gw_wait_loads_and_sync<(GW_STAGES - 2) * (LOADS_A + LOADS_W)>();
  fetch_a(0, 0, fa[0]);
  int kt = 0;
  // every tile of this loop has GW_STAGES - 1 tiles behind it
  for (; kt + 2 * GW_STAGES - 2 < k_tiles; kt += GW_STAGES) {
    run_tile(kt, std::integral_constant<int, 0>{}, std::true_type{});
    run_tile(kt + 1, std::integral_constant<int, 1>{}, std::true_type{});
    run_tile(kt + 2, std::integral_constant<int, 2>{}, std::true_type{});
    if constexpr (GW_STAGES > 3) run_tile(kt + 3, std::integral_constant<int, 3 % GW_STAGES>{}, std::true_type{});
    if constexpr (GW_STAGES > 4) run_tile(kt + 4, std::integral_constant<int, 4 % GW_STAGES>{}, std::true_type{});
  }
  for (; kt < k_tiles; kt += GW_STAGES) {          // the last tiles
    run_tile(kt, std::integral_constant<int, 0>{}, std::false_type{});
    if (kt + 1 < k_tiles) run_tile(kt + 1, std::integral_constant<int, 1>{}, std::false_type{});
    if (kt + 2 < k_tiles) run_tile(kt + 2, std::integral_constant<int, 2>{}, std::false_type{});
    if constexpr (GW_STAGES > 3)
      if (kt + 3 < k_tiles) run_tile(kt + 3, std::integral_constant<int, 3 % GW_STAGES>{}, std::false_type{});
    if constexpr (GW_STAGES > 4)
      if (kt + 4 < k_tiles) run_tile(kt + 4, std::integral_constant<int, 4 % GW_STAGES>{}, std::false_type{});
  }

  // ---- epilogue: every wave is past its last operand reads before LDS is reused (and no
  // assembly read is on its way any more, whichever way the loops were left)
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  store_wave_tile<WM, GW_WN, TOut, EPI>(
      acc, reinterpret_cast<float*>(lds) + wave * 32 * (GW_WN * 32 + 8), lane, m0,
      n0 + wave * (GW_WN * 32), m, n, ldc, c, bias, 0, 1, scatter);
}

// --------------------------------------------------------------------------------- host
// Whether this kernel takes the product: the packed copy of W is there, k is a multiple of 64
// (the copy's tiles), rows of A can be loaded in pieces of 16 bytes, k is long and blocks of
// 64 rows x 256 columns fill most of the chip.  Measured with weights that no cache holds (a
// different copy at every launch, as in a step through many layers), at 2,048 rows: 4096 x 1024
// 28.5 us against 42.4 for the kernel with both operands in LDS, 4800 x 1600 47.4 against 58.1,
// 1600 x 6400 68.0 against 92.5; but 768 x 3072 (three blocks side by side) 29.9 against 27.1,
// and at k = 768 the two are level.  (With the same weights at every launch, out of the L2,
// this kernel looks better than it is.)
bool ps_gemm_nt_bf16_wide_supported(const void* a, const void* w_packed, int m, int n, int k,
                                    int lda) {
  const int64_t blocks = (int64_t)((n + GW_BN - 1) / GW_BN) * ((m + 63) / 64);
  return w_packed != nullptr && k >= 1024 && blocks >= ps_compute_units() * 5 / 8 &&
         k % TB_BK == 0 && lda % 8 == 0 && (reinterpret_cast<uintptr_t>(a) & 15u) == 0 &&
         (reinterpret_cast<uintptr_t>(w_packed) & 15u) == 0;
}

template <int WM, int STAGES, typename TOut>
static int launch_wide(const void* a, const void* wp, const float* bias, void* c, int m, int n,
                       int k, int lda, int ldc, int epilogue, const KvScatter& scatter,
                       hipStream_t s) {
  constexpr int BM = 32 * WM;
  const int tiles_m = (m + BM - 1) / BM;
  const int tiles_n = (n + GW_BN - 1) / GW_BN;
  const int run = (tiles_m * tiles_n + 7) / 8;
  const int64_t rows_along = (int64_t)((run + tiles_n - 1) / tiles_n) * BM + n;
  const int64_t rows_down = (int64_t)((run + tiles_m - 1) / tiles_m) * GW_BN + m;
  const int row_major = rows_along < rows_down ? 1 : 0;
  const int w_tiles16 = (n + 15) / 16;
  dim3 grid(tiles_m * tiles_n);
#define PS_LAUNCH_GW(EPI)                                                                      \
  hipLaunchKernelGGL((gemm_nt_bf16_wide_kernel<WM, STAGES, TOut, EPI>), grid, dim3(256), 0, s,         \
                     (const bf16_t*)a, (const bf16_t*)wp, bias, (TOut*)c, m, n, k, lda, ldc,   \
                     tiles_m, tiles_n, row_major, w_tiles16, scatter)
  switch (epilogue) {
    case PS_EPI_NONE: PS_LAUNCH_GW(PS_EPI_NONE); break;
    case PS_EPI_GELU_TANH: PS_LAUNCH_GW(PS_EPI_GELU_TANH); break;
    case PS_EPI_GELU_ERF: PS_LAUNCH_GW(PS_EPI_GELU_ERF); break;
    case PS_EPI_RESIDUAL: PS_LAUNCH_GW(PS_EPI_RESIDUAL); break;
    default: ps_set_error("ps_linear: unknown epilogue %d", epilogue); return 1;
  }
#undef PS_LAUNCH_GW
  PS_CHECK_LAUNCH("ps_linear(wide, bfloat16)");
  return 0;
}

// rows_per_block: 64 or 32; 0 means 64.  (Blocks of 128 rows measured no faster and need
// more than a wave's 256 vector registers: the compiler then parks values in accumulation
// registers, also weight fragments that the assembly loads have not yet delivered.)
int ps_gemm_nt_bf16_wide(const void* a, const void* w_packed, const float* bias, void* c, int m,
                         int n, int k, int lda, int ldc, int c_dtype, int epilogue,
                         const KvScatter& scatter, int rows_per_block, hipStream_t s) {
  // blocks of 64 rows measured fastest wherever this kernel is ahead at all; blocks of 128
  // rows draw level at shapes of thousands of rows and columns, blocks of 32 rows never do
  if (rows_per_block == 0) rows_per_block = 64;
#define PS_WIDE(WM, ST)                                                                                \
  (c_dtype == PS_F32                                                                                   \
       ? launch_wide<WM, ST, float>(a, w_packed, bias, c, m, n, k, lda, ldc, epilogue, scatter, s)      \
       : launch_wide<WM, ST, bf16_t>(a, w_packed, bias, c, m, n, k, lda, ldc, epilogue, scatter, s))
  // (rings of four and five sets measured no faster than three at any shape: the products do
  // not wait for memory)
  if (rows_per_block == 64) return PS_WIDE(2, 3);
  if (rows_per_block == 32) return PS_WIDE(1, 3);

#undef PS_WIDE
  ps_set_error("ps_linear: the wide product has blocks of 64 or 32 rows, not %d", rows_per_block);
  return 1;
}

// The wide product on its own, for tests and measurements of its block shapes.
extern "C" int ps_gemm_nt_wide(const void* a, const void* w_packed, const float* bias, void* c,
                               int m, int n, int k, int lda, int ldc, int c_dtype, int epilogue,
                               int rows_per_block, void* stream) {
  PS_REQUIRE(m > 0 && n > 0 && k > 0 && k % TB_BK == 0 && lda >= k && ldc >= n && lda % 8 == 0,
             "ps_gemm_nt_wide: bad sizes (m %d, n %d, k %d, lda %d, ldc %d)", m, n, k, lda, ldc);
  PS_REQUIRE(a && w_packed && c && (reinterpret_cast<uintptr_t>(a) & 15u) == 0 &&
                 (reinterpret_cast<uintptr_t>(w_packed) & 15u) == 0,
             "ps_gemm_nt_wide: null or unaligned operand");
  PS_REQUIRE(c_dtype == PS_F32 || c_dtype == PS_BF16, "ps_gemm_nt_wide: unknown output dtype");
  PS_REQUIRE(epilogue != PS_EPI_RESIDUAL || c_dtype == PS_F32,
             "ps_gemm_nt_wide: the residual epilogue needs a float output");
  KvScatter none = {};
  return ps_gemm_nt_bf16_wide(a, w_packed, bias, c, m, n, k, lda, ldc, c_dtype, epilogue, none,
                              rows_per_block, (hipStream_t)stream);
}
