// Matrix products on the matrix cores (MFMA) of gfx950:  C[m, n] = epi(sum_k A[m, k] W[n, k] + b[n]).
//
// Two kernels (the tiled bfloat16 product for many rows with k a multiple of 64 is a file of
// its own, gemm_tiled_bf16.hip; this file dispatches to it).
//
// gemm_nt_tiled_kernel — many rows in float32, and bfloat16 shapes the other tiled kernel does
//   not take.  128 x 128 outputs per 256-thread block, four waves in a 2 x 2 arrangement, each
//   wave 2 x 2 tiles of 32 x 32.  A and W tiles of 64 bytes of k per row go global ->
//   registers -> LDS (two buffers, one barrier per k tile); every lane reads 16 bytes of k for
//   its row from LDS.  For bfloat16 that is the operand of one v_mfma_f32_32x32x16_bf16; for
//   float the four values feed four v_mfma_f32_32x32x2_f32 (both operands use the same
//   assignment of k to lanes and instructions, which is all a dot product needs).  The float
//   instantiation multiplies true 32-bit inputs.
//
// gemm_nt_skinny_kernel — up to 64 rows (decode), bfloat16.  The product is bound by reading W
//   once, and at these sizes by the latency of that one trip to memory, so weights go straight
//   from global memory into MFMA operands and every wave issues all its loads before it
//   multiplies.  A block owns 16 weight rows; its four waves take a quarter of k each (every
//   lane loads 32 contiguous bytes of one row per 64 k) and feed v_mfma_f32_16x16x32_bf16 with
//   the weights as row operand and up to four blocks of 16 activation rows as column operands;
//   the four partial tiles are summed through LDS.  K may also be split over blocks; those
//   partial sums are added into the float output with hardware float atomics (only the
//   residual epilogue allows it).
//
// (The skinny kernel for up to 16 rows with the norm of its input fused in front is a file of
// its own, gemm_skinny_norm.hip.)
//
// All of them can also store the key and value columns of a [q | k | v] output into cache
// pages from their epilogue (KvScatter).
//
// Accumulation is float in all cases.  Shapes that the kernels cannot take (k not a multiple
// of 8 elements, unaligned rows) are refused by ps_gemm_nt_mfma_supported and run on the
// plain kernel instead.
#include "gemm_skinny.h"

typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;

#define TG_BM 128
#define TG_BN 128
#define TG_ROW_BYTES 64   // k bytes per row and stage
#define TG_LDS_STRIDE 80  // padded row stride in bytes (keeps 16-byte alignment)

template <typename T>
struct Mma;

template <>
struct Mma<bf16_t> {
  static constexpr int K_PER_CHUNK = 8;  // elements in 16 bytes
  __device__ static inline void step(const uint4& a, const uint4& b, f32x16& acc) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const bf16x8*>(&a),
                                                  *reinterpret_cast<const bf16x8*>(&b), acc, 0, 0, 0);
  }
};

template <>
struct Mma<float> {
  static constexpr int K_PER_CHUNK = 4;
  __device__ static inline void step(const uint4& a, const uint4& b, f32x16& acc) {
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x), __uint_as_float(b.x), acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y), __uint_as_float(b.y), acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z), __uint_as_float(b.z), acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w), __uint_as_float(b.w), acc, 0, 0, 0);
  }
};

#define TG_DEPTH 4   // k tiles whose global loads are in flight

template <typename T, typename TOut, int EPI>
__global__ __launch_bounds__(256) void gemm_nt_tiled_kernel(
    const T* __restrict__ a, const T* __restrict__ w, const float* __restrict__ bias,
    TOut* __restrict__ c, int m, int n, int k, int lda, int ldc, int tiles_m, int tiles_n,
    int k_splits, int k_chunk, KvScatter scatter) {
  constexpr int KC = Mma<T>::K_PER_CHUNK;            // elements per 16-byte chunk
  constexpr int BK = TG_ROW_BYTES / (int)sizeof(T);  // elements of k per stage
  __shared__ __attribute__((aligned(16))) unsigned char lds[2][(TG_BM + TG_BN) * TG_LDS_STRIDE];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // the same in every lane: scalar
  const int wave_m = wave >> 1;
  const int wave_n = wave & 1;
  // Consecutive block ids run on different XCDs, each with an L2 of its own.  Blocks are
  // renumbered so that every XCD works on a contiguous run of tiles (which share rows of A
  // and, in the next run, rows of W) instead of every XCD fetching every operand tile.
  const int blocks = gridDim.x;
  const int per_xcd = blocks / 8;
  int logical = blockIdx.x;
  if (blockIdx.x < per_xcd * 8) logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  const int tiles = tiles_m * tiles_n;
  const int split = logical / tiles;
  const int tile = logical - split * tiles;
  // walk the tiles column-major in groups of 8 rows, so that a run of blocks reuses W tiles
  const int tile_n = tile / tiles_m;
  const int tile_m = tile - tile_n * tiles_m;
  const int m0 = tile_m * TG_BM;
  const int n0 = tile_n * TG_BN;
  const int k_begin = split * k_chunk;
  const int k_end = k_begin + k_chunk < k ? k_begin + k_chunk : k;

  // global -> register staging: 512 chunks of 16 bytes per operand, two per thread; a ring
  // of TG_DEPTH stages keeps that many k tiles in flight
  uint4 ring_a[TG_DEPTH][2], ring_w[TG_DEPTH][2];
  const int load_row = tid >> 2;           // rows load_row and load_row + 64
  const int load_k = (tid & 3) * KC;
  const T* a_src[2];
  const T* w_src[2];
  bool a_row_ok[2], w_row_ok[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = load_row + i * 64;
    a_row_ok[i] = m0 + row < m;
    w_row_ok[i] = n0 + row < n;
    a_src[i] = a + (int64_t)(a_row_ok[i] ? m0 + row : 0) * lda + load_k;
    w_src[i] = w + (int64_t)(w_row_ok[i] ? n0 + row : 0) * k + load_k;
  }
  auto load_global = [&](uint4* stage_a, uint4* stage_w, int k0) {
    // unconditional loads from clamped addresses, zeroed afterwards
    const bool k_ok = k0 + load_k < k_end;
    const int kk = k_ok ? k0 : k_begin;
    const uint4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      stage_a[i] = *reinterpret_cast<const uint4*>(a_src[i] + kk);
      stage_w[i] = *reinterpret_cast<const uint4*>(w_src[i] + kk);
      if (!(a_row_ok[i] && k_ok)) stage_a[i] = zero;
      if (!(w_row_ok[i] && k_ok)) stage_w[i] = zero;
    }
  };
  auto store_lds = [&](int buffer, const uint4* stage_a, const uint4* stage_w) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int offset = (load_row + i * 64) * TG_LDS_STRIDE + (tid & 3) * 16;
      *reinterpret_cast<uint4*>(&lds[buffer][offset]) = stage_a[i];
      *reinterpret_cast<uint4*>(&lds[buffer][TG_BM * TG_LDS_STRIDE + offset]) = stage_w[i];
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  auto compute = [&](int buffer) {
    // 64 bytes of k per row = two 32-byte halves; lanes 0..31 take the first 16 bytes of a
    // half, lanes 32..63 the second
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      uint4 fa[2], fw[2];
      const int kbyte = half * 32 + (lane >> 5) * 16;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int row = wave_m * 64 + i * 32 + (lane & 31);
        fa[i] = *reinterpret_cast<const uint4*>(&lds[buffer][row * TG_LDS_STRIDE + kbyte]);
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int row = wave_n * 64 + j * 32 + (lane & 31);
        fw[j] = *reinterpret_cast<const uint4*>(
            &lds[buffer][TG_BM * TG_LDS_STRIDE + row * TG_LDS_STRIDE + kbyte]);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) Mma<T>::step(fa[i], fw[j], acc[i][j]);
    }
  };

  const int k_tiles = (k_end - k_begin + BK - 1) / BK;
#pragma unroll
  for (int d = 0; d < TG_DEPTH; ++d) load_global(ring_a[d], ring_w[d], k_begin + d * BK);
  store_lds(0, ring_a[0], ring_w[0]);
  __syncthreads();
  for (int kt0 = 0; kt0 < k_tiles; kt0 += TG_DEPTH) {
#pragma unroll
    for (int d = 0; d < TG_DEPTH; ++d) {
      const int kt = kt0 + d;
      if (kt < k_tiles) {
        // stage d held tile kt, which is in LDS already: refill it with tile kt + TG_DEPTH
        load_global(ring_a[d], ring_w[d], k_begin + (kt + TG_DEPTH) * BK);
        compute(kt & 1);
        // tile kt + 1 left TG_DEPTH - 1 iterations ago
        store_lds((kt + 1) & 1, ring_a[(d + 1) % TG_DEPTH], ring_w[(d + 1) % TG_DEPTH]);
        __syncthreads();
      }
    }
  }

  // element e of a 32 x 32 accumulator: row (e / 4) * 8 + (lane / 32) * 4 + e % 4, column lane % 32
  const bool scatters = EPI == PS_EPI_NONE && scatter.k_pool != nullptr && n0 + TG_BN > scatter.q_cols;
  int col[2];
  float b[2];
  TOut* pool[2] = {nullptr, nullptr};
  int64_t pool_offset[2] = {0, 0};
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    col[j] = n0 + wave_n * 64 + j * 32 + (lane & 31);
    b[j] = (bias && split == 0 && col[j] < n) ? bias[col[j]] : 0.f;
    if (scatters && col[j] < n) pool[j] = kv_scatter_col<TOut>(scatter, col[j], &pool_offset[j]);
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int row = m0 + wave_m * 64 + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
      if (row >= m) continue;
      // the page slot of a row is looked up once for all its columns
      const int64_t slot = scatters ? kv_scatter_row(scatter, row) : -1;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        if (col[j] >= n) continue;
        float v = apply_activation<EPI>(acc[i][j][e] + b[j]);
        TOut* dst = c + (int64_t)row * ldc + col[j];
        if (EPI == PS_EPI_RESIDUAL) {
          if (k_splits > 1) {
            unsafeAtomicAdd(reinterpret_cast<float*>(dst), v);
            continue;
          }
          v += to_float<TOut>(*dst);
        }
        *dst = from_float<TOut>(v);
        if (pool[j] != nullptr && slot >= 0) pool[j][slot + pool_offset[j]] = from_float<TOut>(v);
      }
    }
  }
}

// ------------------------------------------------------------------------------- skinny
// Each row's largest value and its column among the block's NT tiles, from the partial tiles
// that the epilogue has just summed (the same sum in the same order, so the value is the one
// stored), raised into the row's keys; the last block to finish turns keys into tokens.
template <int MB, int NT>
__device__ inline void skinny_top_choice(float (*partial)[SK_WAVES][MB][4][64], const float* bias,
                                         int m, int n, int n0, int row0, const TopChoice& top) {
  __shared__ int s_last;
  const int col_in = threadIdx.x & 15;
  const int row_in = threadIdx.x >> 4;
  const int i = col_in & 3;
  const int lane = (col_in >> 2) * 16 + row_in;
  const int block = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
#pragma unroll
  for (int b = 0; b < MB; ++b) {
    const int row = row0 + b * 16 + row_in;
    unsigned long long best = 0;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int col = n0 + j * 16 + col_in;
      if (col < n && row < m) {
        const float v = partial[j][0][b][i][lane] + partial[j][1][b][i][lane] +
                        partial[j][2][b][i][lane] + partial[j][3][b][i][lane] +
                        (bias != nullptr ? bias[col] : 0.f);
        const unsigned long long key = top_choice_key(v, col);
        best = key > best ? key : best;
      }
    }
    // the 16 threads of a row are 16 consecutive lanes of one wave
#pragma unroll
    for (int off = 8; off >= 1; off >>= 1) {
      const unsigned long long other = __shfl_xor(best, off, 64);
      best = other > best ? other : best;
    }
    // (reading the key first, to skip an atomic that would change nothing, costs a trip to
    // memory of its own and measured 3 us slower at 1,571 blocks)
    if (col_in == 0 && row < m)
      __hip_atomic_fetch_max(top_choice_slot(top, row, block & (PS_TOP_SLOTS - 1)), best,
                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  // the block's maxima have been performed before its ticket is drawn
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (threadIdx.x == 0) {
    // Atomics on one address are performed one after the other, some ten nanoseconds each:
    // a block draws from one of PS_TOP_SLOTS counters, and only the last of each draws from
    // the common one.
    const int blocks = gridDim.x * gridDim.y * gridDim.z;
    const int group = block & (PS_TOP_SLOTS - 1);
    const int in_group = (blocks - group + PS_TOP_SLOTS - 1) / PS_TOP_SLOTS;
    const int groups = blocks < PS_TOP_SLOTS ? blocks : PS_TOP_SLOTS;
    int last = __hip_atomic_fetch_add(top_choice_ticket(top, 1 + group), 1, __ATOMIC_RELAXED,
                                      __HIP_MEMORY_SCOPE_AGENT) == in_group - 1;
    if (last)
      last = __hip_atomic_fetch_add(top_choice_ticket(top, 0), 1, __ATOMIC_RELAXED,
                                    __HIP_MEMORY_SCOPE_AGENT) == groups - 1;
    s_last = last;
  }
  __syncthreads();
  if (!s_last) return;
  // 16 threads per row, one key each
  for (int base = 0; base < m; base += 64 * SK_WAVES / PS_TOP_SLOTS) {
    const int row = base + (int)threadIdx.x / PS_TOP_SLOTS;
    unsigned long long best = 0;
    if (row < m) {
      unsigned long long* slot = top_choice_slot(top, row, threadIdx.x & (PS_TOP_SLOTS - 1));
      best = __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(slot, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
#pragma unroll
    for (int off = 8; off >= 1; off >>= 1) {
      const unsigned long long other = __shfl_xor(best, off, 64);
      best = other > best ? other : best;
    }
    if (row < m && (threadIdx.x & (PS_TOP_SLOTS - 1)) == 0)
      top.tokens[row] = (int)(0xFFFFFFFFu - (unsigned int)(best & 0xFFFFFFFFull));
  }
  if (threadIdx.x <= PS_TOP_SLOTS)
    __hip_atomic_store(top_choice_ticket(top, threadIdx.x), 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <typename TOut, int EPI, int MB, int NT, int UNROLL>
__global__ __launch_bounds__(64 * SK_WAVES) void gemm_nt_skinny_kernel(
    const bf16_t* __restrict__ a, const bf16_t* __restrict__ w, const float* __restrict__ bias,
    TOut* __restrict__ c, int m, int n, int k, int lda, int ldc, int k_chunk, int k_splits,
    KvScatter scatter, const bf16_t* __restrict__ wp, int layouts, TopChoice top) {
  // layouts: bit 0, the rows of A lie in the packed order (packed_offset); bit 1, C is to be
  // written in it.
  // NT tiles of 16 columns per block share the loads of the rows of A: with very many
  // columns (the output head) those loads, though they come from the L2, are as many bytes
  // as the weights themselves.
  __shared__ float partial[NT][SK_WAVES][MB][4][64];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // the same in every lane: scalar
  const int n0 = blockIdx.x * 16 * NT;
  const int split = blockIdx.y;
  const int row0 = blockIdx.z * (MB * 16);
  const int k_begin = split * k_chunk;
  const int k_end = k_begin + k_chunk < k ? k_begin + k_chunk : k;
  const int sub = lane & 15;
  const int group = lane >> 4;
  const bf16_t* w_ptr[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int w_row = n0 + j * 16 + sub < n ? n0 + j * 16 + sub : n - 1;
    w_ptr[j] = w + (int64_t)w_row * k + group * 16;
    if (wp != nullptr) {
      // packed copy: the 16 x 64 tile of step s lies in the order in which the lanes hold it,
      // first the halves of the first product, then those of the second (1 KB each)
      const int tiles = (n + 15) / 16;
      const int tile = n0 / 16 + j < tiles ? n0 / 16 + j : tiles - 1;
      w_ptr[j] = wp + (int64_t)tile * (k / 64) * 1024 + lane * 8;
    }
  }
  const bf16_t* a_ptr[MB];
#pragma unroll
  for (int b = 0; b < MB; ++b) {
    const int row = row0 + b * 16 + sub < m ? row0 + b * 16 + sub : m - 1;
    a_ptr[b] = a + (int64_t)row * lda + group * 16;
    if (layouts & 1) a_ptr[b] = a + (int64_t)(row >> 4) * (k / 64) * 1024 + lane * 8;
  }
  f32x4 acc[NT][MB];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int b = 0; b < MB; ++b) acc[j][b] = f32x4{0.f, 0.f, 0.f, 0.f};

  const uint4 zero = {0u, 0u, 0u, 0u};
  // wave `wave` takes the 64-k steps wave, wave + 4, ... of the block's range
  for (int k0 = k_begin + wave * 64; k0 < k_end; k0 += SK_WAVES * UNROLL * 64) {
    uint4 wf[UNROLL][NT][2], xf[UNROLL][MB][2];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int ku = k0 + u * SK_WAVES * 64;
      const int kk = ku + group * 16;
      const bool first = kk < k_end;
      const bool second = kk + 8 < k_end;
      // unconditional loads from a clamped offset, zeroed afterwards: loads under a branch
      // would not be issued together
      const int o0 = first ? ku : k_begin - group * 16;
      const int o1 = second ? ku + 8 : k_begin - group * 16;
      // (packed: k is a multiple of 64, so a step is whole or absent)
      const int p0 = wp != nullptr ? (first ? (ku / 64) * 1024 : 0) : o0;
      const int p1 = wp != nullptr ? p0 + 512 : o1;
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        wf[u][j][0] = *reinterpret_cast<const uint4*>(w_ptr[j] + p0);
        wf[u][j][1] = *reinterpret_cast<const uint4*>(w_ptr[j] + p1);
      }
      const int q0 = (layouts & 1) ? (first ? (ku / 64) * 1024 : 0) : o0;
      const int q1 = (layouts & 1) ? q0 + 512 : o1;
#pragma unroll
      for (int b = 0; b < MB; ++b) {
        xf[u][b][0] = *reinterpret_cast<const uint4*>(a_ptr[b] + q0);
        xf[u][b][1] = *reinterpret_cast<const uint4*>(a_ptr[b] + q1);
      }
      if (!first) {
#pragma unroll
        for (int j = 0; j < NT; ++j) wf[u][j][0] = zero;
#pragma unroll
        for (int b = 0; b < MB; ++b) xf[u][b][0] = zero;
      }
      if (!second) {
#pragma unroll
        for (int j = 0; j < NT; ++j) wf[u][j][1] = zero;
#pragma unroll
        for (int b = 0; b < MB; ++b) xf[u][b][1] = zero;
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int b = 0; b < MB; ++b)
#pragma unroll
          for (int h = 0; h < 2; ++h)
            acc[j][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                *reinterpret_cast<const bf16x8*>(&wf[u][j][h]),
                *reinterpret_cast<const bf16x8*>(&xf[u][b][h]), acc[j][b], 0, 0, 0);
  }

#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int b = 0; b < MB; ++b)
#pragma unroll
      for (int i = 0; i < 4; ++i) partial[j][wave][b][i][lane] = acc[j][b][i];
  __syncthreads();
  // element i of a 16 x 16 accumulator: weight row (lane / 16) * 4 + i, activation row lane % 16
#pragma unroll
  for (int j = 0; j < NT; ++j)
    skinny_epilogue<TOut, EPI, MB>(partial[j], bias, c, m, n, ldc, n0 + j * 16, row0, split,
                                   k_splits, scatter, layouts & 2);
  if (EPI == PS_EPI_NONE && sizeof(TOut) == 4 && top.keys != nullptr)
    skinny_top_choice<MB, NT>(partial, bias, m, n, n0, row0, top);
}

// --------------------------------------------------------------------------------- host
bool ps_gemm_nt_bf16_tiled_supported(const void* a, const void* w, int m, int k, int lda);
bool ps_gemm_nt_bf16_wide_supported(const void* a, const void* w_packed, int m, int n, int k, int lda);
int ps_gemm_nt_bf16_wide(const void* a, const void* w_packed, const float* bias, void* c, int m,
                         int n, int k, int lda, int ldc, int c_dtype, int epilogue,
                         const KvScatter& scatter, int rows_per_block, hipStream_t s);
int ps_gemm_nt_bf16_tiled(const void* a, const void* w, const float* bias, void* c, int m, int n,
                          int k, int lda, int ldc, int c_dtype, int epilogue,
                          const KvScatter& scatter, hipStream_t s);

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

bool ps_gemm_nt_mfma_supported(const void* a, const void* w, int k, int lda, int dtype) {
  const int per_chunk = dtype == PS_BF16 ? 8 : 4;
  return k % per_chunk == 0 && lda % per_chunk == 0 && aligned16(a) && aligned16(w);
}

template <typename T, typename TOut>
static int launch_tiled(const void* a, const void* w, const float* bias, void* c, int m, int n,
                        int k, int lda, int ldc, int epilogue, const KvScatter& scatter,
                        hipStream_t s) {
  const int tiles_m = (m + TG_BM - 1) / TG_BM;
  const int tiles_n = (n + TG_BN - 1) / TG_BN;
  // Few tiles leave compute units idle: where partial sums can be added in place (residual
  // epilogue) k is split over blocks until about three blocks per unit are in flight.
  constexpr int bk = TG_ROW_BYTES / (int)sizeof(T);
  int k_splits = 1;
  if (epilogue == PS_EPI_RESIDUAL) {
    const int wanted = (3 * ps_compute_units() + tiles_m * tiles_n - 1) / (tiles_m * tiles_n);
    const int possible = k / (8 * bk) > 0 ? k / (8 * bk) : 1;
    k_splits = wanted < possible ? wanted : possible;
  }
  int k_chunk = (k + k_splits - 1) / k_splits;
  k_chunk = (k_chunk + bk - 1) / bk * bk;
  k_splits = (k + k_chunk - 1) / k_chunk;
  dim3 grid(tiles_m * tiles_n * k_splits);
#define PS_LAUNCH_TG(EPI)                                                                    \
  hipLaunchKernelGGL((gemm_nt_tiled_kernel<T, TOut, EPI>), grid, dim3(256), 0, s, (const T*)a, \
                     (const T*)w, bias, (TOut*)c, m, n, k, lda, ldc, tiles_m, tiles_n,       \
                     k_splits, k_chunk, scatter)
  switch (epilogue) {
    case PS_EPI_NONE: PS_LAUNCH_TG(PS_EPI_NONE); break;
    case PS_EPI_GELU_TANH: PS_LAUNCH_TG(PS_EPI_GELU_TANH); break;
    case PS_EPI_GELU_ERF: PS_LAUNCH_TG(PS_EPI_GELU_ERF); break;
    case PS_EPI_RESIDUAL: PS_LAUNCH_TG(PS_EPI_RESIDUAL); break;
    default: ps_set_error("ps_linear: unknown epilogue %d", epilogue); return 1;
  }
#undef PS_LAUNCH_TG
  PS_CHECK_LAUNCH("ps_linear(tiled)");
  return 0;
}

template <typename TOut, int EPI>
static void launch_skinny_mb(const void* a, const void* w, const float* bias, void* c, int m,
                             int n, int k, int lda, int ldc, int k_chunk, int k_splits,
                             const KvScatter& scatter, const bf16_t* wp, int layouts,
                             bool two_tiles, const TopChoice& top, hipStream_t s) {
  // Rows go 16 to an accumulator, up to four accumulators to a block.  Where the columns and
  // the k ranges give few blocks, the rows are spread over more of them (every one reads the
  // same weights, which the L2 absorbs; blocks that differ only in z run on one XCD when the
  // number of column blocks is a multiple of 8).
  const int row_blocks = (m + 15) / 16;
  const int grid_xy = ((n + 15) / 16) * k_splits;
  // (up to three blocks per compute unit: 64 x 2304 x 768 with weights from memory takes 5.0 us
  // with its rows on four blocks, 6.2 us on one)
  int z = 3 * ps_compute_units() / grid_xy;
  z = z < 1 ? 1 : (z > row_blocks ? row_blocks : z);
  if (z < (row_blocks + 3) / 4) z = (row_blocks + 3) / 4;   // (a block holds at most four accumulators of 16 rows)
  const int per = (row_blocks + z - 1) / z;
  dim3 grid((n + 15) / 16, k_splits, (row_blocks + per - 1) / per);
  dim3 block(64 * SK_WAVES);
  // a k range of up to 768 (GPT-2's width) needs three steps per wave, not four: a step that
  // is not there would still be fetched from a clamped address
  const bool three = k_chunk <= SK_WAVES * 3 * 64;
#define PS_LAUNCH_SKU(MB, NT, UNROLL)                                                          \
  hipLaunchKernelGGL((gemm_nt_skinny_kernel<TOut, EPI, MB, NT, UNROLL>), grid, block, 0, s,    \
                     (const bf16_t*)a, (const bf16_t*)w, bias, (TOut*)c, m, n, k, lda, ldc,    \
                     k_chunk, k_splits, scatter, wp, layouts, top)
#define PS_LAUNCH_SK(MB)                                                                       \
  do {                                                                                         \
    if (three) PS_LAUNCH_SKU(MB, 1, 3);                                                        \
    else PS_LAUNCH_SKU(MB, 1, SK_UNROLL);                                                      \
  } while (0)
  if (two_tiles && per >= 2) {
    // very many blocks (wide models): two tiles of columns per block halve what the blocks
    // fetch of the rows of A, which at 17 to 64 rows is most of their traffic; the range of k
    // is one round of 2 to 5 steps per wave (chosen by the caller)
    if constexpr (EPI == PS_EPI_RESIDUAL) {
      grid.x = (n + 31) / 32;
      const int steps = (k_chunk + SK_WAVES * 64 - 1) / (SK_WAVES * 64);
#define PS_LAUNCH_TT(MB)                                                                       \
  do {                                                                                         \
    if (steps <= 2) PS_LAUNCH_SKU(MB, 2, 2);                                                   \
    else if (steps == 3) PS_LAUNCH_SKU(MB, 2, 3);                                              \
    else if (steps == 4) PS_LAUNCH_SKU(MB, 2, 4);                                              \
    else PS_LAUNCH_SKU(MB, 2, 5);                                                              \
  } while (0)
      if (per == 2) PS_LAUNCH_TT(2);
      else if (per == 3) PS_LAUNCH_TT(3);
      else PS_LAUNCH_TT(4);
#undef PS_LAUNCH_TT
    }
  } else if (per <= 2 && k_splits == 1 && n >= 16 * 1024) {
    // the output head: two tiles of columns per block (also at 17 to 32 rows: 50,257 x 768 at
    // 17 rows takes 27 us with one tile per block)
    grid.x = (n + 31) / 32;
    if (per <= 1) {
      if (three) PS_LAUNCH_SKU(1, 2, 3);
      else PS_LAUNCH_SKU(1, 2, SK_UNROLL);
    } else {
      if (three) PS_LAUNCH_SKU(2, 2, 3);
      else PS_LAUNCH_SKU(2, 2, SK_UNROLL);
    }
  } else if (per <= 1 && k_chunk > SK_WAVES * SK_UNROLL * 64) {
    // up to 16 rows leave registers for twice the loads: a k of up to 2048 in one round
    hipLaunchKernelGGL((gemm_nt_skinny_kernel<TOut, EPI, 1, 1, 2 * SK_UNROLL>), grid, block, 0, s,
                       (const bf16_t*)a, (const bf16_t*)w, bias, (TOut*)c, m, n, k, lda, ldc,
                       k_chunk, k_splits, scatter, wp, layouts, top);
  } else if (per <= 1) PS_LAUNCH_SK(1);
  else if (per == 2) PS_LAUNCH_SK(2);
  else if (per == 3) PS_LAUNCH_SK(3);
  else PS_LAUNCH_SK(4);
#undef PS_LAUNCH_SK
#undef PS_LAUNCH_SKU
}

template <typename TOut>
static int launch_skinny(const void* a, const void* w, const float* bias, void* c, int m, int n,
                         int k, int lda, int ldc, int epilogue, const KvScatter& scatter,
                         const bf16_t* wp, int layouts, const TopChoice& top, hipStream_t s) {
  if (k % 64 != 0) wp = nullptr;   // the packed copy exists for whole steps of 64 only
  // A block covers 1024 k with one round of loads.  Longer k is split over blocks where the
  // partial sums can be added in place (residual epilogue), else the block loops.
  int k_splits = 1;
  if (epilogue == PS_EPI_RESIDUAL && k > 1024) k_splits = (k + 1023) / 1024;
  int k_chunk = (k + k_splits - 1) / k_splits;
  k_chunk = (k_chunk + 255) / 256 * 256;
  k_splits = (k + k_chunk - 1) / k_chunk;
  // More rows than 16 and half as many blocks again as compute units: two column tiles per
  // block, and ranges of k such that the blocks come to one per compute unit or just under
  // (a unit with two blocks takes twice as long as one with one), each range one round of a
  // wave's loads: 1280 k at 64 x 1600 x 6400 (250 blocks: 11.7 us with weights from memory,
  // against 13.7 with ranges of 640 and 17.7 with one tile and ranges of 1024), 1024 at 64 x
  // 1280 x 5120 (200 blocks: 10.7 against 13.2); at 1024 x 4096 and below the single tile
  // stays ahead.
  const bool two_tiles = epilogue == PS_EPI_RESIDUAL && m > 16 && k_splits > 1 &&
                         (int64_t)((n + 15) / 16) * k_splits >= ps_compute_units() * 3 / 2;
  if (two_tiles) {
    const int tiles32 = (n + 31) / 32;
    const int wanted = ps_compute_units() / tiles32 > 1 ? ps_compute_units() / tiles32 : 1;
    k_chunk = ((k + wanted - 1) / wanted + 255) / 256 * 256;
    k_chunk = k_chunk < 512 ? 512 : (k_chunk > 1280 ? 1280 : k_chunk);
    k_splits = (k + k_chunk - 1) / k_chunk;
  }
#define PS_SKINNY_CASE(EPI)                                                                      \
  case EPI:                                                                                      \
    launch_skinny_mb<TOut, EPI>(a, w, bias, c, m, n, k, lda, ldc, k_chunk, k_splits, scatter, wp, \
                                layouts, two_tiles, top, s);                                     \
    break
  switch (epilogue) {
    PS_SKINNY_CASE(PS_EPI_NONE);
    PS_SKINNY_CASE(PS_EPI_GELU_TANH);
    PS_SKINNY_CASE(PS_EPI_GELU_ERF);
    PS_SKINNY_CASE(PS_EPI_RESIDUAL);
    default: ps_set_error("ps_linear: unknown epilogue %d", epilogue); return 1;
  }
#undef PS_SKINNY_CASE
  PS_CHECK_LAUNCH("ps_linear(skinny)");
  return 0;
}

// Whether ps_gemm_nt_mfma takes the skinny kernel for this product.
// Up to 64 rows the skinny kernel has every load of a block in flight at once, which counts
// when the weights come from memory and not from a cache; the tiled kernel walks k tile by
// tile and wins only where there are tiles enough to fill the chip (the output head).
// A k beyond one round of the skinny kernel's loads makes it loop; there the tiled kernel
// with its ring of stages is ahead, except where partial sums of a split k can be
// added in place (residual epilogue), which keeps every block at one round.
bool ps_gemm_nt_mfma_skinny(const void* a, const void* w, int m, int n, int k, int lda, int dtype,
                            int epilogue) {
  if (dtype != PS_BF16) return false;
  // Somewhat more rows with the residual epilogue (the projections of a step that mixes a
  // short prompt portion with decoded tokens): ranges of k over blocks and atomic adds still
  // beat the tiled kernel's few blocks walking a long k, until the adds and the rows that every
  // block fetches outweigh it (rows x columns, with weights from memory: 128 x 768 x 3072 9.3
  // against 14.7 us, 224 rows 12.3 against 14.5, 256 rows 15.8; 128 x 1024 x 4096 11.7 against
  // 16.6, 192 rows 16.7 against 18.3; 128 x 1600 x 6400 21.3 against 27.2, 160 rows 27.5 against
  // 26.9; with a short k 128 x 768 x 768 4.6 against 5.8, 192 x 1024 x 1024 6.5 against 6.8, 96 x
  // 1600 x 1600 9.2 against 9.3, 112 rows 10.6 against 9.4).
  if (m > 64)
    return epilogue == PS_EPI_RESIDUAL && m <= 224 && n < 64 * 256 &&
           (int64_t)m * n <= (k >= 2048 ? 200000 : 160000);
  const bool skinny_k = n < 64 * 256 && (epilogue == PS_EPI_RESIDUAL || k <= 1024 || m <= 16);
  return skinny_k || !ps_gemm_nt_bf16_tiled_supported(a, w, m, k, lda);
}

int ps_gemm_nt_mfma(const void* a, const void* w, const float* bias, void* c, int m, int n, int k,
                    int lda, int ldc, int dtype, int c_dtype, int epilogue,
                    const KvScatter& scatter, const void* w_packed, int layouts,
                    const TopChoice& top, hipStream_t s) {
  const bf16_t* wp = (const bf16_t*)w_packed;
  if (ps_gemm_nt_mfma_skinny(a, w, m, n, k, lda, dtype, epilogue)) {
    if (c_dtype == PS_F32)
      return launch_skinny<float>(a, w, bias, c, m, n, k, lda, ldc, epilogue, scatter, wp, layouts,
                                  top, s);
    return launch_skinny<bf16_t>(a, w, bias, c, m, n, k, lda, ldc, epilogue, scatter, wp, layouts,
                                 top, s);
  }
  if (layouts != 0) {
    ps_set_error("ps_linear: packed activations go with the skinny product only (m %d, n %d, k %d)",
                 m, n, k);
    return 1;
  }
  if (dtype == PS_BF16 && ps_gemm_nt_bf16_wide_supported(a, wp, m, n, k, lda))
    return ps_gemm_nt_bf16_wide(a, wp, bias, c, m, n, k, lda, ldc, c_dtype, epilogue, scatter, 0, s);
  if (dtype == PS_BF16 && ps_gemm_nt_bf16_tiled_supported(a, w, m, k, lda))
    return ps_gemm_nt_bf16_tiled(a, w, bias, c, m, n, k, lda, ldc, c_dtype, epilogue, scatter, s);
  if (dtype == PS_F32 && c_dtype == PS_F32)
    return launch_tiled<float, float>(a, w, bias, c, m, n, k, lda, ldc, epilogue, scatter, s);
  if (dtype == PS_BF16 && c_dtype == PS_F32)
    return launch_tiled<bf16_t, float>(a, w, bias, c, m, n, k, lda, ldc, epilogue, scatter, s);
  if (dtype == PS_BF16 && c_dtype == PS_BF16)
    return launch_tiled<bf16_t, bf16_t>(a, w, bias, c, m, n, k, lda, ldc, epilogue, scatter, s);
  ps_set_error("ps_linear: unsupported dtype pair (in %d, out %d)", dtype, c_dtype);
  return 1;
}
