// C[m, n] = epilogue(sum_k A[m, k] W[n, k] + bias[n]) with float multiply-adds.
//
// The true 32-bit matrix product of the engine (no reduced-precision matrix mode): every
// product and every sum is an IEEE float operation, summed over k in ascending order inside
// one thread, so a row's result does not depend on how many other rows the call has.  Also
// the fallback of the bfloat16 path for shapes that the MFMA kernel refuses.
//
// Tile: 64 x 64 outputs per 256-thread block, 16 k per stage through LDS, 4 x 4 outputs per
// thread.  Any m, n, k and any row strides; loads are bounds-checked and zero-filled.
//
// Up to 16 rows of float (a decode step of the 32-bit path) take a second kernel: the tiled one
// would run on n / 64 blocks that each walk the whole k in stages of 16, a few dozen blocks
// bound by the latency of hundreds of dependent trips (8 rows x 2304 x 768: 70 us).  Here a
// wave owns a few output columns, its lanes stride over k with 16-byte loads of the weights
// (each read once, as the step's bytes are the weights') and of the rows (which the caches
// hold), every lane sums its share in ascending k, and the lanes' sums are added in a fixed
// tree: a row's result does not depend on the other rows here either.
#include "common.h"
#include "pagedserve_hip.h"

#define SG_BM 64
#define SG_BN 64
#define SG_BK 16

template <typename TIn, typename TOut, int EPI>
__global__ __launch_bounds__(256) void gemm_nt_simple_kernel(
    const TIn* __restrict__ a, const TIn* __restrict__ w, const float* __restrict__ bias,
    TOut* __restrict__ c, int m, int n, int k, int lda, int ldc) {
  __shared__ float a_tile[SG_BK][SG_BM + 4];
  __shared__ float w_tile[SG_BK][SG_BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid & 15;   // 4 output columns each
  const int ty = tid >> 4;   // 4 output rows each
  const int m0 = blockIdx.y * SG_BM;
  const int n0 = blockIdx.x * SG_BN;
  const int load_row = tid >> 2;        // 0..63
  const int load_k = (tid & 3) * 4;     // 0, 4, 8, 12

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < k; k0 += SG_BK) {
    {
      const int row = m0 + load_row;
      const TIn* src = a + (int64_t)row * lda + k0 + load_k;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        a_tile[load_k + i][load_row] =
            (row < m && k0 + load_k + i < k) ? to_float<TIn>(src[i]) : 0.f;
    }
    {
      const int row = n0 + load_row;
      const TIn* src = w + (int64_t)row * k + k0 + load_k;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        w_tile[load_k + i][load_row] =
            (row < n && k0 + load_k + i < k) ? to_float<TIn>(src[i]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < SG_BK; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = a_tile[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = w_tile[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = m0 + ty * 4 + i;
    if (row >= m) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = n0 + tx * 4 + j;
      if (col >= n) continue;
      float v = acc[i][j];
      if (bias != nullptr) v += bias[col];
      v = apply_activation<EPI>(v);
      TOut* dst = c + (int64_t)row * ldc + col;
      if (EPI == PS_EPI_RESIDUAL) v += to_float<TOut>(*dst);
      *dst = from_float<TOut>(v);
    }
  }
}

// MR: rows held in registers (m <= MR); COLS: output columns per wave.  A lane walks k in
// steps of 256 values and asks for 4 / COLS such steps of its COLS weight rows at once (four
// 16-byte loads in flight whatever COLS is); the sums are formed in the order of k either way,
// so the result does not depend on COLS.
template <int EPI, int MR, int COLS>
__global__ __launch_bounds__(256) void gemm_nt_f32_rows_kernel(
    const float* __restrict__ a, const float* __restrict__ w, const float* __restrict__ bias,
    float* __restrict__ c, int m, int n, int k, int lda, int ldc) {
  constexpr int AHEAD = 4 / COLS;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int col0 = (blockIdx.x * 4 + wave) * COLS;
  if (col0 >= n) return;
  const float* w_row[COLS];
#pragma unroll
  for (int j = 0; j < COLS; ++j) w_row[j] = w + (int64_t)(col0 + j < n ? col0 + j : n - 1) * k;
  const float* a_row[MR];
#pragma unroll
  for (int r = 0; r < MR; ++r) a_row[r] = a + (int64_t)(r < m ? r : m - 1) * lda;
  float acc[COLS][MR];
#pragma unroll
  for (int j = 0; j < COLS; ++j)
#pragma unroll
    for (int r = 0; r < MR; ++r) acc[j][r] = 0.f;
  for (int k0 = lane * 4; k0 < k; k0 += 256 * AHEAD) {
    float4 wv[AHEAD][COLS];
#pragma unroll
    for (int u = 0; u < AHEAD; ++u)
#pragma unroll
      for (int j = 0; j < COLS; ++j)
        wv[u][j] = k0 + 256 * u < k ? *reinterpret_cast<const float4*>(w_row[j] + k0 + 256 * u)
                                    : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) {
      if (k0 + 256 * u >= k) break;
#pragma unroll
      for (int r = 0; r < MR; ++r) {
        const float4 av = *reinterpret_cast<const float4*>(a_row[r] + k0 + 256 * u);
#pragma unroll
        for (int j = 0; j < COLS; ++j) {
          acc[j][r] = fmaf(av.x, wv[u][j].x, acc[j][r]);
          acc[j][r] = fmaf(av.y, wv[u][j].y, acc[j][r]);
          acc[j][r] = fmaf(av.z, wv[u][j].z, acc[j][r]);
          acc[j][r] = fmaf(av.w, wv[u][j].w, acc[j][r]);
        }
      }
    }
  }
  // every lane receives every total; lane j * MR + r finishes output (row r, column col0 + j)
  float mine = 0.f;
#pragma unroll
  for (int j = 0; j < COLS; ++j)
#pragma unroll
    for (int r = 0; r < MR; ++r) {
      const float total = wave_sum(acc[j][r]);
      if (lane == j * MR + r) mine = total;
    }
  static_assert(COLS * MR <= 64, "one output per lane");
  const int j = lane / MR;
  const int r = lane - j * MR;
  const int col = col0 + j;
  if (j >= COLS || r >= m || col >= n) return;
  float v = mine;
  if (bias != nullptr) v += bias[col];
  v = apply_activation<EPI>(v);
  float* dst = c + (int64_t)r * ldc + col;
  if (EPI == PS_EPI_RESIDUAL) v += *dst;
  *dst = v;
}

static bool rows_kernel_takes(const void* a, const void* w, int m, int k, int lda) {
  return m >= 1 && m <= 16 && k % 4 == 0 && lda % 4 == 0 &&
         (reinterpret_cast<uintptr_t>(a) & 15u) == 0 && (reinterpret_cast<uintptr_t>(w) & 15u) == 0;
}

static int launch_f32_rows(const void* a, const void* w, const float* bias, void* c, int m, int n,
                           int k, int lda, int ldc, int epilogue, hipStream_t s) {
#define PS_LAUNCH_FR(EPI, MR, COLS)                                                              \
  hipLaunchKernelGGL((gemm_nt_f32_rows_kernel<EPI, MR, COLS>), dim3((n + 4 * COLS - 1) / (4 * COLS)), \
                     dim3(256), 0, s, (const float*)a, (const float*)w, bias, (float*)c, m, n, k, \
                     lda, ldc)
  // Columns per wave by the blocks they leave: a block of four waves per compute unit counts
  // for more than the reuse of the rows (8 x 768 x 3072 on 48 blocks of 4 columns a wave took
  // 31 us, twelve trips to memory one after the other).
  const int units = ps_compute_units();
  const int cols = (n + 15) / 16 >= 3 * units / 4 ? 4 : (n + 7) / 8 >= 3 * units / 4 ? 2 : 1;
#define PS_LAUNCH_FR_M(EPI)                                   \
  do {                                                        \
    if (m <= 4) {                                             \
      if (cols == 4) PS_LAUNCH_FR(EPI, 4, 4);                 \
      else if (cols == 2) PS_LAUNCH_FR(EPI, 4, 2);            \
      else PS_LAUNCH_FR(EPI, 4, 1);                           \
    } else if (m <= 8) {                                      \
      if (cols == 4) PS_LAUNCH_FR(EPI, 8, 4);                 \
      else if (cols == 2) PS_LAUNCH_FR(EPI, 8, 2);            \
      else PS_LAUNCH_FR(EPI, 8, 1);                           \
    } else {                                                  \
      if (cols >= 2) PS_LAUNCH_FR(EPI, 16, 2);                \
      else PS_LAUNCH_FR(EPI, 16, 1);                          \
    }                                                         \
  } while (0)
  switch (epilogue) {
    case PS_EPI_NONE: PS_LAUNCH_FR_M(PS_EPI_NONE); break;
    case PS_EPI_GELU_TANH: PS_LAUNCH_FR_M(PS_EPI_GELU_TANH); break;
    case PS_EPI_GELU_ERF: PS_LAUNCH_FR_M(PS_EPI_GELU_ERF); break;
    case PS_EPI_RESIDUAL: PS_LAUNCH_FR_M(PS_EPI_RESIDUAL); break;
    default: ps_set_error("ps_gemm_nt: unknown epilogue %d", epilogue); return 1;
  }
#undef PS_LAUNCH_FR_M
#undef PS_LAUNCH_FR
  PS_CHECK_LAUNCH("ps_gemm_nt(float rows)");
  return 0;
}

template <typename TIn, typename TOut>
static int launch_simple(const void* a, const void* w, const float* bias, void* c, int m, int n,
                         int k, int lda, int ldc, int epilogue, hipStream_t s) {
  dim3 grid((n + SG_BN - 1) / SG_BN, (m + SG_BM - 1) / SG_BM);
#define PS_LAUNCH_SG(EPI)                                                                     \
  hipLaunchKernelGGL((gemm_nt_simple_kernel<TIn, TOut, EPI>), grid, dim3(256), 0, s,          \
                     (const TIn*)a, (const TIn*)w, bias, (TOut*)c, m, n, k, lda, ldc)
  switch (epilogue) {
    case PS_EPI_NONE: PS_LAUNCH_SG(PS_EPI_NONE); break;
    case PS_EPI_GELU_TANH: PS_LAUNCH_SG(PS_EPI_GELU_TANH); break;
    case PS_EPI_GELU_ERF: PS_LAUNCH_SG(PS_EPI_GELU_ERF); break;
    case PS_EPI_RESIDUAL: PS_LAUNCH_SG(PS_EPI_RESIDUAL); break;
    default: ps_set_error("ps_gemm_nt: unknown epilogue %d", epilogue); return 1;
  }
#undef PS_LAUNCH_SG
  PS_CHECK_LAUNCH("ps_gemm_nt(simple)");
  return 0;
}

int ps_gemm_nt_simple(const void* a, const void* w, const float* bias, void* c, int m, int n,
                      int k, int lda, int ldc, int dtype, int c_dtype, int epilogue,
                      hipStream_t s) {
  if (dtype == PS_F32 && c_dtype == PS_F32 && rows_kernel_takes(a, w, m, k, lda))
    return launch_f32_rows(a, w, bias, c, m, n, k, lda, ldc, epilogue, s);
  if (dtype == PS_F32 && c_dtype == PS_F32)
    return launch_simple<float, float>(a, w, bias, c, m, n, k, lda, ldc, epilogue, s);
  if (dtype == PS_BF16 && c_dtype == PS_F32)
    return launch_simple<bf16_t, float>(a, w, bias, c, m, n, k, lda, ldc, epilogue, s);
  if (dtype == PS_BF16 && c_dtype == PS_BF16)
    return launch_simple<bf16_t, bf16_t>(a, w, bias, c, m, n, k, lda, ldc, epilogue, s);
  ps_set_error("ps_gemm_nt: unsupported dtype pair (in %d, out %d)", dtype, c_dtype);
  return 1;
}
