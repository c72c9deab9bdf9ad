// C[m, n] = epilogue(sum_k A[m, k] W[n, k] + bias[n]) with float multiply-adds.
//
// The true 32-bit matrix product of the engine (no reduced-precision matrix mode): every
// product and every sum is an IEEE float operation, summed over k in ascending order inside
// one thread, so a row's result does not depend on how many other rows the call has.  Also
// the fallback of the bfloat16 path for shapes that the MFMA kernel refuses.
//
// Tile: 64 x 64 outputs per 256-thread block, 16 k per stage through LDS, 4 x 4 outputs per
// thread.  Any m, n, k and any row strides; loads are bounds-checked and zero-filled.
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
  if (dtype == PS_F32 && c_dtype == PS_F32)
    return launch_simple<float, float>(a, w, bias, c, m, n, k, lda, ldc, epilogue, s);
  if (dtype == PS_BF16 && c_dtype == PS_F32)
    return launch_simple<bf16_t, float>(a, w, bias, c, m, n, k, lda, ldc, epilogue, s);
  if (dtype == PS_BF16 && c_dtype == PS_BF16)
    return launch_simple<bf16_t, bf16_t>(a, w, bias, c, m, n, k, lda, ldc, epilogue, s);
  ps_set_error("ps_gemm_nt: unsupported dtype pair (in %d, out %d)", dtype, c_dtype);
  return 1;
}
