// Entry point of the matrix products: checks the operands and picks the kernel.
#include "common.h"
#include "pagedserve_hip.h"

int ps_gemm_nt_simple(const void* a, const void* w, const float* bias, void* c, int m, int n,
                      int k, int lda, int ldc, int dtype, int c_dtype, int epilogue,
                      hipStream_t s);
int ps_gemm_nt_mfma(const void* a, const void* w, const float* bias, void* c, int m, int n, int k,
                    int lda, int ldc, int dtype, int c_dtype, int epilogue, hipStream_t s);
bool ps_gemm_nt_mfma_supported(const void* a, const void* w, int k, int lda, int dtype);

extern "C" int ps_gemm_nt(const void* a, const void* w, const float* bias, void* c, int m, int n,
                          int k, int lda, int ldc, int dtype, int c_dtype, int epilogue,
                          void* stream) {
  PS_REQUIRE(m >= 0 && n > 0 && k > 0, "ps_gemm_nt: bad sizes (m %d, n %d, k %d)", m, n, k);
  PS_REQUIRE(lda >= k && ldc >= n, "ps_gemm_nt: row strides (lda %d, ldc %d) smaller than rows",
             lda, ldc);
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_gemm_nt: unknown dtype %d", dtype);
  PS_REQUIRE(c_dtype == PS_F32 || c_dtype == PS_BF16, "ps_gemm_nt: unknown output dtype %d",
             c_dtype);
  PS_REQUIRE(!(dtype == PS_F32 && c_dtype == PS_BF16),
             "ps_gemm_nt: float operands with bfloat16 output are not supported");
  PS_REQUIRE(epilogue != PS_EPI_RESIDUAL || c_dtype == PS_F32,
             "ps_gemm_nt: the residual epilogue needs a float output");
  if (m == 0) return 0;
  // Matrix cores when the operands allow 16-byte loads; in float only for many rows (the
  // tile is 128 rows high), else the plain kernel.
  const bool mfma = ps_gemm_nt_mfma_supported(a, w, k, lda, dtype) &&
                    (dtype == PS_BF16 || m >= 96);
  if (mfma)
    return ps_gemm_nt_mfma(a, w, bias, c, m, n, k, lda, ldc, dtype, c_dtype, epilogue,
                           (hipStream_t)stream);
  return ps_gemm_nt_simple(a, w, bias, c, m, n, k, lda, ldc, dtype, c_dtype, epilogue,
                           (hipStream_t)stream);
}
