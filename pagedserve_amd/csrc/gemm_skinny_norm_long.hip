// Norm + skinny product as one launch: the instantiations for k of 1025 to 1792 (5 steps of
// 64 k per wave for up to 1280, 7 for up to 1792: the widths of GPT-2 large and XL).

#include "gemm_skinny_norm.h"

int ps_norm_gemm_fused_long(const NormPrologue& norm, const void* w, const float* bias, void* c,
                            int m, int n, int k, int ldc, int c_dtype, int epilogue,
                            const KvScatter& scatter, const void* w_packed, hipStream_t s) {
  return skinny_norm_by_type<5, 7>(norm, w, bias, c, m, n, k, ldc, c_dtype, epilogue, scatter,
                                   w_packed, s);
}
