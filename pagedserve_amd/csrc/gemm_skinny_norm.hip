// Norm + skinny product as one launch: the instantiations for k up to 1024 (3 steps of 64 k
// per wave for up to 768, GPT-2's width, 4 for 1024) and the entry that picks between these
// and the ones for longer k.

#include "gemm_skinny_norm.h"

int ps_norm_gemm_fused_long(const NormPrologue& norm, const void* w, const float* bias, void* c,
                            int m, int n, int k, int ldc, int c_dtype, int epilogue,
                            const KvScatter& scatter, const void* w_packed, hipStream_t s);

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Whether norm + product run as one launch.
// Every block normalises the rows again, so the fusion only pays while there are few blocks
// (for the output head of 50,257 columns it measured 1 % slower per decode step than the
// norm kernel in front of the two-tile skinny product).
bool ps_norm_gemm_fusable(const void* w, const NormPrologue& norm, int m, int n, int k, int dtype) {
  return dtype == PS_BF16 && m <= 16 && n <= 8192 && k <= SN_MAX_K && k % 8 == 0 &&
         norm.ldh % 4 == 0 && aligned16(w) && aligned16(norm.h) && aligned16(norm.gamma) &&
         (norm.beta == nullptr || aligned16(norm.beta));
}

int ps_norm_gemm_fused(const NormPrologue& norm, const void* w, const float* bias, void* c, int m,
                       int n, int k, int ldc, int c_dtype, int epilogue, const KvScatter& scatter,
                       const void* w_packed, hipStream_t s) {
  if (k > SK_WAVES * 4 * 64)
    return ps_norm_gemm_fused_long(norm, w, bias, c, m, n, k, ldc, c_dtype, epilogue, scatter,
                                   w_packed, s);
  return skinny_norm_by_type<3, 4>(norm, w, bias, c, m, n, k, ldc, c_dtype, epilogue, scatter,
                                   w_packed, s);
}
