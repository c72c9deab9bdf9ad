// Entry points of the linear layers: check the operands, pick the kernels, and fuse a norm in
// front and the key/value scatter behind the product where the chosen kernel can.
#include "common.h"
#include "linear.h"
#include "pagedserve_hip.h"

int ps_gemm_nt_simple(const void* a, const void* w, const float* bias, void* c, int m, int n,
                      int k, int lda, int ldc, int dtype, int c_dtype, int epilogue,
                      hipStream_t s);
int ps_gemm_nt_mfma(const void* a, const void* w, const float* bias, void* c, int m, int n, int k,
                    int lda, int ldc, int dtype, int c_dtype, int epilogue,
                    const KvScatter& scatter, const void* w_packed, int layouts,
                    const TopChoice& top, hipStream_t s);
bool ps_gemm_nt_mfma_skinny(const void* a, const void* w, int m, int n, int k, int lda, int dtype,
                            int epilogue);
int ps_norm_layout(const float* x, const int* rows, const float* gamma, const float* beta,
                   void* out, int n_rows, int width, float eps, int rms, int out_dtype,
                   int packed, hipStream_t s);
int ps_norm_gemm_fused(const NormPrologue& norm, const void* w, const float* bias, void* c, int m,
                       int n, int k, int ldc, int c_dtype, int epilogue, const KvScatter& scatter,
                       const void* w_packed, hipStream_t s);
bool ps_gemm_nt_mfma_supported(const void* a, const void* w, int k, int lda, int dtype);
bool ps_norm_gemm_fusable(const void* w, const NormPrologue& norm, int m, int n, int k, int dtype);

// The size of the argument block, so that a caller that lays it out by hand can check that
// it agrees with this library.
extern "C" int ps_linear_args_size(void) { return (int)sizeof(PsLinearArgs); }

extern "C" int ps_linear(const PsLinearArgs* p, void* stream) {
  PS_REQUIRE(p != nullptr, "ps_linear: no arguments");
  const int m = p->m, n = p->n, k = p->k;
  PS_REQUIRE(m >= 0 && n > 0 && k > 0, "ps_linear: bad sizes (m %d, n %d, k %d)", m, n, k);
  PS_REQUIRE(p->ldc >= n, "ps_linear: output row stride %d smaller than n %d", p->ldc, n);
  PS_REQUIRE(p->dtype == PS_F32 || p->dtype == PS_BF16, "ps_linear: unknown dtype %d", p->dtype);
  PS_REQUIRE(p->c_dtype == PS_F32 || p->c_dtype == PS_BF16, "ps_linear: unknown output dtype %d",
             p->c_dtype);
  PS_REQUIRE(!(p->dtype == PS_F32 && p->c_dtype == PS_BF16),
             "ps_linear: float operands with bfloat16 output are not supported");
  PS_REQUIRE(p->epilogue >= PS_EPI_NONE && p->epilogue <= PS_EPI_RESIDUAL,
             "ps_linear: unknown epilogue %d", p->epilogue);
  PS_REQUIRE(p->epilogue != PS_EPI_RESIDUAL || p->c_dtype == PS_F32,
             "ps_linear: the residual epilogue needs a float output");
  PS_REQUIRE(p->w != nullptr && p->c != nullptr, "ps_linear: null matrix");
  const bool has_norm = p->norm_h != nullptr;
  if (has_norm) {
    PS_REQUIRE(p->gamma != nullptr && p->eps > 0.f && p->ldh >= k,
               "ps_linear: the norm needs gamma, a positive eps and rows of at least k values");
  } else {
    PS_REQUIRE(p->a != nullptr && p->lda >= k, "ps_linear: input rows shorter than k");
  }
  KvScatter scatter = {};
  if (p->k_pool != nullptr) {
    PS_REQUIRE(p->v_pool && p->tok_item && p->tok_pos && p->tables, "ps_linear: incomplete scatter");
    PS_REQUIRE(p->epilogue == PS_EPI_NONE && p->c_dtype == p->dtype,
               "ps_linear: the key/value scatter needs a plain epilogue and output of the cache's type");
    PS_REQUIRE(p->q_cols >= 0 && p->kv_cols > 0 && p->q_cols + 2 * p->kv_cols == n &&
                   p->head_dim > 0 && p->kv_heads * p->head_dim == p->kv_cols &&
                   p->page_size > 0 && p->num_pages > 0 && p->table_width > 0,
               "ps_linear: scatter sizes do not describe a [q | k | v] output of %d columns", n);
    scatter.k_pool = p->k_pool;
    scatter.v_pool = p->v_pool;
    scatter.tok_item = p->tok_item;
    scatter.tok_pos = p->tok_pos;
    scatter.tables = p->tables;
    scatter.table_width = p->table_width;
    scatter.q_cols = p->q_cols;
    scatter.kv_cols = p->kv_cols;
    scatter.head_dim = p->head_dim;
    scatter.kv_heads = p->kv_heads;
    scatter.page_size = p->page_size;
    scatter.num_pages = p->num_pages;
    scatter.cache_only = p->scatter_only;
    scatter.page_shift = -1;
    if ((p->page_size & (p->page_size - 1)) == 0) {
      scatter.page_shift = 0;
      while ((1 << scatter.page_shift) < p->page_size) ++scatter.page_shift;
    }
  }
  if (p->top_tokens != nullptr) {
    PS_REQUIRE(p->top_keys != nullptr && p->top_ticket != nullptr && p->top_done != nullptr,
               "ps_linear: choosing tokens needs keys, a ticket and a place for the answer");
    PS_REQUIRE(p->epilogue == PS_EPI_NONE && p->c_dtype == PS_F32 && scatter.k_pool == nullptr,
               "ps_linear: tokens are chosen from a plain float output");
    *p->top_done = 0;
  }
  if (m == 0) return 0;
  hipStream_t s = (hipStream_t)stream;

  const void* a = p->a;
  int lda = p->lda;
  if (p->c_layout != nullptr) *p->c_layout = 0;
  // 17 to 64 rows of bfloat16: activations may travel in the packed order (linear.h)
  const bool decode_rows = p->dtype == PS_BF16 && m > 16 && m <= 64;
  const int padded_rows = (m + 15) / 16 * 16;
  int layouts = 0;
  if (p->a_packed) {
    PS_REQUIRE(!has_norm && decode_rows && k % 64 == 0,
               "ps_linear: packed input rows go with 17 to 64 bfloat16 rows and k a multiple of 64");
    layouts |= 1;
  }
  if (has_norm) {
    NormPrologue norm = {p->norm_h, p->norm_rows, p->gamma, p->beta, p->eps, p->rms, p->ldh};
    if (ps_norm_gemm_fusable(p->w, norm, m, n, k, p->dtype)) {
      return ps_norm_gemm_fused(norm, p->w, p->bias, p->c, m, n, k, p->ldc, p->c_dtype,
                                p->epilogue, scatter, p->w_packed, s);
    }
    PS_REQUIRE(p->norm_out != nullptr, "ps_linear: scratch for the normed rows is needed");
    PS_REQUIRE(p->ldh == k, "ps_linear: unfused norm needs dense rows (ldh %d, k %d)", p->ldh, k);
    const bool pack_norm = decode_rows && k % 64 == 0 && k <= 2048 &&
                           p->norm_out_rows >= padded_rows &&
                           ps_gemm_nt_mfma_skinny(p->norm_out, p->w, m, n, k, k, p->dtype, p->epilogue);
    int status = ps_norm_layout(p->norm_h, p->norm_rows, p->gamma, p->beta, p->norm_out, m, k,
                                p->eps, p->rms, p->dtype, pack_norm ? 1 : 0, s);
    if (status != 0) return status;
    a = p->norm_out;
    lda = k;
    if (pack_norm) layouts |= 1;
  }
  // Matrix cores when the operands allow 16-byte loads; in float only for many rows (the
  // tile is 128 rows high), else the plain kernel.
  const bool mfma = ps_gemm_nt_mfma_supported(a, p->w, k, lda, p->dtype) &&
                    (p->dtype == PS_BF16 || m >= 96);
  if (mfma) {
    if (p->c_packed_request && decode_rows && p->c_dtype == PS_BF16 && n % 64 == 0 &&
        p->epilogue != PS_EPI_RESIDUAL && scatter.k_pool == nullptr && p->c_rows >= padded_rows &&
        p->ldc == n && p->c_layout != nullptr &&
        ps_gemm_nt_mfma_skinny(a, p->w, m, n, k, lda, p->dtype, p->epilogue)) {
      layouts |= 2;
      *p->c_layout = 1;
    }
    TopChoice top = {};
    if (p->top_tokens != nullptr && ps_gemm_nt_mfma_skinny(a, p->w, m, n, k, lda, p->dtype, p->epilogue)) {
      top.keys = reinterpret_cast<unsigned long long*>(p->top_keys);
      top.ticket = p->top_ticket;
      top.tokens = p->top_tokens;
      *p->top_done = 1;
    }
    return ps_gemm_nt_mfma(a, p->w, p->bias, p->c, m, n, k, lda, p->ldc, p->dtype, p->c_dtype,
                           p->epilogue, scatter, p->dtype == PS_BF16 ? p->w_packed : nullptr,
                           layouts, top, s);
  }
  PS_REQUIRE(layouts == 0, "ps_linear: packed input rows need operands that the matrix-core kernels take");
  int status = ps_gemm_nt_simple(a, p->w, p->bias, p->c, m, n, k, lda, p->ldc, p->dtype,
                                 p->c_dtype, p->epilogue, s);
  if (status != 0 || scatter.k_pool == nullptr) return status;
  // the plain kernel has no scatter: store the key and value columns in a second launch
  const size_t element = p->dtype == PS_BF16 ? 2 : 4;
  const char* base = (const char*)p->c;
  return ps_kv_write(base + (size_t)p->q_cols * element,
                     base + (size_t)(p->q_cols + p->kv_cols) * element, p->ldc, p->k_pool,
                     p->v_pool, p->tok_item, p->tok_pos, p->tables, p->table_width, m,
                     p->kv_heads, p->head_dim, p->page_size, p->num_pages, p->dtype, stream);
}

extern "C" int ps_gemm_nt(const void* a, const void* w, const float* bias, void* c, int m, int n,
                          int k, int lda, int ldc, int dtype, int c_dtype, int epilogue,
                          void* stream) {
  PsLinearArgs args = {};
  args.a = a;
  args.w = w;
  args.bias = bias;
  args.c = c;
  args.m = m;
  args.n = n;
  args.k = k;
  args.lda = lda;
  args.ldc = ldc;
  args.dtype = dtype;
  args.c_dtype = c_dtype;
  args.epilogue = epilogue;
  return ps_linear(&args, stream);
}
