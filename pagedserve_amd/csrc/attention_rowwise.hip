// Paged attention, one wave per (token, head): the plain kernel of the engine.
//
// For the token at position p of its request it visits keys max(0, p - window + 1) .. p
// through the request's block table, 64 keys at a time: each lane scores one key
// (q . k * scale), the wave keeps the running maximum and sum of an online softmax
// (reference: src/kernels/triton_paged_attention.py:219-223,275-331), and each lane
// accumulates the weighted values of the head dimensions it owns.  Scores, softmax state and
// accumulators are float whatever the storage type.  Used for every token in the 32-bit path
// and as the fallback for shapes the tiled kernels refuse; it reads keys that the step has
// already stored, so prompt portions, whole prompts and decoded tokens are the same case.
#include <math.h>

#include "common.h"
#include "pagedserve_hip.h"

#define AR_MAX_DIMS 4  // head_dim <= 256

template <typename T>
__global__ __launch_bounds__(64) void attention_rowwise_kernel(
    const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k_pool,
    const T* __restrict__ v_pool, T* __restrict__ out, int64_t out_stride,
    const int* __restrict__ tok_list, const int* __restrict__ tok_item,
    const int* __restrict__ tok_pos, const int* __restrict__ tables, int table_width, int heads,
    int kv_heads, int head_dim, int page_size, int num_pages, float scale, int window) {
  __shared__ float q_row[256];
  __shared__ float prob[64];
  __shared__ int64_t key_base[64];

  const int t = tok_list ? tok_list[blockIdx.x] : blockIdx.x;
  const int head = blockIdx.y;
  const int kv_head = head / (heads / kv_heads);
  const int lane = threadIdx.x;
  const int pos = tok_pos[t];
  const int* table = tables + (int64_t)tok_item[t] * table_width;
  const int first_key = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int end_key = pos + 1;

  for (int i = lane; i < head_dim; i += 64)
    q_row[i] = to_float<T>(q[(int64_t)t * q_stride + (int64_t)head * head_dim + i]);
  __syncthreads();

  float running_max = -INFINITY;
  float running_sum = 0.f;
  float acc[AR_MAX_DIMS] = {0.f, 0.f, 0.f, 0.f};

  for (int k0 = first_key; k0 < end_key; k0 += 64) {
    const int key = k0 + lane;
    float score = -INFINITY;
    int64_t base = -1;
    if (key < end_key) {
      const int logical = key / page_size;
      const int page = logical < table_width ? table[logical] : -1;
      if (page >= 0 && page < num_pages) {
        base = (((int64_t)page * kv_heads + kv_head) * page_size + (key - logical * page_size)) *
               head_dim;
        const T* k_row = k_pool + base;
        float dot = 0.f;
        for (int i = 0; i < head_dim; ++i) dot = fmaf(q_row[i], to_float<T>(k_row[i]), dot);
        score = dot * scale;
      }
    }
    const float chunk_max = wave_max(score);
    const float new_max = fmaxf(running_max, chunk_max);
    // new_max is -inf only if no key has been visible so far; then nothing accumulates.
    const float correction = (new_max == -INFINITY) ? 1.f : expf(running_max - new_max);
    const float p = (score == -INFINITY) ? 0.f : expf(score - new_max);
    running_sum = running_sum * correction + wave_sum(p);
    running_max = new_max;
    __syncthreads();
    prob[lane] = p;
    key_base[lane] = base;
    __syncthreads();
    const int count = (end_key - k0) < 64 ? (end_key - k0) : 64;
#pragma unroll
    for (int d = 0; d < AR_MAX_DIMS; ++d) {
      const int dim = lane + d * 64;
      if (dim < head_dim) {
        float a = acc[d] * correction;
        for (int j = 0; j < count; ++j) {
          const int64_t vb = key_base[j];
          if (vb >= 0) a = fmaf(prob[j], to_float<T>(v_pool[vb + dim]), a);
        }
        acc[d] = a;
      }
    }
  }

#pragma unroll
  for (int d = 0; d < AR_MAX_DIMS; ++d) {
    const int dim = lane + d * 64;
    if (dim < head_dim)
      out[(int64_t)t * out_stride + (int64_t)head * head_dim + dim] =
          from_float<T>(acc[d] / running_sum);
  }
}

extern "C" int ps_attention_rowwise(const void* q, int64_t q_stride, const void* k_pool,
                                    const void* v_pool, void* out, int64_t out_stride,
                                    const int* tok_list, const int* tok_item, const int* tok_pos,
                                    const int* tables, int table_width, int tokens, int heads,
                                    int kv_heads,
                                    int head_dim, int page_size, int num_pages, float scale,
                                    int window, int dtype, void* stream) {
  PS_REQUIRE(tokens >= 0 && heads > 0 && kv_heads > 0 && page_size > 0 && num_pages > 0 &&
                 table_width > 0,
             "ps_attention_rowwise: bad sizes");
  PS_REQUIRE(heads % kv_heads == 0, "ps_attention_rowwise: heads (%d) must be a multiple of kv_heads (%d)",
             heads, kv_heads);
  PS_REQUIRE(head_dim > 0 && head_dim <= 64 * AR_MAX_DIMS,
             "ps_attention_rowwise: head_dim %d must lie in 1..%d", head_dim, 64 * AR_MAX_DIMS);
  PS_REQUIRE(window >= 0, "ps_attention_rowwise: negative window");
  PS_REQUIRE(heads <= 65535, "ps_attention_rowwise: too many heads");
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_attention_rowwise: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  dim3 grid(tokens, heads);
  if (dtype == PS_F32)
    hipLaunchKernelGGL(attention_rowwise_kernel<float>, grid, dim3(64), 0, s, (const float*)q,
                       q_stride, (const float*)k_pool, (const float*)v_pool, (float*)out,
                       out_stride, tok_list, tok_item, tok_pos, tables, table_width, heads, kv_heads,
                       head_dim, page_size, num_pages, scale, window);
  else
    hipLaunchKernelGGL(attention_rowwise_kernel<bf16_t>, grid, dim3(64), 0, s, (const bf16_t*)q,
                       q_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool, (bf16_t*)out,
                       out_stride, tok_list, tok_item, tok_pos, tables, table_width, heads, kv_heads,
                       head_dim, page_size, num_pages, scale, window);
  PS_CHECK_LAUNCH("ps_attention_rowwise");
  return 0;
}
