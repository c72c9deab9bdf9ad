// Split-KV paged attention for single queries: the decode kernel.
//
// One 256-thread block per (query token, head, split).  A token's visible keys are cut into
// `splits` contiguous ranges so that a small batch still fills the chip (the reference's
// Triton kernel runs one program per (request, head), src/kernels/triton_paged_attention.py:
// 84-86, which leaves most CUs idle at batch 1).  Inside a block, LPK lanes share one key:
// each lane loads 8 consecutive head dimensions of it (16 bytes of bfloat16), so a wave's
// load of 64/LPK keys is one contiguous run inside a page; the partial dot products are
// summed over the LPK lanes with shuffles.  Every lane group keeps its own online-softmax
// state (running max m, sum l, 8 accumulators; float, as in src/kernels/
// triton_paged_attention.py:219-223) over the keys it visits and the states are merged once
// at the end: across lane groups by shuffles, across the four waves through LDS.  With one
// split the block writes the output; otherwise it writes (acc, m, l) and
// attention_reduce_kernel merges the splits.  Without an output tensor (out == nullptr) the
// records (acc, m, l) are all that is written, whatever the number of splits: the kernel in
// attention_merge_linear.hip merges them inside the output projection.
#include <math.h>

#include <mutex>

#include "common.h"
#include "pagedserve_hip.h"


#include "attention_decode_block.h"

// out = sum_s acc_s 2^{m_s - M} / sum_s l_s 2^{m_s - M} (the maxima are in units of log 2).  One wave per (token, head); lane s
// first fetches (m_s, l_s) of split s (splits <= 64), so the weights cost one trip to memory.
template <typename T>
__global__ __launch_bounds__(64) void attention_reduce_kernel(
    const float* __restrict__ partial, T* __restrict__ out, int64_t out_stride,
    const int* __restrict__ tok_list, int heads, int head_dim, int splits) {
  const int n = blockIdx.x;
  const int head = blockIdx.y;
  const int lane = threadIdx.x;
  const int t = tok_list ? tok_list[n] : n;
  const int stride = head_dim + 2;
  const float* src = partial + ((int64_t)n * heads + head) * splits * stride;
  const float m_s = lane < splits ? src[lane * stride + head_dim] : -INFINITY;
  const float l_s = lane < splits ? src[lane * stride + head_dim + 1] : 0.f;
  const float total_m = wave_max(m_s);
  const float weight = (m_s == -INFINITY) ? 0.f : exp2_fast<T>(m_s - total_m);
  const float total_l = wave_sum(l_s * weight);
  // Every lane takes part in every round, also where head_dim leaves it no dimension: the
  // weights travel by shuffles, and a shuffle only reads lanes that execute it.
  for (int d0 = 0; d0 < head_dim; d0 += 64) {
    const int d = d0 + lane;
    const bool mine = d < head_dim;
    const int safe_d = mine ? d : 0;
    float value = 0.f;
    for (int s = 0; s < splits; ++s)
      value = fmaf(src[s * stride + safe_d], __shfl(weight, s, 64), value);
    if (mine)
      out[(int64_t)t * out_stride + (int64_t)head * head_dim + d] = from_float<T>(value / total_l);
  }
}

template <typename T>
static int launch_decode(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                         void* out, int64_t out_stride, float* partial, const int* tok_list,
                         const int* tok_item, const int* tok_pos, const int* tables,
                         int table_width, int count, int heads, int kv_heads, int head_dim,
                         int page_size, int num_pages, float scale, int window, int splits,
                         int waves, hipStream_t s) {
  int page_shift = -1;
  if ((page_size & (page_size - 1)) == 0) {
    page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
  }
  dim3 grid(count, heads, splits);
#define PS_LAUNCH_ADN(LPK, WAVES, NT)                                                            \
  hipLaunchKernelGGL((attention_decode_kernel<T, LPK, WAVES, (WAVES == 16 && sizeof(T) == 2 ? 8 : 4), NT>), grid, \
                     dim3(64 * WAVES), 0, s,                                                     \
                     (const T*)q, q_stride, (const T*)k_pool, (const T*)v_pool, (T*)out,         \
                     out_stride, partial, tok_list, tok_item, tok_pos, tables, table_width,      \
                     heads, kv_heads, head_dim, page_size, page_shift, num_pages,                \
                     scale * 1.4426950408889634f, window, splits)
  // more blocks than compute units: the step is bound by memory bandwidth, not by one round trip
  const bool streaming = sizeof(T) == 2 && (int64_t)count * heads * splits > ps_compute_units();
#define PS_LAUNCH_ADW(LPK, WAVES)          \
  do {                                     \
    if (streaming) {                       \
      PS_LAUNCH_ADN(LPK, WAVES, true);     \
    } else {                               \
      PS_LAUNCH_ADN(LPK, WAVES, false);    \
    }                                      \
  } while (0)
#define PS_LAUNCH_AD(LPK)            \
  do {                               \
    if (waves == 16) {               \
      PS_LAUNCH_ADW(LPK, 16);        \
    } else {                         \
      PS_LAUNCH_ADW(LPK, 4);         \
    }                                \
  } while (0)
  const int lanes = head_dim / 8;
  if (lanes <= 2) PS_LAUNCH_AD(2);
  else if (lanes <= 4) PS_LAUNCH_AD(4);
  else if (lanes <= 8) PS_LAUNCH_AD(8);
  else if (lanes <= 16) PS_LAUNCH_AD(16);
  else PS_LAUNCH_AD(32);
#undef PS_LAUNCH_AD
#undef PS_LAUNCH_ADW
#undef PS_LAUNCH_ADN
  PS_CHECK_LAUNCH("ps_attention_decode");
  if (splits > 1 && out != nullptr) {
    hipLaunchKernelGGL(attention_reduce_kernel<T>, dim3(count, heads), dim3(64), 0, s, partial,
                       (T*)out, out_stride, tok_list, heads, head_dim, splits);
    PS_CHECK_LAUNCH("ps_attention_decode(reduce)");
  }
  return 0;
}

static int check_decode_sizes(const char* who, int count, int heads, int kv_heads, int head_dim,
                              int page_size, int num_pages, int table_width, int window,
                              int splits, int waves, int dtype) {
  PS_REQUIRE(count >= 0 && heads > 0 && kv_heads > 0 && page_size > 0 && num_pages > 0 &&
                 table_width > 0,
             "%s: bad sizes", who);
  PS_REQUIRE(heads % kv_heads == 0, "%s: heads (%d) must be a multiple of kv_heads (%d)", who,
             heads, kv_heads);
  // a lane fetches eight consecutive head dimensions of a key in one piece
  PS_REQUIRE(head_dim > 0 && head_dim % 8 == 0 && head_dim <= 256,
             "%s: head_dim %d must be a multiple of 8 up to 256 (ps_attention_rowwise takes "
             "every head size)", who, head_dim);
  PS_REQUIRE(window >= 0, "%s: negative window", who);
  PS_REQUIRE(splits >= 1 && splits <= 64 && heads <= 65535,
             "%s: splits %d / heads %d out of range", who, splits, heads);
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "%s: unknown dtype %d", who, dtype);
  PS_REQUIRE(waves == 4 || waves == 16, "%s: blocks have 4 or 16 waves, not %d", who, waves);
  return 0;
}

// ---- the variant that allocates nothing ------------------------------------------------------
// The partial results of the key ranges live in a file-scope device array instead of a buffer
// that the caller allocates.  Every GPU holds its own copy of the array at its own address;
// the name below is only the host's handle for hipGetSymbolAddress, never a kernel argument.
static __device__ __align__(256) float scratch[PS_DECODE_STATIC_SCRATCH_FLOATS];

#define PS_MAX_DEVICES 64
static std::mutex g_scratch_mutex;
static float* g_scratch_ptr[PS_MAX_DEVICES];   // per device: where its copy of `scratch` lies

// The address of the current device's copy (looked up once per device), or null with the
// error set.
static float* static_scratch_of_current_device() {
  int device = -1;
  hipError_t status = hipGetDevice(&device);
  if (status != hipSuccess || device < 0 || device >= PS_MAX_DEVICES) {
    ps_set_error("ps_attention_decode_static: no current device (%s)",
                 status == hipSuccess ? "index out of range" : hipGetErrorString(status));
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[device] == nullptr) {
    void* address = nullptr;
    status = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));
    if (status != hipSuccess || address == nullptr) {
      ps_set_error("ps_attention_decode_static: hipGetSymbolAddress failed on device %d: %s",
                   device, hipGetErrorString(status));
      return nullptr;
    }
    g_scratch_ptr[device] = static_cast<float*>(address);
  }
  return g_scratch_ptr[device];
}

extern "C" int ps_attention_decode_static(const void* q, int64_t q_stride, const void* k_pool,
                                          const void* v_pool, void* out, int64_t out_stride,
                                          const int* tok_list, const int* tok_item,
                                          const int* tok_pos, const int* tables, int table_width,
                                          int count, int heads, int kv_heads, int head_dim,
                                          int page_size, int num_pages, float scale, int window,
                                          int splits, int waves, int dtype, void* stream) {
  if (check_decode_sizes("ps_attention_decode_static", count, heads, kv_heads, head_dim, page_size,
                         num_pages, table_width, window, splits, waves, dtype))
    return 1;
  PS_REQUIRE(out != nullptr, "ps_attention_decode_static: no output tensor");
  float* partial = nullptr;
  if (splits > 1) {
    const int64_t need = (int64_t)count * heads * splits * (head_dim + 2);
    PS_REQUIRE(need <= (int64_t)PS_DECODE_STATIC_SCRATCH_FLOATS,
               "ps_attention_decode_static: %d tokens x %d heads x %d splits x (%d + 2) = %lld "
               "floats of partial results exceed the static scratch of %lld floats; use fewer "
               "splits or ps_attention_decode with a buffer of the caller",
               count, heads, splits, head_dim, (long long)need,
               (long long)PS_DECODE_STATIC_SCRATCH_FLOATS);
    partial = static_scratch_of_current_device();
    if (partial == nullptr) return 3;
  }
  if (count == 0) return 0;
  // Nothing in the scratch has to start at zero: every (token, head, range) block writes its
  // whole record (accumulators, maximum, sum) before the merge kernel reads it, also when its
  // range holds no key.
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PS_F32)
    return launch_decode<float>(q, q_stride, k_pool, v_pool, out, out_stride, partial, tok_list,
                                tok_item, tok_pos, tables, table_width, count, heads, kv_heads,
                                head_dim, page_size, num_pages, scale, window, splits, waves, s);
  return launch_decode<bf16_t>(q, q_stride, k_pool, v_pool, out, out_stride, partial, tok_list,
                               tok_item, tok_pos, tables, table_width, count, heads, kv_heads,
                               head_dim, page_size, num_pages, scale, window, splits, waves, s);
}

// The partial records only (see pagedserve_hip.h).
extern "C" int ps_attention_decode_partial(const void* q, int64_t q_stride, const void* k_pool,
                                           const void* v_pool, float* partial,
                                           int64_t partial_floats, const int* tok_list,
                                           const int* tok_item, const int* tok_pos,
                                           const int* tables, int table_width, int count,
                                           int heads, int kv_heads, int head_dim, int page_size,
                                           int num_pages, float scale, int window, int splits,
                                           int waves, int dtype, void* stream) {
  if (check_decode_sizes("ps_attention_decode_partial", count, heads, kv_heads, head_dim,
                         page_size, num_pages, table_width, window, splits, waves, dtype))
    return 1;
  const int64_t need = (int64_t)count * heads * splits * (head_dim + 2);
  PS_REQUIRE(partial != nullptr && partial_floats >= need,
             "ps_attention_decode_partial: the records need %lld floats", (long long)need);
  if (count == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PS_F32)
    return launch_decode<float>(q, q_stride, k_pool, v_pool, nullptr, 0, partial, tok_list,
                                tok_item, tok_pos, tables, table_width, count, heads, kv_heads,
                                head_dim, page_size, num_pages, scale, window, splits, waves, s);
  return launch_decode<bf16_t>(q, q_stride, k_pool, v_pool, nullptr, 0, partial, tok_list,
                               tok_item, tok_pos, tables, table_width, count, heads, kv_heads,
                               head_dim, page_size, num_pages, scale, window, splits, waves, s);
}

extern "C" int ps_attention_decode(const void* q, int64_t q_stride, const void* k_pool,
                                   const void* v_pool, void* out, int64_t out_stride,
                                   float* partial, int64_t partial_floats, const int* tok_list,
                                   const int* tok_item, const int* tok_pos, const int* tables,
                                   int table_width, int count, int heads, int kv_heads,
                                   int head_dim, int page_size, int num_pages, float scale,
                                   int window, int splits, int waves, int dtype, void* stream) {
  if (check_decode_sizes("ps_attention_decode", count, heads, kv_heads, head_dim, page_size,
                         num_pages, table_width, window, splits, waves, dtype))
    return 1;
  PS_REQUIRE(out != nullptr, "ps_attention_decode: no output tensor");
  if (splits > 1) {
    const int64_t need = (int64_t)count * heads * splits * (head_dim + 2);
    PS_REQUIRE(partial != nullptr && partial_floats >= need,
               "ps_attention_decode: %lld floats of scratch needed for %d splits, %lld given",
               (long long)need, splits, (long long)partial_floats);
  }
  if (count == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PS_F32)
    return launch_decode<float>(q, q_stride, k_pool, v_pool, out, out_stride, partial, tok_list,
                                tok_item, tok_pos, tables, table_width, count, heads, kv_heads,
                                head_dim, page_size, num_pages, scale, window, splits, waves, s);
  return launch_decode<bf16_t>(q, q_stride, k_pool, v_pool, out, out_stride, partial, tok_list,
                               tok_item, tok_pos, tables, table_width, count, heads, kv_heads,
                               head_dim, page_size, num_pages, scale, window, splits, waves, s);
}
