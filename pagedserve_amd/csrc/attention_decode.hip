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


// Eight consecutive elements as they lie in memory; widened to float when they are used, so
// that many of them can be in flight without filling the register file.
template <typename T>
struct Raw8;

template <>
struct Raw8<float> {
  float4 a, b;
  template <bool NT>
  __device__ inline void load(const float* p) {
    a = *reinterpret_cast<const float4*>(p);
    b = *reinterpret_cast<const float4*>(p + 4);
  }
  __device__ inline void widen(float* out) const {
    out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w;
    out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
  }
};

template <>
struct Raw8<bf16_t> {
  uint4 raw;
  // NT: a load that leaves no line behind in the caches.  Keys and values are read once per
  // step; with more blocks than compute units, where memory bandwidth is the limit, such loads
  // measured 13 % faster (5.7 against 5.0 TB/s at 64 requests); with fewer blocks, where the
  // latency of a block's one round of loads is the limit, slightly slower.
  template <bool NT>
  __device__ inline void load(const bf16_t* p) {
    if constexpr (NT) {
      typedef __attribute__((ext_vector_type(4))) uint32_t vec_t;
      const vec_t v = __builtin_nontemporal_load(reinterpret_cast<const vec_t*>(p));
      raw = make_uint4(v.x, v.y, v.z, v.w);
    } else {
      raw = *reinterpret_cast<const uint4*>(p);
    }
  }
  __device__ inline void widen(float* out) const {
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      out[2 * i] = __uint_as_float(w[i] << 16);
      out[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
};

// 2^x (the arguments here are never positive).  Scores are kept in units of log 2, so that no
// multiplication precedes it.  The 32-bit path takes the library's exp2f, which is exact to an
// ulp over the whole range, tiny results included; bfloat16 storage takes the bare hardware
// instruction.
template <typename T>
__device__ inline float exp2_fast(float x) {
  if constexpr (sizeof(T) == 4) return exp2f(x);
  else return __builtin_amdgcn_exp2f(x);
}

// Over the lanes that hold the same head dimensions (l ^ LPK, l ^ 2 LPK, ... l ^ 32): the
// maximum, then the sums of the states scaled to it.
template <int LPK>
__device__ inline float groups_max(float v) {
  if (LPK <= 1) v = xor_max<1>(v);
  if (LPK <= 2) v = xor_max<2>(v);
  if (LPK <= 4) v = xor_max<4>(v);
  if (LPK <= 8) v = xor_max<8>(v);
  if (LPK <= 16) v = xor_max<16>(v);
  return xor_max<32>(v);
}
template <int LPK>
__device__ inline float groups_sum(float v) {
  if (LPK <= 1) v = xor_sum<1>(v);
  if (LPK <= 2) v = xor_sum<2>(v);
  if (LPK <= 4) v = xor_sum<4>(v);
  if (LPK <= 8) v = xor_sum<8>(v);
  if (LPK <= 16) v = xor_sum<16>(v);
  return xor_sum<32>(v);
}

template <typename T, int LPK, int AD_WAVES, int AD_UNROLL, bool NT>
__global__ __launch_bounds__(64 * AD_WAVES) void attention_decode_kernel(
    const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k_pool,
    const T* __restrict__ v_pool, T* __restrict__ out, int64_t out_stride,
    float* __restrict__ partial, const int* __restrict__ tok_list,
    const int* __restrict__ tok_item, const int* __restrict__ tok_pos,
    const int* __restrict__ tables, int table_width, int heads, int kv_heads, int head_dim,
    int page_size, int page_shift, int num_pages, float scale_log2, int window, int splits) {
  constexpr int GROUPS = 64 / LPK;               // keys per wave load
  constexpr int KEYS_PER_WAVE = GROUPS * AD_UNROLL;
  __shared__ float s_acc[AD_WAVES][256];
  __shared__ float s_ml[AD_WAVES][2];

  const int n = blockIdx.x;
  const int head = blockIdx.y;
  const int split = blockIdx.z;
  const int t = tok_list ? tok_list[n] : n;
  const int kv_head = head / (heads / kv_heads);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // the same in every lane: scalar
  const int group = lane / LPK;
  const int dim0 = (lane % LPK) * 8;
  const bool has_dims = dim0 < head_dim;

  // tok_item == null: token t is item t (a step of single tokens only).  The row of the
  // block table is then known without a load, and when it is short its entries are asked for
  // at once, beside the position, instead of behind it: one trip to memory less on the way to
  // the first keys (lane l holds entries l and l + 64; the lanes hand them to each other).
  const bool direct = tok_item == nullptr;
  const bool prefetched = direct && table_width <= 128;
  int held0 = 0, held1 = 0;
  if (prefetched) {
    const int* row = tables + (int64_t)t * table_width;
    held0 = row[lane < table_width ? lane : table_width - 1];
    if (table_width > 64) held1 = row[lane + 64 < table_width ? lane + 64 : table_width - 1];
  }
  const int pos = tok_pos[t];
  const int* table = tables + (int64_t)(direct ? t : tok_item[t]) * table_width;
  const int first_key = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int end_key = pos + 1;
  int chunk = (end_key - first_key + splits - 1) / splits;
  chunk = (chunk + KEYS_PER_WAVE - 1) / KEYS_PER_WAVE * KEYS_PER_WAVE;
  const int range_begin = first_key + split * chunk;
  const int range_end = range_begin + chunk < end_key ? range_begin + chunk : end_key;

  float qf[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
    qf[i] = has_dims ? to_float<T>(q[(int64_t)t * q_stride + (int64_t)head * head_dim + dim0 + i])
                     : 0.f;

  float m = -INFINITY, l = 0.f;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  for (int base = range_begin + wave * KEYS_PER_WAVE; base < range_end;
       base += AD_WAVES * KEYS_PER_WAVE) {
    Raw8<T> kr[AD_UNROLL], vr[AD_UNROLL];
    bool valid[AD_UNROLL];
    // Every load is unconditional from a clamped address and masked afterwards, so that the
    // table entries, then all keys and values of the iteration, travel together.
    int page[AD_UNROLL], within[AD_UNROLL];
#pragma unroll
    for (int u = 0; u < AD_UNROLL; ++u) {
      const int key = base + u * GROUPS + group;
      const int safe_key = key < range_end ? key : range_end - 1;
      const int logical = page_shift >= 0 ? (safe_key >> page_shift) : safe_key / page_size;
      within[u] = safe_key - logical * page_size;
      const int entry = logical < table_width ? logical : table_width - 1;
      if (prefetched) {
        const int low = __shfl(held0, entry & 63, 64);
        page[u] = low;
        if (table_width > 64) {
          const int high = __shfl(held1, entry & 63, 64);
          page[u] = entry < 64 ? low : high;
        }
      } else {
        page[u] = table[entry];
      }
      valid[u] = key < range_end && logical < table_width;
    }
#pragma unroll
    for (int u = 0; u < AD_UNROLL; ++u) {
      valid[u] = valid[u] && page[u] >= 0 && page[u] < num_pages;
      const int safe_page = valid[u] ? page[u] : 0;
      const int64_t offset =
          (((int64_t)safe_page * kv_heads + kv_head) * page_size + within[u]) * head_dim +
          (has_dims ? dim0 : 0);
      kr[u].template load<NT>(k_pool + offset);
      vr[u].template load<NT>(v_pool + offset);
    }
    float s[AD_UNROLL];
    float m_new = m;
#pragma unroll
    for (int u = 0; u < AD_UNROLL; ++u) {
      float kf[8];
      kr[u].widen(kf);
      float dot = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) dot = fmaf(qf[i], kf[i], dot);
      if (!has_dims) dot = 0.f;
      if (LPK <= 16) {
        dot = lanes_sum<(LPK <= 16 ? LPK : 16)>(dot);
      } else {
        dot = lanes_sum<16>(dot);
        dot += __shfl_xor(dot, 16, 64);
      }
      s[u] = valid[u] ? dot * scale_log2 : -INFINITY;
      m_new = fmaxf(m_new, s[u]);
    }
    if (m_new != -INFINITY) {
      const float correction = (m == -INFINITY) ? 0.f : exp2_fast<T>(m - m_new);
      l *= correction;
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] *= correction;
#pragma unroll
      for (int u = 0; u < AD_UNROLL; ++u) {
        const float p = valid[u] ? exp2_fast<T>(s[u] - m_new) : 0.f;
        l += p;
        float vf[8];
        vr[u].widen(vf);
        // a masked key was loaded from a clamped address and may hold anything, also NaN
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = valid[u] ? fmaf(p, vf[i], acc[i]) : acc[i];
      }
      m = m_new;
    }
  }
  if (!has_dims) {
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  }

  // merge the lane groups of this wave: every state is scaled to the wave's maximum, then
  // the sums run over the lanes that hold the same head dimensions
  {
    const float wave_m = groups_max<LPK>(m);
    const float c = (m == -INFINITY) ? 0.f : exp2_fast<T>(m - wave_m);
    l = groups_sum<LPK>(l * c);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = groups_sum<LPK>(acc[i] * c);
    m = wave_m;
  }
  if (group == 0 && has_dims) {
#pragma unroll
    for (int i = 0; i < 8; ++i) s_acc[wave][dim0 + i] = acc[i];
  }
  if (lane == 0) {
    s_ml[wave][0] = m;
    s_ml[wave][1] = l;
  }
  __syncthreads();

  // merge the waves: one thread per head dimension
  const int d = threadIdx.x;
  if (d >= 256) return;
  float block_m = -INFINITY;
#pragma unroll
  for (int w = 0; w < AD_WAVES; ++w) block_m = fmaxf(block_m, s_ml[w][0]);
  float block_l = 0.f, value = 0.f;
#pragma unroll
  for (int w = 0; w < AD_WAVES; ++w) {
    const float c = (s_ml[w][0] == -INFINITY) ? 0.f : exp2_fast<T>(s_ml[w][0] - block_m);
    block_l += s_ml[w][1] * c;
    if (d < head_dim) value += s_acc[w][d] * c;
  }
  if (splits == 1 && out != nullptr) {
    if (d < head_dim)
      out[(int64_t)t * out_stride + (int64_t)head * head_dim + d] = from_float<T>(value / block_l);
  } else {
    float* dst = partial + (((int64_t)n * heads + head) * splits + split) * (head_dim + 2);
    if (d < head_dim) dst[d] = value;
    if (d == 0) {
      dst[head_dim] = block_m;
      dst[head_dim + 1] = block_l;
    }
  }
}

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
