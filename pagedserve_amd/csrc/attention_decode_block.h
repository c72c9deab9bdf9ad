// The decode attention's block (see attention_decode.hip for the method): shared by the kernel
// of that file and by the kernel of attention_mixed.hip, which runs such blocks beside the
// blocks of the tiled prefill attention in one launch.
#pragma once
#include <math.h>

#include "common.h"

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

// What a block of this kernel keeps in LDS, in floats: the waves' accumulators and their (m, l).
template <int AD_WAVES>
struct DecodeLds {
  float acc[AD_WAVES][256];
  float ml[AD_WAVES][2];
};

// The work of one block: token n of the list, one head, one range of its keys.  The caller
// provides the block's LDS (the kernel below its own; a kernel that runs blocks of several
// kinds in one launch a share of what all of them need).
template <typename T, int LPK, int AD_WAVES, int AD_UNROLL, bool NT>
__device__ __forceinline__ void attention_decode_block(
    DecodeLds<AD_WAVES>& lds, const int n, const int head, const int split,
    const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k_pool,
    const T* __restrict__ v_pool, T* __restrict__ out, int64_t out_stride,
    float* __restrict__ partial, const int* __restrict__ tok_list,
    const int* __restrict__ tok_item, const int* __restrict__ tok_pos,
    const int* __restrict__ tables, int table_width, int heads, int kv_heads, int head_dim,
    int page_size, int page_shift, int num_pages, float scale_log2, int window, int splits) {
  constexpr int GROUPS = 64 / LPK;               // keys per wave load
  constexpr int KEYS_PER_WAVE = GROUPS * AD_UNROLL;
  float (&s_acc)[AD_WAVES][256] = lds.acc;
  float (&s_ml)[AD_WAVES][2] = lds.ml;

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

template <typename T, int LPK, int AD_WAVES, int AD_UNROLL, bool NT>
__global__ __launch_bounds__(64 * AD_WAVES) void attention_decode_kernel(
    const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k_pool,
    const T* __restrict__ v_pool, T* __restrict__ out, int64_t out_stride,
    float* __restrict__ partial, const int* __restrict__ tok_list,
    const int* __restrict__ tok_item, const int* __restrict__ tok_pos,
    const int* __restrict__ tables, int table_width, int heads, int kv_heads, int head_dim,
    int page_size, int page_shift, int num_pages, float scale_log2, int window, int splits) {
  __shared__ DecodeLds<AD_WAVES> lds;
  attention_decode_block<T, LPK, AD_WAVES, AD_UNROLL, NT>(
      lds, blockIdx.x, blockIdx.y, blockIdx.z, q, q_stride, k_pool, v_pool, out, out_stride, partial,
      tok_list, tok_item, tok_pos, tables, table_width, heads, kv_heads, head_dim, page_size,
      page_shift, num_pages, scale_log2, window, splits);
}

