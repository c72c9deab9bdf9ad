// Paged attention of items with several tokens (prompt portions) in true 32-bit.
//
// A block of four waves per (tile of 64 queries, head).  Keys and values come 64 at a time
// through the request's block table into LDS, as floats; the 64 x 64 scores of a tile are
// plain fused multiply-adds in registers (a thread owns 4 queries x 4 keys; no matrix mode
// of reduced precision), the softmax runs online per query row in float with the library's
// expf (reference: src/kernels/triton_paged_attention.py:219-223,275-331), the probabilities
// go through LDS, and a thread accumulates 4 queries x its 4 (or 8) head dimensions.  Every
// key is read once per 64 queries where the one-wave-per-token kernel reads it once per query
// (a prefill of 2 x 1,024 tokens at 12 heads of 64: 110 against 750 us a layer).
//
// The tiles are those of the bfloat16 kernel (`tile_item`, `tile_q0`: the item of each tile and
// its first query within the item's tokens of this step), and so are the rules: query i of an
// item whose cached length after the step is L and which brings n tokens stands at position
// L - n + i and sees keys max(0, position - window + 1) .. position.
//
// Head sizes that are multiples of 4 up to 128; others stay with the one-wave-per-token
// kernel.
#include <math.h>

#include "common.h"
#include "pagedserve_hip.h"

#define AF_TILE 64       // queries of a block, and keys per turn of its loop
#define AF_MAX_DIM 128
#define AF_P_STRIDE 68   // floats from row to row of the probabilities in LDS

// DV: float4 groups of head dimensions per thread (thread tx owns groups tx and tx + 16)
template <int DV>
__global__ __launch_bounds__(256) void attention_tiled_f32_kernel(
    const float* __restrict__ q, int64_t q_stride, const float* __restrict__ k_pool,
    const float* __restrict__ v_pool, float* __restrict__ out, int64_t out_stride,
    const int* __restrict__ tile_item, const int* __restrict__ tile_q0,
    const int* __restrict__ cu_tokens, const int* __restrict__ kv_lens,
    const int* __restrict__ tables, int table_width, int heads, int kv_heads, int head_dim,
    int page_size, int num_pages, float scale, int window) {
  constexpr int STRIDE = 64 * DV + 4;   // floats from row to row of q, k and v in LDS
  __shared__ __attribute__((aligned(16))) float s_q[AF_TILE * STRIDE];
  __shared__ __attribute__((aligned(16))) float s_k[AF_TILE * STRIDE];
  __shared__ __attribute__((aligned(16))) float s_v[AF_TILE * STRIDE];
  __shared__ __attribute__((aligned(16))) float s_p[AF_TILE * AF_P_STRIDE];
  __shared__ int64_t s_base[AF_TILE];   // first value of each key's row in the pools, or -1

  const int tid = threadIdx.x;
  const int tx = tid & 15;    // keys tx + 16 j of a turn of the loop; dimension groups tx + 16 v
  const int ty = tid >> 4;    // queries 4 ty + i of the tile
  const int tile_index = blockIdx.x / heads;
  const int head = blockIdx.x - tile_index * heads;
  const int kv_head = head / (heads / kv_heads);
  const int d4 = head_dim >> 2;

  const int item = tile_item[tile_index];
  const int q0 = tile_q0[tile_index];
  const int tok0 = cu_tokens[item];
  const int count = cu_tokens[item + 1] - tok0;
  const int start = kv_lens[item] - count;   // position of the portion's first token
  const int* table = tables + (int64_t)item * table_width;
  const int last_q = q0 + AF_TILE - 1 < count ? q0 + AF_TILE - 1 : count - 1;
  const int key_end = start + last_q + 1;
  int key_begin = 0;
  if (window > 0 && start + q0 - window + 1 > 0) key_begin = start + q0 - window + 1;

  // the tile's queries; rows beyond the item's tokens are zeros and never stored
  for (int index = tid; index < AF_TILE * d4; index += 256) {
    const int row = index / d4;
    const int f = index - row * d4;
    float4 value = make_float4(0.f, 0.f, 0.f, 0.f);
    if (q0 + row < count)
      value = *reinterpret_cast<const float4*>(q + (int64_t)(tok0 + q0 + row) * q_stride +
                                               (int64_t)head * head_dim + 4 * f);
    *reinterpret_cast<float4*>(&s_q[row * STRIDE + 4 * f]) = value;
  }

  int q_pos[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) q_pos[i] = q0 + 4 * ty + i < count ? start + q0 + 4 * ty + i : -1;
  float run_max[4], run_sum[4];
  float4 acc[DV][4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    run_max[i] = -INFINITY;
    run_sum[i] = 0.f;
#pragma unroll
    for (int v = 0; v < DV; ++v) acc[v][i] = make_float4(0.f, 0.f, 0.f, 0.f);
  }

  for (int k0 = key_begin; k0 < key_end; k0 += AF_TILE) {
    // (the 64 keys before have been read: the barrier at the end of the loop)
    if (tid < AF_TILE) {
      const int key = k0 + tid;
      int64_t base = -1;
      if (key < key_end) {
        const int logical = key / page_size;
        const int page = logical < table_width ? table[logical] : -1;
        if (page >= 0 && page < num_pages)
          base = (((int64_t)page * kv_heads + kv_head) * page_size + (key - logical * page_size)) *
                 head_dim;
      }
      s_base[tid] = base;
    }
    __syncthreads();
    for (int index = tid; index < AF_TILE * d4; index += 256) {
      const int row = index / d4;
      const int f = index - row * d4;
      const int64_t base = s_base[row];
      float4 key_values = make_float4(0.f, 0.f, 0.f, 0.f), values = key_values;
      if (base >= 0) {
        key_values = *reinterpret_cast<const float4*>(k_pool + base + 4 * f);
        values = *reinterpret_cast<const float4*>(v_pool + base + 4 * f);
      }
      *reinterpret_cast<float4*>(&s_k[row * STRIDE + 4 * f]) = key_values;
      *reinterpret_cast<float4*>(&s_v[row * STRIDE + 4 * f]) = values;
    }
    __syncthreads();

    // scores of queries 4 ty + i against keys k0 + tx + 16 j
    float s[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) s[i][j] = 0.f;
    for (int f = 0; f < d4; ++f) {
      float4 a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = *reinterpret_cast<const float4*>(&s_q[(4 * ty + i) * STRIDE + 4 * f]);
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = *reinterpret_cast<const float4*>(&s_k[(tx + 16 * j) * STRIDE + 4 * f]);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          s[i][j] = fmaf(a[i].x, b[j].x, s[i][j]);
          s[i][j] = fmaf(a[i].y, b[j].y, s[i][j]);
          s[i][j] = fmaf(a[i].z, b[j].z, s[i][j]);
          s[i][j] = fmaf(a[i].w, b[j].w, s[i][j]);
        }
    }
    bool key_ok[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) key_ok[j] = s_base[tx + 16 * j] >= 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float tile_max = -INFINITY;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int key = k0 + tx + 16 * j;
        const bool visible = key_ok[j] && key <= q_pos[i] && (window <= 0 || q_pos[i] - key < window);
        s[i][j] = visible ? s[i][j] * scale : -INFINITY;
        tile_max = fmaxf(tile_max, s[i][j]);
      }
      // the 16 threads of a row are 16 neighbouring lanes of one wave
#pragma unroll
      for (int mask = 8; mask >= 1; mask >>= 1) tile_max = fmaxf(tile_max, __shfl_xor(tile_max, mask, 16));
      const float new_max = fmaxf(run_max[i], tile_max);
      // new_max is -inf only while no key has been visible; then nothing accumulates
      const float correction = new_max == -INFINITY ? 1.f : expf(run_max[i] - new_max);
      float tile_sum = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float p = s[i][j] == -INFINITY ? 0.f : expf(s[i][j] - new_max);
        s_p[(4 * ty + i) * AF_P_STRIDE + tx + 16 * j] = p;
        tile_sum += p;
      }
#pragma unroll
      for (int mask = 8; mask >= 1; mask >>= 1) tile_sum += __shfl_xor(tile_sum, mask, 16);
      run_sum[i] = run_sum[i] * correction + tile_sum;
      run_max[i] = new_max;
#pragma unroll
      for (int v = 0; v < DV; ++v) {
        acc[v][i].x *= correction;
        acc[v][i].y *= correction;
        acc[v][i].z *= correction;
        acc[v][i].w *= correction;
      }
    }
    __syncthreads();

    // weighted values: queries 4 ty + i, dimension groups tx + 16 v
    for (int j4 = 0; j4 < AF_TILE / 4; ++j4) {
      float4 p[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) p[i] = *reinterpret_cast<const float4*>(&s_p[(4 * ty + i) * AF_P_STRIDE + 4 * j4]);
#pragma unroll
      for (int v = 0; v < DV; ++v) {
        const int f = tx + 16 * v;
        if (f < d4) {
          float4 value[4];
#pragma unroll
          for (int jj = 0; jj < 4; ++jj)
            value[jj] = *reinterpret_cast<const float4*>(&s_v[(4 * j4 + jj) * STRIDE + 4 * f]);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float w[4] = {p[i].x, p[i].y, p[i].z, p[i].w};
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
              acc[v][i].x = fmaf(w[jj], value[jj].x, acc[v][i].x);
              acc[v][i].y = fmaf(w[jj], value[jj].y, acc[v][i].y);
              acc[v][i].z = fmaf(w[jj], value[jj].z, acc[v][i].z);
              acc[v][i].w = fmaf(w[jj], value[jj].w, acc[v][i].w);
            }
          }
        }
      }
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (q_pos[i] < 0) continue;
    const float inverse = run_sum[i] > 0.f ? 1.f / run_sum[i] : 0.f;
    float* row = out + (int64_t)(tok0 + q0 + 4 * ty + i) * out_stride + (int64_t)head * head_dim;
#pragma unroll
    for (int v = 0; v < DV; ++v) {
      const int f = tx + 16 * v;
      if (f < d4)
        *reinterpret_cast<float4*>(row + 4 * f) =
            make_float4(acc[v][i].x * inverse, acc[v][i].y * inverse, acc[v][i].z * inverse,
                        acc[v][i].w * inverse);
    }
  }
}

extern "C" int ps_attention_tiled_f32_supported(int head_dim) {
  return head_dim >= 4 && head_dim <= AF_MAX_DIM && head_dim % 4 == 0;
}

extern "C" int ps_attention_tiled_f32_tile() { return AF_TILE; }

extern "C" int ps_attention_tiled_f32(const void* q, int64_t q_stride, const void* k_pool,
                                      const void* v_pool, void* out, int64_t out_stride,
                                      const int* tile_item, const int* tile_q0, int tiles,
                                      const int* cu_tokens, const int* kv_lens, const int* tables,
                                      int table_width, int heads, int kv_heads, int head_dim,
                                      int page_size, int num_pages, float scale, int window,
                                      void* stream) {
  PS_REQUIRE(tiles >= 0 && heads > 0 && kv_heads > 0 && page_size > 0 && num_pages > 0 &&
                 table_width > 0,
             "ps_attention_tiled_f32: bad sizes");
  PS_REQUIRE(ps_attention_tiled_f32_supported(head_dim),
             "ps_attention_tiled_f32: head_dim %d must be a multiple of 4 up to %d "
             "(ps_attention_rowwise takes every size)", head_dim, AF_MAX_DIM);
  PS_REQUIRE(heads % kv_heads == 0,
             "ps_attention_tiled_f32: heads (%d) must be a multiple of kv_heads (%d)", heads, kv_heads);
  PS_REQUIRE(window >= 0 && scale > 0.f, "ps_attention_tiled_f32: bad window or scale");
  PS_REQUIRE((q_stride % 4) == 0 && (out_stride % 4) == 0 && ((uintptr_t)q % 16) == 0 &&
                 ((uintptr_t)out % 16) == 0 && ((uintptr_t)k_pool % 16) == 0 &&
                 ((uintptr_t)v_pool % 16) == 0,
             "ps_attention_tiled_f32: rows of q, out and the pools must allow 16-byte accesses");
  const int64_t blocks = (int64_t)tiles * heads;
  PS_REQUIRE(blocks < ((int64_t)1 << 31), "ps_attention_tiled_f32: too many blocks");
  if (blocks == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
#define PS_LAUNCH_AF(DV)                                                                          \
  hipLaunchKernelGGL(attention_tiled_f32_kernel<DV>, dim3((unsigned)blocks), dim3(256), 0, s,     \
                     (const float*)q, q_stride, (const float*)k_pool, (const float*)v_pool,       \
                     (float*)out, out_stride, tile_item, tile_q0, cu_tokens, kv_lens, tables,     \
                     table_width, heads, kv_heads, head_dim, page_size, num_pages, scale, window)
  if (head_dim <= 64) {
    PS_LAUNCH_AF(1);
  } else {
    PS_LAUNCH_AF(2);
  }
#undef PS_LAUNCH_AF
  PS_CHECK_LAUNCH("ps_attention_tiled_f32");
  return 0;
}
