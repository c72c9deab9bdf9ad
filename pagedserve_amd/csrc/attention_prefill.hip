// Tiled paged attention for prompt portions on the matrix cores (bfloat16).
//
// One 256-thread block per (tile of 64 queries of one request, head); each of the four waves
// owns 16 consecutive queries.  Keys and values are visited 64 at a time through the request's
// block table, from the first key any query of the tile may see to the tile's last position
// (the portion's own keys are already in the pages, so a whole prompt, a later portion and a
// portion that starts in the middle of a page are one case).  Per key tile:
//
//   * all threads copy the K tile [64 keys][head_dim] into LDS as it lies in the pages, and
//     the V tile transposed to [head_dim][64 keys], so that both products find their reduction
//     dimension contiguous;
//   * S^T = K Q^T with v_mfma_f32_16x16x32_bf16: keys are the rows, queries the columns, so a
//     lane ends up with 4 keys x its own query per 16-key block — the same (query, key-group)
//     ownership that the second product needs for its column operand;
//   * scale, causal/window mask, online softmax in float per query (running max and sum, as
//     src/kernels/triton_paged_attention.py:275-331), probabilities rounded to bfloat16;
//   * O^T += V^T P^T with the same instruction: head dimensions are the rows, queries the
//     columns, 32 keys per instruction.
//
// head_dim is any multiple of 16 up to 128 (odd multiples are zero-padded to 32 for the first
// product); other sizes run on the row-wise kernel.
#include <math.h>

#include "common.h"
#include "pagedserve_hip.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

#define AP_KEYS 64      // keys per tile
#define AP_QUERIES 64   // queries per block
#define AP_V_STRIDE (AP_KEYS * 2 + 16)

__device__ inline uint32_t pack_bf16(float lo, float hi) { return pack2_bf16(lo, hi); }

template <int NDB>  // head_dim / 16
__global__ __launch_bounds__(256) void attention_prefill_kernel(
    const bf16_t* __restrict__ q, int64_t q_stride, const bf16_t* __restrict__ k_pool,
    const bf16_t* __restrict__ v_pool, bf16_t* __restrict__ out, int64_t out_stride,
    const int* __restrict__ tile_item, const int* __restrict__ tile_q0,
    const int* __restrict__ cu_tokens, const int* __restrict__ kv_lens,
    const int* __restrict__ tables, int table_width, int heads, int kv_heads, int page_size,
    int page_shift, int num_pages, float scale, int window) {
  constexpr int HD = NDB * 16;
  constexpr int NDQ = (NDB + 1) / 2;   // 32-wide steps over the head dimension
  constexpr int HDP = NDQ * 32;
  constexpr int K_STRIDE = HDP * 2 + 16;
  __shared__ __attribute__((aligned(16))) unsigned char k_lds[AP_KEYS * K_STRIDE];
  __shared__ __attribute__((aligned(16))) unsigned char v_lds[HD * AP_V_STRIDE];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int sub = lane & 15;     // query of this lane within the wave
  const int group = lane >> 4;   // which quarter of a reduction dimension
  const int head = blockIdx.y;
  const int kv_head = head / (heads / kv_heads);

  // later tiles of a request see more keys: start them first
  const int tile_index = gridDim.x - 1 - blockIdx.x;
  const int item = tile_item[tile_index];
  const int q0 = tile_q0[tile_index];
  const int tok0 = cu_tokens[item];
  const int count = cu_tokens[item + 1] - tok0;
  const int start = kv_lens[item] - count;   // position of the portion's first token
  const int* table = tables + (int64_t)item * table_width;

  const int qi = q0 + wave * 16 + sub;
  const bool q_valid = qi < count;
  const int q_pos = q_valid ? start + qi : -1;
  const int wave_first = start + q0 + wave * 16;
  const int wave_last_q = q0 + wave * 16 + 15 < count ? q0 + wave * 16 + 15 : count - 1;
  const int wave_last = start + wave_last_q;
  const bool wave_active = q0 + wave * 16 < count;
  const int tile_last_q = q0 + AP_QUERIES - 1 < count ? q0 + AP_QUERIES - 1 : count - 1;
  const int key_end = start + tile_last_q + 1;
  int key_begin = 0;
  if (window > 0 && start + q0 - window + 1 > 0) key_begin = start + q0 - window + 1;

  // zero the padding columns of the K tile once (odd NDB)
  if (HDP > HD) {
    for (int i = tid; i < AP_KEYS * (HDP - HD) / 8; i += 256) {
      const int key = i / ((HDP - HD) / 8);
      const int chunk = i % ((HDP - HD) / 8);
      *reinterpret_cast<uint4*>(&k_lds[key * K_STRIDE + (HD + chunk * 8) * 2]) = uint4{0u, 0u, 0u, 0u};
    }
  }

  // queries as column operand of the first product: lane (query sub, dims dq*32 + group*8 ..)
  uint4 qf[NDQ];
#pragma unroll
  for (int dq = 0; dq < NDQ; ++dq) {
    const int d = dq * 32 + group * 8;
    qf[dq] = (q_valid && d < HD)
                 ? *reinterpret_cast<const uint4*>(q + (int64_t)(tok0 + qi) * q_stride +
                                                   (int64_t)head * HD + d)
                 : uint4{0u, 0u, 0u, 0u};
  }

  // Scores are kept in units of log 2 (scale * log2(e) folded into one factor), so that
  // every exponential is one v_exp_f32; probabilities are rounded to bfloat16 right after.
  const float scale_log2 = scale * 1.4426950408889634f;
  float m = -INFINITY, l = 0.f;
  f32x4 acc[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db) acc[db] = f32x4{0.f, 0.f, 0.f, 0.f};

  // Each thread moves CHUNKS 16-byte pieces of a K tile and of a V tile; the next tile's
  // pieces are loaded into registers while the current tile is being multiplied.
  constexpr int CHUNKS = (AP_KEYS * NDB * 2 + 255) / 256;
  uint4 k_next[CHUNKS], v_next[CHUNKS];
  int page_next[CHUNKS];
  // The address of a key needs its page, which is a load of its own: pages are fetched one
  // tile further ahead than keys, so neither trip to memory is waited for.
  auto fetch_pages = [&](int k0) {
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) {
      const int c = tid + i * 256;
      const int key_local = c % AP_KEYS;
      const int key = k0 + key_local;
      const int safe_key = key < key_end ? key : key_end - 1;
      const int logical = page_shift >= 0 ? (safe_key >> page_shift) : safe_key / page_size;
      page_next[i] = logical < table_width ? table[logical] : -1;
    }
  };
  auto fetch_tile = [&](int k0) {
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) {
      // piece c = (8 head dimensions dc, key c % 64): the lanes of a wave hold 64 consecutive
      // keys of the same dimensions, so the transposed V stores below do not collide in LDS
      const int c = tid + i * 256;
      const int dc = c / AP_KEYS;
      const int key_local = c - dc * AP_KEYS;
      const int key = k0 + key_local;
      // unconditional loads from clamped addresses, zeroed afterwards
      const int safe_key = key < key_end ? key : key_end - 1;
      const int logical = page_shift >= 0 ? (safe_key >> page_shift) : safe_key / page_size;
      const int page = page_next[i];
      const bool ok = key < key_end && dc < NDB * 2 && page >= 0 && page < num_pages;
      const int64_t offset =
          (((int64_t)(ok ? page : 0) * kv_heads + kv_head) * page_size +
           (safe_key - logical * page_size)) * HD + (dc < NDB * 2 ? dc : 0) * 8;
      k_next[i] = *reinterpret_cast<const uint4*>(k_pool + offset);
      v_next[i] = *reinterpret_cast<const uint4*>(v_pool + offset);
      if (!ok) {
        k_next[i] = uint4{0u, 0u, 0u, 0u};
        v_next[i] = uint4{0u, 0u, 0u, 0u};
      }
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) {
      const int c = tid + i * 256;
      const int dc = c / AP_KEYS;
      const int key_local = c - dc * AP_KEYS;
      if (dc >= NDB * 2) continue;
      *reinterpret_cast<uint4*>(&k_lds[key_local * K_STRIDE + dc * 16]) = k_next[i];
      const uint32_t words[4] = {v_next[i].x, v_next[i].y, v_next[i].z, v_next[i].w};
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint16_t value = (uint16_t)(words[j >> 1] >> ((j & 1) * 16));
        *reinterpret_cast<uint16_t*>(&v_lds[(dc * 8 + j) * AP_V_STRIDE + key_local * 2]) = value;
      }
    }
  };

  const int k_first = key_begin / AP_KEYS * AP_KEYS;
  fetch_pages(k_first);
  fetch_tile(k_first);
  if (k_first + AP_KEYS < key_end) fetch_pages(k_first + AP_KEYS);
  for (int k0 = k_first; k0 < key_end; k0 += AP_KEYS) {
    __syncthreads();   // the previous tile has been consumed
    store_tile();
    __syncthreads();
    if (k0 + AP_KEYS < key_end) {
      fetch_tile(k0 + AP_KEYS);   // in flight during the products
      if (k0 + 2 * AP_KEYS < key_end) fetch_pages(k0 + 2 * AP_KEYS);
    }
    // skip tiles that no query of this wave can see
    if (!wave_active || k0 > wave_last) continue;
    if (window > 0 && k0 + AP_KEYS - 1 < wave_first - window + 1) continue;

    // S^T: 4 blocks of 16 keys; lane holds keys kb*16 + group*4 + i of its own query
    float s[4][4];
    float tile_max = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      f32x4 sacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int dq = 0; dq < NDQ; ++dq) {
        const uint4 kf = *reinterpret_cast<const uint4*>(
            &k_lds[(kb * 16 + sub) * K_STRIDE + (dq * 32 + group * 8) * 2]);
        sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(&kf),
                                                       *reinterpret_cast<const bf16x8*>(&qf[dq]),
                                                       sacc, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = k0 + kb * 16 + group * 4 + i;
        const bool visible = key <= q_pos && (window <= 0 || q_pos - key < window);
        s[kb][i] = visible ? sacc[i] * scale_log2 : -INFINITY;
        tile_max = fmaxf(tile_max, s[kb][i]);
      }
    }
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, 64));
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, 64));
    const float m_new = fmaxf(m, tile_max);
    if (m_new == -INFINITY) {
      // nothing visible to this query so far; other lanes of the wave may differ, so the
      // products below still run with zero probabilities
    }
    const float correction =
        (m == -INFINITY || m_new == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m - m_new);
    float tile_sum = 0.f;
    uint32_t pw[4][2];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      float p[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        p[i] = (s[kb][i] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(s[kb][i] - m_new);
        tile_sum += p[i];
      }
      pw[kb][0] = pack_bf16(p[0], p[1]);
      pw[kb][1] = pack_bf16(p[2], p[3]);
    }
    tile_sum += __shfl_xor(tile_sum, 16, 64);
    tile_sum += __shfl_xor(tile_sum, 32, 64);
    l = l * correction + tile_sum;
    m = m_new;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[db][i] *= correction;

    // O^T += V^T P^T, 32 keys per instruction: keys {kp*32 + group*4 + i} and
    // {kp*32 + 16 + group*4 + i}, the same eight for both operands
#pragma unroll
    for (int kp = 0; kp < 2; ++kp) {
      const uint4 pf = {pw[2 * kp][0], pw[2 * kp][1], pw[2 * kp + 1][0], pw[2 * kp + 1][1]};
#pragma unroll
      for (int db = 0; db < NDB; ++db) {
        const unsigned char* v_row = &v_lds[(db * 16 + sub) * AP_V_STRIDE];
        const uint2 lo = *reinterpret_cast<const uint2*>(v_row + (kp * 32 + group * 4) * 2);
        const uint2 hi = *reinterpret_cast<const uint2*>(v_row + (kp * 32 + 16 + group * 4) * 2);
        const uint4 vf = {lo.x, lo.y, hi.x, hi.y};
        acc[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(&vf),
                                                         *reinterpret_cast<const bf16x8*>(&pf),
                                                         acc[db], 0, 0, 0);
      }
    }
  }

  // element i of an accumulator: head dimension db*16 + group*4 + i of query `sub`
  if (q_valid && l > 0.f) {
    const float inv = 1.0f / l;
    bf16_t* dst = out + (int64_t)(tok0 + qi) * out_stride + (int64_t)head * HD;
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
      uint2 packed;
      packed.x = pack_bf16(acc[db][0] * inv, acc[db][1] * inv);
      packed.y = pack_bf16(acc[db][2] * inv, acc[db][3] * inv);
      *reinterpret_cast<uint2*>(dst + db * 16 + group * 4) = packed;
    }
  }
}

extern "C" int ps_attention_prefill(const void* q, int64_t q_stride, const void* k_pool,
                                    const void* v_pool, void* out, int64_t out_stride,
                                    const int* tile_item, const int* tile_q0, int tiles,
                                    const int* cu_tokens, const int* kv_lens, const int* tables,
                                    int table_width, int heads, int kv_heads, int head_dim,
                                    int page_size, int num_pages, float scale, int window,
                                    int dtype, void* stream) {
  PS_REQUIRE(tiles >= 0 && heads > 0 && kv_heads > 0 && page_size > 0 && num_pages > 0 &&
                 table_width > 0,
             "ps_attention_prefill: bad sizes");
  PS_REQUIRE(dtype == PS_BF16, "ps_attention_prefill: bfloat16 only (dtype %d)", dtype);
  PS_REQUIRE(heads % kv_heads == 0,
             "ps_attention_prefill: heads (%d) must be a multiple of kv_heads (%d)", heads, kv_heads);
  PS_REQUIRE(head_dim > 0 && head_dim % 16 == 0 && head_dim <= 128,
             "ps_attention_prefill: head_dim %d must be a multiple of 16 up to 128", head_dim);
  PS_REQUIRE(window >= 0 && heads <= 65535, "ps_attention_prefill: bad window or head count");
  PS_REQUIRE((q_stride % 8) == 0 && ((uintptr_t)q % 16) == 0 && (out_stride % 4) == 0 &&
                 ((uintptr_t)out % 8) == 0,
             "ps_attention_prefill: q and out rows must allow 16- and 8-byte accesses");
  if (tiles == 0) return 0;
  int page_shift = -1;
  if ((page_size & (page_size - 1)) == 0) {
    page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
  }
  hipStream_t s = (hipStream_t)stream;
  dim3 grid(tiles, heads);
#define PS_LAUNCH_AP(NDB)                                                                       \
  hipLaunchKernelGGL((attention_prefill_kernel<NDB>), grid, dim3(256), 0, s, (const bf16_t*)q,  \
                     q_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool, (bf16_t*)out,      \
                     out_stride, tile_item, tile_q0, cu_tokens, kv_lens, tables, table_width,   \
                     heads, kv_heads, page_size, page_shift, num_pages, scale, window)
  switch (head_dim / 16) {
    case 1: PS_LAUNCH_AP(1); break;
    case 2: PS_LAUNCH_AP(2); break;
    case 3: PS_LAUNCH_AP(3); break;
    case 4: PS_LAUNCH_AP(4); break;
    case 5: PS_LAUNCH_AP(5); break;
    case 6: PS_LAUNCH_AP(6); break;
    case 7: PS_LAUNCH_AP(7); break;
    default: PS_LAUNCH_AP(8); break;
  }
#undef PS_LAUNCH_AP
  PS_CHECK_LAUNCH("ps_attention_prefill");
  return 0;
}
