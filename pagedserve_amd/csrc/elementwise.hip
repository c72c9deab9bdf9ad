// Embedding(+position table) add, LayerNorm / RMS norm with row gather, and the scatter of
// new keys and values into cache pages.  All arithmetic is float; storage may be bfloat16.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "common.h"
#include "linear.h"
#include "pagedserve_hip.h"

// ---------------------------------------------------------------- error channel
static thread_local char g_error[512] = "";

void ps_set_error(const char* fmt, ...) {
  va_list args;
  va_start(args, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, args);
  va_end(args);
}

extern "C" const char* ps_last_error(void) { return g_error; }

extern "C" int ps_device_info(int* compute_units, int* lds_bytes, char* arch, int arch_len) {
  int device = 0;
  hipError_t status = hipGetDevice(&device);
  PS_REQUIRE(status == hipSuccess, "ps_device_info: %s", hipGetErrorString(status));
  hipDeviceProp_t prop;
  status = hipGetDeviceProperties(&prop, device);
  PS_REQUIRE(status == hipSuccess, "ps_device_info: %s", hipGetErrorString(status));
  if (compute_units) *compute_units = prop.multiProcessorCount;
  if (lds_bytes) *lds_bytes = (int)prop.sharedMemPerBlock;
  if (arch && arch_len > 0) {
    strncpy(arch, prop.gcnArchName, arch_len - 1);
    arch[arch_len - 1] = 0;
  }
  return 0;
}

// Compute units of the current device, asked once per device: launch shapes follow it.
int ps_compute_units() {
  static int cached[64];
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 256;
  if (cached[device] == 0) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) != hipSuccess || prop.multiProcessorCount <= 0) return 256;
    cached[device] = prop.multiProcessorCount;
  }
  return cached[device];
}

// ---------------------------------------------------------------- embedding
// h0[t] = scale * wte[id[t]] + wpe[pos[t]]  (reference: src/model/paged_decoder.py:306-314,
// where the scale is 1).
// The id of token t is ids[t], or carried[src[t]] where src[t] >= 0: a token that an earlier
// step chose on the device and that the host has not seen yet.
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const T* __restrict__ pos_table,
                             const int* __restrict__ ids, const int* __restrict__ src,
                             const int* __restrict__ carried, const int* __restrict__ positions,
                             float* __restrict__ out, int width, int vocab, float scale) {
  const int t = blockIdx.x;
  int id = ids[t];
  if (src != nullptr) {
    const int from = src[t];
    if (from >= 0) id = carried[from];
  }
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);   // never a read outside the table
  const T* row = table + (int64_t)id * width;
  float* dst = out + (int64_t)t * width;
  if (pos_table != nullptr) {
    const T* prow = pos_table + (int64_t)positions[t] * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x)
      dst[i] = to_float<T>(row[i]) * scale + to_float<T>(prow[i]);
  } else {
    for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = to_float<T>(row[i]) * scale;
  }
}

extern "C" int ps_embed(const void* table, const void* pos_table, const int* ids, const int* src,
                        const int* carried, const int* positions, float* out, int tokens,
                        int width, int vocab, int max_positions, float scale, int dtype,
                        void* stream) {
  PS_REQUIRE(tokens >= 0 && width > 0 && vocab > 0, "ps_embed: bad sizes (tokens %d, width %d)",
             tokens, width);
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_embed: unknown dtype %d", dtype);
  PS_REQUIRE(pos_table == nullptr || max_positions > 0, "ps_embed: position table without rows");
  PS_REQUIRE(src == nullptr || carried != nullptr, "ps_embed: carried tokens are missing");
  if (tokens == 0) return 0;
  const int threads = width >= 256 ? 256 : 64;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PS_F32)
    hipLaunchKernelGGL(embed_kernel<float>, dim3(tokens), dim3(threads), 0, s, (const float*)table,
                       (const float*)pos_table, ids, src, carried, positions, out, width, vocab,
                       scale);
  else
    hipLaunchKernelGGL(embed_kernel<bf16_t>, dim3(tokens), dim3(threads), 0, s,
                       (const bf16_t*)table, (const bf16_t*)pos_table, ids, src, carried,
                       positions, out, width, vocab, scale);
  PS_CHECK_LAUNCH("ps_embed");
  return 0;
}

// ---------------------------------------------------------------- norms
// mean, centred values, biased variance of the centred values, rsqrt(var + eps), scale and
// shift (reference: src/kernels/triton_residual_layernorm.py:25-39).
//
// norm_wave_kernel: one wave per row, the row held in registers (width <= 64 * VPT): one
// trip to memory, reductions by shuffles, no barrier.  norm_block_kernel: one block per row,
// the row read three times (it stays in cache), any width.
template <typename T, bool RMS, int VPT>
__global__ __launch_bounds__(256) void norm_wave_kernel(
    const float* __restrict__ x, const int* __restrict__ rows, const float* __restrict__ gamma,
    const float* __restrict__ beta, T* __restrict__ out, int n_rows, int width, float eps,
    int packed) {
  const int lane = threadIdx.x & 63;
  const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= n_rows) return;
  const float* src = x + (int64_t)(rows ? rows[r] : r) * width;
  // Loads are unconditional (index clamped, value selected afterwards): a load under a
  // branch would wait for the one before it, and the row would cost VPT trips to memory.
  float v[VPT], g[VPT], b[VPT];
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int col = lane + i * 64;
    const int safe = col < width ? col : width - 1;
    v[i] = src[safe];
    g[i] = gamma[safe];
    b[i] = (!RMS && beta != nullptr) ? beta[safe] : 0.f;
  }
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    if (lane + i * 64 >= width) v[i] = 0.f;
    sum += v[i];
  }
  float mean = 0.f;
  if (!RMS) mean = wave_sum(sum) / (float)width;
  float sq = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int col = lane + i * 64;
    const float c = col < width ? v[i] - mean : 0.f;
    v[i] = c;
    sq += c * c;
  }
  const float inv_std = 1.0f / sqrtf(wave_sum(sq) / (float)width + eps);
  T* dst = out + (int64_t)r * width;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int col = lane + i * 64;
    if (col >= width) continue;
    const T y = from_float<T>(v[i] * inv_std * g[i] + b[i]);
    if (packed) out[packed_offset(r, col, width)] = y;
    else dst[col] = y;
  }
}

// norm_row_kernel: one block of four waves per row, the row held in registers (width <= 256 *
// VPT), the two sums met through LDS.  For few wide rows (a decode step of a wide model): a
// wave alone would hold 25 values per lane at 1,600 columns and ask for them one after the
// other, four waves ask for 7 each.
template <typename T, bool RMS, int VPT>
__global__ __launch_bounds__(256) void norm_row_kernel(
    const float* __restrict__ x, const int* __restrict__ rows, const float* __restrict__ gamma,
    const float* __restrict__ beta, T* __restrict__ out, int width, float eps, int packed) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const float* src = x + (int64_t)(rows ? rows[r] : r) * width;
  float v[VPT], g[VPT], b[VPT];
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int col = threadIdx.x + i * 256;
    const int safe = col < width ? col : width - 1;
    v[i] = src[safe];
    g[i] = gamma[safe];
    b[i] = (!RMS && beta != nullptr) ? beta[safe] : 0.f;
  }
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    if ((int)threadIdx.x + i * 256 >= width) v[i] = 0.f;
    sum += v[i];
  }
  float mean = 0.f;
  if (!RMS) mean = block_sum(sum, scratch) / (float)width;
  float sq = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int col = threadIdx.x + i * 256;
    const float c = col < width ? v[i] - mean : 0.f;
    v[i] = c;
    sq += c * c;
  }
  const float inv_std = 1.0f / sqrtf(block_sum(sq, scratch) / (float)width + eps);
  T* dst = out + (int64_t)r * width;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int col = threadIdx.x + i * 256;
    if (col >= width) continue;
    const T y = from_float<T>(v[i] * inv_std * g[i] + b[i]);
    if (packed) out[packed_offset(r, col, width)] = y;
    else dst[col] = y;
  }
}

template <typename T, bool RMS>
__global__ void norm_block_kernel(const float* __restrict__ x, const int* __restrict__ rows,
                                  const float* __restrict__ gamma, const float* __restrict__ beta,
                                  T* __restrict__ out, int width, float eps) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const float* src = x + (int64_t)(rows ? rows[r] : r) * width;
  T* dst = out + (int64_t)r * width;
  float mean = 0.f;
  if (!RMS) {
    float partial = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) partial += src[i];
    mean = block_sum(partial, scratch) / (float)width;
  }
  float partial = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float c = src[i] - mean;
    partial += c * c;
  }
  const float variance = block_sum(partial, scratch) / (float)width;
  const float inv_std = 1.0f / sqrtf(variance + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = (src[i] - mean) * inv_std * gamma[i];
    if (!RMS && beta != nullptr) v += beta[i];
    dst[i] = from_float<T>(v);
  }
}

template <typename T, bool RMS>
static void launch_norm(const float* x, const int* rows, const float* gamma, const float* beta,
                        void* out, int n_rows, int width, float eps, int packed, hipStream_t s) {
  const int per_lane = (width + 63) / 64;
  const dim3 grid((n_rows + 3) / 4);
  if (n_rows <= 64 && per_lane > 12 && per_lane <= 32) {
    // few wide rows: a block of four waves per row
#define PS_LAUNCH_NR(VPT)                                                                          \
  hipLaunchKernelGGL((norm_row_kernel<T, RMS, VPT>), dim3(n_rows), dim3(256), 0, s, x, rows, gamma, \
                     beta, (T*)out, width, eps, packed)
    if (per_lane <= 16) PS_LAUNCH_NR(4);
    else PS_LAUNCH_NR(8);
#undef PS_LAUNCH_NR
    return;
  }
#define PS_LAUNCH_NW(VPT)                                                                       \
  hipLaunchKernelGGL((norm_wave_kernel<T, RMS, VPT>), grid, dim3(256), 0, s, x, rows, gamma, beta, \
                     (T*)out, n_rows, width, eps, packed)
  if (per_lane <= 2) PS_LAUNCH_NW(2);
  else if (per_lane <= 4) PS_LAUNCH_NW(4);
  else if (per_lane <= 8) PS_LAUNCH_NW(8);
  else if (per_lane <= 12) PS_LAUNCH_NW(12);
  else if (per_lane <= 16) PS_LAUNCH_NW(16);
  else if (per_lane <= 32) PS_LAUNCH_NW(32);
  else
    hipLaunchKernelGGL((norm_block_kernel<T, RMS>), dim3(n_rows), dim3(256), 0, s, x, rows, gamma,
                       beta, (T*)out, width, eps);
#undef PS_LAUNCH_NW
}

// The norm with its rows written row by row (packed == 0) or in the operand order of the
// skinny product (packed_offset in linear.h; needs width a multiple of 64 up to 2048 and room
// for the row count rounded up to 16).
int ps_norm_layout(const float* x, const int* rows, const float* gamma, const float* beta,
                   void* out, int n_rows, int width, float eps, int rms, int out_dtype,
                   int packed, hipStream_t s) {
  PS_REQUIRE(n_rows >= 0 && width > 0, "ps_norm: bad sizes (rows %d, width %d)", n_rows, width);
  PS_REQUIRE(out_dtype == PS_F32 || out_dtype == PS_BF16, "ps_norm: unknown dtype %d", out_dtype);
  PS_REQUIRE(eps > 0.f, "ps_norm: eps must be positive");
  PS_REQUIRE(!packed || (width % 64 == 0 && width <= 2048),
             "ps_norm: the packed layout needs a width that is a multiple of 64 up to 2048");
  if (n_rows == 0) return 0;
  if (out_dtype == PS_F32) {
    if (rms) launch_norm<float, true>(x, rows, gamma, beta, out, n_rows, width, eps, packed, s);
    else launch_norm<float, false>(x, rows, gamma, beta, out, n_rows, width, eps, packed, s);
  } else {
    if (rms) launch_norm<bf16_t, true>(x, rows, gamma, beta, out, n_rows, width, eps, packed, s);
    else launch_norm<bf16_t, false>(x, rows, gamma, beta, out, n_rows, width, eps, packed, s);
  }
  PS_CHECK_LAUNCH("ps_norm");
  return 0;
}

extern "C" int ps_norm(const float* x, const int* rows, const float* gamma, const float* beta,
                       void* out, int n_rows, int width, float eps, int rms, int out_dtype,
                       void* stream) {
  return ps_norm_layout(x, rows, gamma, beta, out, n_rows, width, eps, rms, out_dtype, 0,
                        (hipStream_t)stream);
}

// ---------------------------------------------------------------- key/value scatter
// Token t of request r at position p is stored at (page = table[r][p / page], offset =
// p % page) (reference: src/model/kv_manager.py:303-308,403-404).
template <typename T>
__global__ void kv_write_kernel(const T* __restrict__ k, const T* __restrict__ v, int64_t stride,
                                T* __restrict__ k_pool, T* __restrict__ v_pool,
                                const int* __restrict__ tok_item, const int* __restrict__ tok_pos,
                                const int* __restrict__ tables, int table_width, int kv_heads,
                                int head_dim, int page_size, int num_pages) {
  const int t = blockIdx.x;
  const int pos = tok_pos[t];
  const int logical = pos / page_size;
  if (logical >= table_width) return;
  const int page = tables[(int64_t)tok_item[t] * table_width + logical];
  if (page < 0 || page >= num_pages) return;
  const int offset = pos - logical * page_size;
  const int row = kv_heads * head_dim;
  for (int i = threadIdx.x; i < row; i += blockDim.x) {
    const int head = i / head_dim;
    const int dim = i - head * head_dim;
    const int64_t dst = (((int64_t)page * kv_heads + head) * page_size + offset) * head_dim + dim;
    k_pool[dst] = k[(int64_t)t * stride + i];
    v_pool[dst] = v[(int64_t)t * stride + i];
  }
}

extern "C" int ps_kv_write(const void* k, const void* v, int64_t stride, void* k_pool,
                           void* v_pool, const int* tok_item, const int* tok_pos,
                           const int* tables, int table_width, int tokens, int kv_heads,
                           int head_dim, int page_size, int num_pages, int dtype, void* stream) {
  PS_REQUIRE(tokens >= 0 && kv_heads > 0 && head_dim > 0 && page_size > 0 && num_pages > 0 &&
                 table_width > 0,
             "ps_kv_write: bad sizes");
  PS_REQUIRE(stride >= (int64_t)kv_heads * head_dim, "ps_kv_write: row stride too small");
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_kv_write: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  const int row = kv_heads * head_dim;
  const int threads = row >= 256 ? 256 : 64;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PS_F32)
    hipLaunchKernelGGL(kv_write_kernel<float>, dim3(tokens), dim3(threads), 0, s, (const float*)k,
                       (const float*)v, stride, (float*)k_pool, (float*)v_pool, tok_item, tok_pos,
                       tables, table_width, kv_heads, head_dim, page_size, num_pages);
  else
    hipLaunchKernelGGL(kv_write_kernel<bf16_t>, dim3(tokens), dim3(threads), 0, s,
                       (const bf16_t*)k, (const bf16_t*)v, stride, (bf16_t*)k_pool,
                       (bf16_t*)v_pool, tok_item, tok_pos, tables, table_width, kv_heads, head_dim,
                       page_size, num_pages);
  PS_CHECK_LAUNCH("ps_kv_write");
  return 0;
}
