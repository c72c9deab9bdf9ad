// Token selection from float logits: argmax (ties to the lowest id, as torch.argmax on
// the reference's path, src/scheduler/orca_scheduler.py:250) or a draw from
// softmax(logits / temperature) by inverse CDF.  The uniform number of a row is made by the
// host from (seed, request, step), so a draw does not depend on what else is in the batch.
//
// One 1024-thread block per row.  The maximum is found with coalesced strided reads, sixteen
// of them in flight per thread.  For a
// draw, wave w owns the contiguous id range [w * seg, (w + 1) * seg): it sums
// exp((l - max) / T) over its range 64 ids at a time, thread 0 picks the range that holds
// uniform * total, and that wave walks its range again with a prefix sum over each 64 ids to
// find the first id whose cumulative mass exceeds the goal.
#include <math.h>

#include "common.h"
#include "pagedserve_hip.h"

#define SM_THREADS 1024
#define SM_WAVES (SM_THREADS / 64)
#define SM_LOADS 16   // a row of 16,384 logits is one trip to memory for the maximum

__global__ __launch_bounds__(SM_THREADS) void sample_kernel(
    const float* __restrict__ logits, int64_t ld, const float* __restrict__ inv_temperature,
    const float* __restrict__ uniform, int* __restrict__ tokens, int vocab) {
  __shared__ float s_val[SM_WAVES];
  __shared__ int s_idx[SM_WAVES];
  __shared__ float s_sum[SM_WAVES];
  __shared__ int s_choice;
  __shared__ float s_before;
  __shared__ float s_goal;

  const int r = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const float* row = logits + (int64_t)r * ld;

  // maximum and its first index
  float best = -INFINITY;
  int best_idx = vocab;
  for (int i0 = tid; i0 < vocab; i0 += SM_LOADS * SM_THREADS) {
    float v[SM_LOADS];
#pragma unroll
    for (int u = 0; u < SM_LOADS; ++u) {   // all loads in flight, index clamped, masked below
      const int i = i0 + u * SM_THREADS;
      v[u] = row[i < vocab ? i : vocab - 1];
    }
#pragma unroll
    for (int u = 0; u < SM_LOADS; ++u) {
      const int i = i0 + u * SM_THREADS;
      if (i < vocab && v[u] > best) {
        best = v[u];
        best_idx = i;
      }
    }
  }
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) {
    const float other = __shfl_xor(best, offset, 64);
    const int other_idx = __shfl_xor(best_idx, offset, 64);
    if (other > best || (other == best && other_idx < best_idx)) {
      best = other;
      best_idx = other_idx;
    }
  }
  if (lane == 0) {
    s_val[wave] = best;
    s_idx[wave] = best_idx;
  }
  __syncthreads();
  float row_max = s_val[0];
  int row_argmax = s_idx[0];
#pragma unroll
  for (int w = 1; w < SM_WAVES; ++w) {
    if (s_val[w] > row_max || (s_val[w] == row_max && s_idx[w] < row_argmax)) {
      row_max = s_val[w];
      row_argmax = s_idx[w];
    }
  }
  if (row_argmax >= vocab) row_argmax = 0;
  const float inv_t = inv_temperature ? inv_temperature[r] : 0.f;
  if (inv_t <= 0.f) {
    if (tid == 0) tokens[r] = row_argmax;
    return;
  }

  // unnormalised probabilities exp((l - max) / T), summed per wave range
  const int seg = ((vocab + SM_WAVES - 1) / SM_WAVES + 63) / 64 * 64;
  const int begin = wave * seg;
  const int end = begin + seg < vocab ? begin + seg : vocab;
  float partial = 0.f;
  for (int i = begin + lane; i < end; i += 64) partial += expf((row[i] - row_max) * inv_t);
  partial = wave_sum(partial);
  if (lane == 0) s_sum[wave] = partial;
  __syncthreads();
  if (tid == 0) {
    float total = 0.f;
    for (int w = 0; w < SM_WAVES; ++w) total += s_sum[w];
    const float goal = uniform[r] * total;
    float before = 0.f;
    int choice = -1;
    for (int w = 0; w < SM_WAVES; ++w) {
      if (s_sum[w] > 0.f && before + s_sum[w] > goal) {
        choice = w;
        break;
      }
      before += s_sum[w];
    }
    if (choice < 0) {
      // rounding left the goal at or beyond the total: the last non-empty range takes it
      choice = SM_WAVES - 1;
      while (choice > 0 && s_sum[choice] <= 0.f) --choice;
      before = 0.f;
      for (int w = 0; w < choice; ++w) before += s_sum[w];
    }
    s_choice = choice;
    s_before = before;
    s_goal = goal;
  }
  __syncthreads();
  if (wave != s_choice) return;
  float running = s_before;
  const float goal = s_goal;
  int token = -1;
  int last_positive = -1;
  for (int base = begin; base < end && token < 0; base += 64) {
    const int i = base + lane;
    const float e = i < end ? expf((row[i] - row_max) * inv_t) : 0.f;
    float prefix = e;  // inclusive prefix sum over the wave
#pragma unroll
    for (int offset = 1; offset < 64; offset <<= 1) {
      const float other = __shfl_up(prefix, offset, 64);
      if (lane >= offset) prefix += other;
    }
    const unsigned long long hits = __ballot(i < end && e > 0.f && running + prefix > goal);
    const unsigned long long positive = __ballot(i < end && e > 0.f);
    if (positive) last_positive = base + 63 - __clzll(positive);
    if (hits) token = base + __ffsll((long long)hits) - 1;
    running += __shfl(prefix, 63, 64);
  }
  if (token < 0) token = last_positive >= 0 ? last_positive : row_argmax;
  if (lane == 0) tokens[r] = token;
}

extern "C" int ps_sample(const float* logits, int64_t ld, const float* inv_temperature,
                         const float* uniform, int* tokens, int rows, int vocab, void* stream) {
  PS_REQUIRE(rows >= 0 && vocab > 0 && ld >= vocab, "ps_sample: bad sizes (rows %d, vocab %d)",
             rows, vocab);
  PS_REQUIRE(inv_temperature == nullptr || uniform != nullptr,
             "ps_sample: temperatures without uniform numbers");
  if (rows == 0) return 0;
  hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SM_THREADS), 0, (hipStream_t)stream, logits,
                     ld, inv_temperature, uniform, tokens, vocab);
  PS_CHECK_LAUNCH("ps_sample");
  return 0;
}
