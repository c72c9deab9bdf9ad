// Token selection from float logits: argmax (ties to the lowest id, as torch.argmax on
// the reference's path, src/scheduler/orca_scheduler.py:250) or a draw from
// softmax(logits / temperature) by inverse CDF.  The uniform number of a row is made by the
// host from (seed, request, step), so a draw does not depend on what else is in the batch.
// One 256-thread block per row; thread i owns the contiguous id range [i*c, (i+1)*c), which
// fixes the order of every sum.
#include <math.h>

#include "common.h"
#include "pagedserve_hip.h"

#define SM_THREADS 256

__global__ __launch_bounds__(SM_THREADS) void sample_kernel(
    const float* __restrict__ logits, int64_t ld, const float* __restrict__ inv_temperature,
    const float* __restrict__ uniform, int* __restrict__ tokens, int vocab) {
  __shared__ float s_val[SM_THREADS];
  __shared__ int s_idx[SM_THREADS];
  __shared__ float s_sum[SM_THREADS];
  __shared__ int s_choice;
  __shared__ float s_before;
  __shared__ float s_goal;

  const int r = blockIdx.x;
  const int tid = threadIdx.x;
  const float* row = logits + (int64_t)r * ld;
  const int chunk = (vocab + SM_THREADS - 1) / SM_THREADS;
  const int begin = tid * chunk;
  const int end = begin + chunk < vocab ? begin + chunk : vocab;

  // maximum and its first index
  float best = -INFINITY;
  int best_idx = vocab;
  for (int i = begin; i < end; ++i) {
    const float v = row[i];
    if (v > best) {
      best = v;
      best_idx = i;
    }
  }
  s_val[tid] = best;
  s_idx[tid] = best_idx;
  __syncthreads();
  for (int stride = SM_THREADS / 2; stride > 0; stride >>= 1) {
    if (tid < stride) {
      const float other = s_val[tid + stride];
      const int other_idx = s_idx[tid + stride];
      if (other > s_val[tid] || (other == s_val[tid] && other_idx < s_idx[tid])) {
        s_val[tid] = other;
        s_idx[tid] = other_idx;
      }
    }
    __syncthreads();
  }
  const float row_max = s_val[0];
  const int row_argmax = s_idx[0] < vocab ? s_idx[0] : 0;
  const float inv_t = inv_temperature ? inv_temperature[r] : 0.f;
  if (inv_t <= 0.f) {
    if (tid == 0) tokens[r] = row_argmax;
    return;
  }

  // unnormalised probabilities exp((l - max) / T), summed per thread range
  float partial = 0.f;
  for (int i = begin; i < end; ++i) partial += expf((row[i] - row_max) * inv_t);
  s_sum[tid] = partial;
  __syncthreads();
  if (tid == 0) {
    float total = 0.f;
    for (int i = 0; i < SM_THREADS; ++i) total += s_sum[i];
    const float goal = uniform[r] * total;
    float before = 0.f;
    int choice = -1;
    for (int i = 0; i < SM_THREADS; ++i) {
      if (s_sum[i] > 0.f && before + s_sum[i] > goal) {
        choice = i;
        break;
      }
      before += s_sum[i];
    }
    if (choice < 0) {
      // rounding left the goal at or beyond the total: the last non-empty range takes it
      choice = SM_THREADS - 1;
      while (choice > 0 && s_sum[choice] <= 0.f) --choice;
      before = 0.f;
      for (int i = 0; i < choice; ++i) before += s_sum[i];
    }
    s_choice = choice;
    s_before = before;
    s_goal = goal;
  }
  __syncthreads();
  if (tid == s_choice) {
    float running = s_before;
    int token = end - 1 >= begin ? end - 1 : row_argmax;
    for (int i = begin; i < end; ++i) {
      running += expf((row[i] - row_max) * inv_t);
      if (running > s_goal) {
        token = i;
        break;
      }
    }
    tokens[r] = token;
  }
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
