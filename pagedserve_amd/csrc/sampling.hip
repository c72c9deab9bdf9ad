// Token selection from float logits: argmax (ties to the lowest id, as torch.argmax on
// the reference's path, src/scheduler/orca_scheduler.py:250) or a draw from
// softmax(logits / temperature) by inverse CDF.  The uniform number of a row is made by the
// host from (seed, request, step), so a draw does not depend on what else is in the batch.
//
// One 1024-thread block per row.  Wave w owns the contiguous id range [w * seg, (w + 1) * seg).
// Up to 65,536 ids a row is read once: every lane asks for all its logits at the start (ids
// begin + 64 j + lane, up to 64 of them) and keeps them in registers for the maximum, for the
// exponentials and their sums, and for the walk through the range that holds uniform * total.
// That walk is made by the lanes side by side: the range's exponentials are turned through
// LDS so that every lane holds a run of consecutive ids, sums its run, and looks in it for the
// first id whose cumulative mass exceeds the goal.  (A wave that read its range again for
// each of these, 64 ids at a time and each read behind the one before, took 36 us for 8 rows
// of 50,257 ids where this takes 9.)  Longer rows take the kernel that reads three times.
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

// The same with every logit of the row in registers (PER of them per lane: vocab <= 1024 PER).
template <int PER>
__global__ __launch_bounds__(SM_THREADS) void sample_resident_kernel(
    const float* __restrict__ logits, int64_t ld, const float* __restrict__ inv_temperature,
    const float* __restrict__ uniform, int* __restrict__ tokens, int vocab) {
  __shared__ float s_val[SM_WAVES];
  __shared__ int s_idx[SM_WAVES];
  __shared__ float s_sum[SM_WAVES];
  __shared__ float s_turn[PER * 66];        // the chosen range, id by id (+ a gap per 32 ids)

  const int r = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const float* row = logits + (int64_t)r * ld;
  const int seg = ((vocab + SM_WAVES - 1) / SM_WAVES + 63) / 64 * 64;   // ids per wave
  const int begin = wave * seg;
  const int per = seg / 64;                                             // ids per lane, <= PER
  // places of the range that hold an id: p < limit (none for a wave beyond the row's end)
  const int limit = vocab - begin < seg ? (vocab - begin > 0 ? vocab - begin : 0) : seg;
  // (asked for now, so that they are there when the maximum is known)
  const float inv_t = inv_temperature ? inv_temperature[r] : 0.f;
  const float draw = (inv_temperature && uniform) ? uniform[r] : 0.f;

  float v[PER];
#pragma unroll
  for (int j = 0; j < PER; ++j) {   // all loads in flight, index clamped, masked below
    const int p = j * 64 + lane;
    v[j] = row[p < limit ? begin + p : vocab - 1];
  }
  // maximum and its first index (a lane's ids rise with j)
  float best = -INFINITY;
  int best_idx = vocab;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int p = j * 64 + lane;
    if (p < limit && v[j] > best) {
      best = v[j];
      best_idx = begin + p;
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
  if (inv_t <= 0.f) {
    if (tid == 0) tokens[r] = row_argmax;
    return;
  }

  // unnormalised probabilities exp((l - max) / T) = 2^((l - max) log2(e) / T) in place, summed
  // per wave range.  The exponential is the hardware's (v_exp_f32, within an ulp or two): the
  // library's takes some twenty instructions, 6 us for a row of 50,257 on one compute unit.
  const float scale = inv_t * 1.4426950408889634f;
  float partial = 0.f;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int p = j * 64 + lane;
    v[j] = p < limit ? __builtin_amdgcn_exp2f((v[j] - row_max) * scale) : 0.f;
    partial += v[j];
  }
  partial = wave_sum(partial);
  if (lane == 0) s_sum[wave] = partial;
  __syncthreads();
  // every wave finds the range that holds the goal (the same sums in the same order)
  float total = 0.f;
#pragma unroll
  for (int w = 0; w < SM_WAVES; ++w) total += s_sum[w];
  const float goal = draw * total;
  float before = 0.f;
  int choice = -1;
#pragma unroll
  for (int w = 0; w < SM_WAVES; ++w) {
    if (choice < 0) {
      if (s_sum[w] > 0.f && before + s_sum[w] > goal) choice = w;
      else before += s_sum[w];
    }
  }
  if (choice < 0) {
    // rounding left the goal at or beyond the total: the last non-empty range takes it
    choice = SM_WAVES - 1;
    while (choice > 0 && s_sum[choice] <= 0.f) --choice;
    before = 0.f;
    for (int w = 0; w < choice; ++w) before += s_sum[w];
  }
  if (wave != choice) return;

  // Place p of the range (id begin + p) goes to s_turn[p + p / 32]; lane l then owns places
  // l * per .. l * per + per - 1.  The gap keeps lanes that are `per` places apart off one bank.
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    if (j < per) {
      const int p = j * 64 + lane;
      s_turn[p + (p >> 5)] = v[j];
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // one wave: its own writes are all it reads
  const int first = lane * per;
  float mine = 0.f;
#pragma unroll
  for (int q = 0; q < PER; ++q) {   // the lane's run, all reads in flight (v is free again)
    const int p = first + q;
    v[q] = q < per ? s_turn[p + (p >> 5)] : 0.f;
  }
#pragma unroll
  for (int q = 0; q < PER; ++q) mine += v[q];
  float prefix = mine;   // inclusive prefix sum of the lanes' runs
#pragma unroll
  for (int offset = 1; offset < 64; offset <<= 1) {
    const float other = __shfl_up(prefix, offset, 64);
    if (lane >= offset) prefix += other;
  }
  float running = before + (prefix - mine);
  int hit = -1, last_positive = -1;
#pragma unroll
  for (int q = 0; q < PER; ++q) {
    running += v[q];
    if (v[q] > 0.f) {
      last_positive = begin + first + q;
      if (hit < 0 && running > goal) hit = begin + first + q;
    }
  }
  // the first hit in id order is the hit of the lowest lane that has one
  const unsigned long long hits = __ballot(hit >= 0);
  const unsigned long long positive = __ballot(last_positive >= 0);
  int token;
  if (hits) {
    token = __shfl(hit, __ffsll((long long)hits) - 1, 64);
  } else if (positive) {
    token = __shfl(last_positive, 63 - __clzll(positive), 64);
  } else {
    token = row_argmax;
  }
  if (lane == 0) tokens[r] = token;
}

extern "C" int ps_sample(const float* logits, int64_t ld, const float* inv_temperature,
                         const float* uniform, int* tokens, int rows, int vocab, void* stream) {
  PS_REQUIRE(rows >= 0 && vocab > 0 && ld >= vocab, "ps_sample: bad sizes (rows %d, vocab %d)",
             rows, vocab);
  PS_REQUIRE(inv_temperature == nullptr || uniform != nullptr,
             "ps_sample: temperatures without uniform numbers");
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (vocab <= 16 * SM_THREADS)
    hipLaunchKernelGGL(sample_resident_kernel<16>, dim3(rows), dim3(SM_THREADS), 0, s, logits, ld,
                       inv_temperature, uniform, tokens, vocab);
  else if (vocab <= 52 * SM_THREADS)   // (GPT-2's 50,257 ids: 50 a lane)
    hipLaunchKernelGGL(sample_resident_kernel<52>, dim3(rows), dim3(SM_THREADS), 0, s, logits, ld,
                       inv_temperature, uniform, tokens, vocab);
  else if (vocab <= 64 * SM_THREADS)
    hipLaunchKernelGGL(sample_resident_kernel<64>, dim3(rows), dim3(SM_THREADS), 0, s, logits, ld,
                       inv_temperature, uniform, tokens, vocab);
  else
    hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SM_THREADS), 0, s, logits, ld,
                       inv_temperature, uniform, tokens, vocab);
  PS_CHECK_LAUNCH("ps_sample");
  return 0;
}
