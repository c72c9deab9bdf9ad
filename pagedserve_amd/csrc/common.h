// Shared device helpers for the gfx950 kernels: storage types, conversions,
// wave64 reductions and the error channel of the C interface.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define PS_WAVE 64

// Storage dtypes of the C interface.
enum PsDtype { PS_F32 = 0, PS_BF16 = 1 };

// Epilogues of the matrix products.
enum PsEpilogue {
  PS_EPI_NONE = 0,       // C = A W^T + b
  PS_EPI_GELU_TANH = 1,  // C = gelu_tanh(A W^T + b)
  PS_EPI_GELU_ERF = 2,   // C = gelu_erf(A W^T + b)
  PS_EPI_RESIDUAL = 3,   // C(float) += A W^T + b   (C holds the residual stream)
};

struct bf16_t {
  uint16_t bits;
};

__host__ __device__ inline float bf16_to_float(bf16_t v) {
  union {
    uint32_t u;
    float f;
  } c;
  c.u = ((uint32_t)v.bits) << 16;
  return c.f;
}

// Round to nearest, ties to even; NaN stays NaN.  On the device this is the hardware
// conversion of gfx950 (v_cvt_pk_bf16_f32).
__host__ __device__ inline bf16_t float_to_bf16(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
  bf16_t native;
  native.bits = __builtin_bit_cast(uint16_t, (__bf16)f);
  return native;
#endif
  union {
    uint32_t u;
    float f;
  } c;
  c.f = f;
  bf16_t out;
  if ((c.u & 0x7fffffffu) > 0x7f800000u) {
    out.bits = (uint16_t)((c.u >> 16) | 0x0040u);
    return out;
  }
  uint32_t rounding = 0x7fffu + ((c.u >> 16) & 1u);
  out.bits = (uint16_t)((c.u + rounding) >> 16);
  return out;
}

// Two floats to two bfloat16 in one 32-bit word (lo in the low half).
__device__ inline uint32_t pack2_bf16(float lo, float hi) {
  typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2_t;
  typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
  const f32x2_t pair = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2_t));
}

template <typename T>
__device__ inline float to_float(T v);
template <>
__device__ inline float to_float<float>(float v) {
  return v;
}
template <>
__device__ inline float to_float<bf16_t>(bf16_t v) {
  return bf16_to_float(v);
}

template <typename T>
__device__ inline T from_float(float v);
template <>
__device__ inline float from_float<float>(float v) {
  return v;
}
template <>
__device__ inline bf16_t from_float<bf16_t>(float v) {
  return float_to_bf16(v);
}

// Lane exchanges inside a row of 16 lanes run on the vector unit itself (DPP), not through
// the LDS crossbar that __shfl_xor uses: a reduction over a wave is four such steps, then the
// four row results are read as scalars.  CTRL: 0xB1 / 0x4E swap neighbours / pairs inside a
// quad, 0x141 / 0x140 mirror a half row / a row.
template <int CTRL>
__device__ inline float lane_exchange(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

// Sum over aligned groups of N lanes (N = 2, 4, 8 or 16); every lane receives its group's sum.
template <int N>
__device__ inline float lanes_sum(float v) {
  static_assert(N == 1 || N == 2 || N == 4 || N == 8 || N == 16, "groups inside a row of 16 lanes");
  if (N >= 2) v += lane_exchange<0xB1>(v);
  if (N >= 4) v += lane_exchange<0x4E>(v);
  if (N >= 8) v += lane_exchange<0x141>(v);
  if (N >= 16) v += lane_exchange<0x140>(v);
  return v;
}

template <int N>
__device__ inline float lanes_max(float v) {
  static_assert(N == 1 || N == 2 || N == 4 || N == 8 || N == 16, "groups inside a row of 16 lanes");
  if (N >= 2) v = fmaxf(v, lane_exchange<0xB1>(v));
  if (N >= 4) v = fmaxf(v, lane_exchange<0x4E>(v));
  if (N >= 8) v = fmaxf(v, lane_exchange<0x141>(v));
  if (N >= 16) v = fmaxf(v, lane_exchange<0x140>(v));
  return v;
}

// The sum / maximum of a lane's value and that of the lane 32 further (or back): one swap of
// the wave's halves (v_permlane32_swap) instead of a trip through LDS.
__device__ inline float halves_sum(float v) {
  const int bits = __builtin_bit_cast(int, v);
  const auto both = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
  return __builtin_bit_cast(float, (int)both[0]) + __builtin_bit_cast(float, (int)both[1]);
}

__device__ inline float halves_max(float v) {
  const int bits = __builtin_bit_cast(int, v);
  const auto both = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
  return fmaxf(__builtin_bit_cast(float, (int)both[0]), __builtin_bit_cast(float, (int)both[1]));
}

// The sum / maximum of a lane's value and that of lane (l ^ OFFSET), for OFFSET = 8, 16 or 32
// without a trip through LDS (a rotation inside the row of 16 lanes, a swap of rows, a swap of
// the wave's halves); other offsets go through the shuffle.
template <int OFFSET>
__device__ inline float lane_xor(float v) {
  return __shfl_xor(v, OFFSET, 64);
}
template <int OFFSET>
__device__ inline float xor_sum(float v) {
  if (OFFSET == 8) return v + lane_exchange<0x128>(v);
  if (OFFSET == 16) {
    const int bits = __builtin_bit_cast(int, v);
    const auto both = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
    return __builtin_bit_cast(float, (int)both[0]) + __builtin_bit_cast(float, (int)both[1]);
  }
  if (OFFSET == 32) return halves_sum(v);
  return v + lane_xor<OFFSET>(v);
}
template <int OFFSET>
__device__ inline float xor_max(float v) {
  if (OFFSET == 8) return fmaxf(v, lane_exchange<0x128>(v));
  if (OFFSET == 16) {
    const int bits = __builtin_bit_cast(int, v);
    const auto both = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
    return fmaxf(__builtin_bit_cast(float, (int)both[0]), __builtin_bit_cast(float, (int)both[1]));
  }
  if (OFFSET == 32) return halves_max(v);
  return fmaxf(v, lane_xor<OFFSET>(v));
}

__device__ inline float read_lane(float v, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// Every lane receives the sum / the maximum over the wave.
__device__ inline float wave_sum(float v) {
  v = lanes_sum<16>(v);
  return (read_lane(v, 0) + read_lane(v, 16)) + (read_lane(v, 32) + read_lane(v, 48));
}

__device__ inline float wave_max(float v) {
  v = lanes_max<16>(v);
  return fmaxf(fmaxf(read_lane(v, 0), read_lane(v, 16)), fmaxf(read_lane(v, 32), read_lane(v, 48)));
}

// Sum over a block of up to 1024 threads; every thread receives the total.
// `scratch` holds at least 16 floats of shared memory.
__device__ inline float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (PS_WAVE - 1);
  const int wave = threadIdx.x / PS_WAVE;
  const int waves = (blockDim.x + PS_WAVE - 1) / PS_WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int i = 0; i < waves; ++i) total += scratch[i];
  return total;
}

__device__ inline float gelu_tanh_f(float u) {
  const float k = 0.7978845608028654f;  // sqrt(2/pi)
  return 0.5f * u * (1.0f + tanhf(k * (u + 0.044715f * u * u * u)));
}

__device__ inline float gelu_erf_f(float u) {
  return 0.5f * u * (1.0f + erff(u * 0.7071067811865476f));
}

template <int EPI>
__device__ inline float apply_activation(float v) {
  if (EPI == PS_EPI_GELU_TANH) return gelu_tanh_f(v);
  if (EPI == PS_EPI_GELU_ERF) return gelu_erf_f(v);
  return v;
}

// ---- error channel -------------------------------------------------------
void ps_set_error(const char* fmt, ...);

#define PS_REQUIRE(cond, ...)   \
  do {                          \
    if (!(cond)) {              \
      ps_set_error(__VA_ARGS__); \
      return 1;                 \
    }                           \
  } while (0)

#define PS_CHECK_LAUNCH(name)                                              \
  do {                                                                     \
    hipError_t launch_error_ = hipGetLastError();                          \
    if (launch_error_ != hipSuccess) {                                     \
      ps_set_error("%s: launch failed: %s", name, hipGetErrorString(launch_error_)); \
      return 2;                                                            \
    }                                                                      \
  } while (0)

// Compute units of the current device (asked once per device; elementwise.hip).
int ps_compute_units();
