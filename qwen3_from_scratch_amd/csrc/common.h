// Shared device helpers for the gfx950 kernels: bfloat16 conversion, wave and
// block reductions for 64-wide wavefronts, and the dtype dispatch used by the
// extern "C" entry points.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define Q3_WAVE 64

enum Q3DType { Q3_F32 = 0, Q3_BF16 = 1 };

// Refusals of the host-side launchers (HIP's own codes are positive and small).
#define Q3_ERR_BAD_ARGUMENT 10001
#define Q3_ERR_UNSUPPORTED 10002

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

// Round to nearest, ties to even; NaN stays NaN.
__host__ __device__ inline bf16_t float_to_bf16(float f) {
  union {
    uint32_t u;
    float f;
  } c;
  c.f = f;
  bf16_t r;
  if ((c.u & 0x7fffffffu) > 0x7f800000u) {
    r.bits = (uint16_t)((c.u >> 16) | 0x0040u);
    return r;
  }
  uint32_t lsb = (c.u >> 16) & 1u;
  c.u += 0x7fffu + lsb;
  r.bits = (uint16_t)(c.u >> 16);
  return r;
}

__device__ inline float to_float(float v) { return v; }
__device__ inline float to_float(bf16_t v) { return bf16_to_float(v); }

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

__device__ inline float wave_sum(float v) {
#pragma unroll
  for (int off = Q3_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, Q3_WAVE);
  return v;
}

__device__ inline float wave_max(float v) {
#pragma unroll
  for (int off = Q3_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, Q3_WAVE));
  return v;
}

// The maximum (sum) over the four lanes l, l ^ 16, l ^ 32, l ^ 48, in all of them: two lane
// swaps in the vector unit (rows of 16 lanes, then halves of 32) instead of two round trips
// through shared memory, which is what a shuffle by 16 or 32 lanes compiles to.
__device__ inline float quad_rows_max(float v) {
  unsigned u = __float_as_uint(v);
  auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  u = __float_as_uint(v);
  auto b = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

// The same for values that are never NaN (matrix results, minus infinity): the maximum instruction as it is.
// The compiler's own first makes a quiet NaN of either operand, one instruction each.
__device__ inline float max_of_numbers(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
__device__ inline float quad_rows_max_of_numbers(float v) {
  unsigned u = __float_as_uint(v);
  auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  v = max_of_numbers(__uint_as_float(a[0]), __uint_as_float(a[1]));
  u = __float_as_uint(v);
  auto b = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return max_of_numbers(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

__device__ inline float quad_rows_sum(float v) {
  unsigned u = __float_as_uint(v);
  auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  u = __float_as_uint(v);
  auto b = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// Sum over a block of up to 1024 threads; every thread gets the result.
// `scratch` holds at least 17 floats of shared memory.
__device__ inline float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (Q3_WAVE - 1);
  const int wave = threadIdx.x / Q3_WAVE;
  const int waves = (blockDim.x + Q3_WAVE - 1) / Q3_WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int i = 0; i < waves; ++i) total += scratch[i];
  return total;
}

#define Q3_DISPATCH_DTYPE(code, T, ...)              \
  do {                                               \
    if ((code) == Q3_F32) {                          \
      typedef float T;                               \
      __VA_ARGS__;                                   \
    } else if ((code) == Q3_BF16) {                  \
      typedef bf16_t T;                              \
      __VA_ARGS__;                                   \
    } else {                                         \
      return Q3_ERR_BAD_ARGUMENT;                    \
    }                                                \
  } while (0)

static inline int q3_launch_status() { return (int)hipGetLastError(); }
