// The per-head preparation of queries and keys, RMSNorm over the head and then the NeoX
// rotation of the pairs (d, d + D / 2), in pieces of eight pairs. Two kernels share it: the
// one that prepares a whole step's heads, and the decoding attention kernel, which prepares
// its own rows. Every product and sum is written with the rounding it is meant to have, so
// that both give the same bits whatever the compiler would contract elsewhere.
#pragma once

#include "common.h"

union Half8 {
  uint4 u;
  bf16_t e[8];
};

template <typename W>
__device__ inline void load_weights8(const W* w, float (&o)[8]);
template <>
__device__ inline void load_weights8<float>(const float* w, float (&o)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(w), b = *reinterpret_cast<const float4*>(w + 4);
  o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
}
template <>
__device__ inline void load_weights8<bf16_t>(const bf16_t* w, float (&o)[8]) {
  Half8 h;
  h.u = *reinterpret_cast<const uint4*>(w);
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = bf16_to_float(h.e[i]);
}

// a[i]^2 + b[i]^2 summed over the eight pairs in ascending order.
__device__ __forceinline__ float pairs_sum_of_squares(const float (&a)[8], const float (&b)[8]) {
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    s = __fmaf_rn(a[i], a[i], s);
    s = __fmaf_rn(b[i], b[i], s);
  }
  return s;
}

// rsqrt(mean + eps) of a head whose squares sum to `ss`.
__device__ __forceinline__ float head_norm_scale(float ss, int D, float eps) {
  return rsqrtf(__fadd_rn(__fdiv_rn(ss, (float)D), eps));
}

// x * scale * weight for eight pairs.
__device__ __forceinline__ void pairs_normalise(float (&a)[8], float (&b)[8], float scale, const float (&wa)[8],
                                                const float (&wb)[8]) {
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = __fmul_rn(__fmul_rn(a[i], scale), wa[i]);
    b[i] = __fmul_rn(__fmul_rn(b[i], scale), wb[i]);
  }
}

// (a, b) -> (a cos - b sin, b cos + a sin) for eight pairs.
__device__ __forceinline__ void pairs_rotate(float (&a)[8], float (&b)[8], const float (&cs)[8],
                                             const float (&sn)[8]) {
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float ya = __fmaf_rn(a[i], cs[i], -__fmul_rn(b[i], sn[i]));
    const float yb = __fmaf_rn(b[i], cs[i], __fmul_rn(a[i], sn[i]));
    a[i] = ya;
    b[i] = yb;
  }
}
