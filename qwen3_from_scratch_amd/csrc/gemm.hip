// out = x @ weight^T with float32 accumulation: x (M, K), weight (N, K), out (M, N).
#include "common.h"

// ---------------------------------------------------------------------------
// float32: plain fused multiply-adds, no matrix-core mode of reduced precision.
// A block of 256 threads computes a 64 x 64 tile of out; each thread a 4 x 4
// patch, summing over k in ascending order, so an output element's value does
// not depend on which rows share its batch.
// ---------------------------------------------------------------------------
#define F32_BM 64
#define F32_BN 64
#define F32_BK 16

__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ a,
                                                       const float* __restrict__ w,
                                                       float* __restrict__ out, int M, int N, int K) {
  __shared__ float as[F32_BK][F32_BM + 4];
  __shared__ float ws[F32_BK][F32_BN + 4];
  const int t = threadIdx.x;
  const int m0 = blockIdx.y * F32_BM;
  const int n0 = blockIdx.x * F32_BN;
  const int tm = (t / 16) * 4;  // this thread's rows within the tile
  const int tn = (t % 16) * 4;  // and columns
  // loader coordinates: 64 rows x 16 k per tile, 4 elements per thread
  const int lr = t / 4;          // row 0..63
  const int lk = (t % 4) * 4;    // k offset 0, 4, 8, 12
  const bool vec = (K % 4) == 0;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += F32_BK) {
    float av[4] = {0.f, 0.f, 0.f, 0.f}, wv[4] = {0.f, 0.f, 0.f, 0.f};
    const int gm = m0 + lr, gn = n0 + lr, gk = k0 + lk;
    if (gm < M) {
      const float* p = a + (size_t)gm * K + gk;
      if (vec && gk + 3 < K) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        av[0] = v.x; av[1] = v.y; av[2] = v.z; av[3] = v.w;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (gk + i < K) av[i] = p[i];
      }
    }
    if (gn < N) {
      const float* p = w + (size_t)gn * K + gk;
      if (vec && gk + 3 < K) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        wv[0] = v.x; wv[1] = v.y; wv[2] = v.z; wv[3] = v.w;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (gk + i < K) wv[i] = p[i];
      }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      as[lk + i][lr] = av[i];
      ws[lk + i][lr] = wv[i];
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < F32_BK; ++kk) {
      float ar[4], wr[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) ar[i] = as[kk][tm + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wr[j] = ws[kk][tn + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(ar[i], wr[j], acc[i][j]);
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gm = m0 + tm + i;
    if (gm >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + tn + j;
      if (gn < N) out[(size_t)gm * N + gn] = acc[i][j];
    }
  }
}

extern "C" int q3_linear(const void* x, const void* weight, void* out, int M, int N, int K, int in_dtype,
                         int out_dtype, hipStream_t stream) {
  if (M <= 0 || N <= 0 || K <= 0) return Q3_ERR_BAD_ARGUMENT;
  if (in_dtype == Q3_F32) {
    if (out_dtype != Q3_F32) return Q3_ERR_BAD_ARGUMENT;
    const dim3 grid((N + F32_BN - 1) / F32_BN, (M + F32_BM - 1) / F32_BM);
    if (grid.y > 65535) return Q3_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(gemm_f32_kernel, grid, dim3(256), 0, stream, (const float*)x, (const float*)weight,
                       (float*)out, M, N, K);
    return q3_launch_status();
  }
  return Q3_ERR_UNSUPPORTED;
}
