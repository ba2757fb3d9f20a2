// What this GPU delivers, measured: the rate at which a kernel can read memory that no cache
// holds, and the rate of the bfloat16 matrix instruction with operands in registers. The
// benchmark prices its steps against these beside the published peaks.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

// Every thread reads 16 bytes at a time, a block's threads consecutive addresses; the sum keeps
// the loads alive, the store never happens for a buffer of zeros.
__global__ __launch_bounds__(256) void probe_read_kernel(const float4* __restrict__ buffer, size_t count,
                                                         float* __restrict__ sink) {
  float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (; i + 3 * stride < count; i += 4 * stride) {   // four loads in flight per thread
    const float4 a = buffer[i], b = buffer[i + stride], c = buffer[i + 2 * stride], d = buffer[i + 3 * stride];
    sum.x += a.x + b.x + c.x + d.x;
    sum.y += a.y + b.y + c.y + d.y;
    sum.z += a.z + b.z + c.z + d.z;
    sum.w += a.w + b.w + c.w + d.w;
  }
  for (; i < count; i += stride) {
    const float4 a = buffer[i];
    sum.x += a.x; sum.y += a.y; sum.z += a.z; sum.w += a.w;
  }
  if (sum.x + sum.y + sum.z + sum.w == 12345.f) sink[0] = sum.x;
}

// Eight independent chains of v_mfma_f32_16x16x32_bf16 per wavefront, `iters` rounds. The instruction is
// written as assembly with the accumulator as one in/out operand: left to the compiler, the loop came out with
// some forty moves between the two register files per round, and the rate read 1.4 PFLOP/s where the
// instruction alone delivers what the other form does.
__global__ __launch_bounds__(256) void probe_mfma_kernel(int iters, float* __restrict__ sink) {
  bf16x8_t a, b;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    a[j] = (__bf16)(0.001f * (float)(threadIdx.x & 7));
    b[j] = (__bf16)(0.002f * (float)(j + 1));
  }
  f32x4_t acc[8];
#pragma unroll
  for (int c = 0; c < 8; ++c) acc[c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int c = 0; c < 8; ++c)
      asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(acc[c]) : "v"(a), "v"(b));
  }
  float total = 0.f;
#pragma unroll
  for (int c = 0; c < 8; ++c) total += acc[c][0] + acc[c][1] + acc[c][2] + acc[c][3];
  if (total == 12345.f) sink[0] = total;
}

// The same with v_mfma_f32_32x32x16_bf16 (32,768 operations each), four chains of sixteen accumulators.
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
__global__ __launch_bounds__(256) void probe_mfma32_kernel(int iters, float* __restrict__ sink) {
  bf16x8_t a, b;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    a[j] = (__bf16)(0.001f * (float)(threadIdx.x & 7));
    b[j] = (__bf16)(0.002f * (float)(j + 1));
  }
  f32x16_t acc[4];
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[c][j] = 0.f;
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[c], 0, 0, 0);
  }
  float total = 0.f;
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int j = 0; j < 16; ++j) total += acc[c][j];
  if (total == 12345.f) sink[0] = total;
}

// Reads `bytes` (a multiple of 16) of `buffer` once. `sink`: one float, never written for a buffer of zeros.
extern "C" int q3_probe_read(const void* buffer, size_t bytes, float* sink, int blocks, hipStream_t stream) {
  if (!buffer || !sink || bytes < 16 || bytes % 16 || blocks < 1 || blocks > 65535 * 16) return Q3_ERR_BAD_ARGUMENT;
  hipLaunchKernelGGL(probe_read_kernel, dim3(blocks), dim3(256), 0, stream, (const float4*)buffer, bytes / 16, sink);
  return q3_launch_status();
}

// `blocks` blocks of four wavefronts, each wavefront `iters` x 8 matrix instructions of 16 x 16 x 32
// (2 x 16 x 16 x 32 = 16,384 floating-point operations each). Returns the operations launched in *flops.
// `shape` 0: 16 x 16 x 32; 1: 32 x 32 x 16 in four chains (32,768 operations each).
extern "C" int q3_probe_mfma(int blocks, int iters, int shape, float* sink, double* flops, hipStream_t stream) {
  if (!sink || !flops || blocks < 1 || blocks > 1 << 20 || iters < 1 || shape < 0 || shape > 1) return Q3_ERR_BAD_ARGUMENT;
  if (shape == 0)
    hipLaunchKernelGGL(probe_mfma_kernel, dim3(blocks), dim3(256), 0, stream, iters, sink);
  else
    hipLaunchKernelGGL(probe_mfma32_kernel, dim3(blocks), dim3(256), 0, stream, iters, sink);
  *flops = (double)blocks * 4.0 * (double)iters * (shape == 0 ? 8.0 * 16384.0 : 4.0 * 32768.0);
  return q3_launch_status();
}
