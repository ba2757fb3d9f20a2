// Embedding row gather and the SwiGLU activation.
#include "common.h"

// out[t, :] = float(table[ids[t], :]). An id outside the table gives a row of
// zeros (the host refuses such ids before launching; this only keeps the
// kernel inside its operands).
template <typename T>
__global__ void embed_rows_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                                  float* __restrict__ out, int H, int V) {
  const int t = blockIdx.x;
  const int id = ids[t];
  const bool ok = id >= 0 && id < V;
  const T* row = table + (size_t)(ok ? id : 0) * H;
  float* dst = out + (size_t)t * H;
  for (int j = threadIdx.x; j < H; j += blockDim.x) dst[j] = ok ? to_float(row[j]) : 0.f;
}

// out[t, j] = silu(gate[t, j]) * up[t, j] for rows that interleave the two:
// gate_up[t, 2j] = gate[t, j], gate_up[t, 2j + 1] = up[t, j].
// silu(g) = g / (1 + exp(-g)), evaluated in float32 and rounded once.
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int I) {
  const int t = blockIdx.y;
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= I) return;
  const T* row = gate_up + (size_t)t * 2 * I;
  const float g = to_float(row[2 * j]);
  const float u = to_float(row[2 * j + 1]);
  out[(size_t)t * I + j] = from_float<T>(g / (1.f + expf(-g)) * u);
}

// The same, eight outputs per thread with 16-byte loads and stores; bfloat16, I a multiple of 8.
__global__ void swiglu_vec8_kernel(const bf16_t* __restrict__ gate_up, bf16_t* __restrict__ out, int I) {
  const int t = blockIdx.y;
  const int j = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (j >= I) return;
  const bf16_t* row = gate_up + (size_t)t * 2 * I + 2 * j;
  union {
    uint4 u;
    bf16_t e[8];
  } a, b, o;
  a.u = *reinterpret_cast<const uint4*>(row);
  b.u = *reinterpret_cast<const uint4*>(row + 8);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float g0 = bf16_to_float(a.e[2 * i]), g1 = bf16_to_float(b.e[2 * i]);
    o.e[i] = float_to_bf16(g0 / (1.f + expf(-g0)) * bf16_to_float(a.e[2 * i + 1]));
    o.e[4 + i] = float_to_bf16(g1 / (1.f + expf(-g1)) * bf16_to_float(b.e[2 * i + 1]));
  }
  *reinterpret_cast<uint4*>(out + (size_t)t * I + j) = o.u;
}

extern "C" int q3_embed_rows(const int* ids, const void* table, float* out, int T, int H, int V,
                             int table_dtype, hipStream_t stream) {
  if (T <= 0 || H <= 0 || V <= 0) return Q3_ERR_BAD_ARGUMENT;
  const int threads = H >= 1024 ? 256 : (H >= 256 ? 128 : 64);
  Q3_DISPATCH_DTYPE(table_dtype, TT,
                    hipLaunchKernelGGL(embed_rows_kernel<TT>, dim3(T), dim3(threads), 0, stream, ids,
                                       (const TT*)table, out, H, V));
  return q3_launch_status();
}

extern "C" int q3_swiglu(const void* gate_up, void* out, int T, int I, int dtype, hipStream_t stream) {
  if (T <= 0 || I <= 0 || T > 65535 * 32) return Q3_ERR_BAD_ARGUMENT;
  const int threads = 256;
  // blockIdx.y carries the row; rows beyond 65535 are covered by several launches
  for (int t0 = 0; t0 < T; t0 += 65535) {
    const int rows = T - t0 < 65535 ? T - t0 : 65535;
    if (dtype == Q3_BF16 && I % 8 == 0) {
      const int per_row = I / 8;
      const int vt = per_row >= 256 ? 256 : 64;
      hipLaunchKernelGGL(swiglu_vec8_kernel, dim3((per_row + vt - 1) / vt, rows), dim3(vt), 0, stream,
                         (const bf16_t*)gate_up + (size_t)t0 * 2 * I, (bf16_t*)out + (size_t)t0 * I, I);
      continue;
    }
    Q3_DISPATCH_DTYPE(dtype, TT,
                      hipLaunchKernelGGL(swiglu_kernel<TT>, dim3((I + threads - 1) / threads, rows),
                                         dim3(threads), 0, stream,
                                         (const TT*)gate_up + (size_t)t0 * 2 * I, (TT*)out + (size_t)t0 * I, I));
  }
  return q3_launch_status();
}
