// RMSNorm over the float32 residual stream, with the pending residual addition
// and an optional row selection folded in.
#include "common.h"

// One block per output row r; source row s = rows ? rows[r] : r.
//   v = x[s] (+ delta[s]);  if write_back: x[s] = v
//   out[r] = v * rsqrt(mean(v^2) + eps) * weight        (all float32, rounded once)
// The row is kept in shared memory between the two passes when it fits
// (`cached` floats), otherwise it is formed again from its sources.
template <typename T, typename W>
__global__ void rmsnorm_kernel(float* __restrict__ x, const T* __restrict__ delta,
                               const W* __restrict__ weight, const int* __restrict__ rows,
                               T* __restrict__ out, int H, int n_src, float eps, int write_back,
                               int cached) {
  extern __shared__ float smem[];
  float* red = smem;            // 32 floats for the reduction
  float* row = smem + 32;       // `cached` floats
  const int r = blockIdx.x;
  int s = rows ? rows[r] : r;
  if (s < 0 || s >= n_src) s = 0;  // the host checks rows; stay inside the operands regardless
  float* xs = x + (size_t)s * H;
  const T* ds = delta ? delta + (size_t)s * H : nullptr;
  float acc = 0.f;
  for (int j = threadIdx.x; j < H; j += blockDim.x) {
    float v = xs[j];
    if (ds) v += to_float(ds[j]);
    if (j < cached) row[j] = v;
    acc += v * v;
  }
  const float total = block_sum(acc, red);
  const float scale = rsqrtf(total / (float)H + eps);
  T* o = out + (size_t)r * H;
  for (int j = threadIdx.x; j < H; j += blockDim.x) {
    float v;
    if (j < cached) {
      v = row[j];
    } else {
      v = xs[j];
      if (ds) v += to_float(ds[j]);
    }
    if (write_back) xs[j] = v;
    o[j] = from_float<T>(v * scale * to_float(weight[j]));
  }
}

// The same for row lengths that are a multiple of 4 and fit the block's registers:
// 16-byte loads, the row held in registers between the two passes.
__device__ inline float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ inline float4 load4(const bf16_t* p) {
  union {
    uint2 u;
    bf16_t e[4];
  } pk;
  pk.u = *reinterpret_cast<const uint2*>(p);
  return make_float4(bf16_to_float(pk.e[0]), bf16_to_float(pk.e[1]), bf16_to_float(pk.e[2]), bf16_to_float(pk.e[3]));
}
__device__ inline void store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ inline void store4(bf16_t* p, float4 v) {
  union {
    uint2 u;
    bf16_t e[4];
  } pk;
  pk.e[0] = float_to_bf16(v.x);
  pk.e[1] = float_to_bf16(v.y);
  pk.e[2] = float_to_bf16(v.z);
  pk.e[3] = float_to_bf16(v.w);
  *reinterpret_cast<uint2*>(p) = pk.u;
}

#define NORM_CHUNKS 4
template <typename T, typename W>
__global__ void rmsnorm_vec_kernel(float* __restrict__ x, const T* __restrict__ delta,
                                   const W* __restrict__ weight, const int* __restrict__ rows,
                                   T* __restrict__ out, int H, int n_src, float eps, int write_back) {
  __shared__ float red[32];
  const int r = blockIdx.x;
  int s = rows ? rows[r] : r;
  if (s < 0 || s >= n_src) s = 0;
  float* xs = x + (size_t)s * H;
  const T* ds = delta ? delta + (size_t)s * H : nullptr;
  const int H4 = H >> 2;
  float4 v[NORM_CHUNKS], wv[NORM_CHUNKS];
  float acc = 0.f;
#pragma unroll
  for (int c = 0; c < NORM_CHUNKS; ++c) {
    const int j = threadIdx.x + c * blockDim.x;
    if (j < H4) {
      wv[c] = load4(weight + 4 * j);  // needed only after the sum; asked for now so that it has arrived by then
      v[c] = load4(xs + 4 * j);
      if (ds) {
        const float4 d = load4(ds + 4 * j);
        v[c].x += d.x; v[c].y += d.y; v[c].z += d.z; v[c].w += d.w;
      }
      acc += v[c].x * v[c].x + v[c].y * v[c].y + v[c].z * v[c].z + v[c].w * v[c].w;
    }
  }
  const float total = block_sum(acc, red);
  const float scale = rsqrtf(total / (float)H + eps);
  T* o = out + (size_t)r * H;
#pragma unroll
  for (int c = 0; c < NORM_CHUNKS; ++c) {
    const int j = threadIdx.x + c * blockDim.x;
    if (j < H4) {
      if (write_back) store4(xs + 4 * j, v[c]);
      const float4 w = wv[c];
      store4(o + 4 * j, make_float4(v[c].x * scale * w.x, v[c].y * scale * w.y, v[c].z * scale * w.z,
                                    v[c].w * scale * w.w));
    }
  }
}

template <typename T, typename W>
static int launch_rmsnorm(float* x, const void* delta, const void* weight, const int* rows, void* out,
                          int n_out, int n_src, int H, float eps, int write_back, hipStream_t stream) {
  if (H % 4 == 0 && H / 4 <= 1024 * NORM_CHUNKS) {
    int threads = 64;
    while (threads < 1024 && threads * NORM_CHUNKS < H / 4) threads *= 2;
    hipLaunchKernelGGL((rmsnorm_vec_kernel<T, W>), dim3(n_out), dim3(threads), 0, stream, x, (const T*)delta,
                       (const W*)weight, rows, (T*)out, H, n_src, eps, write_back);
    return q3_launch_status();
  }
  int threads = 64;
  while (threads < 1024 && threads * 4 < H) threads *= 2;
  const int cached = H <= 12000 ? H : 12000;  // 48 KB of the row at most
  const size_t smem = (size_t)(32 + cached) * sizeof(float);
  hipLaunchKernelGGL((rmsnorm_kernel<T, W>), dim3(n_out), dim3(threads), smem, stream, x, (const T*)delta,
                     (const W*)weight, rows, (T*)out, H, n_src, eps, write_back, cached);
  return q3_launch_status();
}

extern "C" int q3_rmsnorm(float* x, const void* delta, const void* weight, const int* rows, void* out,
                          int n_out, int n_src, int H, float eps, int act_dtype, int w_dtype,
                          int write_back, hipStream_t stream) {
  if (n_out <= 0 || n_src <= 0 || H <= 0) return Q3_ERR_BAD_ARGUMENT;
  if (write_back && rows) return Q3_ERR_BAD_ARGUMENT;  // a row named twice would be added twice
  Q3_DISPATCH_DTYPE(act_dtype, TT, Q3_DISPATCH_DTYPE(w_dtype, WW, return (launch_rmsnorm<TT, WW>(
      x, delta, weight, rows, out, n_out, n_src, H, eps, write_back, stream))));
  return Q3_ERR_BAD_ARGUMENT;
}
