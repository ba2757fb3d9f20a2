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

template <typename T, typename W>
static int launch_rmsnorm(float* x, const void* delta, const void* weight, const int* rows, void* out,
                          int n_out, int n_src, int H, float eps, int write_back, hipStream_t stream) {
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
