// One token per row of float32 logits: arg-max, or a draw from the softmax at a
// temperature, optionally among the k best, as the arg-max of
// logit / temperature + Gumbel noise.
#include "common.h"
#include "sampling.h"

#include <math.h>

#include <mutex>

// Philox-4x32 with 10 rounds (Salmon et al., "Parallel random numbers: as easy
// as 1, 2, 3"): a counter-based generator, so the noise of (seed, counter,
// column) does not depend on which rows share the launch.
__device__ inline void philox4x32_10(uint32_t c[4], uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    const uint32_t hi0 = __umulhi(0xD2511F53u, c[0]), lo0 = 0xD2511F53u * c[0];
    const uint32_t hi1 = __umulhi(0xCD9E8D57u, c[2]), lo1 = 0xCD9E8D57u * c[2];
    const uint32_t n0 = hi1 ^ c[1] ^ k0, n2 = hi0 ^ c[3] ^ k1;
    c[0] = n0; c[1] = lo1; c[2] = n2; c[3] = lo0;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
}

// Larger float <=> larger key.
__device__ inline uint32_t order_key(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

struct Best {
  float value;
  int index;
};

__device__ inline Best better(Best a, Best b) {
  if (b.value > a.value || (b.value == a.value && b.index < a.index)) return b;
  return a;
}

__device__ inline Best block_best(Best mine, Best* scratch) {
#pragma unroll
  for (int off = Q3_WAVE / 2; off > 0; off >>= 1) {
    Best other;
    other.value = __shfl_xor(mine.value, off, Q3_WAVE);
    other.index = __shfl_xor(mine.index, off, Q3_WAVE);
    mine = better(mine, other);
  }
  const int lane = threadIdx.x & (Q3_WAVE - 1), wave = threadIdx.x / Q3_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = mine;
  __syncthreads();
  Best total = scratch[0];
  for (int i = 1; i < (int)(blockDim.x / Q3_WAVE); ++i) total = better(total, scratch[i]);
  return total;
}

// Three kernels, so that a row's vocabulary is read by many blocks:
// 1. (only if some row restricts the draw to its k best) per row, the key of the k-th largest
//    logit by a radix select over the four bytes; zero, which every key passes, otherwise;
// 2. per (row, chunk of the vocabulary), the best candidate of the chunk: the largest logit,
//    or the largest logit / temperature + Gumbel noise among those that pass;
// 3. per row, the best of the chunks' candidates.
// The best of bests does not depend on the chunking, and the noise of a column is keyed by
// (seed, counter, column) alone, so the token is the one a single pass would give.
__global__ __launch_bounds__(1024) void sample_threshold_kernel(const float* __restrict__ logits,
                                                                const float* __restrict__ temperature,
                                                                const int* __restrict__ top_k,
                                                                uint32_t* __restrict__ threshold, int V) {
  __shared__ unsigned int hist[256];
  __shared__ uint32_t sh_prefix, sh_remaining;
  const int r = blockIdx.x;
  const float* row = logits + (size_t)r * V;
  const int k = top_k[r];
  if (!(temperature[r] > 0.f) || k <= 0 || k >= V) {
    if (threadIdx.x == 0) threshold[r] = 0;
    return;
  }
  uint32_t prefix = 0, mask = 0;
  uint32_t remaining = (uint32_t)k;
  for (int shift = 24; shift >= 0; shift -= 8) {
    for (int i = threadIdx.x; i < 256; i += blockDim.x) hist[i] = 0;
    __syncthreads();
    for (int j = threadIdx.x; j < V; j += blockDim.x) {
      const uint32_t key = order_key(row[j]);
      if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      uint32_t left = remaining;
      int bin = 255;
      for (; bin > 0; --bin) {
        if (hist[bin] >= left) break;
        left -= hist[bin];
      }
      sh_prefix = prefix | ((uint32_t)bin << shift);
      sh_remaining = left;
    }
    __syncthreads();
    prefix = sh_prefix;
    remaining = sh_remaining;
    mask |= 255u << shift;
    __syncthreads();
  }
  if (threadIdx.x == 0) threshold[r] = prefix;
}

// grid (chunks, R), 256 threads; `chunk` columns per block, a multiple of 4 (the generator
// makes four columns' noise at a time).
__global__ __launch_bounds__(256) void sample_partial_kernel(const float* __restrict__ logits,
                                                             const float* __restrict__ temperature,
                                                             const long long* __restrict__ seed,
                                                             const int* __restrict__ counter,
                                                             const uint32_t* __restrict__ threshold,
                                                             Best* __restrict__ partial, int V, int chunk) {
  __shared__ Best best_scratch[4];
  const int r = blockIdx.y;
  const float* row = logits + (size_t)r * V;
  const float temp = temperature[r];
  const int c0 = blockIdx.x * chunk, c1 = min(V, c0 + chunk);
  Best mine;
  mine.value = -INFINITY;
  mine.index = 0x7fffffff;
  if (!(temp > 0.f)) {
    for (int j = c0 + threadIdx.x; j < c1; j += blockDim.x) {
      Best c;
      c.value = row[j];
      c.index = j;
      mine = better(mine, c);
    }
  } else {
    const uint32_t pass = threshold ? threshold[r] : 0u;
    const unsigned long long sd = (unsigned long long)seed[r];
    const uint32_t k0 = (uint32_t)sd, k1 = (uint32_t)(sd >> 32);
    const uint32_t step = (uint32_t)counter[r];
    const float inv_t = 1.f / temp;
    for (int j4 = c0 + threadIdx.x * 4; j4 < c1; j4 += blockDim.x * 4) {
      uint32_t c[4] = {(uint32_t)(j4 >> 2), step, 0u, 0u};
      philox4x32_10(c, k0, k1);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int j = j4 + i;
        if (j >= c1) break;
        const float x = row[j];
        if (order_key(x) < pass) continue;
        const float u = ((float)(c[i] >> 9) + 0.5f) * (1.f / 8388608.f);  // in (0, 1), exact
        Best cand;
        cand.value = x * inv_t - logf(-logf(u));
        cand.index = j;
        mine = better(mine, cand);
      }
    }
  }
  const Best total = block_best(mine, best_scratch);
  if (threadIdx.x == 0) partial[(size_t)r * gridDim.x + blockIdx.x] = total;
}

// grid R, 64 threads.
__global__ __launch_bounds__(64) void sample_final_kernel(const Best* __restrict__ partial, int chunks,
                                                          int* __restrict__ out, int V) {
  const int r = blockIdx.x;
  Best mine;
  mine.value = -INFINITY;
  mine.index = 0x7fffffff;
  for (int i = threadIdx.x; i < chunks; i += 64) mine = better(mine, partial[(size_t)r * chunks + i]);
#pragma unroll
  for (int off = Q3_WAVE / 2; off > 0; off >>= 1) {
    Best other;
    other.value = __shfl_xor(mine.value, off, Q3_WAVE);
    other.index = __shfl_xor(mine.index, off, Q3_WAVE);
    mine = better(mine, other);
  }
  if (threadIdx.x == 0) out[r] = mine.index < V ? mine.index : 0;
}

// How many chunks `q3_sample` cuts a row into, and the bytes of workspace it needs.
extern "C" int q3_sample_chunks(int V) {
  int chunks = (V + 1023) / 1024;
  return chunks < 1 ? 1 : (chunks > 256 ? 256 : chunks);
}

extern "C" long q3_sample_workspace(int R, int V) {
  return (long)R * q3_sample_chunks(V) * (long)sizeof(Best) + (long)R * (long)sizeof(uint32_t);
}

static int launch_sample(const float* logits, const float* temperature, const int* top_k, const long long* seed,
                         const int* counter, int* out, int R, int V, int with_top_k, void* workspace,
                         hipStream_t stream) {
  const int chunks = q3_sample_chunks(V);
  const int chunk = ((V + chunks - 1) / chunks + 3) / 4 * 4;
  Best* partial = static_cast<Best*>(workspace);
  uint32_t* threshold = reinterpret_cast<uint32_t*>(partial + (size_t)R * chunks);
  if (with_top_k) {
    int threads = 64;
    while (threads < 1024 && threads * 4 < V) threads *= 2;
    hipLaunchKernelGGL(sample_threshold_kernel, dim3(R), dim3(threads), 0, stream, logits, temperature, top_k,
                       threshold, V);
  }
  hipLaunchKernelGGL(sample_partial_kernel, dim3(chunks, R), dim3(256), 0, stream, logits, temperature, seed, counter,
                     with_top_k ? threshold : nullptr, partial, V, chunk);
  hipLaunchKernelGGL(sample_final_kernel, dim3(R), dim3(64), 0, stream, partial, chunks, out, V);
  return q3_launch_status();
}

// `with_top_k`: 0 if the caller knows that no row restricts its draw (the select is skipped).
// `workspace`: q3_sample_workspace(R, V) bytes, 8-byte aligned.
extern "C" int q3_sample(const float* logits, const float* temperature, const int* top_k,
                         const long long* seed, const int* counter, int* out, int R, int V,
                         int with_top_k, void* workspace, hipStream_t stream) {
  if (R <= 0 || V <= 0 || workspace == nullptr) return Q3_ERR_BAD_ARGUMENT;
  if (R > 65535) return Q3_ERR_UNSUPPORTED;
  return launch_sample(logits, temperature, top_k, seed, counter, out, R, V, with_top_k, workspace, stream);
}

// ---- the same without a workspace from the caller (see sampling.h) ------------------------
// The chunks' candidates and the rows' thresholds live in this array, one copy on every GPU that
// loads the library, held until the process ends. Host code never uses the array's name as an
// address: it asks each device for its copy's address once and passes that to the kernels.
static __device__ __align__(256) unsigned char scratch[Q3_SAMPLE_STATIC_BYTES];

#define Q3_MAX_DEVICES 64
static std::mutex scratch_lock;
static void* scratch_of_device[Q3_MAX_DEVICES];   // null until the device's first call

extern "C" int q3_sample_static(const float* logits, const float* temperature, const int* top_k,
                                const long long* seed, const int* counter, int* out, int R, int V,
                                int with_top_k, hipStream_t stream) {
  if (R <= 0 || V <= 0 || !logits || !temperature || !top_k || !seed || !counter || !out) return Q3_ERR_BAD_ARGUMENT;
  if (R > 65535 || q3_sample_workspace(R, V) > (long)Q3_SAMPLE_STATIC_BYTES) return Q3_ERR_UNSUPPORTED;
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return (int)e;
  if (device < 0 || device >= Q3_MAX_DEVICES) return Q3_ERR_UNSUPPORTED;
  void* workspace = nullptr;
  {
    std::lock_guard<std::mutex> hold(scratch_lock);
    if (scratch_of_device[device] == nullptr) {   // this device's copy of the array, asked for with it current
      void* ptr = nullptr;
      e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
      if (e != hipSuccess) return (int)e;
      if (ptr == nullptr) return Q3_ERR_UNSUPPORTED;
      scratch_of_device[device] = ptr;
    }
    workspace = scratch_of_device[device];
  }
  // every word the kernels read from the array they have written in this call (a candidate per
  // row and chunk, a threshold per row where a selection is asked for): nothing needs clearing
  return launch_sample(logits, temperature, top_k, seed, counter, out, R, V, with_top_k, workspace, stream);
}
