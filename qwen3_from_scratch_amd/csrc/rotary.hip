// Rotary position encoding: the [cos | sin] table, and the fused pass over a
// step's qkv rows: per-head RMSNorm of q and k, rotation, and the cache write.
#include "common.h"

// table[p, i] = cos(p * inv_freq[i]), table[p, half + i] = sin(p * inv_freq[i]).
// The angle is the float32 product, as a float32 outer product would give it;
// cosf and sinf are the full-range float32 routines (no fast-math variants).
__global__ void rope_table_kernel(const float* __restrict__ inv_freq, float* __restrict__ table,
                                  int max_pos, int half) {
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)max_pos * half) return;
  const int p = (int)(idx / half);
  const int i = (int)(idx % half);
  const float angle = (float)p * inv_freq[i];
  table[(size_t)p * 2 * half + i] = cosf(angle);
  table[(size_t)p * 2 * half + half + i] = sinf(angle);
}

// One wavefront per (token, head). Heads 0..Hq-1 are queries, the next Hkv keys,
// the last Hkv values.
//   q: y = rotate(rmsnorm(x) * wq), written back in place
//   k: y = rotate(rmsnorm(x) * wk), stored to the key cache
//   v: stored to the value cache as it is
// rotate pairs element i with i + R/2 for i < R/2 (R = rotary_dim) and leaves
// elements >= R alone: y_i = x_i c - x_{i+R/2} s, y_{i+R/2} = x_{i+R/2} c + x_i s.
// The cache row of token t is page block_table[seq_index[t], pos / page], slot
// pos % page. Keys are laid out (pages, Hkv, page, D); values are transposed
// within the page, (pages, Hkv, D, page), so element j of a value row goes to
// [page, head, j, slot]. Everything is float32 until the single rounding at the
// store.
template <typename T, typename W, int PER_LANE>
__global__ void qk_norm_rope_store_kernel(T* __restrict__ qkv, const W* __restrict__ q_weight,
                                          const W* __restrict__ k_weight, float eps,
                                          const float* __restrict__ table, int rotary_dim, int max_pos,
                                          const int* __restrict__ positions,
                                          const int* __restrict__ seq_index,
                                          const int* __restrict__ block_table, int bt_stride, int bt_rows,
                                          T* __restrict__ k_cache, T* __restrict__ v_cache, int page_size,
                                          int num_pages, int Hq, int Hkv, int D) {
  const int lane = threadIdx.x & (Q3_WAVE - 1);
  const int head = blockIdx.y * (blockDim.x / Q3_WAVE) + threadIdx.x / Q3_WAVE;
  const int t = blockIdx.x;
  const int heads = Hq + 2 * Hkv;
  if (head >= heads) return;
  T* src = qkv + ((size_t)t * heads + head) * D;
  const int pos = positions[t];

  // where a key or value row goes, or nullptr if it is not stored
  T* dst = nullptr;
  int dst_stride = 1;  // distance between consecutive elements of the row at dst
  if (head >= Hq && k_cache != nullptr) {
    const int b = seq_index[t];
    const int blk = pos / page_size;
    if (b >= 0 && b < bt_rows && blk < bt_stride && pos >= 0) {
      const int page = block_table[(size_t)b * bt_stride + blk];
      if (page >= 0 && page < num_pages) {
        if (head < Hq + Hkv) {
          dst = k_cache + (((size_t)page * Hkv + (head - Hq)) * page_size + (pos % page_size)) * D;
        } else {
          dst = v_cache + ((size_t)page * Hkv + (head - Hq - Hkv)) * D * page_size + (pos % page_size);
          dst_stride = page_size;
        }
      }
    }
  }

  if (head >= Hq + Hkv) {  // a value head: copy
    if (dst)
      for (int j = lane; j < D; j += Q3_WAVE) dst[(size_t)j * dst_stride] = src[j];
    return;
  }

  const W* w = head < Hq ? q_weight : k_weight;
  float v[PER_LANE];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < PER_LANE; ++k) {
    const int j = lane + k * Q3_WAVE;
    v[k] = j < D ? to_float(src[j]) : 0.f;
    ss += v[k] * v[k];
  }
  if (w != nullptr) {
    ss = wave_sum(ss);
    const float scale = rsqrtf(ss / (float)D + eps);
#pragma unroll
    for (int k = 0; k < PER_LANE; ++k) {
      const int j = lane + k * Q3_WAVE;
      if (j < D) v[k] = v[k] * scale * to_float(w[j]);
    }
  }
  T* o = head < Hq ? src : dst;
  if (o == nullptr) return;
  const int half = rotary_dim / 2;
  const bool turn = table != nullptr && pos >= 0 && pos < max_pos;
  // element j's partner lives in lane (j +- half) % 64, register (j +- half) / 64:
  // exchange through shared memory rather than assume half is a multiple of 64
  __shared__ float stage[4][PER_LANE * Q3_WAVE];
  float* mine = stage[threadIdx.x / Q3_WAVE];
#pragma unroll
  for (int k = 0; k < PER_LANE; ++k) mine[lane + k * Q3_WAVE] = v[k];
  // the partner's value is written by another lane of this wavefront only
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
  for (int k = 0; k < PER_LANE; ++k) {
    const int j = lane + k * Q3_WAVE;
    if (j >= D) continue;
    float y = v[k];
    if (turn && j < rotary_dim) {
      const float* cs = table + (size_t)pos * rotary_dim;
      if (j < half) {
        y = v[k] * cs[j] - mine[j + half] * cs[half + j];
      } else {
        y = v[k] * cs[j - half] + mine[j - half] * cs[j];
      }
    }
    o[j] = from_float<T>(y);
  }
}

extern "C" int q3_rope_table(const float* inv_freq, float* table, int max_pos, int half,
                             hipStream_t stream) {
  if (max_pos <= 0 || half <= 0) return Q3_ERR_BAD_ARGUMENT;
  const long n = (long)max_pos * half;
  hipLaunchKernelGGL(rope_table_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, inv_freq,
                     table, max_pos, half);
  return q3_launch_status();
}

template <typename T, typename W>
static int launch_qk(void* qkv, const void* qw, const void* kw, float eps, const float* table,
                     int rotary_dim, int max_pos, const int* positions, const int* seq_index,
                     const int* block_table, int bt_stride, int bt_rows, void* k_cache, void* v_cache,
                     int page_size, int num_pages, int T_, int Hq, int Hkv, int D, hipStream_t stream) {
  const int heads = Hq + 2 * Hkv;
  const dim3 grid(T_, (heads + 3) / 4);
  const dim3 block(4 * Q3_WAVE);
#define Q3_QK_LAUNCH(N)                                                                                 \
  hipLaunchKernelGGL((qk_norm_rope_store_kernel<T, W, N>), grid, block, 0, stream, (T*)qkv,             \
                     (const W*)qw, (const W*)kw, eps, table, rotary_dim, max_pos, positions, seq_index, \
                     block_table, bt_stride, bt_rows, (T*)k_cache, (T*)v_cache, page_size, num_pages,   \
                     Hq, Hkv, D)
  if (D <= 64) {
    Q3_QK_LAUNCH(1);
  } else if (D <= 128) {
    Q3_QK_LAUNCH(2);
  } else if (D <= 256) {
    Q3_QK_LAUNCH(4);
  } else if (D <= 512) {
    Q3_QK_LAUNCH(8);
  } else {
    return Q3_ERR_UNSUPPORTED;
  }
#undef Q3_QK_LAUNCH
  return q3_launch_status();
}

extern "C" int q3_qk_norm_rope_store(void* qkv, const void* q_weight, const void* k_weight, int w_dtype,
                                     float eps, const float* table, int rotary_dim, int max_pos,
                                     const int* positions, const int* seq_index, const int* block_table,
                                     int bt_stride, int bt_rows, void* k_cache, void* v_cache,
                                     int page_size, int num_pages, int T_, int Hq, int Hkv, int D,
                                     int act_dtype, hipStream_t stream) {
  if (T_ <= 0 || Hq <= 0 || Hkv <= 0 || D <= 0 || (Hq + 2 * Hkv + 3) / 4 > 65535) return Q3_ERR_BAD_ARGUMENT;
  if (table && (rotary_dim <= 0 || rotary_dim % 2 || rotary_dim > D)) return Q3_ERR_BAD_ARGUMENT;
  if (k_cache && (!v_cache || !block_table || page_size <= 0)) return Q3_ERR_BAD_ARGUMENT;
  if ((q_weight == nullptr) != (k_weight == nullptr)) return Q3_ERR_BAD_ARGUMENT;
  Q3_DISPATCH_DTYPE(act_dtype, TT, Q3_DISPATCH_DTYPE(w_dtype, WW, return (launch_qk<TT, WW>(
      qkv, q_weight, k_weight, eps, table, rotary_dim, max_pos, positions, seq_index, block_table,
      bt_stride, bt_rows, k_cache, v_cache, page_size, num_pages, T_, Hq, Hkv, D, stream))));
  return Q3_ERR_BAD_ARGUMENT;
}
