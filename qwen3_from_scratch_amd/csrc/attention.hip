// Causal softmax attention of packed query rows over paged keys and values.
//
// Layout: caches are (pages, Hkv, page, D); sequence b's key j lives in page
// block_table[b, j / page] at row j % page. Query row i of a sequence with q_len
// rows and kv_len keys sits at position kv_len - q_len + i and sees keys at
// positions <= its own, and, with a window w > 0, only those fewer than w behind.
#include "common.h"

#include <math.h>

// ---------------------------------------------------------------------------
// The general kernel: any head size that is a multiple of 16 up to 256, any
// page size, float32 or bfloat16 storage, float32 arithmetic throughout
// (scores, softmax statistics, probabilities and the output accumulation).
// One block serves BM = 16 query rows of one query head against tiles of
// BN = 32 keys. Tiles start at absolute key positions that are multiples of
// BN, so the order of a row's accumulation does not depend on how the
// sequence was cut into steps.
// ---------------------------------------------------------------------------
#define GEN_BM 16
#define GEN_BN 32

template <typename T>
__global__ __launch_bounds__(256) void attn_general_kernel(
    const T* __restrict__ q, int q_stride, T* __restrict__ out, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, int num_pages, const int* __restrict__ block_table, int bt_stride,
    const int* __restrict__ cu_q, const int* __restrict__ kv_lens, int Hq, int Hkv, int D, int page,
    float scale, int window) {
  extern __shared__ float smem[];
  const int b = blockIdx.z;
  const int h = blockIdx.y;
  const int q0 = cu_q[b];
  const int q_len = cu_q[b + 1] - q0;
  const int m0 = blockIdx.x * GEN_BM;
  if (m0 >= q_len) return;
  const int kv_len = kv_lens[b];
  const int rows = min(GEN_BM, q_len - m0);
  const int first_pos = kv_len - q_len + m0;
  const int g = h / (Hq / Hkv);

  float* qs = smem;                         // [BM][D]
  float* kv = qs + GEN_BM * D;              // [BN][D + 1]
  float* ps = kv + GEN_BN * (D + 1);        // [BM][BN + 1]
  const int ldk = D + 1;
  const int t = threadIdx.x;
  const int r = t >> 4;    // query row of this thread
  const int sub = t & 15;  // its place among the 16 threads of the row
  const int nd = D >> 4;   // output columns per thread

  for (int idx = t; idx < GEN_BM * D; idx += 256) {
    const int rr = idx / D, d = idx - rr * D;
    qs[idx] = rr < rows ? to_float(q[(size_t)(q0 + m0 + rr) * q_stride + (size_t)h * D + d]) : 0.f;
  }

  float acc[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  const int my_pos = first_pos + r;
  const bool my_row = r < rows;

  const int k_end = first_pos + rows;  // one past the last key any row of the tile sees
  int k_begin = 0;
  if (window > 0) k_begin = max(0, first_pos - window + 1);
  k_begin -= k_begin % GEN_BN;

  for (int kt = k_begin; kt < k_end; kt += GEN_BN) {
    __syncthreads();
    // keys of this tile -> shared memory (zeros beyond k_end or for pages given back)
    for (int jj = r; jj < GEN_BN; jj += 16) {
      const int kj = kt + jj;
      const T* src = nullptr;
      if (kj < k_end) {
        const int pg = block_table[(size_t)b * bt_stride + kj / page];
        if (pg >= 0 && pg < num_pages) src = k_cache + (((size_t)pg * Hkv + g) * page + kj % page) * D;
      }
      for (int d = sub; d < D; d += 16) kv[jj * ldk + d] = src ? to_float(src[d]) : 0.f;
    }
    __syncthreads();
    float s[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int jj = sub + 16 * u;
      const int kj = kt + jj;
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot += qs[r * D + d] * kv[jj * ldk + d];
      bool seen = my_row && kj <= my_pos && kj < k_end;
      if (window > 0 && my_pos - kj >= window) seen = false;
      s[u] = seen ? dot * scale : -INFINITY;
    }
    float tile_max = fmaxf(s[0], s[1]);
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) tile_max = fmaxf(tile_max, __shfl_xor(tile_max, off, Q3_WAVE));
    const float m_new = fmaxf(m_run, tile_max);
    float alpha = 1.f, p[2] = {0.f, 0.f};
    if (m_new > -INFINITY) {
      alpha = expf(m_run - m_new);
      p[0] = expf(s[0] - m_new);
      p[1] = expf(s[1] - m_new);
    }
    float tile_sum = p[0] + p[1];
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) tile_sum += __shfl_xor(tile_sum, off, Q3_WAVE);
    l_run = l_run * alpha + tile_sum;
    m_run = m_new;
    ps[r * (GEN_BN + 1) + sub] = p[0];
    ps[r * (GEN_BN + 1) + sub + 16] = p[1];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] *= alpha;
    __syncthreads();
    // values of this tile replace the keys
    for (int jj = r; jj < GEN_BN; jj += 16) {
      const int kj = kt + jj;
      const T* src = nullptr;
      if (kj < k_end) {
        const int pg = block_table[(size_t)b * bt_stride + kj / page];
        if (pg >= 0 && pg < num_pages) src = v_cache + (((size_t)pg * Hkv + g) * page + kj % page) * D;
      }
      for (int d = sub; d < D; d += 16) kv[jj * ldk + d] = src ? to_float(src[d]) : 0.f;
    }
    __syncthreads();
    for (int jj = 0; jj < GEN_BN; ++jj) {
      const float pj = ps[r * (GEN_BN + 1) + jj];
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (i < nd) acc[i] += pj * kv[jj * ldk + sub + 16 * i];
    }
  }
  if (my_row) {
    const float inv = 1.f / l_run;
    T* o = out + (size_t)(q0 + m0 + r) * ((size_t)Hq * D) + (size_t)h * D;
#pragma unroll
    for (int i = 0; i < 16; ++i)
      if (i < nd) o[sub + 16 * i] = from_float<T>(acc[i] * inv);
  }
}

template <typename T>
static int launch_general(const void* q, int q_stride, void* out, const void* k_cache, const void* v_cache,
                          int num_pages, const int* block_table, int bt_stride, const int* cu_q,
                          const int* kv_lens, int B, int Hq, int Hkv, int D, int page, float scale,
                          int window, int max_q_len, hipStream_t stream) {
  const size_t smem = (size_t)(GEN_BM * D + GEN_BN * (D + 1) + GEN_BM * (GEN_BN + 1)) * sizeof(float);
  const dim3 grid((max_q_len + GEN_BM - 1) / GEN_BM, Hq, B);
  hipLaunchKernelGGL(attn_general_kernel<T>, grid, dim3(256), smem, stream, (const T*)q, q_stride, (T*)out,
                     (const T*)k_cache, (const T*)v_cache, num_pages, block_table, bt_stride, cu_q, kv_lens,
                     Hq, Hkv, D, page, scale, window);
  return q3_launch_status();
}

extern "C" int q3_paged_attention(const void* q, int q_stride, void* out, const void* k_cache,
                                  const void* v_cache, int num_pages, const int* block_table,
                                  int bt_stride, const int* cu_q, const int* kv_lens, int B, int T_, int Hq,
                                  int Hkv, int D, int page, float scale, int window, int max_q_len,
                                  int max_kv_len, int dtype, hipStream_t stream) {
  if (B <= 0 || T_ <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || page <= 0 || max_q_len <= 0)
    return Q3_ERR_BAD_ARGUMENT;
  if (D % 16 || D < 16 || D > 256) return Q3_ERR_UNSUPPORTED;
  if (B > 65535 || Hq > 65535) return Q3_ERR_UNSUPPORTED;
  (void)max_kv_len;
  Q3_DISPATCH_DTYPE(dtype, TT, return launch_general<TT>(q, q_stride, out, k_cache, v_cache, num_pages,
                                                        block_table, bt_stride, cu_q, kv_lens, B, Hq, Hkv,
                                                        D, page, scale, window, max_q_len, stream));
  return Q3_ERR_BAD_ARGUMENT;
}
