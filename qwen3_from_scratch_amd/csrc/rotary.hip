// Rotary position encoding: the [cos | sin] table, and the fused pass over a
// step's qkv rows: per-head RMSNorm of q and k, rotation, and the cache write.
#include "common.h"
#include "qk_prepare.h"

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

// ---------------------------------------------------------------------------
// The same work for bfloat16 with 16-byte accesses, for head sizes 16, 32, 64,
// 128 and 256 with full or no rotation: a query or key head is served by D / 16
// lanes, each holding eight elements of the head's first half and the eight
// that pair with them in the second half; values are transposed page by page
// through shared memory by a second kernel.
// ---------------------------------------------------------------------------
// grid (T, ceil(heads / heads_per_block)), 256 threads; LPH = D / 16 lanes per head. With
// STORE_V the value heads are handled here too, element by element into the transposed
// cache (for steps of few tokens, where a second launch would cost more than it saves).
template <typename W, int LPH, bool STORE_V>
__device__ __forceinline__ void qk_vec_body(
    int t, int head_block, bf16_t* __restrict__ qkv, const W* __restrict__ q_weight, const W* __restrict__ k_weight,
    float eps, const float* __restrict__ table, int max_pos, const int* __restrict__ positions,
    const int* __restrict__ seq_index, const int* __restrict__ block_table, int bt_stride, int bt_rows,
    bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache, int page_size, int num_pages, int Hq, int Hkv) {
  constexpr int D = LPH * 16, HALF = D / 2;
  const int head = head_block * (256 / LPH) + threadIdx.x / LPH;
  const int c = threadIdx.x % LPH;  // which eight of the half
  if (head >= Hq + (STORE_V ? 2 : 1) * Hkv) return;
  bf16_t* src = qkv + ((size_t)t * (Hq + 2 * Hkv) + head) * D;
  const int pos = positions[t];
  Half8 x1, x2;
  x1.u = *reinterpret_cast<const uint4*>(src + 8 * c);
  x2.u = *reinterpret_cast<const uint4*>(src + HALF + 8 * c);
  if (STORE_V && head >= Hq + Hkv) {
    if (v_cache == nullptr) return;
    const int sq = seq_index[t];
    const int blk = pos / page_size;
    if (sq < 0 || sq >= bt_rows || blk >= bt_stride || pos < 0) return;
    const int page = block_table[(size_t)sq * bt_stride + blk];
    if (page < 0 || page >= num_pages) return;
    bf16_t* o = v_cache + ((size_t)page * Hkv + (head - Hq - Hkv)) * D * page_size + (pos % page_size);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      o[(size_t)(8 * c + i) * page_size] = x1.e[i];
      o[(size_t)(HALF + 8 * c + i) * page_size] = x2.e[i];
    }
    return;
  }
  float a[8], b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = bf16_to_float(x1.e[i]);
    b[i] = bf16_to_float(x2.e[i]);
  }
  const W* w = head < Hq ? q_weight : k_weight;
  if (w != nullptr) {
    float ss = pairs_sum_of_squares(a, b);
#pragma unroll
    for (int off = LPH / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, Q3_WAVE);
    float wa[8], wb[8];
    load_weights8<W>(w + 8 * c, wa);
    load_weights8<W>(w + HALF + 8 * c, wb);
    pairs_normalise(a, b, head_norm_scale(ss, D, eps), wa, wb);
  }
  if (table != nullptr && pos >= 0 && pos < max_pos) {
    float cs[8], sn[8];
    load_weights8<float>(table + (size_t)pos * D + 8 * c, cs);
    load_weights8<float>(table + (size_t)pos * D + HALF + 8 * c, sn);
    pairs_rotate(a, b, cs, sn);
  }
  bf16_t* dst = src;
  if (head >= Hq) {
    dst = nullptr;
    if (k_cache != nullptr) {
      const int sq = seq_index[t];
      const int blk = pos / page_size;
      if (sq >= 0 && sq < bt_rows && blk < bt_stride && pos >= 0) {
        const int page = block_table[(size_t)sq * bt_stride + blk];
        if (page >= 0 && page < num_pages)
          dst = k_cache + (((size_t)page * Hkv + (head - Hq)) * page_size + (pos % page_size)) * D;
      }
    }
  }
  if (dst == nullptr) return;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    x1.e[i] = float_to_bf16(a[i]);
    x2.e[i] = float_to_bf16(b[i]);
  }
  *reinterpret_cast<uint4*>(dst + 8 * c) = x1.u;
  *reinterpret_cast<uint4*>(dst + HALF + 8 * c) = x2.u;
}

template <typename W, int LPH, bool STORE_V>
__global__ __launch_bounds__(256) void qk_norm_rope_store_vec_kernel(
    bf16_t* __restrict__ qkv, const W* __restrict__ q_weight, const W* __restrict__ k_weight, float eps,
    const float* __restrict__ table, int max_pos, const int* __restrict__ positions,
    const int* __restrict__ seq_index, const int* __restrict__ block_table, int bt_stride, int bt_rows,
    bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache, int page_size, int num_pages, int Hq, int Hkv) {
  qk_vec_body<W, LPH, STORE_V>(blockIdx.x, blockIdx.y, qkv, q_weight, k_weight, eps, table, max_pos, positions,
                               seq_index, block_table, bt_stride, bt_rows, k_cache, v_cache, page_size, num_pages,
                               Hq, Hkv);
}

// Values of this step into the transposed value cache, the work of one block for (logical
// page j of the step's span, key head, sequence): the rows of the up to
// `page_size` (<= 64) tokens that fall in the page are staged in shared memory and
// written as rows of the page, 16 bytes at a time where eight neighbouring slots
// are all written in this step, element by element otherwise.
template <int D>
__device__ __forceinline__ void store_values_body(
    int span_page, int g, int b, bf16_t (*tile)[D + 8], const bf16_t* __restrict__ qkv,
    const int* __restrict__ cu_q, const int* __restrict__ kv_lens, const int* __restrict__ block_table,
    int bt_stride, bf16_t* __restrict__ v_cache, int page_size, int num_pages, int Hq, int Hkv) {
  const int q0 = cu_q[b];
  const int q_len = cu_q[b + 1] - q0;
  if (q_len <= 0) return;
  const int first_pos = kv_lens[b] - q_len;
  const int blk = first_pos / page_size + span_page;        // logical page
  const int lo = max(first_pos, blk * page_size);           // positions written in it: [lo, hi)
  const int hi = min(first_pos + q_len, (blk + 1) * page_size);
  if (lo >= hi) return;
  const int page = block_table[(size_t)b * bt_stride + blk];
  if (page < 0 || page >= num_pages) return;
  const int heads = Hq + 2 * Hkv;
  const int n = hi - lo;
  for (int idx = threadIdx.x; idx < n * (D / 8); idx += 256) {
    const int r = idx / (D / 8), c = idx % (D / 8);
    const bf16_t* row = qkv + ((size_t)(q0 + lo - first_pos + r) * heads + Hq + Hkv + g) * D;
    *reinterpret_cast<uint4*>(&tile[r][8 * c]) = *reinterpret_cast<const uint4*>(row + 8 * c);
  }
  __syncthreads();
  const int slot_lo = lo - blk * page_size;
  bf16_t* base = v_cache + ((size_t)page * Hkv + g) * D * page_size;
  const int groups = page_size / 8;  // 16-byte groups of slots per row (page_size is a multiple of 8 here)
  for (int idx = threadIdx.x; idx < D * groups; idx += 256) {
    const int d = idx / groups, s8 = (idx % groups) * 8;
    if (s8 + 8 <= slot_lo || s8 >= slot_lo + n) continue;
    bf16_t* o = base + (size_t)d * page_size + s8;
    if (s8 >= slot_lo && s8 + 8 <= slot_lo + n) {
      Half8 h;
#pragma unroll
      for (int i = 0; i < 8; ++i) h.e[i] = tile[s8 - slot_lo + i][d];
      *reinterpret_cast<uint4*>(o) = h.u;
    } else {
      for (int i = 0; i < 8; ++i) {
        const int r = s8 + i - slot_lo;
        if (r >= 0 && r < n) o[i] = tile[r][d];
      }
    }
  }
}

// Both kinds of block in one launch, for steps of many tokens: the first `value_blocks` blocks
// (span_pages x Hkv x B of them) transpose values, the others prepare queries and keys. The
// two touch different parts of qkv and different caches, so they need no order, and a launch
// of its own for the values, which is short on work per block, would only add its latency.
template <typename W, int LPH>
__global__ __launch_bounds__(256) void qk_and_values_kernel(
    bf16_t* __restrict__ qkv, const W* __restrict__ q_weight, const W* __restrict__ k_weight, float eps,
    const float* __restrict__ table, int max_pos, const int* __restrict__ positions,
    const int* __restrict__ seq_index, const int* __restrict__ block_table, int bt_stride, int bt_rows,
    bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache, int page_size, int num_pages, int Hq, int Hkv,
    const int* __restrict__ cu_q, const int* __restrict__ kv_lens, int span_pages, int value_blocks,
    int head_blocks) {
  constexpr int D = LPH * 16;
  __shared__ bf16_t tile[64][D + 8];
  int id = blockIdx.x;
  if (id < value_blocks) {
    const int span_page = id % span_pages, g = (id / span_pages) % Hkv, b = id / (span_pages * Hkv);
    store_values_body<D>(span_page, g, b, tile, qkv, cu_q, kv_lens, block_table, bt_stride, v_cache, page_size,
                         num_pages, Hq, Hkv);
    return;
  }
  id -= value_blocks;
  qk_vec_body<W, LPH, false>(id / head_blocks, id % head_blocks, qkv, q_weight, k_weight, eps, table, max_pos,
                             positions, seq_index, block_table, bt_stride, bt_rows, k_cache, v_cache, page_size,
                             num_pages, Hq, Hkv);
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

template <typename W>
static int launch_qk_vec(void* qkv, const void* qw, const void* kw, float eps, const float* table, int max_pos,
                         const int* positions, const int* seq_index, const int* block_table, int bt_stride,
                         int bt_rows, void* k_cache, void* v_cache, int page_size, int num_pages, int T_, int Hq,
                         int Hkv, int D, const int* cu_q, const int* kv_lens, int B, int max_q_len,
                         hipStream_t stream) {
  const bool few = max_q_len < 8;  // values element by element by the lanes that prepare queries and keys
  const bool values_apart = v_cache != nullptr && !few;
  const int nheads = Hq + (few ? 2 : 1) * Hkv;
  const int span_pages = values_apart ? (max_q_len + page_size - 1) / page_size + 1 : 0;
  const long value_blocks = values_apart ? (long)span_pages * Hkv * B : 0;
#define Q3_QKV_LAUNCH(LPH)                                                                                    \
  do {                                                                                                        \
    const int head_blocks = (nheads + 256 / LPH - 1) / (256 / LPH);                                           \
    if (values_apart) {                                                                                       \
      const long blocks = value_blocks + (long)T_ * head_blocks;                                              \
      if (blocks > 0x7fffffffL) return Q3_ERR_UNSUPPORTED;                                                    \
      hipLaunchKernelGGL((qk_and_values_kernel<W, LPH>), dim3((unsigned)blocks), dim3(256), 0, stream,        \
                         (bf16_t*)qkv, (const W*)qw, (const W*)kw, eps, table, max_pos, positions, seq_index, \
                         block_table, bt_stride, bt_rows, (bf16_t*)k_cache, (bf16_t*)v_cache, page_size,      \
                         num_pages, Hq, Hkv, cu_q, kv_lens, span_pages, (int)value_blocks, head_blocks);      \
    } else if (few) {                                                                                         \
      hipLaunchKernelGGL((qk_norm_rope_store_vec_kernel<W, LPH, true>), dim3(T_, head_blocks), dim3(256), 0,  \
                         stream, (bf16_t*)qkv, (const W*)qw, (const W*)kw, eps, table, max_pos, positions,    \
                         seq_index, block_table, bt_stride, bt_rows, (bf16_t*)k_cache, (bf16_t*)v_cache,      \
                         page_size, num_pages, Hq, Hkv);                                                      \
    } else {                                                                                                  \
      hipLaunchKernelGGL((qk_norm_rope_store_vec_kernel<W, LPH, false>), dim3(T_, head_blocks), dim3(256), 0, \
                         stream, (bf16_t*)qkv, (const W*)qw, (const W*)kw, eps, table, max_pos, positions,    \
                         seq_index, block_table, bt_stride, bt_rows, (bf16_t*)k_cache, (bf16_t*)v_cache,      \
                         page_size, num_pages, Hq, Hkv);                                                      \
    }                                                                                                         \
  } while (0)
  switch (D) {
    case 16: Q3_QKV_LAUNCH(1); break;
    case 32: Q3_QKV_LAUNCH(2); break;
    case 64: Q3_QKV_LAUNCH(4); break;
    case 128: Q3_QKV_LAUNCH(8); break;
    case 256: Q3_QKV_LAUNCH(16); break;
    default: return Q3_ERR_UNSUPPORTED;
  }
#undef Q3_QKV_LAUNCH
  return q3_launch_status();
}

// `cu_q`, `kv_lens`, `B`, `max_q_len` describe the step's sequences (they may be null / 0: then
// only the one-wavefront-per-head kernel is used). `max_kv_len`: what the host knows of the
// step's last position + 1 (0: nothing); a step that would pass the rotation table's end is
// refused, since a row without its rotation is a wrong answer, not an error anyone sees.
extern "C" int q3_qk_norm_rope_store(void* qkv, const void* q_weight, const void* k_weight, int w_dtype,
                                     float eps, const float* table, int rotary_dim, int max_pos,
                                     const int* positions, const int* seq_index, const int* block_table,
                                     int bt_stride, int bt_rows, void* k_cache, void* v_cache,
                                     int page_size, int num_pages, int T_, int Hq, int Hkv, int D,
                                     int act_dtype, const int* cu_q, const int* kv_lens, int B, int max_q_len,
                                     int max_kv_len, hipStream_t stream) {
  if (table && max_kv_len > max_pos) return Q3_ERR_BAD_ARGUMENT;
  if (T_ <= 0 || Hq <= 0 || Hkv <= 0 || D <= 0 || (Hq + 2 * Hkv + 3) / 4 > 65535) return Q3_ERR_BAD_ARGUMENT;
  if (table && (rotary_dim <= 0 || rotary_dim % 2 || rotary_dim > D)) return Q3_ERR_BAD_ARGUMENT;
  if (k_cache && (!v_cache || !block_table || page_size <= 0)) return Q3_ERR_BAD_ARGUMENT;
  if ((q_weight == nullptr) != (k_weight == nullptr)) return Q3_ERR_BAD_ARGUMENT;
  const bool pow2_head = D == 16 || D == 32 || D == 64 || D == 128 || D == 256;
  const bool vec = act_dtype == Q3_BF16 && pow2_head && (!table || rotary_dim == D) &&
                   (!k_cache || (cu_q && kv_lens && B > 0 && B <= 65535 && max_q_len > 0 && page_size % 8 == 0 &&
                                 page_size <= 64));
  if (vec) {
    Q3_DISPATCH_DTYPE(w_dtype, WW, return (launch_qk_vec<WW>(
        qkv, q_weight, k_weight, eps, table, max_pos, positions, seq_index, block_table, bt_stride, bt_rows,
        k_cache, v_cache, page_size, num_pages, T_, Hq, Hkv, D, cu_q, kv_lens, B, max_q_len, stream)));
  }
  Q3_DISPATCH_DTYPE(act_dtype, TT, Q3_DISPATCH_DTYPE(w_dtype, WW, return (launch_qk<TT, WW>(
      qkv, q_weight, k_weight, eps, table, rotary_dim, max_pos, positions, seq_index, block_table,
      bt_stride, bt_rows, k_cache, v_cache, page_size, num_pages, T_, Hq, Hkv, D, stream))));
  return Q3_ERR_BAD_ARGUMENT;
}
