// Causal softmax attention of packed query rows over paged keys and values.
//
// Layout: the key cache is (pages, Hkv, page, D), the value cache is transposed
// within the page, (pages, Hkv, D, page); sequence b's key j lives in page
// block_table[b, j / page] at slot j % page. Query row i of a sequence with q_len
// rows and kv_len keys sits at position kv_len - q_len + i and sees keys at
// positions <= its own, and, with a window w > 0, only those fewer than w behind.
#include "common.h"
#include "qk_prepare.h"

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
        if (pg >= 0 && pg < num_pages) src = v_cache + ((size_t)pg * Hkv + g) * D * page + kj % page;
      }
      for (int d = sub; d < D; d += 16) kv[jj * ldk + d] = src ? to_float(src[(size_t)d * page]) : 0.f;
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


// ---------------------------------------------------------------------------
// The matrix-core kernels: bfloat16, head size 64 or 128, page size a multiple
// of 16. One wavefront works on query rows in blocks of 16 against tiles of 32
// keys, with v_mfma_f32_16x16x32_bf16:
//
//   S^T (keys x rows)  = K (keys x d) . Q^T (d x rows)        A = K rows, B = Q rows
//   O^T (d x rows)    += V^T (d x keys) . P^T (keys x rows)   A = V^T rows, B = P
//
// Both products put the query row in the lane's low four bits (lane % 16), so
// the softmax statistics of a row, its probabilities and its output
// accumulators all live in the same lanes and nothing is transposed. A lane of
// group g = lane / 16 holds, after S^T, the scores of keys 4g..4g+3 of each of
// the tile's two 16-key blocks; these eight are exactly the keys its P operand
// multiplies, and the value cache is transposed within the page so that the
// matching V^T operand is two 8-byte loads. K operands are 16-byte loads. No
// shared memory is used on the way from the cache to the matrix cores.
//
// A "row" is a (token, query head of the group) pair: row r of a workgroup is
// token r / G, head r % G of the key head's group, so that all heads of a group
// share each key and value load.
// ---------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

union Pack16 {
  uint4 u;
  uint2 h[2];
  bf16x8_t v;
  __bf16 e[8];
};

#define FAST_TILE 32

// v_exp_f32: 2^x without the library routine's handling of results below the
// normal range, which are zero for our purposes (arguments are <= 0).
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// The softmax update of one block of 16 rows for one 32-key tile. s: this lane's
// eight raw scores (two key blocks of four). Scores enter scaled by scale_log2
// only inside the exponent: p = 2^(s * scale - m), with m the running maximum of
// s * scale. `full` says that every key of the tile is visible to every row of
// the wavefront, so no masking is needed. Returns the probabilities as the P
// operand and rescales the accumulators only if some row's maximum moved.
template <int NB>
__device__ __forceinline__ Pack16 softmax_step(const f32x4_t (&s)[2], bool full, int key0, int grp, int row_pos,
                                               int window, float scale_log2, float& m_run, float& l_run,
                                               f32x4_t (&acc)[NB]) {
  float v[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = s[j >> 2][j & 3];
  if (!full) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int key = key0 + 16 * (j >> 2) + 4 * grp + (j & 3);
      bool seen = key <= row_pos;
      if (window > 0 && row_pos - key >= window) seen = false;
      if (!seen) v[j] = -INFINITY;
    }
  }
  float mx = fmaxf(fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3])), fmaxf(fmaxf(v[4], v[5]), fmaxf(v[6], v[7])));
  mx = quad_rows_max(mx);
  const float m_new = fmaxf(m_run, mx * scale_log2);
  Pack16 p;
  float sum = 0.f;
  if (m_new > -INFINITY) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float e = fast_exp2(fmaf(v[j], scale_log2, -m_new));
      sum += e;
      p.e[j] = (__bf16)e;
    }
  } else {
    p.u = make_uint4(0, 0, 0, 0);
  }
  const bool moved = m_new != m_run;
  if (__builtin_amdgcn_ballot_w64(moved) != 0) {
    const float alpha = m_new > -INFINITY ? fast_exp2(m_run - m_new) : 1.f;
    l_run *= alpha;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[nb] *= alpha;
    m_run = m_new;
  }
  l_run += sum;
  return p;
}

// Where the two 16-key blocks of the tile that starts at key0 lie in the caches
// (nullptr for a block past the sequence's end or in a page given back), from
// this lane's point of view: its K row and its V^T row.
struct TileAddr {
  const bf16_t* k[2];
  const bf16_t* v[2];
};

__device__ __forceinline__ TileAddr tile_addr(const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
                                              int num_pages, const int* __restrict__ bt_row, int Hkv, int g_kv,
                                              int page, int D, int key0, int kv_len) {
  const int lane = threadIdx.x & 63;
  const int col = lane & 15, grp = lane >> 4;
  TileAddr t;
#pragma unroll
  for (int kb = 0; kb < 2; ++kb) {
    const int kbase = key0 + 16 * kb;
    t.k[kb] = nullptr;
    t.v[kb] = nullptr;
    if (kbase < kv_len) {
      const int pg = bt_row[kbase / page];
      if (pg >= 0 && pg < num_pages) {
        const int slot0 = kbase % page;
        t.k[kb] = k_cache + (((size_t)pg * Hkv + g_kv) * page + slot0 + col) * D + 8 * grp;
        t.v[kb] = v_cache + (((size_t)pg * Hkv + g_kv) * D + col) * page + slot0 + 4 * grp;
      }
    }
  }
  return t;
}

// The same in two halves, for a block that does not have the sequence's length in hand yet:
// the table entries of a tile's two blocks of 16 keys (-1 where the table has none: entries past
// a sequence's pages are -1), and the addresses from them. Keys past the sequence's end inside
// its last page hold anything; the caller masks them.
struct TilePages {
  int pg[2];
};

__device__ __forceinline__ TilePages tile_pages(const int* __restrict__ bt_row, int bt_stride, int page, int key0) {
  TilePages p;
#pragma unroll
  for (int kb = 0; kb < 2; ++kb) {
    const int entry = (key0 + 16 * kb) / page;
    p.pg[kb] = entry < bt_stride ? bt_row[entry] : -1;
  }
  return p;
}

__device__ __forceinline__ TileAddr tile_addr_of(const TilePages& p, const bf16_t* __restrict__ k_cache,
                                                 const bf16_t* __restrict__ v_cache, int num_pages, int Hkv, int g_kv,
                                                 int page, int D, int key0) {
  const int lane = threadIdx.x & 63;
  const int col = lane & 15, grp = lane >> 4;
  TileAddr t;
#pragma unroll
  for (int kb = 0; kb < 2; ++kb) {
    t.k[kb] = nullptr;
    t.v[kb] = nullptr;
    const int pg = p.pg[kb];
    if (pg >= 0 && pg < num_pages) {
      const int slot0 = (key0 + 16 * kb) % page;
      t.k[kb] = k_cache + (((size_t)pg * Hkv + g_kv) * page + slot0 + col) * D + 8 * grp;
      t.v[kb] = v_cache + (((size_t)pg * Hkv + g_kv) * D + col) * page + slot0 + 4 * grp;
    }
  }
  return t;
}

// The K operands of a tile: [key block][d step].
template <int D>
__device__ __forceinline__ void load_keys(Pack16 (&a)[2][D / 32], const TileAddr& t) {
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int i = 0; i < D / 32; ++i) {
      if (t.k[kb])
        a[kb][i].u = *reinterpret_cast<const uint4*>(t.k[kb] + 32 * i);
      else
        a[kb][i].u = make_uint4(0, 0, 0, 0);
    }
}

// Scores, softmax update and value accumulation of one 32-key tile for QB
// blocks of 16 rows, with the tile's K operands already in registers. row_pos[qb]:
// position of this lane's row, below zero for a row that does not exist. m, l:
// running maximum (log2 domain) and this lane's share of the running sum. The
// value loads are issued first and meet the probabilities after the softmax.
// The V^T operands of a tile, one per block of 16 output columns.
template <int D>
__device__ __forceinline__ void load_values(Pack16 (&vt)[D / 16], const TileAddr& t, int page) {
#pragma unroll
  for (int nb = 0; nb < D / 16; ++nb)
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      if (t.v[kb])
        vt[nb].h[kb] = *reinterpret_cast<const uint2*>(t.v[kb] + (size_t)16 * nb * page);
      else
        vt[nb].h[kb] = make_uint2(0, 0);
    }
}

template <int D, int QB>
__device__ __forceinline__ void attend_tile(const Pack16 (&qreg)[QB][D / 32], const Pack16 (&a)[2][D / 32],
                                            Pack16 (&vt)[D / 16], int key0, int kv_len,
                                            const int (&row_pos)[QB], int window, float scale_log2,
                                            f32x4_t (&acc)[QB][D / 16], float (&m_run)[QB], float (&l_run)[QB]) {
  const int lane = threadIdx.x & 63;
  const int grp = lane >> 4;
  f32x4_t s[QB][2];
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      f32x4_t c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < D / 32; ++i)
        c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[kb][i].v, qreg[qb][i].v, c, 0, 0, 0);
      s[qb][kb] = c;
    }
  Pack16 p[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb)
    p[qb] = softmax_step<D / 16>(s[qb], false, key0, grp, row_pos[qb], window, scale_log2, m_run[qb], l_run[qb],
                                 acc[qb]);
  if (key0 + FAST_TILE > kv_len) {  // slots past the sequence's end hold anything: zero them, 0 * NaN is NaN
#pragma unroll
    for (int nb = 0; nb < D / 16; ++nb)
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (key0 + 16 * (j >> 2) + 4 * grp + (j & 3) >= kv_len) vt[nb].e[j] = (__bf16)0.f;
  }
#pragma unroll
  for (int nb = 0; nb < D / 16; ++nb)
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
      acc[qb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vt[nb].v, p[qb].v, acc[qb][nb], 0, 0, 0);
}

// All tiles first, first + step, ... below last for one wavefront: the value loads of a
// tile and the key loads of the next one are issued before the tile's arithmetic. The
// first tile's keys are loaded by the caller (`first_tile_keys`), who may have other work
// to do while they travel.
template <int D>
__device__ __forceinline__ TileAddr first_tile_keys(Pack16 (&a_cur)[2][D / 32], const bf16_t* __restrict__ k_cache,
                                                    const bf16_t* __restrict__ v_cache, int num_pages,
                                                    const int* __restrict__ bt_row, int Hkv, int g_kv, int page,
                                                    int first, int last, int kv_len) {
  TileAddr t{};
  if (first >= last) return t;
  t = tile_addr(k_cache, v_cache, num_pages, bt_row, Hkv, g_kv, page, D, first * FAST_TILE, kv_len);
  load_keys<D>(a_cur, t);
  return t;
}

template <int D, int QB>
__device__ __forceinline__ void attend_tiles(const Pack16 (&qreg)[QB][D / 32], Pack16 (&a_cur)[2][D / 32],
                                             TileAddr t_cur, const bf16_t* __restrict__ k_cache,
                                             const bf16_t* __restrict__ v_cache, int num_pages,
                                             const int* __restrict__ bt_row, int Hkv, int g_kv, int page, int first,
                                             int last, int step, int kv_len, const int (&row_pos)[QB], int window,
                                             float scale_log2, f32x4_t (&acc)[QB][D / 16], float (&m_run)[QB],
                                             float (&l_run)[QB]) {
  if (first >= last) return;
  Pack16 a_nxt[2][D / 32], vt[D / 16];
  for (int t = first; t < last; t += step) {
    load_values<D>(vt, t_cur, page);
    const bool more = t + step < last;
    if (more) {
      t_cur = tile_addr(k_cache, v_cache, num_pages, bt_row, Hkv, g_kv, page, D, (t + step) * FAST_TILE, kv_len);
      load_keys<D>(a_nxt, t_cur);
    }
    attend_tile<D, QB>(qreg, a_cur, vt, t * FAST_TILE, kv_len, row_pos, window, scale_log2, acc, m_run, l_run);
    if (more) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < D / 32; ++i) a_cur[kb][i] = a_nxt[kb][i];
    }
  }
}

// The same walk for a wavefront whose tiles are known before the sequence's length is (tiles
// first, first + step, ... of the whole sequence): the caller has the first tile's keys on their
// and values on their way (`a_cur`, `v_cur`) and the second tile's table entries asked for (`p_nxt`);
// every turn asks for the table entries two tiles ahead, so that no key load waits for a table load.
template <int D, int QB>
__device__ __forceinline__ void attend_tiles_ahead(const Pack16 (&qreg)[QB][D / 32], Pack16 (&a_cur)[2][D / 32],
                                                   Pack16 (&v_cur)[D / 16], TilePages p_nxt,
                                                   const bf16_t* __restrict__ k_cache,
                                                   const bf16_t* __restrict__ v_cache, int num_pages,
                                                   const int* __restrict__ bt_row, int bt_stride, int Hkv, int g_kv,
                                                   int page, int first, int last, int step, int kv_len,
                                                   const int (&row_pos)[QB], int window, float scale_log2,
                                                   f32x4_t (&acc)[QB][D / 16], float (&m_run)[QB],
                                                   float (&l_run)[QB]) {
  if (first >= last) return;
  // a tile's keys and values are asked for together, a whole tile before they are used: a
  // wavefront with two or three tiles (few requests, each over a few thousand keys) then waits
  // for memory once per tile, not twice
  Pack16 a_nxt[2][D / 32], v_nxt[D / 16];
  for (int t = first; t < last; t += step) {
    const bool more = t + step < last;
    if (more) {
      const TileAddr t_nxt = tile_addr_of(p_nxt, k_cache, v_cache, num_pages, Hkv, g_kv, page, D, (t + step) * FAST_TILE);
      load_keys<D>(a_nxt, t_nxt);
      load_values<D>(v_nxt, t_nxt, page);
      p_nxt = tile_pages(bt_row, bt_stride, page, (t + 2 * step) * FAST_TILE);
    }
    attend_tile<D, QB>(qreg, a_cur, v_cur, t * FAST_TILE, kv_len, row_pos, window, scale_log2, acc, m_run, l_run);
    if (more) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < D / 32; ++i) a_cur[kb][i] = a_nxt[kb][i];
#pragma unroll
      for (int nb = 0; nb < D / 16; ++nb) v_cur[nb] = v_nxt[nb];
    }
  }
}

// ---- sequences with few rows (q_len * G <= 16): decoding ---------------------
// grid (splits, Hkv, B), 256 threads. The four wavefronts of a block take the
// tiles of the block's share of the keys in turn and are merged through shared
// memory; with more than one split the block leaves an unnormalised partial
// result (maximum, sum, accumulator) in the workspace for the reduction kernel.
// With PREP the kernel also does what the preparation kernel does for a step of single
// tokens (q_len = 1 everywhere): `q` is then the step's raw [q | k | v] rows. Every block
// normalises and rotates its own query rows on the way into the registers. If the step's
// key and value are to be stored (`prep.k_cache`), the block of the last split (the one
// with the fewest tiles) normalises and rotates the new key, writes it and the new value
// into the cache for later steps, and adds the new key's share of the result itself, from
// shared memory (one score per row, the value as it is) when it merges its wavefronts. No
// block reads the new position from the cache: they read what earlier steps wrote, so no
// read waits for a write.
// Without a window (AHEAD) a wavefront's tiles are every (4 x splits)-th of the whole sequence,
// so its first tile is known before the sequence's length is, and a tile's keys and values
// travel together, one tile ahead of their use. Measured at batch 8 over 2,100 keys: 25.2 us
// with the merge against 26.0 before; with 2, 4, 16, 32 splits instead of 8: 33, 27, 31, 48 us;
// one request: 14 us (16 or 32 splits), which is what two launches and their chains of
// dependent loads (length, table entry, keys; then the partial results) cost with no data at all.
struct DecodePrep {
  const void* q_weight;  // (D,) or null: no norm
  const void* k_weight;
  float eps;
  const float* table;    // (max_pos, D): cos | sin, or null: no rotation
  int max_pos;
  bf16_t* k_cache;       // writable views of the caches, or null: nothing is stored
  bf16_t* v_cache;
};

// One query row's operand registers from its raw values: lane (col, grp) holds elements
// 32 i + 8 grp + j; the pairs (d, d + D / 2) are registers i and i + D / 64 of the same lane.
// The sums take the order of the preparation kernel's butterfly (its lane c = 4 i + grp).
template <int D, typename W>
__device__ __forceinline__ void prepare_query(Pack16 (&qreg)[D / 32], const W* weight, float eps,
                                              const float* table_row, int grp) {
  constexpr int HI = D / 64;
  float a[HI][8], b[HI][8];
#pragma unroll
  for (int i = 0; i < HI; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      a[i][j] = (float)qreg[i].e[j];
      b[i][j] = (float)qreg[i + HI].e[j];
    }
  if (weight != nullptr) {
    float ss = pairs_sum_of_squares(a[0], b[0]);
    if constexpr (HI == 2) ss += pairs_sum_of_squares(a[1], b[1]);
    ss += __shfl_xor(ss, 32, 64);
    ss += __shfl_xor(ss, 16, 64);
    const float scale = head_norm_scale(ss, D, eps);
#pragma unroll
    for (int i = 0; i < HI; ++i) {
      float wa[8], wb[8];
      load_weights8<W>(weight + 32 * i + 8 * grp, wa);
      load_weights8<W>(weight + D / 2 + 32 * i + 8 * grp, wb);
      pairs_normalise(a[i], b[i], scale, wa, wb);
    }
  }
  if (table_row != nullptr) {
#pragma unroll
    for (int i = 0; i < HI; ++i) {
      float cs[8], sn[8];
      load_weights8<float>(table_row + 32 * i + 8 * grp, cs);
      load_weights8<float>(table_row + D / 2 + 32 * i + 8 * grp, sn);
      pairs_rotate(a[i], b[i], cs, sn);
    }
  }
#pragma unroll
  for (int i = 0; i < HI; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      qreg[i].e[j] = (__bf16)a[i][j];
      qreg[i + HI].e[j] = (__bf16)b[i][j];
    }
}

// The new key of head g_kv (the first D / 16 lanes of the block's last wavefront, as the
// preparation kernel's lanes) and the new value (the first D / 16 lanes of the wavefront
// before it) of the token whose raw row is `row`, into
// slot pos % page of `pg` (if there is such a page) and, as the cache's rounded numbers, into
// shared memory.
template <int D, typename W>
__device__ __forceinline__ void store_new_key_value(const bf16_t* row, int Hq, int Hkv, int g_kv, const W* k_weight,
                                                    float eps, const float* table_row, bf16_t* k_cache,
                                                    bf16_t* v_cache, int pg, int page, int slot, float* sh_k,
                                                    float* sh_v) {
  constexpr int LPH = D / 16, HALF = D / 2;
  const int t = threadIdx.x;
  if (t >= 192 && t < 192 + LPH) {
    const int c = t - 192;
    const bf16_t* src = row + (size_t)(Hq + g_kv) * D;
    Half8 x1, x2;
    x1.u = *reinterpret_cast<const uint4*>(src + 8 * c);
    x2.u = *reinterpret_cast<const uint4*>(src + HALF + 8 * c);
    float a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      a[i] = bf16_to_float(x1.e[i]);
      b[i] = bf16_to_float(x2.e[i]);
    }
    if (k_weight != nullptr) {
      float ss = pairs_sum_of_squares(a, b);
#pragma unroll
      for (int off = LPH / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
      float wa[8], wb[8];
      load_weights8<W>(k_weight + 8 * c, wa);
      load_weights8<W>(k_weight + HALF + 8 * c, wb);
      pairs_normalise(a, b, head_norm_scale(ss, D, eps), wa, wb);
    }
    if (table_row != nullptr) {
      float cs[8], sn[8];
      load_weights8<float>(table_row + 8 * c, cs);
      load_weights8<float>(table_row + HALF + 8 * c, sn);
      pairs_rotate(a, b, cs, sn);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      x1.e[i] = float_to_bf16(a[i]);
      x2.e[i] = float_to_bf16(b[i]);
      sh_k[8 * c + i] = bf16_to_float(x1.e[i]);
      sh_k[HALF + 8 * c + i] = bf16_to_float(x2.e[i]);
    }
    if (pg >= 0) {
      bf16_t* dst = k_cache + (((size_t)pg * Hkv + g_kv) * page + slot) * D;
      *reinterpret_cast<uint4*>(dst + 8 * c) = x1.u;
      *reinterpret_cast<uint4*>(dst + HALF + 8 * c) = x2.u;
    }
  } else if (t >= 128 && t < 128 + LPH) {
    const int c = t - 128;
    const bf16_t* src = row + (size_t)(Hq + Hkv + g_kv) * D;
    Half8 x1, x2;
    x1.u = *reinterpret_cast<const uint4*>(src + 8 * c);
    x2.u = *reinterpret_cast<const uint4*>(src + HALF + 8 * c);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      sh_v[8 * c + i] = bf16_to_float(x1.e[i]);
      sh_v[HALF + 8 * c + i] = bf16_to_float(x2.e[i]);
    }
    if (pg >= 0) {
      bf16_t* o = v_cache + ((size_t)pg * Hkv + g_kv) * D * page + slot;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        o[(size_t)(8 * c + i) * page] = x1.e[i];
        o[(size_t)(HALF + 8 * c + i) * page] = x2.e[i];
      }
    }
  }
}

template <int D, bool PREP, typename W, bool AHEAD>
__global__ __launch_bounds__(256) void attn_decode_kernel(
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, int num_pages, const int* __restrict__ block_table, int bt_stride,
    const int* __restrict__ cu_q, const int* __restrict__ kv_lens, int Hq, int Hkv, int page, float scale_log2,
    int window, int splits, float* __restrict__ ws_acc, float* __restrict__ ws_ml, DecodePrep prep) {
  const int b = blockIdx.z, g_kv = blockIdx.y, split = blockIdx.x;
  const int G = Hq / Hkv;
  // a step of single tokens (PREP): sequence b's token is row b, and nothing is read to know it
  const int q0 = PREP ? b : cu_q[b];
  const int q_len = PREP ? 1 : cu_q[b + 1] - q0;
  if (q_len <= 0 || q_len * G > 16) return;  // the other kernel's sequence
  const int* bt_row = block_table + (size_t)b * bt_stride;
  // Without a window a wavefront's tiles are first, first + step, ... of the whole sequence, known
  // before its length is: the table entries and then the keys of the first tile are asked for
  // beside the length, not after it.
  // (AHEAD: the host launches this form when there is no window.)
  constexpr bool ahead = AHEAD;
  const int kv_len = kv_lens[b];
  const int wave_of_block = threadIdx.x >> 6;
  const int ahead_first = split * 4 + wave_of_block, ahead_step = 4 * splits;
  Pack16 a_first[2][D / 32], v_first[ahead ? D / 16 : 1];
  TileAddr t_first{};
  TilePages p_second{};
  if constexpr (ahead) {
    t_first = tile_addr_of(tile_pages(bt_row, bt_stride, page, ahead_first * FAST_TILE), k_cache, v_cache, num_pages,
                           Hkv, g_kv, page, D, ahead_first * FAST_TILE);
    load_keys<D>(a_first, t_first);
    load_values<D>(v_first, t_first, page);
    p_second = tile_pages(bt_row, bt_stride, page, (ahead_first + ahead_step) * FAST_TILE);
  }
  if (PREP && (q_len != 1 || kv_len < 1)) {
    // not a step of single tokens (the host sends no such row): the row's output is zero, and
    // the merge finds an empty share in this block's place, not whatever the workspace held
    for (int i = threadIdx.x; i < q_len * G * D; i += blockDim.x) {
      const int r = i / D, d = i - r * D;
      if (splits == 1) {
        out[(size_t)(q0 + r / G) * Hq * D + (size_t)(g_kv * G + r % G) * D + d] = float_to_bf16(0.f);
      } else {
        const size_t slot = (((size_t)b * Hkv + g_kv) * splits + split) * 16 + r;
        ws_acc[slot * D + d] = 0.f;
        if (d == 0) {
          ws_ml[slot * 2] = -INFINITY;
          ws_ml[slot * 2 + 1] = 0.f;
        }
      }
    }
    return;
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int rows = q_len * G;
  const int first_pos = kv_len - q_len;
  // the new key is not in the cache yet: the last split's block brings it
  const bool fresh = PREP && prep.k_cache != nullptr;
  const bool brings_new = fresh && split == splits - 1;  // uniform in the block
  const float* table_row = nullptr;
  if constexpr (PREP) {
    if (prep.table != nullptr && first_pos < prep.max_pos) table_row = prep.table + (size_t)first_pos * D;
  }
  __shared__ float sh_k[PREP ? D : 1], sh_v[PREP ? D : 1];

  Pack16 qreg[1][D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i) {
    if (col < rows)
      qreg[0][i].u = *reinterpret_cast<const uint4*>(q + (size_t)(q0 + col / G) * q_stride +
                                                    (size_t)(g_kv * G + col % G) * D + 32 * i + 8 * grp);
    else
      qreg[0][i].u = make_uint4(0, 0, 0, 0);
  }

  // with a fresh key the cache is read up to the position before it: the rows then stand one
  // position earlier for the masks, and the window, which counts the new key, is one shorter
  const int kv_seen = fresh ? kv_len - 1 : kv_len;
  const int win = (fresh && window > 0) ? window - 1 : window;
  int row_pos[1];
  row_pos[0] = col < rows ? first_pos + col / G - (fresh ? 1 : 0) : -1;
  int tile_lo = 0;
  if (window > 0) tile_lo = max(0, first_pos - window + 1) / FAST_TILE;
  int tile_hi = (kv_seen + FAST_TILE - 1) / FAST_TILE;
  if (fresh && window == 1) tile_hi = tile_lo;  // the new key alone is visible
  const int per_split = (max(tile_hi - tile_lo, 0) + splits - 1) / splits;
  const int t0 = tile_lo + split * per_split;
  const int t1 = min(tile_hi, t0 + per_split);
  // the first tile's keys are on their way while the query rows are prepared
  if constexpr (!ahead)
    t_first = first_tile_keys<D>(a_first, k_cache, v_cache, num_pages, bt_row, Hkv, g_kv, page, t0 + wave, t1, kv_seen);
  float m_new = -INFINITY;  // in the last wavefront: the new key's score for this lane's row
  if constexpr (PREP) {
    prepare_query<D, W>(qreg[0], static_cast<const W*>(prep.q_weight), prep.eps, table_row, grp);
    if (brings_new) {
      // the last two wavefronts, which have the fewest tiles, lend a few lanes: the key and the
      // value into the cache for later steps, and into shared memory for this one (the value
      // is read after the barriers of the merge, the key after the barrier below)
      const int blk = first_pos / page;
      int pg = blk < bt_stride ? bt_row[blk] : -1;
      if (pg >= num_pages) pg = -1;
      store_new_key_value<D, W>(q + (size_t)q0 * q_stride, Hq, Hkv, g_kv, static_cast<const W*>(prep.k_weight),
                                prep.eps, table_row, prep.k_cache, prep.v_cache, pg, page, first_pos % page, sh_k,
                                sh_v);
      __syncthreads();  // the key is in shared memory for all lanes that read it (brings_new is the block's)
      if (wave == 3) {
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < D / 32; ++i)
#pragma unroll
          for (int j = 0; j < 8; ++j) dot = fmaf((float)qreg[0][i].e[j], sh_k[32 * i + 8 * grp + j], dot);
        dot += __shfl_xor(dot, 16, 64);
        dot += __shfl_xor(dot, 32, 64);
        if (col < rows) m_new = dot * scale_log2;
      }
    }
  }

  f32x4_t acc[1][D / 16];
#pragma unroll
  for (int nb = 0; nb < D / 16; ++nb) acc[0][nb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m_run[1] = {-INFINITY}, l_run[1] = {0.f};
  if constexpr (ahead)
    attend_tiles_ahead<D, 1>(qreg, a_first, v_first, p_second, k_cache, v_cache, num_pages, bt_row, bt_stride, Hkv,
                             g_kv, page, ahead_first, tile_hi, ahead_step, kv_seen, row_pos, win, scale_log2, acc,
                             m_run, l_run);
  else
    attend_tiles<D, 1>(qreg, a_first, t_first, k_cache, v_cache, num_pages, bt_row, Hkv, g_kv, page, t0 + wave, t1, 4,
                       kv_seen, row_pos, win, scale_log2, acc, m_run, l_run);

  // this lane's sum covers its own keys only
  float l = l_run[0];
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);

  // the merge of the four wavefronts, and of the new key as a fifth contribution of one key:
  // its score is its maximum, its sum is one, its accumulator is the value itself
  __shared__ float sh_m[5][16], sh_l[4][16];
  __shared__ float sh_acc[4][16][D + 4];
  if (grp == 0) {
    sh_m[wave][col] = m_run[0];
    sh_l[wave][col] = l;
  }
  if (wave == 3 && grp == 0) sh_m[4][col] = m_new;
  __syncthreads();
  float m_all = fmaxf(fmaxf(sh_m[0][col], sh_m[1][col]), fmaxf(sh_m[2][col], sh_m[3][col]));
  m_all = fmaxf(m_all, sh_m[4][col]);
  const float w_mine = m_run[0] > -INFINITY ? exp2f(m_run[0] - m_all) : 0.f;
  if (col < rows) {
#pragma unroll
    for (int nb = 0; nb < D / 16; ++nb)
#pragma unroll
      for (int j = 0; j < 4; ++j) sh_acc[wave][col][16 * nb + 4 * grp + j] = acc[0][nb][j] * w_mine;
  }
  __syncthreads();
  // 256 threads: thread -> (row = t / 16, d = t % 16 + 16 k)
  const int r = threadIdx.x >> 4, dd = threadIdx.x & 15;
  if (r >= rows) return;
  const float m5 = sh_m[4][r];
  const float mr = fmaxf(fmaxf(fmaxf(sh_m[0][r], sh_m[1][r]), fmaxf(sh_m[2][r], sh_m[3][r])), m5);
  const float w5 = m5 > -INFINITY ? exp2f(m5 - mr) : 0.f;
  float lr = w5;
#pragma unroll
  for (int w = 0; w < 4; ++w) lr += sh_m[w][r] > -INFINITY ? sh_l[w][r] * exp2f(sh_m[w][r] - mr) : 0.f;
  const int token = q0 + r / G, head = g_kv * G + r % G;
  if (splits == 1) {
    const float inv = 1.f / lr;
    for (int d = dd; d < D; d += 16) {
      float o = sh_acc[0][r][d] + sh_acc[1][r][d] + sh_acc[2][r][d] + sh_acc[3][r][d];
      if (PREP && w5 > 0.f) o += sh_v[d] * w5;
      out[(size_t)token * Hq * D + (size_t)head * D + d] = float_to_bf16(o * inv);
    }
  } else {
    const size_t slot = (((size_t)b * Hkv + g_kv) * splits + split) * 16 + r;
    for (int d = dd; d < D; d += 16) {
      float o = sh_acc[0][r][d] + sh_acc[1][r][d] + sh_acc[2][r][d] + sh_acc[3][r][d];
      if (PREP && w5 > 0.f) o += sh_v[d] * w5;
      ws_acc[slot * D + d] = o;
    }
    if (dd == 0) {
      ws_ml[slot * 2] = mr;
      ws_ml[slot * 2 + 1] = lr;
    }
  }
}

// Merge the splits' partial results: grid (Hkv, B), 256 threads; splits <= 64.
// (A kernel of its own rather than the work of the decode kernel's last-arriving
// block: the device-scope fences that needs write back and invalidate each XCD's
// L2, which measured three times slower than this second launch.)
// The kernel is a chain of latencies, so it asks for as much as it can at once: a thread
// owns four neighbouring output elements and every `groups`-th split (groups = as many as
// 256 threads allow), loads its first eight partial accumulators before anything else,
// then the maxima and sums, from which a wavefront forms a row's weights (a split per lane)
// and leaves them in shared memory; the groups' sums meet there too.
#define MAX_SPLITS 64
#define REDUCE_BATCH 8
template <int D>
__global__ __launch_bounds__(256) void attn_decode_reduce_kernel(
    bf16_t* __restrict__ out, const int* __restrict__ cu_q, int Hq, int Hkv, int splits,
    const float* __restrict__ ws_acc, const float* __restrict__ ws_ml) {
  __shared__ float sh_w[16][MAX_SPLITS];
  __shared__ float4 sh_part[256];
  const int b = blockIdx.y, g_kv = blockIdx.x;
  const int G = Hq / Hkv;
  const int q0 = cu_q ? cu_q[b] : b;                     // no cu_q: a step of single tokens, row b is sequence b's
  const int q_len = cu_q ? cu_q[b + 1] - q0 : 1;
  if (q_len <= 0 || q_len * G > 16) return;
  const int rows = q_len * G;
  const size_t base = ((size_t)b * Hkv + g_kv) * splits;
  const int cols = rows * (D / 4);                       // float4 columns of the output
  const int groups = cols <= 256 ? 256 / cols : 1;       // threads per column, each with its share of the splits
  const int t = threadIdx.x;
  const int grp = cols <= 256 ? t / cols : 0;
  const int c0 = cols <= 256 ? t - grp * cols : t;
  const bool active = grp < groups;

  // this thread's first column: its first batch of partial accumulators is asked for now
  float4 first[REDUCE_BATCH];
#pragma unroll
  for (int k = 0; k < REDUCE_BATCH; ++k) {
    const int s = grp + k * groups;
    first[k] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (active && c0 < cols && s < splits) {
      const int r = c0 / (D / 4), d = 4 * (c0 - r * (D / 4));
      first[k] = *reinterpret_cast<const float4*>(ws_acc + ((base + s) * 16 + r) * D + d);
    }
  }
  // the splits' weights, a row per wavefront at a time: lane s holds split s
  {
    const int lane = t & 63, wave = t >> 6;
    for (int r = wave; r < rows; r += 4) {
      float2 ml = make_float2(-INFINITY, 0.f);
      if (lane < splits) ml = *reinterpret_cast<const float2*>(ws_ml + ((base + lane) * 16 + r) * 2);
      const float m_all = wave_max(ml.x);
      const float e = ml.x > -INFINITY ? exp2f(ml.x - m_all) : 0.f;
      const float l_all = wave_sum(ml.y * e);
      if (lane < splits) sh_w[r][lane] = l_all > 0.f ? e / l_all : 0.f;   // a row that saw no key at all: zeros
    }
  }
  __syncthreads();
  for (int c = c0; c < cols; c += 256) {   // one pass unless there are more columns than threads
    const int r = c / (D / 4), d = 4 * (c - r * (D / 4));
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    if (active) {
      for (int k0 = 0; grp + k0 * groups < splits; k0 += REDUCE_BATCH) {
        float4 a[REDUCE_BATCH];
#pragma unroll
        for (int k = 0; k < REDUCE_BATCH; ++k) {
          const int s = grp + (k0 + k) * groups;
          if (c == c0 && k0 == 0)
            a[k] = first[k];
          else
            a[k] = s < splits ? *reinterpret_cast<const float4*>(ws_acc + ((base + s) * 16 + r) * D + d)
                              : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int k = 0; k < REDUCE_BATCH; ++k) {  // an empty split's partial is zero and so is its weight
          const int s = grp + (k0 + k) * groups;
          const float w = s < splits ? sh_w[r][s] : 0.f;
          o.x += a[k].x * w; o.y += a[k].y * w; o.z += a[k].z * w; o.w += a[k].w * w;
        }
      }
    }
    if (groups > 1) {
      if (active && grp > 0) sh_part[t] = o;
      __syncthreads();
      if (grp == 0) {
        for (int g2 = 1; g2 < groups; ++g2) {
          const float4 p = sh_part[g2 * cols + c];
          o.x += p.x; o.y += p.y; o.z += p.z; o.w += p.w;
        }
      }
    }
    if (grp == 0) {
      const int token = q0 + r / G, head = g_kv * G + r % G;
      union {
        uint2 u;
        bf16_t e[4];
      } pk;
      pk.e[0] = float_to_bf16(o.x); pk.e[1] = float_to_bf16(o.y);
      pk.e[2] = float_to_bf16(o.z); pk.e[3] = float_to_bf16(o.w);
      *reinterpret_cast<uint2*>(out + (size_t)token * Hq * D + (size_t)head * D + d) = pk.u;
    }
  }
}

// ---- sequences with many rows: portions of prompts ----------------------------
// grid (Hkv, row tiles, B), 256 threads; a block owns 128 / G tokens x G heads,
// each wavefront 32 rows of them (two blocks of 16). The block's threads bring
// each 64-key tile from the cache into shared memory once, with loads that write
// shared memory directly (no registers in between), the next tile's while the
// current tile is worked on; the wavefronts read their matrix-core operands from
// there. The 16-byte pieces of a tile are placed so that the sixteen rows an operand
// read touches fall in different banks (see PrefillSmem). Two stages of a 64-key
// tile take 64 KB of the CU's 160 KB, so two blocks share a CU. The key head is the
// grid's fastest index: consecutive blocks go to the XCDs in turn, so with eight key heads
// each XCD's L2 holds one head's keys and values, which all its blocks read (with the row
// tile fastest, every XCD read every head and 8 MB went through each 4 MB L2). A head's
// blocks take their row tiles in an order that lets the blocks which come to share a CU
// add up to about the same work. Block-table entries are copied to
// shared memory PREFILL_PAGES at a time, so that no cache load waits for a table load.
#define PREFILL_PAGES 512
// (measured for one 2,048-token prompt at head size 128: 64-key tiles in two stages 94 us, 32-key
// tiles in four stages, which have three tiles on their way, 116 us; three stages of 64 keys
// leave room for one block a CU only, 184 us. With the address tables in shared memory, which took
// some hundred vector instructions per tile out of the copies: 78 us, and 682 for 8,192 tokens.
// The same kernel rewritten around v_mfma_f32_32x32x16_bf16 (a wavefront's 32 rows one operand, the
// two lanes of a row exchanging runs of four probabilities by v_permlane32_swap so that each holds
// eight consecutive keys, values as D rows of 64 keys in shared memory) was correct and took 71 us
// and 690, 9,100 for 32,768 tokens; with blocks of 256 rows, eight wavefronts and three stages,
// which halve the tiles' traffic from the L2 to the CUs, 90, 698 and 8,960. So neither the matrix
// instruction's form nor that traffic is what bounds it. Time stamps around the phases of one wavefront
// (the kernel runs at 1.77 GHz): per tile the copy's issue 580 cycles, the first product 870, the softmax
// 1,360, the second product 880, waits 160, about 4,600 with the loop around them, in which the SIMD serves
// two wavefronts; the 64 matrix instructions of a tile take 1,024 cycles of the matrix pipe and its 265
// other vector instructions about 1,200 of the vector unit: each works about half the time, and they
// overlap only in part. The rewrite was not kept: its gain is within what boxes differ by from 4,096 tokens on.)
#define PF_TILE 64    // keys per tile
#define PF_STAGES 2  // tiles in shared memory: one being worked on, the others on their way
template <int D, int TILE>
struct PrefillSmem {
  // A stage holds a tile's keys (TILE rows of D) and values (D rows of TILE), both as
  // 16-byte pieces in an order chosen so that the matrix-core operand reads spread over all
  // banks without padding (the loads that fill a stage write whole kilobytes, see below).
  // A window is 256 bytes. Keys: a window = RPW rows of CPR pieces; piece c of row r sits at
  // place (r % RPW) * CPR + (c ^ (window % CPR)) of window r / RPW. Values (a piece = eight
  // keys of one 16-key block): sixteen rows' pieces of the tile's first half of blocks are
  // followed by the same rows' pieces of its second half (two planes), so that the two 8-byte
  // reads that make one operand of the second product (four keys of block h, four of block
  // h + blocks / 2) are a fixed, short distance apart and one instruction fetches both. A
  // plane's sixteen rows are VPR windows of VRW rows of VPR pieces (q = 2 * (block in the
  // plane) + half); piece q of row d sits at place (d % VRW) * VPR + (q ^ window) of its window.
  static constexpr int CPR = D / 8;          // 16-byte pieces per key row
  static constexpr int RPW = 16 / CPR > 0 ? 16 / CPR : 1;   // key rows per window (D <= 128)
  static constexpr int VPR = TILE / 16;      // pieces per value row in a plane
  static constexpr int VRW = 16 / VPR;       // value rows per window
  static constexpr int K_BYTES = TILE * D * 2;
  static constexpr int V_BYTES = D * TILE * 2;
  static constexpr int STAGE = K_BYTES + V_BYTES;
  static constexpr int K_PIECES = K_BYTES / 16, V_PIECES = V_BYTES / 16;
};

// The softmax update of one block of 16 rows for one tile of KB4 16-key blocks: as
// softmax_step; the probabilities come back as the P operands of the tile's 32-key halves.
template <int NB, int KB4>
__device__ __forceinline__ void softmax_tile(const f32x4_t (&s)[KB4], bool full, int key0, int grp, int row_pos,
                                             int window, float scale_log2, float& m_run, float& l_run,
                                             f32x4_t (&acc)[NB], Pack16 (&p)[KB4 / 2]) {
  constexpr int N = 4 * KB4;
  static_assert(N % 2 == 0, "maxima are taken three at a time");
  float v[N];
#pragma unroll
  for (int j = 0; j < N; ++j) v[j] = s[j >> 2][j & 3];
  if (!full) {
    // (the row's position and the lane's first key go through an empty piece of assembly so that the
    // comparisons' operands are worked out here, where they are needed, and not before the branch for
    // every tile)
    int pos = row_pos, first_key = key0 + 4 * grp;
    asm volatile("" : "+v"(pos), "+v"(first_key));
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const int key = first_key + 16 * (j >> 2) + (j & 3);
      bool seen = key <= pos;
      if (window > 0 && pos - key >= window) seen = false;
      if (!seen) v[j] = -INFINITY;
    }
  }
  // the scores are matrix results or minus infinity, never NaN: the three-operand maximum as
  // it is (the compiler's own first makes every operand a quiet NaN, one instruction each)
  // (one statement for a tile of 64 keys: after every statement of assembly the compiler leaves a wait state)
  float mx;
  if constexpr (N == 16) {
    asm("v_max_f32 %0, %1, %2\n\tv_max3_f32 %0, %0, %3, %4\n\tv_max3_f32 %0, %0, %5, %6\n\tv_max3_f32 %0, %0, %7, %8\n\t"
        "v_max3_f32 %0, %0, %9, %10\n\tv_max3_f32 %0, %0, %11, %12\n\tv_max3_f32 %0, %0, %13, %14\n\t"
        "v_max3_f32 %0, %0, %15, %16"
        : "=&v"(mx)
        : "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]), "v"(v[4]), "v"(v[5]), "v"(v[6]), "v"(v[7]), "v"(v[8]), "v"(v[9]),
          "v"(v[10]), "v"(v[11]), "v"(v[12]), "v"(v[13]), "v"(v[14]), "v"(v[15]));
  } else {
    asm("v_max_f32 %0, %1, %2" : "=v"(mx) : "v"(v[0]), "v"(v[1]));
#pragma unroll
    for (int j = 2; j < N; j += 2) asm("v_max3_f32 %0, %1, %2, %3" : "=v"(mx) : "v"(mx), "v"(v[j]), "v"(v[j + 1]));
  }
  mx = quad_rows_max_of_numbers(mx);
  const float m_new = max_of_numbers(m_run, mx * scale_log2);
  // a row that has seen no key yet has minus infinity here and in all its scores: its terms are
  // exp2(-inf - 0) = 0
  const float m_use = m_new > -INFINITY ? m_new : 0.f;
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < N; ++j) {
    const float e = fast_exp2(fmaf(v[j], scale_log2, -m_use));
    sum += e;
    p[(j >> 2) % (KB4 / 2)].e[4 * ((j >> 2) / (KB4 / 2)) + (j & 3)] = (__bf16)e;  // block kb goes with kb + KB4 / 2
  }
  const bool moved = m_new != m_run;
  if (__builtin_amdgcn_ballot_w64(moved) != 0) {
    const float alpha = m_new > -INFINITY ? fast_exp2(m_run - m_new) : 1.f;
    l_run *= alpha;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[nb] *= alpha;
    m_run = m_new;
  }
  l_run += sum;
}

template <int D, int TILE, int STAGES>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void attn_prefill_kernel(
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, int num_pages, const int* __restrict__ block_table, int bt_stride,
    const int* __restrict__ cu_q, const int* __restrict__ kv_lens, int Hq, int Hkv, int page, float scale_log2,
    int window, int tokens_per_block, int key_splits, float* __restrict__ part_acc, float* __restrict__ part_ml) {
  typedef PrefillSmem<D, TILE> SM;
  constexpr int KB4 = TILE / 16;  // 16-key blocks per tile
  __shared__ __attribute__((aligned(16))) unsigned char smem[STAGES * SM::STAGE];
  __shared__ int sh_pages[PREFILL_PAGES];  // the block-table entries of the tiles in hand
  // and the address at which each entry's (page, this key head) begins in either cache: worked out
  // once per entry, so that a tile's load finds its address with one read of this table and one
  // addition of a number the thread keeps for the whole kernel
  __shared__ long long sh_kaddr[PREFILL_PAGES], sh_vaddr[PREFILL_PAGES];
  const int b = blockIdx.z, g_kv = blockIdx.x;
  const int G = Hq / Hkv;
  const int q0 = cu_q[b];
  const int q_len = cu_q[b + 1] - q0;
  if (q_len * G <= 16) return;  // the other kernel's sequence
  const int n_tiles = (q_len + tokens_per_block - 1) / tokens_per_block;
  // with `key_splits` > 1 a row tile's keys are shared out over that many blocks, whose
  // unnormalised results attn_prefill_merge_kernel joins
  const int split = (int)blockIdx.y % key_splits, tile_index = (int)blockIdx.y / key_splits;
  if (tile_index >= n_tiles) return;
  // the first half of a head's blocks takes the row tiles from the sequence's end downwards (the
  // long ones start first), the second half from its start upwards: block i and block
  // i + n / 2, a long and a short one, come to share a CU (measured against plain ascending and
  // descending orders and the mirrored one: 87 us against 95, 89 and 88)
  const int half_tiles = (n_tiles + 1) / 2;
  const int tile = tile_index < half_tiles ? n_tiles - 1 - tile_index : tile_index - half_tiles;
  const int kv_len = kv_lens[b];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int first_pos = kv_len - q_len;
  const int rows_in_block = tokens_per_block * G;  // <= 128

  int row_pos[2], row_tok[2], row_head[2];
  Pack16 qreg[2][D / 32];
  int pos_max = -1, pos_min = 0x7fffffff;
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const int r = wave * 32 + qb * 16 + col;
    const int tok = tile * tokens_per_block + r / G;
    const bool ok = r < rows_in_block && tok < q_len;
    row_tok[qb] = q0 + tok;
    row_head[qb] = g_kv * G + r % G;
    row_pos[qb] = ok ? first_pos + tok : -1;
    if (ok) {
      pos_max = max(pos_max, row_pos[qb]);
      pos_min = min(pos_min, row_pos[qb]);
    }
#pragma unroll
    for (int i = 0; i < D / 32; ++i) {
      if (ok)
        qreg[qb][i].u = *reinterpret_cast<const uint4*>(q + (size_t)row_tok[qb] * q_stride +
                                                       (size_t)row_head[qb] * D + 32 * i + 8 * grp);
      else
        qreg[qb][i].u = make_uint4(0, 0, 0, 0);
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    pos_max = max(pos_max, __shfl_xor(pos_max, off, 64));
    pos_min = min(pos_min, __shfl_xor(pos_min, off, 64));
  }
  // the same in all lanes: kept as scalars, so that what is decided by them per tile is a scalar branch
  pos_max = __builtin_amdgcn_readfirstlane(pos_max);
  pos_min = __builtin_amdgcn_readfirstlane(pos_min);
  f32x4_t acc[2][D / 16];
#pragma unroll
  for (int qb = 0; qb < 2; ++qb)
#pragma unroll
    for (int nb = 0; nb < D / 16; ++nb) acc[qb][nb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m_run[2] = {-INFINITY, -INFINITY}, l_run[2] = {0.f, 0.f};

  // the block's range of tiles: from the window's start of its first row to its last row's position
  const int blk_first_tok = tile * tokens_per_block;
  const int blk_last_tok = min(q_len, blk_first_tok + tokens_per_block) - 1;
  int tile_lo = 0;
  if (window > 0) tile_lo = max(0, first_pos + blk_first_tok - window + 1) / TILE;
  int tile_hi = (first_pos + blk_last_tok) / TILE + 1;
  // and this wavefront's own (a wavefront whose rows do not exist has none)
  int my_lo = tile_lo, my_hi = pos_max >= 0 ? pos_max / TILE + 1 : 0;
  if (window > 0 && pos_max >= 0) my_lo = max(0, pos_min - window + 1) / TILE;
  if (key_splits > 1) {  // this block's share of the range (it may be empty)
    const int share = (tile_hi - tile_lo + key_splits - 1) / key_splits;
    tile_lo = min(tile_hi, tile_lo + split * share);
    tile_hi = min(tile_hi, tile_lo + share);
    my_lo = max(my_lo, tile_lo);
    my_hi = min(my_hi, tile_hi);
  }
  const int* bt_row = block_table + (size_t)b * bt_stride;

  // The copy of a tile from the caches into a stage. Place s (a 16-byte piece) of the keys'
  // or values' part of a stage is filled by thread s % 256 in its turn s / 256: a wavefront's
  // 64 lanes fill one contiguous kilobyte per turn, which is what a load that writes shared
  // memory directly asks for (lane L's 16 bytes land at the wavefront's base + 16 L; the
  // global address is each lane's own). Tiles that lie whole inside the sequence, with no
  // page given back, are copied that way, without passing through registers; the others go
  // through registers, where what lies past the sequence's end is zeroed.
  constexpr int K_TURNS = SM::K_PIECES / 256, V_TURNS = SM::V_PIECES / 256;
  int page_base = 0;  // sh_pages[i] is the table's entry page_base + i
  const int page_shift = 31 - __clz(page);  // the page size is a power of two here
  // which piece of which row a place holds: keys (row of the tile, element offset), values
  // (16-key block, row d, half of the block)
  int k_row[K_TURNS], k_off[K_TURNS], v_kb[V_TURNS], v_d[V_TURNS], v_h[V_TURNS];
#pragma unroll
  for (int j = 0; j < K_TURNS; ++j) {
    const int place = tid + 256 * j, w = place >> 4, u = place & 15;
    k_row[j] = w * SM::RPW + u / SM::CPR;
    k_off[j] = 8 * ((u % SM::CPR) ^ (w % SM::CPR));
  }
#pragma unroll
  for (int j = 0; j < V_TURNS; ++j) {
    const int place = tid + 256 * j, rows16 = place / (SM::VPR * 32), plane = (place / (SM::VPR * 16)) & 1;
    const int w = (place >> 4) % SM::VPR, u = place & 15;
    const int q = (u % SM::VPR) ^ w;
    v_d[j] = 16 * rows16 + SM::VRW * w + u / SM::VPR;
    v_kb[j] = plane * (TILE / 32) + (q >> 1);
    v_h[j] = q & 1;
  }
  const size_t page_elems = (size_t)page * D;  // elements of one (page, head) in either cache
  // What a thread keeps per load of a whole tile: where in the address tables its piece's page stands,
  // counted from the tile's first page, and the piece's byte offset within (page, head). With pages of
  // fewer keys than a tile the tile begins a page and both are fixed; with larger pages the tile lies
  // in one page, at an offset that is the same for all threads and is added per tile.
  const bool small_pages = page < TILE;
  unsigned k_slot[K_TURNS], k_at[K_TURNS], v_slot[V_TURNS], v_at[V_TURNS];
#pragma unroll
  for (int j = 0; j < K_TURNS; ++j) {
    k_slot[j] = small_pages ? 8u * (unsigned)(k_row[j] >> page_shift) : 0u;
    k_at[j] = 2u * (unsigned)((small_pages ? k_row[j] & (page - 1) : k_row[j]) * D + k_off[j]);
  }
#pragma unroll
  for (int j = 0; j < V_TURNS; ++j) {
    const int key = 16 * v_kb[j] + 8 * v_h[j];   // the first of the piece's eight keys, from the tile's first
    v_slot[j] = small_pages ? 8u * (unsigned)(key >> page_shift) : 0u;
    v_at[j] = 2u * (unsigned)(v_d[j] * page + (small_pages ? key & (page - 1) : key));
  }
  // A load of 16 bytes per lane that writes shared memory directly: lane L's bytes land at
  // `lds` + 16 L (`lds` the same in all lanes). It is written as assembly on purpose: for the
  // compiler's own form of this instruction the compiler makes every later read of shared
  // memory wait until no load at all is outstanding, since it cannot tell the stage being
  // filled from the stage being read, and the next tile's copy would not overlap with this
  // tile's work in the same wavefront. What orders these loads against the reads is
  // `wait_for_tile` and the barrier after it.
  typedef __attribute__((address_space(3))) unsigned char* lds_ptr;
  const unsigned smem_lds = (unsigned)(unsigned long)(lds_ptr)smem;
  auto load_to_lds = [&](const void* src, unsigned lds) {
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds) : "memory", "m0");
  };

  auto plain_tile = [&](int t) { return t * TILE + TILE <= kv_len && window == 0; };
  auto copy_direct = [&](int t, int stage) {
    const int key0 = t * TILE;
    // this wavefront's kilobyte of each turn
    const unsigned ks = __builtin_amdgcn_readfirstlane(smem_lds + stage * SM::STAGE + 1024 * wave);
    const unsigned vs = ks + SM::K_BYTES;
    const unsigned first = 8u * (unsigned)((key0 >> page_shift) - page_base);   // the tile's first page in the tables
    const unsigned within = small_pages ? 0u : (unsigned)(key0 & (page - 1));   // the tile's first key in its page
    const unsigned k_in = 2u * within * D, v_in = 2u * within;
    const char* k_table = reinterpret_cast<const char*>(sh_kaddr) + first;
    const char* v_table = reinterpret_cast<const char*>(sh_vaddr) + first;
    long long base[K_TURNS + V_TURNS];
#pragma unroll
    for (int j = 0; j < K_TURNS; ++j) base[j] = *reinterpret_cast<const long long*>(k_table + k_slot[j]);
#pragma unroll
    for (int j = 0; j < V_TURNS; ++j) base[K_TURNS + j] = *reinterpret_cast<const long long*>(v_table + v_slot[j]);
    if (small_pages) {   // a tile begins a page: nothing to add to the thread's own offsets
#pragma unroll
      for (int j = 0; j < K_TURNS; ++j) load_to_lds(reinterpret_cast<const char*>(base[j]) + k_at[j], ks + 4096 * j);
#pragma unroll
      for (int j = 0; j < V_TURNS; ++j)
        load_to_lds(reinterpret_cast<const char*>(base[K_TURNS + j]) + v_at[j], vs + 4096 * j);
    } else {
#pragma unroll
      for (int j = 0; j < K_TURNS; ++j)
        load_to_lds(reinterpret_cast<const char*>(base[j]) + (k_at[j] + k_in), ks + 4096 * j);
#pragma unroll
      for (int j = 0; j < V_TURNS; ++j)
        load_to_lds(reinterpret_cast<const char*>(base[K_TURNS + j]) + (v_at[j] + v_in), vs + 4096 * j);
    }
  };
  auto copy_checked = [&](int t, int stage) {
    const int key0 = t * TILE;
    unsigned char* ks = smem + stage * SM::STAGE;
    unsigned char* vs = ks + SM::K_BYTES;
#pragma unroll
    for (int j = 0; j < K_TURNS; ++j) {
      const int key = key0 + k_row[j];
      uint4 piece = make_uint4(0, 0, 0, 0);  // rows past the end are zero
      if (key < kv_len) {
        const int pg = sh_pages[(key >> page_shift) - page_base];
        if (pg >= 0 && pg < num_pages)
          piece = *reinterpret_cast<const uint4*>(k_cache + (size_t)(pg * Hkv + g_kv) * page_elems +
                                                  ((key & (page - 1)) * D + k_off[j]));
      }
      *reinterpret_cast<uint4*>(ks + 16 * (tid + 256 * j)) = piece;
    }
#pragma unroll
    for (int j = 0; j < V_TURNS; ++j) {
      const int key = key0 + 16 * v_kb[j] + 8 * v_h[j];  // the first of the piece's eight keys
      Pack16 piece;
      piece.u = make_uint4(0, 0, 0, 0);
      if (key < kv_len) {
        const int pg = sh_pages[(key >> page_shift) - page_base];
        if (pg >= 0 && pg < num_pages) {
          piece.u = *reinterpret_cast<const uint4*>(v_cache + (size_t)(pg * Hkv + g_kv) * page_elems +
                                                    (v_d[j] * page + (key & (page - 1))));
          if (key + 8 > kv_len) {  // slots past the end hold anything: zero them (0 * NaN is NaN)
#pragma unroll
            for (int i = 0; i < 8; ++i)
              if (key + i >= kv_len) piece.e[i] = (__bf16)0.f;
          }
        }
      }
      *reinterpret_cast<uint4*>(vs + 16 * (tid + 256 * j)) = piece.u;
    }
  };
  auto copy_tile = [&](int t, int stage) {
    if (plain_tile(t))
      copy_direct(t, stage);
    else
      copy_checked(t, stage);
  };
  // the operand reads' addresses: this lane's window and swizzle for the key rows 16 kb4 + col
  // and for the value rows 16 nb + col
  const int k_lane = (col / SM::RPW) * 256 + (col % SM::RPW) * SM::CPR * 16;
  const int k_swz = (col / SM::RPW) % SM::CPR;
  const int v_lane = (col / SM::VRW) * 256 + (col % SM::VRW) * SM::VPR * 16 + 8 * (grp & 1);
  const int v_swz = (col / SM::VRW) % SM::VPR;
  int k_read[D / 32], v_read[TILE / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i) k_read[i] = k_lane + 16 * ((4 * i + grp) ^ k_swz);
#pragma unroll
  for (int h = 0; h < TILE / 32; ++h) v_read[h] = v_lane + 16 * ((2 * h + (grp >> 1)) ^ v_swz);
  constexpr int LOADS_PER_TILE = K_TURNS + V_TURNS;  // this thread's loads in flight per tile on its way

  // The query rows are used here, before the tile loop, so that the compiler waits for their
  // loads here: a wait it would otherwise place at their first use inside the loop, where it
  // would also wait, every time round, for the next tile's copy (the compiler counts loads,
  // and does not know of those it did not issue).
#pragma unroll
  for (int qb = 0; qb < 2; ++qb)
#pragma unroll
    for (int i = 0; i < D / 32; ++i) asm volatile("" : "+v"(qreg[qb][i].v));

  // tiles are worked through in spans whose table entries fit sh_pages
  const int tiles_per_span = max(1, (PREFILL_PAGES - 4) * page / TILE);
  for (int span_lo = tile_lo; span_lo < tile_hi; span_lo += tiles_per_span) {
    const int span_hi = min(tile_hi, span_lo + tiles_per_span);
    __syncthreads();
    page_base = (span_lo * TILE) >> page_shift;
    {
      const int last_page = min((kv_len - 1) >> page_shift, (span_hi * TILE - 1) >> page_shift);
      for (int i = tid; page_base + i <= last_page; i += 256) {
        const int pg = bt_row[page_base + i];
        sh_pages[i] = pg;
        const long long at = 2 * (long long)(min(max(pg, 0), num_pages - 1) * Hkv + g_kv) * (long long)page_elems;
        sh_kaddr[i] = reinterpret_cast<long long>(k_cache) + at;
        sh_vaddr[i] = reinterpret_cast<long long>(v_cache) + at;
      }
    }
    __syncthreads();
    // STAGES - 1 tiles are on their way at any time: the first ones here, then tile
    // t + STAGES - 1 at the top of tile t's turn, into the stage tile t - 1 has left. Loads
    // complete in the order they were issued, so waiting until no more than the later tiles'
    // loads are outstanding means the next tile has landed.
    auto wait_for_tile = [&](int tiles_after) {
      if (tiles_after <= 0)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      else if (tiles_after == 1)
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LOADS_PER_TILE) : "memory");
      else
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * LOADS_PER_TILE) : "memory");
    };
    static_assert(STAGES >= 2 && STAGES <= 4 && 2 * LOADS_PER_TILE < 64, "the wait counts above");
#pragma unroll
    for (int ahead = 0; ahead < STAGES - 1; ++ahead)
      if (span_lo + ahead < span_hi) copy_tile(span_lo + ahead, ahead);
    wait_for_tile(min(span_hi - span_lo, STAGES - 1) - 1);
    __syncthreads();
    for (int t = span_lo; t < span_hi; ++t) {
      const int stage = (t - span_lo) % STAGES;
      if (t + STAGES - 1 < span_hi) copy_tile(t + STAGES - 1, (t + STAGES - 1 - span_lo) % STAGES);
      if (t >= my_lo && t < my_hi) {
        const unsigned char* ks = smem + stage * SM::STAGE;
        const unsigned char* vs = ks + SM::K_BYTES;
        const int key0 = t * TILE;
        f32x4_t sc[2][KB4];
#pragma unroll
        for (int kb4 = 0; kb4 < KB4; ++kb4) {
          Pack16 a[D / 32];
#pragma unroll
          for (int i = 0; i < D / 32; ++i)
            a[i].u = *reinterpret_cast<const uint4*>(ks + (16 / SM::RPW) * 256 * kb4 + k_read[i]);
#pragma unroll
          for (int qb = 0; qb < 2; ++qb) {
            f32x4_t c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < D / 32; ++i)
              c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i].v, qreg[qb][i].v, c, 0, 0, 0);
            sc[qb][kb4] = c;
          }
        }
        // no key of the tile is hidden from any row of this wavefront?
        const bool full = key0 + TILE - 1 <= pos_min && (window == 0 || pos_max - key0 < window);
        Pack16 p[2][KB4 / 2];
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
          softmax_tile<D / 16, KB4>(sc[qb], full, key0, grp, row_pos[qb], window, scale_log2, m_run[qb], l_run[qb],
                                    acc[qb], p[qb]);
        // the values' operands (keys 4 grp .. 4 grp + 3 of blocks half and half + KB4 / 2) are
        // read one group of output columns ahead of the matrix instructions that use them
        Pack16 vt[4][KB4 / 2];
        auto read_values = [&](int nb, Pack16 (&to)[KB4 / 2]) {
#pragma unroll
          for (int half = 0; half < KB4 / 2; ++half)
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
              // (an empty statement of assembly after each read keeps it a ds_read_b64 of its own: joined by the
              // compiler into one ds_read2st64_b64, two addresses a multiple of 512 bytes apart fall into the
              // same banks, and shared memory takes sixteen cycles per kilobyte, half of them counted as bank
              // conflicts, where two ds_read_b64 take two cycles each; measured with the read pattern alone.
              // These reads were four fifths of the kernel's shared-memory time, and shared memory was its
              // busiest unit.)
              to[half].h[kb] = *reinterpret_cast<const uint2*>(vs + (2 * nb + kb) * SM::VPR * 256 + v_read[half]);
              asm volatile("" ::: "memory");
            }
        };
        read_values(0, vt[0]);
        read_values(1, vt[1]);
#pragma unroll
        for (int nb = 0; nb < D / 16; ++nb) {
          if (nb + 2 < D / 16) read_values(nb + 2, vt[(nb + 2) & 3]);
#pragma unroll
          for (int half = 0; half < KB4 / 2; ++half)
#pragma unroll
            for (int qb = 0; qb < 2; ++qb)
              acc[qb][nb] =
                  __builtin_amdgcn_mfma_f32_16x16x32_bf16(vt[nb & 3][half].v, p[qb][half].v, acc[qb][nb], 0, 0, 0);
        }
        // the order the compiler is to keep (left to itself it reads each operand right before
        // its use, into the same registers, and waits for it every time): four operands (two reads each) ahead
        __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
#pragma unroll
        for (int i = 0; i < (D / 16) * (KB4 / 2) - 4; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
      }
      // this wavefront's share of the next tile has landed; the tiles after it may still travel
      wait_for_tile(min(t + STAGES - 1, span_hi - 1) - (t + 1));
      __syncthreads();
    }
  }
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    float l = l_run[qb];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (row_pos[qb] < 0) continue;
    if (key_splits > 1) {
      const size_t slot = ((size_t)row_tok[qb] * Hq + row_head[qb]) * key_splits + split;
      float* o = part_acc + slot * D + 4 * grp;
#pragma unroll
      for (int nb = 0; nb < D / 16; ++nb)
        *reinterpret_cast<float4*>(o + 16 * nb) =
            make_float4(acc[qb][nb][0], acc[qb][nb][1], acc[qb][nb][2], acc[qb][nb][3]);
      if (grp == 0) *reinterpret_cast<float2*>(part_ml + slot * 2) = make_float2(m_run[qb], l);
      continue;
    }
    const float inv = 1.f / l;
    bf16_t* o = out + (size_t)row_tok[qb] * Hq * D + (size_t)row_head[qb] * D + 4 * grp;
#pragma unroll
    for (int nb = 0; nb < D / 16; ++nb) {
      union {
        uint2 u;
        bf16_t e[4];
      } pk;
#pragma unroll
      for (int j = 0; j < 4; ++j) pk.e[j] = float_to_bf16(acc[qb][nb][j] * inv);
      *reinterpret_cast<uint2*>(o + 16 * nb) = pk.u;
    }
  }
}

// Joins the key splits of attn_prefill_kernel: grid (max_q_len, B), 256 threads; a block takes
// one token of a sequence, a thread four neighbouring output elements of one (token, head)
// row at a time. Sequences of few rows are the decoding kernel's.
template <int D>
__global__ __launch_bounds__(256) void attn_prefill_merge_kernel(bf16_t* __restrict__ out,
                                                                 const int* __restrict__ cu_q, int Hq, int Hkv,
                                                                 int key_splits, const float* __restrict__ part_acc,
                                                                 const float* __restrict__ part_ml) {
  const int b = blockIdx.y;
  const int q0 = cu_q[b], q_len = cu_q[b + 1] - q0;
  if (q_len * (Hq / Hkv) <= 16) return;
  constexpr int PER_ROW = D / 4;  // threads a row takes
  const int first = blockIdx.x;
  if (first >= q_len) return;
  const int rows = Hq;
  for (int i = threadIdx.x; i < rows * PER_ROW; i += 256) {
    const int row = i / PER_ROW, d = 4 * (i % PER_ROW);
    const size_t slot = ((size_t)(q0 + first) * Hq + row) * key_splits;
    float m_all = -INFINITY;
    for (int s = 0; s < key_splits; ++s) m_all = fmaxf(m_all, part_ml[(slot + s) * 2]);
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    float l_all = 0.f;
    for (int s = 0; s < key_splits; ++s) {   // in the splits' order: a fixed order of additions
      const float2 ml = *reinterpret_cast<const float2*>(part_ml + (slot + s) * 2);
      if (ml.x == -INFINITY) continue;       // a split with no key for this row
      const float w = fast_exp2(ml.x - m_all);
      const float4 a = *reinterpret_cast<const float4*>(part_acc + (slot + s) * D + d);
      o.x += a.x * w; o.y += a.y * w; o.z += a.z * w; o.w += a.w * w;
      l_all += ml.y * w;
    }
    const float inv = 1.f / l_all;
    union {
      uint2 u;
      bf16_t e[4];
    } pk;
    pk.e[0] = float_to_bf16(o.x * inv); pk.e[1] = float_to_bf16(o.y * inv);
    pk.e[2] = float_to_bf16(o.z * inv); pk.e[3] = float_to_bf16(o.w * inv);
    *reinterpret_cast<uint2*>(out + ((size_t)(q0 + first) * Hq + row) * D + d) = pk.u;
  }
}

// How the rows and keys of a step's long sequences go over blocks. A block owns 128 rows
// (tokens x heads of a group) and all their keys; with so few rows that the blocks do not fill
// the chip twice (a portion of 512 tokens of one prompt: 128 blocks, each a chain of as many
// tiles as the prefix is long), first the keys are split over up to four blocks, from 2,048
// keys on and as long as a split keeps eight tiles (512 tokens over 3,584 keys: 127 us whole,
// 97 in two, 88 in four; 256 over 7,936: 224, 141, 97; over 512 keys splitting loses), then a
// block's rows are halved, down to one wavefront's 32 (its other wavefronts then only help
// to copy the tiles).
static int prompt_key_splits(int total_tokens, int G, int Hkv, int max_kv_len) {
  const int tpb = 128 / G;
  int ks = 1;
  const int key_tiles = (max_kv_len + PF_TILE - 1) / PF_TILE;
  while (Hkv * ((total_tokens + tpb - 1) / tpb) * ks < 512 && ks < 4 && key_tiles >= 32 && key_tiles / (2 * ks) >= 8)
    ks *= 2;
  return ks;
}

static int prompt_tokens_per_block(int total_tokens, int G, int Hkv, int key_splits) {
  int tpb = 128 / G;
  while (Hkv * ((total_tokens + tpb - 1) / tpb) * key_splits < 256 && (tpb / 2) * G >= 32) tpb /= 2;
  return tpb;
}

template <int D>
static int launch_fast(const void* q, int q_stride, void* out, const void* k_cache, const void* v_cache,
                       int num_pages, const int* block_table, int bt_stride, const int* cu_q, const int* kv_lens,
                       int B, int total_tokens, int Hq, int Hkv, int page, float scale, int window, int max_q_len,
                       int min_q_len, int splits, float* ws_acc, float* ws_ml, int key_splits, float* prompt_ws,
                       hipStream_t stream) {
  const int G = Hq / Hkv;
  const float scale_log2 = scale * 1.4426950408889634f;
  if (min_q_len * G <= 16) {
    if (window == 0)
      hipLaunchKernelGGL((attn_decode_kernel<D, false, float, true>), dim3(splits, Hkv, B), dim3(256), 0, stream,
                         (const bf16_t*)q, q_stride, (bf16_t*)out, (const bf16_t*)k_cache, (const bf16_t*)v_cache,
                         num_pages, block_table, bt_stride, cu_q, kv_lens, Hq, Hkv, page, scale_log2, window, splits,
                         ws_acc, ws_ml, DecodePrep{});
    else
      hipLaunchKernelGGL((attn_decode_kernel<D, false, float, false>), dim3(splits, Hkv, B), dim3(256), 0, stream,
                         (const bf16_t*)q, q_stride, (bf16_t*)out, (const bf16_t*)k_cache, (const bf16_t*)v_cache,
                         num_pages, block_table, bt_stride, cu_q, kv_lens, Hq, Hkv, page, scale_log2, window, splits,
                         ws_acc, ws_ml, DecodePrep{});
    if (splits > 1)
      hipLaunchKernelGGL(attn_decode_reduce_kernel<D>, dim3(Hkv, B), dim3(256), 0, stream, (bf16_t*)out, cu_q, Hq,
                         Hkv, splits, ws_acc, ws_ml);
  }
  if (max_q_len * G > 16) {
    const int tokens_per_block = prompt_tokens_per_block(total_tokens, G, Hkv, key_splits);
    const int tiles = (max_q_len + tokens_per_block - 1) / tokens_per_block;
    if (tiles * key_splits > 65535) return Q3_ERR_UNSUPPORTED;
    float* part_acc = prompt_ws;
    float* part_ml = prompt_ws ? prompt_ws + (size_t)total_tokens * Hq * key_splits * D : nullptr;
    hipLaunchKernelGGL((attn_prefill_kernel<D, PF_TILE, PF_STAGES>), dim3(Hkv, tiles * key_splits, B), dim3(256), 0,
                       stream, (const bf16_t*)q, q_stride, (bf16_t*)out, (const bf16_t*)k_cache,
                       (const bf16_t*)v_cache, num_pages, block_table, bt_stride, cu_q, kv_lens, Hq, Hkv, page,
                       scale_log2, window, tokens_per_block, key_splits, part_acc, part_ml);
    if (key_splits > 1)
      hipLaunchKernelGGL(attn_prefill_merge_kernel<D>, dim3(max_q_len, B), dim3(256), 0, stream,
                         (bf16_t*)out, cu_q, Hq, Hkv, key_splits, part_acc, part_ml);
  }
  return q3_launch_status();
}

template <int D, typename W>
static int launch_decode_prep(const void* qkv, void* out, const void* k_cache, const void* v_cache, int num_pages,
                              const int* block_table, int bt_stride, const int* cu_q, const int* kv_lens, int B,
                              int Hq, int Hkv, int page, float scale, int window, int splits, float* ws_acc,
                              float* ws_ml, const DecodePrep& prep, hipStream_t stream) {
  const float scale_log2 = scale * 1.4426950408889634f;
  if (window == 0)
    hipLaunchKernelGGL((attn_decode_kernel<D, true, W, true>), dim3(splits, Hkv, B), dim3(256), 0, stream,
                       (const bf16_t*)qkv, (Hq + 2 * Hkv) * D, (bf16_t*)out, (const bf16_t*)k_cache,
                       (const bf16_t*)v_cache, num_pages, block_table, bt_stride, cu_q, kv_lens, Hq, Hkv, page,
                       scale_log2, window, splits, ws_acc, ws_ml, prep);
  else
    hipLaunchKernelGGL((attn_decode_kernel<D, true, W, false>), dim3(splits, Hkv, B), dim3(256), 0, stream,
                       (const bf16_t*)qkv, (Hq + 2 * Hkv) * D, (bf16_t*)out, (const bf16_t*)k_cache,
                       (const bf16_t*)v_cache, num_pages, block_table, bt_stride, cu_q, kv_lens, Hq, Hkv, page,
                       scale_log2, window, splits, ws_acc, ws_ml, prep);
  if (splits > 1)
    hipLaunchKernelGGL(attn_decode_reduce_kernel<D>, dim3(Hkv, B), dim3(256), 0, stream, (bf16_t*)out,
                       (const int*)nullptr, Hq, Hkv, splits, ws_acc, ws_ml);
  return q3_launch_status();
}

// Whether the matrix-core kernels take this problem; otherwise the general kernel does.
extern "C" int q3_paged_attention_fast_path(int Hq, int Hkv, int D, int page, int dtype) {
  if (dtype != Q3_BF16) return 0;
  if (D != 64 && D != 128) return 0;
  if (page < 16 || (page & (page - 1))) return 0;  // a power of two, at least 16
  if (Hq % Hkv || Hq / Hkv > 16) return 0;
  return 1;
}

// Floats of workspace the split decoding needs: accumulators, then (max, sum) pairs.
extern "C" long q3_paged_attention_workspace(int B, int Hkv, int D, int splits) {
  return splits > 1 ? (long)B * Hkv * splits * 16 * (D + 2) : 0;
}

// Over how many blocks the keys of a step's long sequences are best split (see above): `T` the
// step's rows, `max_kv_len` the longest of those sequences. With more than one, the workspace
// holds T * Hq * splits * (D + 2) floats: unnormalised outputs, then (max, sum) pairs.
extern "C" int q3_paged_attention_prompt_splits(int T, int Hq, int Hkv, int max_kv_len) {
  if (T <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv) return 1;
  return prompt_key_splits(T, Hq / Hkv, Hkv, max_kv_len);
}

// `splits`, `workspace`: for the sequences of few rows (q3_paged_attention_workspace);
// `prompt_splits` (1, 2 or 4), `prompt_workspace`: for those of many.
extern "C" int q3_paged_attention(const void* q, int q_stride, void* out, const void* k_cache,
                                  const void* v_cache, int num_pages, const int* block_table,
                                  int bt_stride, const int* cu_q, const int* kv_lens, int B, int T_, int Hq,
                                  int Hkv, int D, int page, float scale, int window, int max_q_len,
                                  int min_q_len, int max_kv_len, int dtype, int splits, float* workspace,
                                  int prompt_splits, float* prompt_workspace, hipStream_t stream) {
  if (B <= 0 || T_ <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || page <= 0 || max_q_len <= 0 || min_q_len <= 0 ||
      min_q_len > max_q_len)
    return Q3_ERR_BAD_ARGUMENT;
  if (D % 16 || D < 16 || D > 256) return Q3_ERR_UNSUPPORTED;
  if (B > 65535 || Hq > 65535) return Q3_ERR_UNSUPPORTED;
  if (q3_paged_attention_fast_path(Hq, Hkv, D, page, dtype) && (q_stride % 8) == 0) {
    if (splits < 1 || splits > MAX_SPLITS || (splits > 1 && workspace == nullptr)) return Q3_ERR_BAD_ARGUMENT;
    if (prompt_splits < 1 || prompt_splits > 4 || (prompt_splits > 1 && prompt_workspace == nullptr))
      return Q3_ERR_BAD_ARGUMENT;
    (void)max_kv_len;
    float* ws_acc = workspace;
    float* ws_ml = workspace ? workspace + (size_t)B * Hkv * splits * 16 * D : nullptr;
    if (D == 64)
      return launch_fast<64>(q, q_stride, out, k_cache, v_cache, num_pages, block_table, bt_stride, cu_q, kv_lens,
                             B, T_, Hq, Hkv, page, scale, window, max_q_len, min_q_len, splits, ws_acc, ws_ml,
                             prompt_splits, prompt_workspace, stream);
    return launch_fast<128>(q, q_stride, out, k_cache, v_cache, num_pages, block_table, bt_stride, cu_q, kv_lens, B,
                            T_, Hq, Hkv, page, scale, window, max_q_len, min_q_len, splits, ws_acc, ws_ml,
                            prompt_splits, prompt_workspace, stream);
  }
  Q3_DISPATCH_DTYPE(dtype, TT, return launch_general<TT>(q, q_stride, out, k_cache, v_cache, num_pages,
                                                        block_table, bt_stride, cu_q, kv_lens, B, Hq, Hkv,
                                                        D, page, scale, window, max_q_len, stream));
  return Q3_ERR_BAD_ARGUMENT;
}

// Whether `q3_decode_attention` takes a step of single tokens with these sizes: what the
// matrix-core kernels take, with a rotation (if any) over the whole head.
extern "C" int q3_decode_attention_takes(int Hq, int Hkv, int D, int page, int dtype, int rotary_dim) {
  return q3_paged_attention_fast_path(Hq, Hkv, D, page, dtype) && (rotary_dim == 0 || rotary_dim == D);
}

// A step in which every sequence brings one token, from the raw projections: qkv (B, (Hq +
// 2 Hkv) D) bfloat16 holds [q | k | v] of token b in row b (cu_q[b] = b). Per-head RMSNorm
// of q and k (weights of `w_dtype`, both or neither), rotation by `table` (or null), the new
// key and value written to the caches at position kv_lens[b] - 1 (if `store`), and attention
// over the cache, in one kernel and, with more than one split, the merge of its partial
// results (workspace as for q3_paged_attention). out (B, Hq D) bfloat16. `max_kv_len`: a bound
// on kv_lens that the host knows; a step that would pass the rotation table's end is refused.
extern "C" int q3_decode_attention(const void* qkv, void* out, void* k_cache, void* v_cache, int num_pages,
                                   const int* block_table, int bt_stride, const int* cu_q, const int* kv_lens,
                                   int B, int Hq, int Hkv, int D, int page, float scale, int window, int splits,
                                   float* workspace, const void* q_weight, const void* k_weight, int w_dtype,
                                   float eps, const float* table, int rotary_dim, int max_pos, int store,
                                   int max_kv_len, hipStream_t stream) {
  if (table && max_kv_len > max_pos) return Q3_ERR_BAD_ARGUMENT;
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || page <= 0) return Q3_ERR_BAD_ARGUMENT;
  if (B > 65535) return Q3_ERR_UNSUPPORTED;
  if (!q3_decode_attention_takes(Hq, Hkv, D, page, Q3_BF16, table ? rotary_dim : 0)) return Q3_ERR_UNSUPPORTED;
  if ((q_weight == nullptr) != (k_weight == nullptr)) return Q3_ERR_BAD_ARGUMENT;
  if (q_weight && w_dtype != Q3_F32 && w_dtype != Q3_BF16) return Q3_ERR_BAD_ARGUMENT;
  if (splits < 1 || splits > MAX_SPLITS || (splits > 1 && workspace == nullptr)) return Q3_ERR_BAD_ARGUMENT;
  float* ws_acc = workspace;
  float* ws_ml = workspace ? workspace + (size_t)B * Hkv * splits * 16 * D : nullptr;
  DecodePrep prep{};
  prep.q_weight = q_weight;
  prep.k_weight = k_weight;
  prep.eps = eps;
  prep.table = table;
  prep.max_pos = max_pos;
  prep.k_cache = store ? (bf16_t*)k_cache : nullptr;
  prep.v_cache = store ? (bf16_t*)v_cache : nullptr;
#define Q3_DECODE_PREP(DD, WW)                                                                                    \
  return launch_decode_prep<DD, WW>(qkv, out, k_cache, v_cache, num_pages, block_table, bt_stride, cu_q, kv_lens, \
                                    B, Hq, Hkv, page, scale, window, splits, ws_acc, ws_ml, prep, stream)
  if (D == 64) {
    if (w_dtype == Q3_F32) Q3_DECODE_PREP(64, float);
    Q3_DECODE_PREP(64, bf16_t);
  }
  if (w_dtype == Q3_F32) Q3_DECODE_PREP(128, float);
  Q3_DECODE_PREP(128, bf16_t);
#undef Q3_DECODE_PREP
}
