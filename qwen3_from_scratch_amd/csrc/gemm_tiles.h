// A matrix-core product for many rows, out[M, N] = x[M, K] . w[N, K]^T in bfloat16 with
// float32 accumulation: the counterpart of the reference's own GEMM kernel
// (src/qwen3_from_scratch/kernels/triton/gemm.py:26-274, 128 x 128 tiles, float32
// accumulation), written for gfx950.
//
// A block of WM x WN wavefronts owns a BM x BN tile of the output and walks K in steps of
// 64. Both operands have K contiguous, so a step's slices of x and of w are BM and BN rows of
// 128 bytes. They travel from memory to shared memory by loads that write shared memory
// directly (16 bytes a lane, a wavefront's 64 lanes fill one contiguous kilobyte, eight rows),
// the slices of the next STAGES - 1 steps while the current one is multiplied. Within a row the
// eight 16-byte pieces are placed by an XOR with bits 1..3 of the row number, so that the
// sixteen lanes that read one piece of sixteen consecutive rows (an operand of
// v_mfma_f32_16x16x32_bf16) touch every bank once. The loads are issued as assembly with their
// own wait counts (see attn_prefill_kernel in attention.hip for why).
//
// The weight rows are the matrix instruction's first operand and the rows of x its second, so
// a lane ends with four consecutive outputs of one row of x: pairs (gate, up) for the SwiGLU
// epilogue, eight bytes of bfloat16 for the plain one.
//
// What bounds it (2,048 x 24,576 x 4,096, 256 x 256 tiles, eight wavefronts of 64 x 128): with
// the copies taken out 233 us (1.77 PFLOP/s), with copies that always hit the cache 303, with
// the copies issued and never waited for 328, as it is 323 (1.27; the matrix pipes are busy 59 %
// of the cycles, no bank conflicts), the vendor library's best kernel 279. So it is the copies'
// passage itself, not their latency, that takes the time from the operand reads. The other
// matrix instruction, v_mfma_f32_32x32x16_bf16, runs at 2.4 PFLOP/s from registers where
// this kernel's 16 x 16 x 32 runs at 2.2 (one wavefront a SIMD: 2.25 against 1.8), and in this
// kernel it changed nothing (256 x 256 tiles 417 us beside the library's 312 on a box where the
// 16 x 16 x 32 form took about 375; no bank conflicts, the matrix pipes busy 39 % of the time):
// the time goes to the wait for each step's copies with only two stages in flight, not to
// the multiplications. Tried and not
// kept: steps of 32 in four stages with the next step's operands read while the current one is
// multiplied (385); copies through registers and ds_write (365); wavefront tiles of 128 x 128,
// one wavefront a SIMD (364).
//
// A product with few tiles (576 x 4,096 x 12,288: 160 tiles of 128 x 128 on 256 CUs) shares K
// out over several blocks per tile, whose float32 partial products a second kernel adds in a
// fixed order.
//
// For steps of some tens of rows it carries what the few-row kernel of gemm.hip carries for up
// to sixteen: the division by the rows' root mean square that the norm before the product
// left out (RowScale: in the epilogue, also before SwiGLU, or in the kernel that adds the
// shares of K), and the residual addition with the next norm's preparation
// (tiles_residual_kernel, which takes the float32 partial products, a single share too).
//
// K must be a multiple of 64. Rows of x beyond M and of w beyond N are read from the last
// valid row and never written. Blocks are numbered so that the eight XCDs each take a
// contiguous run of tiles, M fastest: the blocks that share a slice of w run on one XCD at
// about the same time and the slice comes from memory once.

#pragma once

#include "common.h"

namespace tiles {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

union Frag {
  uint4 u;
  bf16x8_t v;
};

enum { EPI_PLAIN = 0, EPI_SWIGLU = 1 };

constexpr int BK = 64;          // k per step: two matrix instructions deep
constexpr int ROW_BYTES = 128;  // a row of a slice

template <int BM, int BN, int WM, int WN, int STAGES>
struct Shape {
  static constexpr int THREADS = 64 * WM * WN;
  static constexpr int STAGE_BYTES = (BM + BN) * ROW_BYTES;
  static constexpr int SMEM_BYTES = STAGES * STAGE_BYTES;
  static constexpr int TURN_ROWS = THREADS / 8;               // rows of a slice that one turn of the block fills
  static constexpr int X_TURNS = BM / TURN_ROWS, W_TURNS = BN / TURN_ROWS;  // loads a thread issues per step
  static constexpr int LOADS = X_TURNS + W_TURNS;
  static constexpr int MI = BM / WM / 16, NJ = BN / WN / 16;  // 16 x 16 blocks of a wavefront's tile
  static_assert(BM % TURN_ROWS == 0 && BN % TURN_ROWS == 0 && (BM / WM) % 16 == 0 && (BN / WN) % 16 == 0, "shape");
};

// four outputs to bfloat16 (round to nearest even, as float_to_bf16: the hardware's conversion)
__device__ inline uint2 pack_bf16x4(f32x4_t c) {
  typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;
  union {
    bf16x4_t v;
    uint2 u;
  } pk;
  pk.v = __builtin_convertvector(c, bf16x4_t);
  return pk.u;
}

// The rows of x may still lack the factor of the norm before this product: they hold
// stream * norm_weight, and `sums` (chunks, rows) holds the rows' sums of squares of the stream in
// partial sums of column chunks (tiles_residual_kernel and the few-row kernel of gemm.hip leave them
// so; `rows` is the distance between two partial sums of one row, the number of rows or more). Row m
// of the product is then multiplied by rsqrt(sum_m * inv_width + eps): (x / rms) @ W^T = (x @ W^T) / rms.
struct RowScale {
  const float* sums = nullptr;
  int chunks = 0, rows = 0;
  float eps = 0.f, inv_width = 0.f;
  // the partial sums are asked for eight at a time (a chain of loads otherwise) and added in the chunks' order
  __device__ float of(int m) const {
    float total = 0.f;
    for (int c0 = 0; c0 < chunks; c0 += 8) {
      float part[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) part[k] = c0 + k < chunks ? sums[(size_t)(c0 + k) * rows + m] : 0.f;
#pragma unroll
      for (int k = 0; k < 8; ++k)
        if (c0 + k < chunks) total += part[k];
    }
    return rsqrtf(total * inv_width + eps);
  }
};

// The sum of `splits` partial products' quads at `at` (`stride` floats apart), added in the splits' order; the
// loads go out eight at a time.
__device__ inline float4 sum_of_shares(const float* __restrict__ partials, size_t at, size_t stride, int splits) {
  float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int s0 = 0; s0 < splits; s0 += 8) {
    float4 part[8];
#pragma unroll
    for (int k = 0; k < 8; ++k)
      if (s0 + k < splits) part[k] = *reinterpret_cast<const float4*>(partials + (size_t)(s0 + k) * stride + at);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      if (s0 + k >= splits) continue;
      if (s0 + k == 0) {
        sum = part[k];
      } else {
        sum.x += part[k].x; sum.y += part[k].y; sum.z += part[k].z; sum.w += part[k].w;
      }
    }
  }
  return sum;
}

// A wavefront's outputs to memory: lane (col, grp) of block (i, j) holds out[m][n .. n + 3] with
// m = m_base + 16 i + col, n = n_base + 16 j + 4 grp.
template <typename OUT, int EPI, int MI, int NJ>
__device__ inline void store_tile(const f32x4_t (&acc)[MI][NJ], OUT* __restrict__ out, int M, int N, int m_base,
                                  int n_base, int col, int grp, const float (&factor)[MI]) {
#pragma unroll
  for (int i = 0; i < MI; ++i) {
    const int m = m_base + 16 * i + col;
    if (m >= M) continue;
    const float r = factor[i];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int n = n_base + 16 * j + 4 * grp;
      if (n >= N) continue;
      const f32x4_t c = acc[i][j] * r;
      if constexpr (EPI == EPI_SWIGLU) {
        // rows of w interleave gate and up (row 2 i gate, row 2 i + 1 up); both are rounded to
        // the activation type first, as a separate activation kernel would have read them
        OUT* o = out + (size_t)m * (N / 2) + n / 2;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
          if (n + 2 * p + 1 < N) {
            const float g = to_float(from_float<OUT>(c[2 * p])), u = to_float(from_float<OUT>(c[2 * p + 1]));
            o[p] = from_float<OUT>(g / (1.f + expf(-g)) * u);
          }
        }
      } else {
        OUT* o = out + (size_t)m * N + n;
        if (n + 3 < N && (N % 4) == 0) {
          if constexpr (sizeof(OUT) == 4) {
            *reinterpret_cast<float4*>(o) = make_float4(c[0], c[1], c[2], c[3]);
          } else {
            *reinterpret_cast<uint2*>(o) = pack_bf16x4(c);
          }
        } else {
#pragma unroll
          for (int q = 0; q < 4; ++q)
            if (n + q < N) o[q] = from_float<OUT>(c[q]);
        }
      }
    }
  }
}

template <typename OUT, int EPI, int BM, int BN, int WM, int WN, int STAGES>
__global__ __launch_bounds__(64 * WM * WN) void gemm_tiles_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                         OUT* __restrict__ out, int M, int N, int K, int tiles_m,
                                                         int tiles_total, int tiles_per_xcd, int steps_per_split,
                                                         float* __restrict__ partials, RowScale scale) {
  typedef Shape<BM, BN, WM, WN, STAGES> S;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  // block -> tile: XCD x (blocks x, x + 8, ...) takes tiles [x * per, (x + 1) * per)
  const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
  const int tile = xcd * tiles_per_xcd + local;
  if (local >= tiles_per_xcd || tile >= tiles_total) return;
  const int m0 = (tile % tiles_m) * BM, n0 = (tile / tiles_m) * BN;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int wm = wave % WM, wn = wave / WM;

  // the copies: in turn j this thread fills place THREADS j + tid of a slice (16 bytes each,
  // row = place / 8), with the piece that the XOR puts there
  const int piece = (tid & 7) ^ ((tid >> 4) & 7);
  const bf16_t* x_src[S::X_TURNS];
  const bf16_t* w_src[S::W_TURNS];
#pragma unroll
  for (int j = 0; j < S::X_TURNS; ++j)
    x_src[j] = x + (size_t)min(m0 + S::TURN_ROWS * j + (tid >> 3), M - 1) * K + 8 * piece;
#pragma unroll
  for (int j = 0; j < S::W_TURNS; ++j)
    w_src[j] = w + (size_t)min(n0 + S::TURN_ROWS * j + (tid >> 3), N - 1) * K + 8 * piece;
  typedef __attribute__((address_space(3))) unsigned char* lds_ptr;
  const unsigned smem_lds = (unsigned)(unsigned long)(lds_ptr)smem;
  auto load_to_lds = [&](const void* src, unsigned lds) {
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds) : "memory", "m0");
  };
  auto copy_step = [&](int kt, int stage) {
    const unsigned base = __builtin_amdgcn_readfirstlane(smem_lds + stage * S::STAGE_BYTES + 1024 * wave);
#pragma unroll
    for (int j = 0; j < S::X_TURNS; ++j) load_to_lds(x_src[j] + (size_t)kt * BK, base + 16 * S::THREADS * j);
#pragma unroll
    for (int j = 0; j < S::W_TURNS; ++j)
      load_to_lds(w_src[j] + (size_t)kt * BK, base + BM * ROW_BYTES + 16 * S::THREADS * j);
  };
  // loads complete in the order they were issued: with no more than the later steps' loads
  // outstanding, this thread's share of the next step has landed
  auto wait_for_step = [&](int steps_after) {
    if (steps_after <= 0)
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else if (steps_after == 1)
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(S::LOADS) : "memory");
    else if (steps_after == 2 || STAGES <= 4)
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * S::LOADS) : "memory");
    else if (steps_after == 3 || STAGES <= 5)
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(STAGES > 4 ? 3 * S::LOADS : 0) : "memory");
    else
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(STAGES > 5 ? 4 * S::LOADS : 0) : "memory");
  };
  static_assert(STAGES >= 2 && STAGES <= 6 && (STAGES - 2) * S::LOADS < 64, "the wait counts above");

  // operand reads: row 16 i + col of this wavefront's half of a slice, pieces 4 s + grp
  const int swz = (col >> 1) & 7;
  int read_off[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) read_off[s] = col * ROW_BYTES + 16 * ((4 * s + grp) ^ swz);
  const int x_half = wm * (BM / WM) * ROW_BYTES, w_half = BM * ROW_BYTES + wn * (BN / WN) * ROW_BYTES;

  f32x4_t acc[S::MI][S::NJ];
#pragma unroll
  for (int i = 0; i < S::MI; ++i)
#pragma unroll
    for (int j = 0; j < S::NJ; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // with K shared out over gridDim.y blocks, this one walks steps first .. first + steps - 1
  const int first = blockIdx.y * steps_per_split;
  const int steps = min(K / BK - first, steps_per_split);
  auto multiply_stage = [&](const unsigned char* st) {
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      Frag xf[S::MI], wf[S::NJ];
#pragma unroll
      for (int i = 0; i < S::MI; ++i)
        xf[i].u = *reinterpret_cast<const uint4*>(st + x_half + 16 * i * ROW_BYTES + read_off[s]);
#pragma unroll
      for (int j = 0; j < S::NJ; ++j)
        wf[j].u = *reinterpret_cast<const uint4*>(st + w_half + 16 * j * ROW_BYTES + read_off[s]);
#pragma unroll
      for (int i = 0; i < S::MI; ++i)
#pragma unroll
        for (int j = 0; j < S::NJ; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[j].v, xf[i].v, acc[i][j], 0, 0, 0);
    }
  };
  float factor[S::MI];
  {
#pragma unroll
    for (int ahead = 0; ahead < STAGES - 1; ++ahead)
      if (ahead < steps) copy_step(first + ahead, ahead);
    // the rows' factors while the first copies are on their way (the wait for them is one for those copies too)
#pragma unroll
    for (int i = 0; i < S::MI; ++i) {
      const int m = m0 + wm * (BM / WM) + 16 * i + col;
      factor[i] = scale.sums && m < M ? scale.of(m) : 1.f;
    }
    for (int kt = 0; kt < steps; ++kt) {
      // step kt has landed in every thread's view, and nobody still reads the stage that the
      // next copy overwrites (step kt - 1's)
      wait_for_step(min(kt + STAGES - 2, steps - 1) - kt);
      __syncthreads();
      if (kt + STAGES - 1 < steps) copy_step(first + kt + STAGES - 1, (kt + STAGES - 1) % STAGES);
      multiply_stage(smem + (kt % STAGES) * S::STAGE_BYTES);
    }
  }
  if (partials)   // a share of K: float32 sums for gemm_tiles_reduce_kernel
    store_tile<float, EPI_PLAIN, S::MI, S::NJ>(acc, partials + (size_t)blockIdx.y * M * N, M, N, m0 + wm * (BM / WM),
                                               n0 + wn * (BN / WN), col, grp, factor);
  else
    store_tile<OUT, EPI, S::MI, S::NJ>(acc, out, M, N, m0 + wm * (BM / WM), n0 + wn * (BN / WN), col, grp, factor);
}

// out = the sum of `splits` float32 partial products (each M x N, N a multiple of 4), added in the
// splits' order: a fixed order of additions. With `scale`, row m is multiplied by its factor
// (see RowScale); with SWIGLU the columns are (gate, up) pairs and out is (M, N / 2).
template <typename OUT, bool SWIGLU>
__global__ __launch_bounds__(256) void gemm_tiles_reduce_kernel(const float* __restrict__ partials, OUT* __restrict__ out,
                                                                size_t quads, int quads_per_row, int splits,
                                                                RowScale scale) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= quads) return;
  const float r = scale.sums ? scale.of((int)(i / quads_per_row)) : 1.f;
  float4 sum = sum_of_shares(partials, 4 * i, 4 * quads, splits);
  sum.x *= r; sum.y *= r; sum.z *= r; sum.w *= r;
  if constexpr (SWIGLU) {
    // both rounded to the activation type first, as a separate activation kernel would have read them
    const float g0 = to_float(from_float<OUT>(sum.x)), u0 = to_float(from_float<OUT>(sum.y));
    const float g1 = to_float(from_float<OUT>(sum.z)), u1 = to_float(from_float<OUT>(sum.w));
    OUT* o = out + 2 * i;
    o[0] = from_float<OUT>(g0 / (1.f + expf(-g0)) * u0);
    o[1] = from_float<OUT>(g1 / (1.f + expf(-g1)) * u1);
  } else if constexpr (sizeof(OUT) == 4) {
    reinterpret_cast<float4*>(out)[i] = sum;
  } else {
    reinterpret_cast<uint2*>(out)[i] = pack_bf16x4(f32x4_t{sum.x, sum.y, sum.z, sum.w});
  }
}

// The product as a residual stream's next addend, with the next norm prepared: the sum of the
// partial products is rounded to bfloat16 (what a separate addition would have read), added
// into `residual` (M, N) float32 in place, (residual * norm_weight) goes to `values` as
// bfloat16, and the row's sum of squares over this block's 1,024 columns to sums[chunk][row]
// (`sums_stride` floats a chunk). Grid (chunks of 1,024 columns, rows), 256 threads, four columns a
// thread; N a multiple of 4.
constexpr int CHUNK_COLUMNS = 1024;
template <typename NW>
__global__ __launch_bounds__(256) void tiles_residual_kernel(const float* __restrict__ partials, int splits,
                                                             float* __restrict__ residual,
                                                             const NW* __restrict__ norm_weight,
                                                             bf16_t* __restrict__ values, float* __restrict__ sums,
                                                             int sums_stride, int M, int N) {
  __shared__ float scratch[17];
  const int m = blockIdx.y, n = blockIdx.x * CHUNK_COLUMNS + 4 * threadIdx.x;
  float ss = 0.f;
  if (n < N) {
    const size_t at = (size_t)m * N + n;
    float4 r = *reinterpret_cast<const float4*>(residual + at);
    const float4 sum = sum_of_shares(partials, at, (size_t)M * N, splits);
    r.x += bf16_to_float(float_to_bf16(sum.x)); r.y += bf16_to_float(float_to_bf16(sum.y));
    r.z += bf16_to_float(float_to_bf16(sum.z)); r.w += bf16_to_float(float_to_bf16(sum.w));
    *reinterpret_cast<float4*>(residual + at) = r;
    union {
      uint2 u;
      bf16_t e[4];
    } pk;
    pk.e[0] = float_to_bf16(r.x * to_float(norm_weight[n]));
    pk.e[1] = float_to_bf16(r.y * to_float(norm_weight[n + 1]));
    pk.e[2] = float_to_bf16(r.z * to_float(norm_weight[n + 2]));
    pk.e[3] = float_to_bf16(r.w * to_float(norm_weight[n + 3]));
    *reinterpret_cast<uint2*>(values + at) = pk.u;
    ss = r.x * r.x + r.y * r.y + r.z * r.z + r.w * r.w;
  }
  const float total = block_sum(ss, scratch);
  if (threadIdx.x == 0) sums[(size_t)blockIdx.x * sums_stride + m] = total;
}

// The tile shapes on offer: (BM, BN, STAGES).
constexpr int NUM_CONFIGS = 9;

// `splits` > 1: K is shared out over that many blocks per tile, which leave float32 partial
// products in `partials` (splits x M x N floats) for a second kernel to add, which also applies
// the epilogue; N a multiple of 4.
// `keep_partials`: the partial products (also a single one) stay in `partials` for the caller's
// own second kernel. `scale`: see RowScale.
template <typename OUT, int EPI, int BM, int BN, int WM, int WN, int STAGES>
int launch_config(const void* x, const void* w, void* out, int M, int N, int K, int splits, float* partials,
                  hipStream_t stream, const RowScale& scale = RowScale(), bool keep_partials = false,
                  int* splits_used = nullptr) {
  typedef Shape<BM, BN, WM, WN, STAGES> S;
  static bool raised[16] = {};   // the dynamic shared-memory limit, once per device
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 16) return Q3_ERR_BAD_ARGUMENT;
  auto kernel = gemm_tiles_kernel<OUT, EPI, BM, BN, WM, WN, STAGES>;
  if (!raised[device]) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, S::SMEM_BYTES);
    if (e != hipSuccess) return (int)e;
    raised[device] = true;
  }
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const long total = (long)tiles_m * tiles_n;
  if (total > (1L << 28)) return Q3_ERR_UNSUPPORTED;
  const int per_xcd = (int)((total + 7) / 8);
  const int steps = K / BK;
  if (splits < 1 || splits > steps || splits > 64) return Q3_ERR_BAD_ARGUMENT;
  if ((splits > 1 || keep_partials) && (N % 4 || partials == nullptr)) return Q3_ERR_BAD_ARGUMENT;
  const int per_split = (steps + splits - 1) / splits;
  const int used = (steps + per_split - 1) / per_split;     // no block without a step
  const bool to_partials = used > 1 || keep_partials;
  hipLaunchKernelGGL(kernel, dim3(8 * per_xcd, used), dim3(S::THREADS), S::SMEM_BYTES, stream, (const bf16_t*)x,
                     (const bf16_t*)w, (OUT*)out, M, N, K, tiles_m, (int)total, per_xcd, per_split,
                     to_partials ? partials : nullptr, to_partials ? RowScale() : scale);
  if (splits_used) *splits_used = used;
  if (to_partials && !keep_partials) {
    const size_t quads = (size_t)M * N / 4;
    hipLaunchKernelGGL((gemm_tiles_reduce_kernel<OUT, EPI == EPI_SWIGLU>), dim3((unsigned)((quads + 255) / 256)),
                       dim3(256), 0, stream, partials, (OUT*)out, quads, N / 4, used, scale);
  }
  return q3_launch_status();
}

// The number of shares of K that fills the chip once for this size and tile shape (1: the
// tiles alone do, or the steps are too few to share out).
inline int splits_that_fill(int config, int M, int N, int K) {
  // tile rows, tile columns, blocks resident at once on 256 CUs (what shared memory allows)
  static const int shape[NUM_CONFIGS][3] = {{128, 128, 512}, {128, 128, 256}, {256, 128, 256}, {256, 256, 256},
                                            {256, 256, 256}, {64, 128, 512}, {64, 128, 768}, {64, 256, 512},
                                            {64, 128, 256}};
  if (config < 0 || config >= NUM_CONFIGS) return 1;
  const int bm = shape[config][0], bn = shape[config][1], slots = shape[config][2];
  const long tiles = (long)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
  int splits = (int)(slots / tiles);
  const int steps = K / BK;
  while (splits > 1 && steps / splits < 8) --splits;           // a share keeps eight steps at least
  return splits < 2 || N % 4 ? 1 : (splits > 16 ? 16 : splits);
}

template <typename OUT, int EPI>
int launch(int config, const void* x, const void* w, void* out, int M, int N, int K, hipStream_t stream,
           int splits = 1, float* partials = nullptr, const RowScale& scale = RowScale(), bool keep_partials = false,
           int* splits_used = nullptr) {
  switch (config) {
    case 0: return launch_config<OUT, EPI, 128, 128, 2, 2, 2>(x, w, out, M, N, K, splits, partials, stream, scale, keep_partials, splits_used);
    case 1: return launch_config<OUT, EPI, 128, 128, 2, 2, 3>(x, w, out, M, N, K, splits, partials, stream, scale, keep_partials, splits_used);
    case 2: return launch_config<OUT, EPI, 256, 128, 4, 2, 2>(x, w, out, M, N, K, splits, partials, stream, scale, keep_partials, splits_used);
    case 3: return launch_config<OUT, EPI, 256, 256, 2, 4, 2>(x, w, out, M, N, K, splits, partials, stream, scale, keep_partials, splits_used);
    case 4: return launch_config<OUT, EPI, 256, 256, 4, 2, 2>(x, w, out, M, N, K, splits, partials, stream, scale, keep_partials, splits_used);
    case 5: return launch_config<OUT, EPI, 64, 128, 1, 4, 3>(x, w, out, M, N, K, splits, partials, stream, scale, keep_partials, splits_used);
    case 6: return launch_config<OUT, EPI, 64, 128, 1, 4, 2>(x, w, out, M, N, K, splits, partials, stream, scale, keep_partials, splits_used);
    case 7: return launch_config<OUT, EPI, 64, 256, 1, 8, 2>(x, w, out, M, N, K, splits, partials, stream, scale, keep_partials, splits_used);
    case 8: return launch_config<OUT, EPI, 64, 128, 1, 4, 5>(x, w, out, M, N, K, splits, partials, stream, scale, keep_partials, splits_used);
  }
  return Q3_ERR_BAD_ARGUMENT;
}

// Whether the kernel takes a product at all.
inline bool takes(int M, int N, int K) { return M > 0 && N > 0 && K >= BK && K % BK == 0; }

}  // namespace tiles
