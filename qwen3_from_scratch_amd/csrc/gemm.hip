// out = x @ weight^T with float32 accumulation: x (M, K), weight (N, K), out (M, N).
#include "common.h"

// ---------------------------------------------------------------------------
// float32: plain fused multiply-adds, no matrix-core mode of reduced precision.
// A block of 256 threads computes a 64 x 64 tile of out; each thread a 4 x 4
// patch, summing over k in ascending order, so an output element's value does
// not depend on which rows share its batch. The same kernel with bfloat16
// operands (read one by one, summed in float32) serves bfloat16 products of any
// size that no matrix-core kernel takes: an inner size that is no multiple of 8.
// ---------------------------------------------------------------------------
#define F32_BM 64
#define F32_BN 64
#define F32_BK 16

template <typename IN, typename OUT>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const IN* __restrict__ a, const IN* __restrict__ w,
                                                       OUT* __restrict__ out, int M, int N, int K) {
  __shared__ float as[F32_BK][F32_BM + 4];
  __shared__ float ws[F32_BK][F32_BN + 4];
  const int t = threadIdx.x;
  const int m0 = blockIdx.y * F32_BM;
  const int n0 = blockIdx.x * F32_BN;
  const int tm = (t / 16) * 4;  // this thread's rows within the tile
  const int tn = (t % 16) * 4;  // and columns
  // loader coordinates: 64 rows x 16 k per tile, 4 elements per thread
  const int lr = t / 4;          // row 0..63
  const int lk = (t % 4) * 4;    // k offset 0, 4, 8, 12
  const bool vec = sizeof(IN) == 4 && (K % 4) == 0;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += F32_BK) {
    float av[4] = {0.f, 0.f, 0.f, 0.f}, wv[4] = {0.f, 0.f, 0.f, 0.f};
    const int gm = m0 + lr, gn = n0 + lr, gk = k0 + lk;
    if (gm < M) {
      const IN* p = a + (size_t)gm * K + gk;
      if (vec && gk + 3 < K) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        av[0] = v.x; av[1] = v.y; av[2] = v.z; av[3] = v.w;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (gk + i < K) av[i] = to_float(p[i]);
      }
    }
    if (gn < N) {
      const IN* p = w + (size_t)gn * K + gk;
      if (vec && gk + 3 < K) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        wv[0] = v.x; wv[1] = v.y; wv[2] = v.z; wv[3] = v.w;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (gk + i < K) wv[i] = to_float(p[i]);
      }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      as[lk + i][lr] = av[i];
      ws[lk + i][lr] = wv[i];
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < F32_BK; ++kk) {
      float ar[4], wr[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) ar[i] = as[kk][tm + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wr[j] = ws[kk][tn + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(ar[i], wr[j], acc[i][j]);
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gm = m0 + tm + i;
    if (gm >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + tn + j;
      if (gn < N) out[(size_t)gm * N + gn] = from_float<OUT>(acc[i][j]);
    }
  }
}


// ---------------------------------------------------------------------------
// bfloat16 with at most 16 rows (and, for small weights, a few groups of 16 rows, each a set of
// blocks of its own: q3_linear_tiled): a weight-streaming kernel. Every weight is
// read once from HBM and that read is the cost; the matrix cores do the sums
// (v_mfma_f32_16x16x32_bf16) with 16 weight rows as the A operand and the rows
// of x as the B operand, so out^T tiles come out with x's row in the lane's low
// bits: lane (m = lane % 16, g = lane / 16) ends with out[m][n0 + 4g .. 4g+3],
// four consecutive outputs of one row.
//
// A wavefront owns a slab of 16 weight rows and a share of K; the `kw`
// wavefronts that share a slab are summed through shared memory in a fixed
// order, so the result does not depend on timing. Loads are 16 bytes per lane;
// a lane's eight k-values are the same in A and B, which is all the product needs.
// K must be a multiple of 8; rows of the weight beyond N and k beyond K read as zero.
// (More rows of x per wavefront were tried, up to 64: the x operand loads then
// compete with the weight loads and the vendor library's kernels are faster.)
//
// With SWIGLU the weight's rows interleave a gate and an up matrix (row 2i gate, row 2i + 1
// up) and the kernel writes silu(gate) * up, out (M, N / 2): a lane's four consecutive
// outputs are two (gate, up) pairs.
// ---------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

union Pack16 {
  uint4 u;
  bf16x8_t v;
};

#define SKINNY_U 8  // k-steps of 32 per loop iteration: eight 16-byte loads of each operand in flight

//
// With TILED the weight is a copy laid out for this kernel, w[slab][k / 32][lane][8] with
// lane = (n % 16) + 16 * ((k % 32) / 8): the A operand of one matrix instruction is then one
// contiguous kilobyte instead of sixteen 64-byte pieces of sixteen rows, which the memory
// system serves about a fifth faster. Rows are padded with zeros to a multiple of 16, and K
// is a multiple of 32.
//
// Two fusions with the norm between two products, both for TILED weights only (`SkinnyFusion`):
// * EPI_RESIDUAL: the product is a residual stream's next addend. The epilogue rounds it to
//   bfloat16 (what a separate addition would have read), adds it into `residual` (M, N) float32
//   in place, writes (residual * norm_weight) as bfloat16 to out: the next norm's rows, weighted
//   but not yet divided by their root mean square; and leaves, per slab of 16 columns, each
//   row's sum of squares in `sums_out` (slabs, 16). A slab's columns belong to one wavefront,
//   so nothing is added twice and no order depends on timing.
// * `row_sums`: the rows of x are such weighted, unscaled rows. The block adds the partial sums
//   (`sums_rows` slabs of 16 rows) in a fixed order and multiplies row m of the product by
//   rsqrt(sum_m * inv_width + eps) before any other epilogue: (x / rms) @ W^T = (x @ W^T) / rms.
enum { EPI_PLAIN = 0, EPI_SWIGLU = 1, EPI_RESIDUAL = 2 };

struct SkinnyFusion {
  const float* row_sums;
  int sums_rows;
  float eps, inv_width;
  float* residual;
  const void* norm_weight;
  int norm_weight_f32;
  float* sums_out;
  int sums_stride;   // floats between two partial sums of a row, in row_sums and in sums_out: 16 or more, in steps of 4
};

#ifndef SKINNY_PAIR_SLABS
#define SKINNY_PAIR_SLABS 384   // from this many slabs on, and with more than eight rows of x, two slabs share a block
#endif
#define SKINNY_PRE 4  // float4 loads of partial sums a thread has in flight beside the main loop's

template <typename OUT, int EPI, bool TILED, bool SCALED, bool GROUPS>
__global__ __launch_bounds__(1024) void gemm_skinny_kernel(const bf16_t* __restrict__ x,
                                                           const bf16_t* __restrict__ w, OUT* __restrict__ out,
                                                           int M, int N, int K, int kw, int k_per_wave,
                                                           SkinnyFusion fu) {
  extern __shared__ float red[];  // [waves][64][4], then [waves][16] for the rows' sums
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int nwaves = blockDim.x >> 6;
  const int sw = nwaves / kw;
  // With GROUPS (more than 16 rows of x, for weights small enough to be read once per 16 rows): rows
  // 16 y .. 16 y + 15 of x, and of everything that has a row per row of x, belong to the blocks with
  // blockIdx.y = y, and a row's partial sums are fu.sums_stride floats apart. Without, the kernel is the
  // one for up to 16 rows, partial sums 16 floats apart.
  const int row0 = GROUPS ? 16 * (int)blockIdx.y : 0;
  const int sums_stride = GROUPS ? fu.sums_stride : 16;
  auto sums_at = [&](int i, int q) {   // rows 4 q .. 4 q + 3 of this group in partial sum i
    if constexpr (GROUPS)
      return reinterpret_cast<const float4*>(fu.row_sums + (size_t)i * sums_stride + row0)[q];
    else
      return reinterpret_cast<const float4*>(fu.row_sums)[i * 4 + q];
  };
  if constexpr (GROUPS) {
    M = min(16, M - row0);
    x += (size_t)row0 * K;
    out += (size_t)row0 * (EPI == EPI_SWIGLU ? N / 2 : N);
    if (EPI == EPI_RESIDUAL) fu.residual += (size_t)row0 * N;
  }
  const int slab = blockIdx.x * sw + wave / kw;
  const int ksplit = wave % kw;
  const int n0 = slab * 16;
  const int k_begin = ksplit * k_per_wave;
  const int k_end = min(K, k_begin + k_per_wave);
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};

  // partial sums of the rows' squares: thread -> (rows 4q .. 4q + 3, slabs i0, i0 + stride, ...)
  constexpr bool scaled = SCALED;
  float4 pre[SKINNY_PRE];
  if (scaled) {
    const int q = threadIdx.x & 3, i0 = threadIdx.x >> 2, stride = blockDim.x >> 2;
#pragma unroll
    for (int u = 0; u < SKINNY_PRE; ++u) {
      const int i = i0 + u * stride;
      pre[u] = i < fu.sums_rows ? sums_at(i, q) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  }
  // the residual and the norm's weights of this lane's four outputs, asked for before the products
  const int n = n0 + 4 * grp;
  float4 res = make_float4(0.f, 0.f, 0.f, 0.f), nw = res;
  const bool owner = EPI == EPI_RESIDUAL && ksplit == 0 && col < M && n + 3 < N;
  if (EPI == EPI_RESIDUAL && owner) {
    res = *reinterpret_cast<const float4*>(fu.residual + (size_t)col * N + n);
    if (fu.norm_weight_f32) {
      nw = *reinterpret_cast<const float4*>(static_cast<const float*>(fu.norm_weight) + n);
    } else {
      union {
        uint2 u;
        bf16_t e[4];
      } pk;
      pk.u = *reinterpret_cast<const uint2*>(static_cast<const bf16_t*>(fu.norm_weight) + n);
      nw = make_float4(bf16_to_float(pk.e[0]), bf16_to_float(pk.e[1]), bf16_to_float(pk.e[2]), bf16_to_float(pk.e[3]));
    }
  }

  const bool row_ok = TILED ? n0 < N : n0 + col < N;
  const bool x_ok = col < M;
  const bf16_t* wp = TILED ? w + (size_t)(row_ok ? slab : 0) * (K / 32) * 512 + lane * 8
                           : w + (size_t)(row_ok ? n0 + col : 0) * K + 8 * grp;
  const bf16_t* xp = x + (size_t)(x_ok ? col : 0) * K + 8 * grp;
  for (int k = k_begin; k < k_end; k += 32 * SKINNY_U) {
    Pack16 a[SKINNY_U], b[SKINNY_U];
#pragma unroll
    for (int u = 0; u < SKINNY_U; ++u) {
      const int kk = k + 32 * u;
      const bool k_ok = kk + 8 * grp + 8 <= k_end;
      if (TILED)
        a[u].u = (row_ok && k_ok) ? *reinterpret_cast<const uint4*>(wp + (size_t)(kk / 32) * 512) : make_uint4(0, 0, 0, 0);
      else
        a[u].u = (row_ok && k_ok) ? *reinterpret_cast<const uint4*>(wp + kk) : make_uint4(0, 0, 0, 0);
      b[u].u = (x_ok && k_ok) ? *reinterpret_cast<const uint4*>(xp + kk) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int u = 0; u < SKINNY_U; ++u) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u].v, b[u].v, acc, 0, 0, 0);
  }
  float* sums = red + (size_t)nwaves * 256;
  if (scaled) {
    float4 s = pre[0];
#pragma unroll
    for (int u = 1; u < SKINNY_PRE; ++u) {
      s.x += pre[u].x; s.y += pre[u].y; s.z += pre[u].z; s.w += pre[u].w;
    }
    const int q = threadIdx.x & 3, stride = blockDim.x >> 2;
    for (int i = (threadIdx.x >> 2) + SKINNY_PRE * stride; i < fu.sums_rows; i += stride) {
      const float4 v = sums_at(i, q);
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
#pragma unroll
    for (int off = 4; off < 64; off <<= 1) {
      s.x += __shfl_xor(s.x, off, 64); s.y += __shfl_xor(s.y, off, 64);
      s.z += __shfl_xor(s.z, off, 64); s.w += __shfl_xor(s.w, off, 64);
    }
    if (lane < 4) *reinterpret_cast<float4*>(sums + wave * 16 + 4 * lane) = s;
  }
  if (kw > 1) {
#pragma unroll
    for (int j = 0; j < 4; ++j) red[(wave * 64 + lane) * 4 + j] = acc[j];
  }
  if (kw > 1 || scaled) __syncthreads();
  if (kw > 1) {
    if (ksplit != 0) return;
    for (int s = 1; s < kw; ++s)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] += red[((wave + s) * 64 + lane) * 4 + j];
  }
  if (scaled) {
    float total = 0.f;
    for (int wv = 0; wv < nwaves; ++wv) total += sums[wv * 16 + col];
    const float r = rsqrtf(total * fu.inv_width + fu.eps);
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[j] *= r;
  }
  if constexpr (EPI == EPI_RESIDUAL) {
    // N is a multiple of 16 here: a slab is whole or absent
    float ss = 0.f;
    if (owner) {
      const float xn[4] = {res.x + bf16_to_float(float_to_bf16(acc[0])), res.y + bf16_to_float(float_to_bf16(acc[1])),
                           res.z + bf16_to_float(float_to_bf16(acc[2])), res.w + bf16_to_float(float_to_bf16(acc[3]))};
      *reinterpret_cast<float4*>(fu.residual + (size_t)col * N + n) = make_float4(xn[0], xn[1], xn[2], xn[3]);
      const float wn[4] = {nw.x, nw.y, nw.z, nw.w};
      union {
        uint2 u;
        bf16_t e[4];
      } pk;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        ss += xn[j] * xn[j];
        pk.e[j] = float_to_bf16(xn[j] * wn[j]);
      }
      *reinterpret_cast<uint2*>(reinterpret_cast<bf16_t*>(out) + (size_t)col * N + n) = pk.u;
    }
    ss += __shfl_xor(ss, 16, 64);
    ss += __shfl_xor(ss, 32, 64);
    if constexpr (GROUPS) {
      if (grp == 0 && n0 < N) fu.sums_out[(size_t)slab * sums_stride + row0 + col] = ss;
    } else {
      if (grp == 0 && n0 < N) fu.sums_out[slab * 16 + col] = ss;
    }
    return;
  }
  if (col >= M) return;
  if constexpr (EPI == EPI_SWIGLU) {
    OUT* o = out + (size_t)col * (N / 2) + n / 2;  // n is even: pairs (n, n + 1) and (n + 2, n + 3)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      if (n + 2 * j + 1 < N) {
        // the separate kernel sees gate and up rounded to the activation dtype: do the same
        const float g = to_float(from_float<OUT>(acc[2 * j])), u = to_float(from_float<OUT>(acc[2 * j + 1]));
        o[j] = from_float<OUT>(g / (1.f + expf(-g)) * u);
      }
    }
    return;
  }
  OUT* o = out + (size_t)col * N + n;
  if (n + 3 < N && (N % 4) == 0) {
    if constexpr (sizeof(OUT) == 4) {
      *reinterpret_cast<float4*>(o) = make_float4(acc[0], acc[1], acc[2], acc[3]);
    } else {
      union {
        uint2 u;
        bf16_t e[4];
      } pk;
#pragma unroll
      for (int j = 0; j < 4; ++j) pk.e[j] = float_to_bf16(acc[j]);
      *reinterpret_cast<uint2*>(o) = pk.u;
    }
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (n + j < N) o[j] = from_float<OUT>(acc[j]);
  }
}

// Two slabs per block from the tile-ordered copy: a wavefront's rows of x (the second operand)
// serve two matrix instructions, so a block reads x once for 32 weight rows instead of 16.
// With 8 to 16 rows of x the one-slab kernel moves as many bytes of x out of the L2 as weights
// out of memory, and that passage, about 7 TB/s over all CUs, is what bounds it (8, 12 and 16
// rows of the 8B layer's products: 85, 97 and 109 us; reading x from several copies changes
// nothing, so it is the volume, not a hot address). With pairs the gate/up product takes 41.6,
// 42.6 and 44.3 us at 8, 12 and 16 rows (one slab a block: 40.7, 46.1, 51.1) and the q/k/v
// product 13.1, 14.8, 15.8 (13.5, 15.7, 17.7): used with more than eight rows, where the pairs
// still give most CUs a block (384 slabs or more). Epilogues: plain and SwiGLU.
// (Four slabs a block, with four or with eight k-steps a turn, were slower: a decode step at batch 16 went from
// 4.91 to 5.32 and 5.40 ms.)
#define PAIR_PRE 2  // fewer partial sums in flight than the one-slab kernel: the registers go to the second slab
template <typename OUT, int EPI, bool SCALED>
__global__ __launch_bounds__(512, 4) void gemm_skinny_pair_kernel(const bf16_t* __restrict__ x,
                                                               const bf16_t* __restrict__ w, OUT* __restrict__ out,
                                                               int M, int N, int K, int kw, int k_per_wave,
                                                               SkinnyFusion fu) {
  static_assert(EPI == EPI_PLAIN || EPI == EPI_SWIGLU, "plain and SwiGLU epilogues");
  extern __shared__ float red[];  // [waves][2][64][4], then [waves][16] for the rows' sums
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int nwaves = blockDim.x >> 6;      // = kw: the block's wavefronts share K
  const int slabs = (N + 15) / 16;
  const int slab0 = 2 * blockIdx.x;
  const bool second = slab0 + 1 < slabs;
  const int k_begin = wave * k_per_wave;
  const int k_end = min(K, k_begin + k_per_wave);
  f32x4_t acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};

  constexpr bool scaled = SCALED;
  float4 pre[PAIR_PRE];
  if (scaled) {
    const int q = threadIdx.x & 3, i0 = threadIdx.x >> 2, stride = blockDim.x >> 2;
#pragma unroll
    for (int u = 0; u < PAIR_PRE; ++u) {
      const int i = i0 + u * stride;
      pre[u] = i < fu.sums_rows ? reinterpret_cast<const float4*>(fu.row_sums)[i * 4 + q] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  }
  const bool x_ok = col < M;
  const size_t slab_elems = (size_t)(K / 32) * 512;
  const bf16_t* wp0 = w + (size_t)slab0 * slab_elems + lane * 8;
  const bf16_t* wp1 = second ? wp0 + slab_elems : wp0;
  const bf16_t* xp = x + (size_t)(x_ok ? col : 0) * K + 8 * grp;
  for (int k = k_begin; k < k_end; k += 32 * SKINNY_U) {
    Pack16 a0[SKINNY_U], a1[SKINNY_U], b[SKINNY_U];
#pragma unroll
    for (int u = 0; u < SKINNY_U; ++u) {
      const int kk = k + 32 * u;
      const bool k_ok = kk + 8 * grp + 8 <= k_end;
      a0[u].u = k_ok ? *reinterpret_cast<const uint4*>(wp0 + (size_t)(kk / 32) * 512) : make_uint4(0, 0, 0, 0);
      a1[u].u = k_ok ? *reinterpret_cast<const uint4*>(wp1 + (size_t)(kk / 32) * 512) : make_uint4(0, 0, 0, 0);
      b[u].u = (x_ok && k_ok) ? *reinterpret_cast<const uint4*>(xp + kk) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int u = 0; u < SKINNY_U; ++u) {
      acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0[u].v, b[u].v, acc[0], 0, 0, 0);
      acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1[u].v, b[u].v, acc[1], 0, 0, 0);
    }
  }
  float* sums = red + (size_t)nwaves * 512;
  if (scaled) {
    float4 s = pre[0];
#pragma unroll
    for (int u = 1; u < PAIR_PRE; ++u) {
      s.x += pre[u].x; s.y += pre[u].y; s.z += pre[u].z; s.w += pre[u].w;
    }
    const int q = threadIdx.x & 3, stride = blockDim.x >> 2;
    for (int i = (threadIdx.x >> 2) + PAIR_PRE * stride; i < fu.sums_rows; i += stride) {
      const float4 v = reinterpret_cast<const float4*>(fu.row_sums)[i * 4 + q];
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
#pragma unroll
    for (int off = 4; off < 64; off <<= 1) {
      s.x += __shfl_xor(s.x, off, 64); s.y += __shfl_xor(s.y, off, 64);
      s.z += __shfl_xor(s.z, off, 64); s.w += __shfl_xor(s.w, off, 64);
    }
    if (lane < 4) *reinterpret_cast<float4*>(sums + wave * 16 + 4 * lane) = s;
  }
  if (nwaves > 1) {
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int j = 0; j < 4; ++j) red[((wave * 2 + h) * 64 + lane) * 4 + j] = acc[h][j];
  }
  if (nwaves > 1 || scaled) __syncthreads();
  if (wave != 0) return;
  // the wavefronts' sums in their order, as the one-slab kernel adds them
  for (int s = 1; s < nwaves; ++s)
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[h][j] += red[((s * 2 + h) * 64 + lane) * 4 + j];
  if (scaled) {
    float total = 0.f;
    for (int wv = 0; wv < nwaves; ++wv) total += sums[wv * 16 + col];
    const float r = rsqrtf(total * fu.inv_width + fu.eps);
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[h][j] *= r;
  }
  if (col >= M) return;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    if (h == 1 && !second) break;
    const int n = (slab0 + h) * 16 + 4 * grp;
    if constexpr (EPI == EPI_SWIGLU) {
      OUT* o = out + (size_t)col * (N / 2) + n / 2;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        if (n + 2 * j + 1 < N) {
          const float g = to_float(from_float<OUT>(acc[h][2 * j])), u = to_float(from_float<OUT>(acc[h][2 * j + 1]));
          o[j] = from_float<OUT>(g / (1.f + expf(-g)) * u);
        }
      }
    } else {
      OUT* o = out + (size_t)col * N + n;
      if (n + 3 < N && (N % 4) == 0) {
        if constexpr (sizeof(OUT) == 4) {
          *reinterpret_cast<float4*>(o) = make_float4(acc[h][0], acc[h][1], acc[h][2], acc[h][3]);
        } else {
          union {
            uint2 u;
            bf16_t e[4];
          } pk;
#pragma unroll
          for (int j = 0; j < 4; ++j) pk.e[j] = float_to_bf16(acc[h][j]);
          *reinterpret_cast<uint2*>(o) = pk.u;
        }
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (n + j < N) o[j] = from_float<OUT>(acc[h][j]);
      }
    }
  }
}

template <typename OUT, int EPI, bool TILED = false, bool SCALED = false>
static int launch_skinny(const void* x, const void* w, void* out, int M, int N, int K, hipStream_t stream,
                         SkinnyFusion fu = SkinnyFusion{}) {
  const int slabs = (N + 15) / 16;
  // One slab per block, its K shared by up to eight wavefronts, each with at least four
  // k-steps (measured on the 8B model's products at 1, 8 and 16 rows: eight beat four and
  // sixteen by a few percent each, and blocks of several slabs are slower); sixteen where
  // there are too few slabs to give every CU a block otherwise.
  const int kw_max = slabs < 256 ? 16 : 8;
  int kw = 1;
  while (kw < kw_max && K / (kw * 2) >= 128) kw *= 2;
  int sw = 1;
  while (sw * kw < 4 && sw * 2 <= slabs) sw *= 2;
  const int step = 32 * SKINNY_U;
  int k_per_wave = (K + kw - 1) / kw;
  k_per_wave = (k_per_wave + step - 1) / step * step;
  const int groups = (M + 15) / 16;   // of 16 rows of x: one, or a few for a small weight (q3_linear_tiled)
  if constexpr (TILED && (EPI == EPI_PLAIN || EPI == EPI_SWIGLU)) {
    if (slabs >= SKINNY_PAIR_SLABS && sw == 1 && M > 8 && groups == 1) {
      const size_t pair_smem = (size_t)kw * (2 * 64 * 4 + 16) * sizeof(float);
      hipLaunchKernelGGL((gemm_skinny_pair_kernel<OUT, EPI, SCALED>), dim3((slabs + 1) / 2), dim3(64 * kw), pair_smem,
                         stream, (const bf16_t*)x, (const bf16_t*)w, (OUT*)out, M, N, K, kw, k_per_wave, fu);
      return q3_launch_status();
    }
  }
  const int blocks = (slabs + sw - 1) / sw;
  const size_t smem = (size_t)sw * kw * (64 * 4 + 16) * sizeof(float);
  if (groups > 1) {
    if constexpr (TILED)
      hipLaunchKernelGGL((gemm_skinny_kernel<OUT, EPI, TILED, SCALED, true>), dim3(blocks, groups), dim3(64 * sw * kw), smem,
                         stream, (const bf16_t*)x, (const bf16_t*)w, (OUT*)out, M, N, K, kw, k_per_wave, fu);
    else
      return Q3_ERR_BAD_ARGUMENT;
  } else {
    hipLaunchKernelGGL((gemm_skinny_kernel<OUT, EPI, TILED, SCALED, false>), dim3(blocks), dim3(64 * sw * kw), smem, stream,
                       (const bf16_t*)x, (const bf16_t*)w, (OUT*)out, M, N, K, kw, k_per_wave, fu);
  }
  return q3_launch_status();
}

// ---------------------------------------------------------------------------
// float32 with few rows (decoding): the tiled kernel above would give a product of 8 x 4096
// 64 blocks; here the weights are streamed once by as many wavefronts as there are groups of
// four weight rows. A wavefront's lanes stride over k four elements at a time (a kilobyte of
// each weight row per turn, and of each row of x, which all wavefronts of a CU read at about
// the same time), every lane keeps 4 x MB sums, and the lanes' sums meet at the end in a fixed
// order: an output's value depends on K alone, not on the rows beside it.
// ---------------------------------------------------------------------------
#define F32_FEW_ROWS 4  // weight rows per wavefront

template <int MB>
__global__ __launch_bounds__(256) void gemm_f32_few_rows_kernel(const float* __restrict__ x,
                                                                const float* __restrict__ w,
                                                                float* __restrict__ out, int M, int N, int K) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = (blockIdx.x * 4 + wave) * F32_FEW_ROWS;
  if (n0 >= N) return;
  float acc[F32_FEW_ROWS][MB];
#pragma unroll
  for (int j = 0; j < F32_FEW_ROWS; ++j)
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[j][m] = 0.f;
  const float* rows[F32_FEW_ROWS];
#pragma unroll
  for (int j = 0; j < F32_FEW_ROWS; ++j) rows[j] = w + (size_t)min(n0 + j, N - 1) * K;  // a row past the end: read, not written
  for (int k = 4 * lane; k < K; k += 256) {
    float4 wv[F32_FEW_ROWS];
#pragma unroll
    for (int j = 0; j < F32_FEW_ROWS; ++j) wv[j] = *reinterpret_cast<const float4*>(rows[j] + k);
#pragma unroll
    for (int m = 0; m < MB; ++m) {
      if (m < M) {
        const float4 xv = *reinterpret_cast<const float4*>(x + (size_t)m * K + k);
#pragma unroll
        for (int j = 0; j < F32_FEW_ROWS; ++j) {
          float a = acc[j][m];
          a = fmaf(xv.x, wv[j].x, a);
          a = fmaf(xv.y, wv[j].y, a);
          a = fmaf(xv.z, wv[j].z, a);
          a = fmaf(xv.w, wv[j].w, a);
          acc[j][m] = a;
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < F32_FEW_ROWS; ++j)
#pragma unroll
    for (int m = 0; m < MB; ++m) {
      const float total = wave_sum(acc[j][m]);
      if (lane == 0 && m < M && n0 + j < N) out[(size_t)m * N + n0 + j] = total;
    }
}

// Whether the weight-streaming kernel takes this product.
extern "C" int q3_linear_is_skinny(int M, int N, int K, int in_dtype) {
  (void)N;  // any number of weight rows
  return in_dtype == Q3_BF16 && M >= 1 && M <= 16 && K % 8 == 0 && K >= 8;
}

extern "C" int q3_linear(const void* x, const void* weight, void* out, int M, int N, int K, int in_dtype,
                         int out_dtype, hipStream_t stream) {
  if (M <= 0 || N <= 0 || K <= 0) return Q3_ERR_BAD_ARGUMENT;
  if (in_dtype == Q3_F32) {
    if (out_dtype != Q3_F32) return Q3_ERR_BAD_ARGUMENT;
    if (M <= 16 && K % 4 == 0) {
      const dim3 few((N + 4 * F32_FEW_ROWS - 1) / (4 * F32_FEW_ROWS));
      if (M <= 4)
        hipLaunchKernelGGL(gemm_f32_few_rows_kernel<4>, few, dim3(256), 0, stream, (const float*)x,
                           (const float*)weight, (float*)out, M, N, K);
      else if (M <= 8)
        hipLaunchKernelGGL(gemm_f32_few_rows_kernel<8>, few, dim3(256), 0, stream, (const float*)x,
                           (const float*)weight, (float*)out, M, N, K);
      else
        hipLaunchKernelGGL(gemm_f32_few_rows_kernel<16>, few, dim3(256), 0, stream, (const float*)x,
                           (const float*)weight, (float*)out, M, N, K);
      return q3_launch_status();
    }
    const dim3 grid((N + F32_BN - 1) / F32_BN, (M + F32_BM - 1) / F32_BM);
    if (grid.y > 65535) return Q3_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((gemm_f32_kernel<float, float>), grid, dim3(256), 0, stream, (const float*)x,
                       (const float*)weight, (float*)out, M, N, K);
    return q3_launch_status();
  }
  if (in_dtype != Q3_BF16 || (out_dtype != Q3_F32 && out_dtype != Q3_BF16)) return Q3_ERR_BAD_ARGUMENT;
  if (!q3_linear_is_skinny(M, N, K, in_dtype)) {   // any size, by plain multiply-adds
    const dim3 grid((N + F32_BN - 1) / F32_BN, (M + F32_BM - 1) / F32_BM);
    if (grid.y > 65535) return Q3_ERR_UNSUPPORTED;
    if (out_dtype == Q3_F32)
      hipLaunchKernelGGL((gemm_f32_kernel<bf16_t, float>), grid, dim3(256), 0, stream, (const bf16_t*)x,
                         (const bf16_t*)weight, (float*)out, M, N, K);
    else
      hipLaunchKernelGGL((gemm_f32_kernel<bf16_t, bf16_t>), grid, dim3(256), 0, stream, (const bf16_t*)x,
                         (const bf16_t*)weight, (bf16_t*)out, M, N, K);
    return q3_launch_status();
  }
  return out_dtype == Q3_F32 ? launch_skinny<float, EPI_PLAIN>(x, weight, out, M, N, K, stream)
                             : launch_skinny<bf16_t, EPI_PLAIN>(x, weight, out, M, N, K, stream);
}

// out (M, N / 2) = silu(gate) * up where x @ weight^T interleaves gate and up columns
// (weight row 2i is gate's row i, row 2i + 1 up's). bfloat16, M <= 16, N even.
extern "C" int q3_linear_swiglu(const void* x, const void* weight, void* out, int M, int N, int K, int dtype,
                                hipStream_t stream) {
  if (M <= 0 || N <= 0 || K <= 0 || N % 2) return Q3_ERR_BAD_ARGUMENT;
  if (!q3_linear_is_skinny(M, N, K, dtype)) return Q3_ERR_UNSUPPORTED;
  return launch_skinny<bf16_t, EPI_SWIGLU>(x, weight, out, M, N, K, stream);
}

// The same products from the tile-ordered copy of the weight (see gemm_skinny_kernel):
// x (M, K) bfloat16, K a multiple of 32. `epilogue`: 0 output (M, N) in `out_dtype`;
// 1 the activation (output (M, N / 2) bfloat16); 2 the residual addition and the next norm's
// preparation (N a multiple of 16; `residual` (M, N) float32 updated in place, `norm_weight`
// (N,) of `norm_w_dtype`, output (M, N) bfloat16 = residual * norm_weight, `sums_out`
// (N / 16, sums_stride) float32). `row_sums` (sums_rows, sums_stride) float32, if not null, says that
// x's rows still lack the factor rsqrt(sum / width + eps), which the product's rows then receive.
// `sums_stride`: floats between two partial sums of one row: 16 for up to 16 rows, else a multiple of 4 and at
// least M rounded up to 16.
// M <= 16, or up to Q3_SKINNY_MAX_ROWS for a weight small enough that reading it once per 16 rows costs
// less than a kernel more (the caller's rule; every group of 16 rows is a set of blocks of its own).
#define Q3_SKINNY_MAX_ROWS 64
extern "C" int q3_linear_tiled_max_rows() { return Q3_SKINNY_MAX_ROWS; }

extern "C" int q3_linear_tiled(const void* x, const void* weight_tiled, void* out, int M, int N, int K,
                               int out_dtype, int epilogue, const float* row_sums, int sums_rows, float eps,
                               int width, float* residual, const void* norm_weight, int norm_w_dtype,
                               float* sums_out, int sums_stride, hipStream_t stream) {
  if (M <= 0 || M > Q3_SKINNY_MAX_ROWS || N <= 0 || K <= 0 || K % 32) return Q3_ERR_BAD_ARGUMENT;
  SkinnyFusion fu{};
  if (row_sums || sums_out) {
    if (sums_stride % 4 || sums_stride < (M + 15) / 16 * 16 || (M <= 16 && sums_stride != 16)) return Q3_ERR_BAD_ARGUMENT;
    fu.sums_stride = sums_stride;
  }
  if (row_sums) {
    if (sums_rows <= 0 || width <= 0) return Q3_ERR_BAD_ARGUMENT;
    fu.row_sums = row_sums;
    fu.sums_rows = sums_rows;
    fu.eps = eps;
    fu.inv_width = 1.f / (float)width;
  }
  if (epilogue == EPI_SWIGLU) {
    if (N % 2 || out_dtype != Q3_BF16) return Q3_ERR_BAD_ARGUMENT;
    return row_sums ? launch_skinny<bf16_t, EPI_SWIGLU, true, true>(x, weight_tiled, out, M, N, K, stream, fu)
                    : launch_skinny<bf16_t, EPI_SWIGLU, true>(x, weight_tiled, out, M, N, K, stream, fu);
  }
  if (epilogue == EPI_RESIDUAL) {
    if (row_sums || N % 16 || out_dtype != Q3_BF16 || !residual || !norm_weight || !sums_out ||
        (norm_w_dtype != Q3_F32 && norm_w_dtype != Q3_BF16))
      return Q3_ERR_BAD_ARGUMENT;
    fu.residual = residual;
    fu.norm_weight = norm_weight;
    fu.norm_weight_f32 = norm_w_dtype == Q3_F32;
    fu.sums_out = sums_out;
    return launch_skinny<bf16_t, EPI_RESIDUAL, true>(x, weight_tiled, out, M, N, K, stream, fu);
  }
  if (epilogue != EPI_PLAIN) return Q3_ERR_BAD_ARGUMENT;
  if (row_sums)
    return out_dtype == Q3_F32
               ? launch_skinny<float, EPI_PLAIN, true, true>(x, weight_tiled, out, M, N, K, stream, fu)
               : launch_skinny<bf16_t, EPI_PLAIN, true, true>(x, weight_tiled, out, M, N, K, stream, fu);
  return out_dtype == Q3_F32 ? launch_skinny<float, EPI_PLAIN, true>(x, weight_tiled, out, M, N, K, stream, fu)
                             : launch_skinny<bf16_t, EPI_PLAIN, true>(x, weight_tiled, out, M, N, K, stream, fu);
}
