// A weight-streaming matrix-core product for some tens of rows of x (17 to 96), out[M, N] =
// x[M, K] . w[N, K]^T in bfloat16 with float32 accumulation, from the tile-ordered copy of the
// weight that the few-row kernel of gemm.hip reads (w[slab][k / 32][lane][8], one contiguous
// kilobyte per matrix instruction). The reference has no kernel for this range of its own: its
// engine sends every projection to the vendor library (src/qwen3_from_scratch/models/self_attn.py:312-342)
// and the feed-forward to one Triton kernel of 128 x 128 tiles
// (src/qwen3_from_scratch/kernels/triton/gemm.py:26-274).
//
// With 17 to 128 rows a product is still bound by the one pass over the weight, but the rows of x
// no longer fit a wavefront's registers, and if every slab of 16 weight rows fetches them from the
// L2 again they pass from the L2 as often as the weight passes from memory (M / 16 times as many
// bytes). Here a block of WS x 2 wavefronts owns WS slabs and walks K in chunks of 256: the chunk
// of x (all rows) goes through shared memory once per block, so x leaves the L2 once per WS slabs;
// each wavefront multiplies its slab's 128 k of the chunk (the weight straight from memory into
// registers, as the first operand of v_mfma_f32_16x16x32_bf16, x from shared memory as the second)
// into MT accumulators of 16 x 16, the weight of the next chunk already on its way. The two
// wavefronts of a slab add up through shared memory in a fixed order. One barrier per chunk.
//
// The product runs whole (no shares of K, no second kernel), with the epilogues of tiles::store_tile:
// the division by the rows' root mean square that the norm before it left out, SwiGLU over interleaved
// (gate, up) rows, bfloat16 or float32 output. It is taken where its blocks fill the chip in one round
// (see slabs_per_block): a block holds a CU alone, all blocks take the same time, and what a second, partly
// filled round costs is more than the kernel saves.
//
// With 9 to 16 rows the few-row kernel of gemm.hip fetches x per slab (or per pair of slabs) and that
// traffic slows it (gate/up 42.5 us at 12 rows, 44.7 at 16); this kernel takes 40 us at any of them, and
// serves that product there too. Below nine rows the few-row kernel is as fast or faster, and the products
// with fewer slabs would need their K shared out and a second kernel, which costs more than it saves.
//
// Measured with cold caches, weights in turn, against the other route for these rows (for a layer's products
// the tiled kernel of gemm_tiles.h with K shared out and its adding kernel, for the vocabulary's what the
// table of sizes names), microseconds at 24 / 48 / 64 / 96 rows:
//   8B gate/up   24,576 x 4,096, 256 blocks of six slabs     40.7 / 41.0 / 41.6 / 47.9   against 46.3 / 53.7 / 52.8 / 61.1
//   14B gate/up  34,816 x 5,120, 544 blocks of four          80.3 / 86.0 / 94.2 / 122.7  against 69.2 / 76.6 / 77.4 / 97.1
//   32B gate/up  51,200 x 5,120, 534 blocks of six          113.6 / 121.0 / 130.0 / 160.5 against 101.2 / 108.9 / 111.3 / 144.5
//   vocabulary   151,936 x 4,096, 1,583 blocks of six       234.6 / 253.1 / 270.9 / 319.3 against 230.2 / 240.3 / 247.6 / 270.6
//   q/k/v with K in two to five shares and a second kernel: equal on the 8B layer, a tenth slower on the others.
// So it wins where one round of blocks covers the product and loses beyond; shares of K never paid, and the
// kernel has none. With the weight loads alone and no arithmetic the 8B gate/up product takes 42 us at 64 rows,
// so it is the stream that takes the time. Two slabs per wavefront: the same; starting every block at another
// chunk changes nothing.
// K must be a multiple of 32 (the tile-ordered copy has no other), N of 2.
#pragma once

#include "gemm_tiles.h"

namespace stream {

using tiles::f32x4_t;
using tiles::Frag;
using tiles::RowScale;

constexpr int WK = 2;            // wavefronts that share a slab's chunk
constexpr int KC = 128;          // k per wavefront per chunk
constexpr int KCB = KC * WK;     // k per chunk
constexpr int STEPS = KC / 32;   // matrix instructions per accumulator per chunk
constexpr int ROW = KCB * 2 + 32;   // bytes of a row of x in shared memory: 32 more than its data. With 16 more the
                                    // operand reads (16 bytes a lane, sixteen rows a group of lanes) took eight cycles of
                                    // shared memory each, four of them counted as bank conflicts; with 32 more four and none
                                    // (measured with the read pattern alone)
constexpr int MOST_ROWS = 96;

constexpr int smem_bytes(int MT, int WS) {
  const int x_bytes = 2 * MT * 16 * ROW, sums_bytes = WS * WK * MT * 64 * 16;
  return x_bytes > sums_bytes ? x_bytes : sums_bytes;
}

template <typename OUT, int EPI, int MT, int WS>
__global__ __launch_bounds__(WS * WK * 64) void gemm_stream_kernel(const bf16_t* __restrict__ x,
                                                                   const bf16_t* __restrict__ wt, OUT* __restrict__ out,
                                                                   int M, int N, int K, RowScale scale) {
  constexpr int THREADS = WS * WK * 64;
  constexpr int ROWS = MT * 16;
  constexpr int PIECES = ROWS * KCB / 8;                        // 16-byte pieces of a chunk of x
  constexpr int PER_THREAD = (PIECES + THREADS - 1) / THREADS;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];   // two chunks of x, ROWS x ROW bytes each
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ws = wave % WS, wk = wave / WS;
  const int col = lane & 15, grp = lane >> 4;
  const int slabs = (N + 15) / 16;
  const int slab = blockIdx.x * WS + ws;
  const bool slab_ok = slab < slabs;
  const int chunks = (K + KCB - 1) / KCB;
  const bf16_t* wp = wt + (size_t)(slab_ok ? slab : 0) * (K / 32) * 512 + lane * 8;

  f32x4_t acc[MT][1];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t][0] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  auto load_w = [&](Frag (&a)[STEPS], int c) {
    const int k0 = c * KCB + wk * KC;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int k = k0 + 32 * s;
      a[s].u = (slab_ok && k < K) ? *reinterpret_cast<const uint4*>(wp + (size_t)(k / 32) * 512) : make_uint4(0, 0, 0, 0);
    }
  };
  auto load_x = [&](uint4 (&r)[PER_THREAD], int c) {
    const int k0 = c * KCB;
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int piece = threadIdx.x + i * THREADS;
      const int row = piece / (KCB / 8), k = k0 + (piece % (KCB / 8)) * 8;
      r[i] = (piece < PIECES && row < M && k < K) ? *reinterpret_cast<const uint4*>(x + (size_t)row * K + k)
                                                   : make_uint4(0, 0, 0, 0);
    }
  };
  auto store_x = [&](const uint4 (&r)[PER_THREAD], int buffer) {
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int piece = threadIdx.x + i * THREADS;
      if (piece < PIECES)
        *reinterpret_cast<uint4*>(lds + buffer * ROWS * ROW + (piece / (KCB / 8)) * ROW + (piece % (KCB / 8)) * 16) = r[i];
    }
  };
  auto multiply = [&](const Frag (&a)[STEPS], int buffer) {
    const unsigned char* base = lds + buffer * ROWS * ROW + col * ROW + (wk * KC + 8 * grp) * 2;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      Frag b[MT];
#pragma unroll
      for (int t = 0; t < MT; ++t) b[t].u = *reinterpret_cast<const uint4*>(base + t * 16 * ROW + s * 64);
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[t][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[s].v, b[t].v, acc[t][0], 0, 0, 0);
    }
  };

  Frag even[STEPS], odd[STEPS];
  uint4 staged[PER_THREAD];
  load_w(even, 0);
  load_x(staged, 0);
  // the rows' factors while the first loads are on their way: the partial sums of squares (few chunks of
  // 1,024 columns from the kernel that adds the tiled kernel's shares of K, hundreds of slabs from the few-row kernel) are
  // added by the whole block, thread (g, r) the chunks g, g + G, ... of row r, then the G sums of a row in
  // their order: a fixed order of additions
  float factor[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) factor[t] = 1.f;
  if (scale.sums) {
    __shared__ float part[THREADS];
    constexpr int G = THREADS / ROWS;
    const int r = threadIdx.x % ROWS, g = threadIdx.x / ROWS;
    float sum = 0.f;
    if (g < G && r < scale.rows)
      for (int c = g; c < scale.chunks; c += G) sum += scale.sums[(size_t)c * scale.rows + r];
    part[threadIdx.x] = sum;
    __syncthreads();
    if (wk == 0) {
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        float total = 0.f;
        for (int g2 = 0; g2 < G; ++g2) total += part[g2 * ROWS + 16 * t + col];
        factor[t] = rsqrtf(total * scale.inv_width + scale.eps);
      }
    }
  }
  store_x(staged, 0);
  for (int c = 0; c < chunks; c += 2) {
    // chunk c: its weight in `even`, its x in buffer 0; the next chunk's loads go out before the wait
    if (c + 1 < chunks) {
      load_w(odd, c + 1);
      load_x(staged, c + 1);
    }
    __syncthreads();            // buffer 0 is written; nobody still reads buffer 1
    multiply(even, 0);
    if (c + 1 >= chunks) break;
    store_x(staged, 1);
    if (c + 2 < chunks) {
      load_w(even, c + 2);
      load_x(staged, c + 2);
    }
    __syncthreads();            // buffer 1 is written; nobody still reads buffer 0
    multiply(odd, 1);
    if (c + 2 < chunks) store_x(staged, 0);
  }
  // the second wavefront of every slab hands its sums over, and the first adds them to its own
  __syncthreads();
  float* sums = reinterpret_cast<float*>(lds);          // [slab of the block][MT][64 lanes][4]
  if (wk > 0) {
#pragma unroll
    for (int t = 0; t < MT; ++t) *reinterpret_cast<f32x4_t*>(sums + ((ws * MT + t) * 64 + lane) * 4) = acc[t][0];
  }
  __syncthreads();
  if (wk > 0 || !slab_ok) return;
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t][0] += *reinterpret_cast<const f32x4_t*>(sums + ((ws * MT + t) * 64 + lane) * 4);
  tiles::store_tile<OUT, EPI, MT, 1>(acc, out, M, N, 0, slab * 16, col, grp, factor);
}

// How many slabs a block takes (6 or 4) so that the blocks fill the chip's `cus` CUs in one round, at least
// three CUs in four busy; 0 where neither does. Up to 16 rows blocks of six only (measured: blocks of four
// are some microseconds slower there).
inline int slabs_per_block(int M, int N, int cus) {
  const int slabs = (N + 15) / 16;
  for (int ws : {6, 4}) {
    const int blocks = (slabs + ws - 1) / ws;
    if (blocks <= cus && 4 * blocks >= 3 * cus) return ws;
    if (M <= 16) break;
  }
  return 0;
}

inline bool takes(int M, int N, int K) { return M > 8 && M <= MOST_ROWS && N >= 16 && K >= KCB && K % 32 == 0 && N % 2 == 0; }

template <typename OUT, int EPI, int MT, int WS>
int launch_shape(const void* x, const void* wt, void* out, int M, int N, int K, hipStream_t stream, const RowScale& scale) {
  constexpr int SMEM = smem_bytes(MT, WS);
  static bool raised[16] = {};   // the dynamic shared-memory limit, once per device
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 16) return Q3_ERR_BAD_ARGUMENT;
  auto kernel = gemm_stream_kernel<OUT, EPI, MT, WS>;
  if (!raised[device]) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, SMEM);
    if (e != hipSuccess) return (int)e;
    raised[device] = true;
  }
  const int blocks = ((N + 15) / 16 + WS - 1) / WS;
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(WS * WK * 64), SMEM, stream, (const bf16_t*)x, (const bf16_t*)wt,
                     (OUT*)out, M, N, K, scale);
  return q3_launch_status();
}

// x (M, K) row-major, wt the tile-ordered copy of w (N, K), `ws` slabs per block; `scale` as for tiles::launch.
template <typename OUT, int EPI>
int launch(int ws, const void* x, const void* wt, void* out, int M, int N, int K, hipStream_t stream,
           const RowScale& scale = RowScale()) {
  if (!takes(M, N, K) || (ws != 6 && ws != 4)) return Q3_ERR_BAD_ARGUMENT;
  const int mt = (M + 15) / 16;
#define Q3_STREAM_SHAPE(MT_)                                                                   \
  return ws == 6 ? launch_shape<OUT, EPI, MT_, 6>(x, wt, out, M, N, K, stream, scale)          \
                 : launch_shape<OUT, EPI, MT_, 4>(x, wt, out, M, N, K, stream, scale)
  switch (mt) {
    case 1: Q3_STREAM_SHAPE(1);
    case 2: Q3_STREAM_SHAPE(2);
    case 3: Q3_STREAM_SHAPE(3);
    case 4: Q3_STREAM_SHAPE(4);
    case 5:
    case 6: Q3_STREAM_SHAPE(6);
  }
#undef Q3_STREAM_SHAPE
  return Q3_ERR_BAD_ARGUMENT;
}

}  // namespace stream
