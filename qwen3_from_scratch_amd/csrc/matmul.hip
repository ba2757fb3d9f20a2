// Matrix products with many rows, out[M, N] = x[M, K] . w[N, K]^T in bfloat16
// with float32 accumulation, through the vendor library (hipBLASLt), as the
// reference's engine uses its vendor library for them
// (src/qwen3_from_scratch/models/linear.py:24-31 calls F.linear).
//
// The library's heuristic returns a ranked list of kernels for a problem; its
// first choice is often not its fastest (for 576 x 5120 x 17408 the first took
// 108 us and the fourth 92; for 2048 x 4096 x 4096, 101 against 55). The first
// time a problem size is seen outside a graph capture, the leading candidates
// are timed on the caller's own operands and the fastest is kept for the life
// of the process. A size first seen during a capture runs the first candidate
// and is tuned at its next eager call. In the model every weight is read once
// a step, with gigabytes of other traffic in between, so a candidate is timed
// with cold caches: a kernel that reads a buffer larger than the last-level
// cache runs before each timed run. Timed warm, products of few rows pick
// kernels that are the fastest only while the weight sits in that cache.
//
// The hand-written tiled kernel (gemm_tiles.h) stands in the same contest: where it takes a
// size (K a multiple of 64) two or three of its tile shapes, chosen by the rows, are timed after
// the library's candidates, each also with K shared out over several blocks per tile where its
// tiles alone would not fill the chip, and a size goes to whichever kernel was the fastest. q3_matmul_set_kernels narrows the
// contest to the library's kernels alone, or to the hand-written ones where they take the size.
//
// One workspace, one such buffer and one buffer for the hand-written kernel's partial products
// per device, allocated at first need and kept. Calls on one
// device share it and the plans: they are serialised by a lock and are meant
// to come from one stream at a time.

#include "common.h"
#include "gemm_tiles.h"

#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#define Q3_ERR_LIBRARY 20000   // + the library's status
#define Q3_DECLINED 1          // q3_tiles_residual: nothing was done, the caller's other way is faster

namespace {

constexpr size_t WORKSPACE_BYTES = 128u << 20;
constexpr size_t EVICT_BYTES = 512u << 20;     // twice the 256 MB last-level cache
constexpr size_t PARTIALS_BYTES = 128u << 20;  // float32 partial products of the hand-written kernel's K shares
constexpr size_t STAGING_BYTES = 64u << 20;
constexpr int EVICT_BLOCKS = 2048, EVICT_THREADS = 256;
constexpr int MAX_CANDIDATES = 64;

// Reads the whole buffer; the store never happens (the buffer holds zeros) but keeps the loads alive.
__global__ void evict_kernel(float4* buffer, size_t count) {
  float sum = 0.f;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x) {
    const float4 v = buffer[i];
    sum += v.x + v.y + v.z + v.w;
  }
  if (sum == 12345.f) buffer[0].x = sum;
}

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t w = nullptr, x = nullptr, out = nullptr;
  hipblasLtMatmulAlgo_t algo;
  bool tuned = false;
  int own = -1;            // the hand-written kernel's tile shape, if that was chosen; else `algo`
  int own_splits = 1;      // and over how many blocks it shares K out
  int candidates = 0, chosen = 0;
  float first_us = 0.f, best_us = 0.f;
};

struct Device {
  hipblasLtHandle_t handle = nullptr;
  void* workspace = nullptr;
  void* evict = nullptr;
  float* partials = nullptr;
  float* staging = nullptr;   // a float32 product on its way to the kernel that divides its rows (q3_tiles_scaled)
  hipEvent_t begin = nullptr, end = nullptr;
  std::map<std::tuple<int, int, int, int>, Plan> plans;
  // what was chosen for a size, by its rows rounded up to a multiple of 32: sizes beyond 64
  // rows that differ only within such a step take the choice of the first one that was timed
  // (a serving loop meets dozens of them, a prompt's portion plus however many requests decode)
  std::map<std::tuple<int, int, int, int>, Plan> chosen_near;
  // (kind, M, N, K) -> (tile shape, shares of K) of the products that carry a norm (q3_tiles_*)
  std::map<std::tuple<int, int, int, int>, std::pair<int, int>> fused;
};

int rows_class(int M) { return M <= 64 ? M : (M + 31) / 32 * 32; }

std::mutex g_lock;
std::map<int, Device> g_devices;
int g_candidates = 16;
enum { KERNELS_BOTH = 0, KERNELS_LIBRARY = 1, KERNELS_OWN = 2 };
int g_kernels = KERNELS_BOTH;
// The tile shapes that enter the contest, by the product's rows (the others never won a size of the 8B, 14B
// and 32B models there): small tiles with three stages where the weights' passage bounds the product, the
// largest where the matrix units do. Each enters a second time with K shared out where its tiles alone would
// not fill the chip.
constexpr int OWN_FEW_ROWS[] = {1, 5}, OWN_SOME_ROWS[] = {0, 1, 2}, OWN_MANY_ROWS[] = {0, 2, 4};
constexpr int MAX_OWN = 6;
inline const int* own_shapes(int M, int& count) {
  if (M <= 256) {
    count = 2;
    return OWN_FEW_ROWS;
  }
  count = 3;
  return M <= 1024 ? OWN_SOME_ROWS : OWN_MANY_ROWS;
}

#define HIP_TRY(call)                    \
  do {                                   \
    hipError_t e_ = (call);              \
    if (e_ != hipSuccess) return (int)e_; \
  } while (0)
#define LT_TRY(call)                                              \
  do {                                                            \
    hipblasStatus_t s_ = (call);                                  \
    if (s_ != HIPBLAS_STATUS_SUCCESS) return Q3_ERR_LIBRARY + (int)s_; \
  } while (0)

int describe(Plan& p, int M, int N, int K, int out_dtype) {
  // Row-major x (M, K), w (N, K), out (M, N) are column-major (K, M), (K, N), (N, M):
  // out_cm = w_cm^T . x_cm.
  const hipDataType out_type = out_dtype == Q3_F32 ? HIP_R_32F : HIP_R_16BF;
  LT_TRY(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
  hipblasOperation_t transposed = HIPBLAS_OP_T, plain = HIPBLAS_OP_N;
  LT_TRY(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &transposed, sizeof(transposed)));
  LT_TRY(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &plain, sizeof(plain)));
  LT_TRY(hipblasLtMatrixLayoutCreate(&p.w, HIP_R_16BF, K, N, K));
  LT_TRY(hipblasLtMatrixLayoutCreate(&p.x, HIP_R_16BF, K, M, K));
  LT_TRY(hipblasLtMatrixLayoutCreate(&p.out, out_type, N, M, N));
  return 0;
}

void forget(Plan& p) {
  if (p.w) (void)hipblasLtMatrixLayoutDestroy(p.w);
  if (p.x) (void)hipblasLtMatrixLayoutDestroy(p.x);
  if (p.out) (void)hipblasLtMatrixLayoutDestroy(p.out);
  if (p.desc) (void)hipblasLtMatmulDescDestroy(p.desc);
  p = Plan();
}

int run_own(Device& d, int config, int splits, const void* x, const void* w, void* out, int M, int N, int K,
            int out_dtype, hipStream_t stream) {
  if (splits > 1 && (!d.partials || (size_t)splits * M * N * sizeof(float) > PARTIALS_BYTES)) return Q3_ERR_UNSUPPORTED;
  return out_dtype == Q3_F32
             ? tiles::launch<float, tiles::EPI_PLAIN>(config, x, w, out, M, N, K, stream, splits, d.partials)
             : tiles::launch<bf16_t, tiles::EPI_PLAIN>(config, x, w, out, M, N, K, stream, splits, d.partials);
}

hipblasStatus_t run(Device& d, const Plan& p, const hipblasLtMatmulAlgo_t& algo, const void* x, const void* w,
                    void* out, hipStream_t stream) {
  const float one = 1.f, zero = 0.f;
  return hipblasLtMatmul(d.handle, p.desc, &one, w, p.w, x, p.x, &zero, out, p.out, out, p.out, &algo, d.workspace,
                         WORKSPACE_BYTES, stream);
}

// The shortest of `reps` runs of `launch`, each with cold caches, in microseconds; negative if it fails.
template <typename Launch>
float time_runs(Device& d, hipStream_t stream, int reps, Launch launch) {
  float best = -1.f;
  for (int r = 0; r < reps; ++r) {
    evict_kernel<<<EVICT_BLOCKS, EVICT_THREADS, 0, stream>>>((float4*)d.evict, EVICT_BYTES / sizeof(float4));
    if (hipEventRecord(d.begin, stream) != hipSuccess) return -1.f;
    if (!launch()) return -1.f;
    if (hipEventRecord(d.end, stream) != hipSuccess || hipEventSynchronize(d.end) != hipSuccess) return -1.f;
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, d.begin, d.end) != hipSuccess) return -1.f;
    if (best < 0.f || ms * 1000.f < best) best = ms * 1000.f;
  }
  return best;
}

float time_candidate(Device& d, const Plan& p, const hipblasLtMatmulAlgo_t& algo, const void* x, const void* w,
                     void* out, hipStream_t stream, int reps) {
  return time_runs(d, stream, reps, [&] { return run(d, p, algo, x, w, out, stream) == HIPBLAS_STATUS_SUCCESS; });
}

int choose(Device& d, Plan& p, const void* x, const void* w, void* out, int M, int N, int K, int out_dtype,
           hipStream_t stream, bool capturing) {
  const bool own_takes = tiles::takes(M, N, K) && g_kernels != KERNELS_LIBRARY;
  if (own_takes && g_kernels == KERNELS_OWN && capturing) {   // untimed: the first shape, timed at the next eager call
    p.candidates = 1;
    p.chosen = 0;
    int count = 0;
    p.own = own_shapes(M, count)[0];
    p.own_splits = 1;
    p.tuned = false;
    return 0;
  }
  hipblasLtMatmulPreference_t pref = nullptr;
  LT_TRY(hipblasLtMatmulPreferenceCreate(&pref));
  size_t bytes = WORKSPACE_BYTES;
  hipblasStatus_t s = hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &bytes,
                                                            sizeof(bytes));
  const int want = capturing ? 1 : g_candidates;
  std::vector<hipblasLtMatmulHeuristicResult_t> found(want);
  int got = 0;
  if (s == HIPBLAS_STATUS_SUCCESS)
    s = hipblasLtMatmulAlgoGetHeuristic(d.handle, p.desc, p.w, p.x, p.out, p.out, pref, want, found.data(), &got);
  (void)hipblasLtMatmulPreferenceDestroy(pref);
  if (s != HIPBLAS_STATUS_SUCCESS) return Q3_ERR_LIBRARY + (int)s;
  if (got == 0) return Q3_ERR_UNSUPPORTED;
  p.candidates = got;
  p.chosen = 0;
  p.own = -1;
  p.own_splits = 1;
  p.algo = found[0].algo;
  p.tuned = !capturing;
  if (capturing || (got == 1 && !own_takes)) return 0;
  if (!d.evict) {
    HIP_TRY(hipMalloc(&d.evict, EVICT_BYTES));
    HIP_TRY(hipMemsetAsync(d.evict, 0, EVICT_BYTES, stream));
  }
  // two passes: all candidates briefly (the first run of each also loads its code), then those
  // near the front again and longer
  // candidates from `got` on are the hand-written kernel's: (tile shape, shares of K)
  int own_config[MAX_OWN], own_splits[MAX_OWN], owns = 0;
  if (own_takes) {
    int count = 0;
    const int* shapes = own_shapes(M, count);
    for (int i = 0; i < count; ++i) {
      own_config[owns] = shapes[i];
      own_splits[owns++] = 1;
      const int splits = tiles::splits_that_fill(shapes[i], M, N, K);
      if (splits < 2 || (size_t)splits * M * N * sizeof(float) > PARTIALS_BYTES) continue;
      if (!d.partials) HIP_TRY(hipMalloc((void**)&d.partials, PARTIALS_BYTES));
      own_config[owns] = shapes[i];
      own_splits[owns++] = splits;
    }
  }
  const int all = got + owns;
  const int first = g_kernels == KERNELS_OWN && own_takes ? got : 0;
  auto time_one = [&](int i, int reps) {
    if (i < got) return time_candidate(d, p, found[i].algo, x, w, out, stream, reps);
    return time_runs(d, stream, reps, [&] {
      return run_own(d, own_config[i - got], own_splits[i - got], x, w, out, M, N, K, out_dtype, stream) == 0;
    });
  };
  std::vector<float> us(all, -1.f);
  float best = -1.f;
  for (int i = first; i < all; ++i) {
    if (time_one(i, 1) < 0.f) continue;     // the first run of a kernel also loads its code
    us[i] = time_one(i, 2);
    if (us[i] > 0.f && (best < 0.f || us[i] < best)) best = us[i];
  }
  if (best < 0.f) return Q3_ERR_UNSUPPORTED;
  for (int i = first; i < all; ++i) {
    if (us[i] < 0.f || us[i] > 1.2f * best) continue;
    const float again = time_one(i, 5);
    if (again > 0.f && again < us[i]) us[i] = again;
  }
  int chosen = -1;
  for (int i = first; i < all; ++i)
    if (us[i] > 0.f && (chosen < 0 || us[i] < us[chosen])) chosen = i;
  p.candidates = all - first;
  p.chosen = chosen - first;
  if (chosen < got) {
    p.algo = found[chosen].algo;
  } else {
    p.own = own_config[chosen - got];
    p.own_splits = own_splits[chosen - got];
  }
  p.first_us = us[first];
  p.best_us = us[chosen];
  return 0;
}

// The product by the plan's kernel.
int run_plan(Device& d, const Plan& p, const void* x, const void* w, void* out, int M, int N, int K, int out_dtype,
             hipStream_t stream) {
  if (p.own >= 0) return run_own(d, p.own, p.own_splits, x, w, out, M, N, K, out_dtype, stream);
  const hipblasStatus_t s = run(d, p, p.algo, x, w, out, stream);
  return s == HIPBLAS_STATUS_SUCCESS ? 0 : Q3_ERR_LIBRARY + (int)s;
}

// out = x @ w^T by whichever kernel the contest chose for the size (the lock is held).
int product(Device& d, const void* x, const void* w, void* out, int M, int N, int K, int out_dtype, hipStream_t stream) {
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  HIP_TRY(hipStreamIsCapturing(stream, &capture));
  const bool capturing = capture != hipStreamCaptureStatusNone;
  if (!d.handle) {
    if (capturing) return (int)hipErrorStreamCaptureUnsupported;   // the first call on a device allocates
    HIP_TRY(hipMalloc(&d.workspace, WORKSPACE_BYTES));
    if (!d.begin) {
      HIP_TRY(hipEventCreate(&d.begin));
      HIP_TRY(hipEventCreate(&d.end));
    }
    LT_TRY(hipblasLtCreate(&d.handle));
  }
  Plan& p = d.plans[std::make_tuple(M, N, K, out_dtype)];
  if (!p.desc) {
    const int status = describe(p, M, N, K, out_dtype);
    if (status) {
      forget(p);
      return status;
    }
  }
  const auto near_key = std::make_tuple(rows_class(M), N, K, out_dtype);
  if (!p.tuned) {
    auto near = d.chosen_near.find(near_key);
    if (near != d.chosen_near.end()) {   // a neighbour's choice, if the library takes it for this size
      p.own = near->second.own;
      p.own_splits = near->second.own_splits;
      p.algo = near->second.algo;
      if (run_plan(d, p, x, w, out, M, N, K, out_dtype, stream) == 0) {
        p.candidates = near->second.candidates;
        p.chosen = near->second.chosen;
        p.first_us = near->second.first_us;
        p.best_us = near->second.best_us;
        p.tuned = true;
        return 0;
      }
    }
  }
  if (!p.candidates || (!p.tuned && !capturing)) {
    const int status = choose(d, p, x, w, out, M, N, K, out_dtype, stream, capturing);
    if (status) {
      forget(p);
      return status;
    }
    if (p.tuned) {
      Plan& kept = d.chosen_near[near_key];   // the choice only: the descriptors stay with their size
      kept.algo = p.algo;
      kept.own = p.own;
      kept.own_splits = p.own_splits;
      kept.candidates = p.candidates;
      kept.chosen = p.chosen;
      kept.first_us = p.first_us;
      kept.best_us = p.best_us;
    }
  }
  return run_plan(d, p, x, w, out, M, N, K, out_dtype, stream);
}

// Tile shape and shares of K for a product of some tens of rows that carries a norm. `kind` tells the
// variants apart (0 plain, 1 SwiGLU, 2 residual); `launch(config, splits)` runs one without side effects and
// returns its status; `other()` does the same work around the contest's product (the vendor library's, mostly)
// and wins where the tiled kernel's tiles fit the size badly: `config` is then LIBRARY. Timed once per size
// with cold caches outside a graph capture; a capture that meets a new size takes the rule of thumb and leaves
// the timing to the next eager call.
constexpr int LIBRARY = -1;
template <typename Launch, typename Other>
int choose_fused(Device& d, int kind, int M, int N, int K, hipStream_t stream, Launch launch, Other other, int& config,
                 int& splits) {
  // rows that differ within a step of eight share a choice: a serving loop meets most of them
  const auto key = std::make_tuple(kind + 4 * g_kernels, (M + 7) / 8 * 8, N, K);
  auto known = d.fused.find(key);
  if (known != d.fused.end()) {
    config = known->second.first;
    splits = known->second.second;
    return 0;
  }
  // 64 x 128 tiles also with five stages: with K shared out they need fewer shares to fill the chip (q/k/v at
  // 64 rows 17.7 us in 5 shares against 21.9 in 8). The 64 x 256 tiles lose here too (gate/up 67 us against 51).
  constexpr int FUSED_SHAPES[] = {1, 5, 8};
  int configs[6], shares[6], n = 0;
  for (int shape : FUSED_SHAPES) {
    const int fill = tiles::splits_that_fill(shape, M, N, K);   // the same for all rows that share the choice
    if (fill > 1 && (size_t)fill * ((M + 7) / 8 * 8) * N * sizeof(float) <= PARTIALS_BYTES) {
      configs[n] = shape;
      shares[n++] = fill;
    }
    configs[n] = shape;
    shares[n++] = 1;
  }
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  HIP_TRY(hipStreamIsCapturing(stream, &capture));
  if (!d.partials) {
    if (capture != hipStreamCaptureStatusNone) return (int)hipErrorStreamCaptureUnsupported;
    HIP_TRY(hipMalloc((void**)&d.partials, PARTIALS_BYTES));
  }
  config = configs[0];
  splits = shares[0];
  if (capture != hipStreamCaptureStatusNone) return 0;
  if (!d.begin) {
    HIP_TRY(hipEventCreate(&d.begin));
    HIP_TRY(hipEventCreate(&d.end));
  }
  if (!d.evict) {
    HIP_TRY(hipMalloc(&d.evict, EVICT_BYTES));
    HIP_TRY(hipMemsetAsync(d.evict, 0, EVICT_BYTES, stream));
  }
  float best = -1.f;
  // the first call of the other way holds that product's own contest: not inside a timed run, whose events it uses
  const bool other_works = g_kernels != KERNELS_OWN && other() == 0;
  for (int i = 0; i < n && !(other_works && g_kernels == KERNELS_LIBRARY); ++i) {
    auto one = [&] { return launch(configs[i], shares[i]) == 0; };
    if (time_runs(d, stream, 1, one) < 0.f) continue;   // the first run also loads the code
    const float us = time_runs(d, stream, 4, one);
    if (us > 0.f && (best < 0.f || us < best)) {
      best = us;
      config = configs[i];
      splits = shares[i];
    }
  }
  if (other_works) {
    const float us = time_runs(d, stream, 4, [&] { return other() == 0; });
    if (us > 0.f && (best < 0.f || us < best)) {
      best = us;
      config = LIBRARY;
      splits = 1;
    }
  }
  if (best < 0.f) return Q3_ERR_UNSUPPORTED;
  d.fused[key] = std::make_pair(config, splits);
  return 0;
}

}  // namespace

// Products of up to 256 rows that carry a norm, by the hand-written tiled kernel (the few-row kernel of
// gemm.hip does the same for up to 16 rows and is faster there; the callers' policy decides which rows come
// here). x (M, K) and w (N, K) bfloat16, K a multiple of 64, N of 4.
//
// q3_tiles_scaled: the rows of x hold stream * norm_weight and still lack the norm's division; `sums`
// (chunks, M) float32 holds the rows' sums of squares of the stream in partial sums, `width` the stream's
// width (= K). out = (x @ w^T) * rsqrt(sum / width + eps) row by row: epilogue 0 gives (M, N) in `out_dtype`,
// 1 (rows of w interleave gate and up) gives (M, N / 2) bfloat16 = silu(gate) * up.
extern "C" int q3_tiles_scaled(const void* x, const void* w, void* out, int M, int N, int K, int out_dtype,
                               int epilogue, const float* sums, int chunks, float eps, int width, void* stream_) {
  if (!x || !w || !out || !sums || M < 1 || M > 256 || N % 4 || !tiles::takes(M, N, K)) return Q3_ERR_BAD_ARGUMENT;
  if (chunks < 1 || width != K) return Q3_ERR_BAD_ARGUMENT;
  const bool swiglu = epilogue == tiles::EPI_SWIGLU;
  if (!swiglu && epilogue != tiles::EPI_PLAIN) return Q3_ERR_BAD_ARGUMENT;
  if (swiglu ? out_dtype != Q3_BF16 : (out_dtype != Q3_BF16 && out_dtype != Q3_F32)) return Q3_ERR_BAD_ARGUMENT;
  hipStream_t stream = (hipStream_t)stream_;
  std::lock_guard<std::mutex> hold(g_lock);
  int device = 0;
  HIP_TRY(hipGetDevice(&device));
  Device& d = g_devices[device];
  tiles::RowScale scale;
  scale.sums = sums;
  scale.chunks = chunks;
  scale.rows = M;
  scale.eps = eps;
  scale.inv_width = 1.f / (float)width;
  auto launch = [&](int config, int splits) {
    if (swiglu)
      return tiles::launch<bf16_t, tiles::EPI_SWIGLU>(config, x, w, out, M, N, K, stream, splits, d.partials, scale);
    if (out_dtype == Q3_F32)
      return tiles::launch<float, tiles::EPI_PLAIN>(config, x, w, out, M, N, K, stream, splits, d.partials, scale);
    return tiles::launch<bf16_t, tiles::EPI_PLAIN>(config, x, w, out, M, N, K, stream, splits, d.partials, scale);
  };
  // the other way: the contest's product in float32, then the kernel that otherwise adds partial products
  // divides (and activates) its rows
  auto other = [&]() {
    if ((size_t)M * N * sizeof(float) > STAGING_BYTES) return Q3_ERR_UNSUPPORTED;
    if (!d.staging) {
      hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
      HIP_TRY(hipStreamIsCapturing(stream, &capture));
      if (capture != hipStreamCaptureStatusNone) return (int)hipErrorStreamCaptureUnsupported;
      HIP_TRY(hipMalloc((void**)&d.staging, STAGING_BYTES));
    }
    const int status = product(d, x, w, d.staging, M, N, K, Q3_F32, stream);
    if (status) return status;
    const size_t quads = (size_t)M * N / 4;
    const dim3 grid((unsigned)((quads + 255) / 256));
    if (swiglu)
      hipLaunchKernelGGL((tiles::gemm_tiles_reduce_kernel<bf16_t, true>), grid, dim3(256), 0, stream, d.staging,
                         (bf16_t*)out, quads, N / 4, 1, scale);
    else if (out_dtype == Q3_F32)
      hipLaunchKernelGGL((tiles::gemm_tiles_reduce_kernel<float, false>), grid, dim3(256), 0, stream, d.staging,
                         (float*)out, quads, N / 4, 1, scale);
    else
      hipLaunchKernelGGL((tiles::gemm_tiles_reduce_kernel<bf16_t, false>), grid, dim3(256), 0, stream, d.staging,
                         (bf16_t*)out, quads, N / 4, 1, scale);
    return q3_launch_status();
  };
  int config = 0, splits = 1;
  const int status = choose_fused(d, swiglu ? 1 : 0, M, N, K, stream, launch, other, config, splits);
  if (status) return status;
  return config == LIBRARY ? other() : launch(config, splits);
}

// q3_tiles_residual: residual (M, N) float32 += bfloat16(x @ w^T) in place; values (M, N) bfloat16 =
// residual * norm_weight; sums (ceil(N / 1024), M) float32 = the rows' sums of squares of the new residual over
// chunks of 1,024 columns: what q3_tiles_scaled takes for the next product. Returns Q3_DECLINED, and has done
// nothing, where the contest's plain product followed by the norm's own kernel is the faster way for this size.
extern "C" int q3_tiles_residual_chunks(int N) { return (N + tiles::CHUNK_COLUMNS - 1) / tiles::CHUNK_COLUMNS; }

extern "C" int q3_tiles_residual(const void* x, const void* w, int M, int N, int K, float* residual,
                                 const void* norm_weight, int norm_weight_dtype, void* values, float* sums,
                                 void* stream_) {
  if (!x || !w || !residual || !norm_weight || !values || !sums) return Q3_ERR_BAD_ARGUMENT;
  if (M < 1 || M > 256 || N % 4 || !tiles::takes(M, N, K)) return Q3_ERR_BAD_ARGUMENT;
  if (norm_weight_dtype != Q3_BF16 && norm_weight_dtype != Q3_F32) return Q3_ERR_BAD_ARGUMENT;
  hipStream_t stream = (hipStream_t)stream_;
  std::lock_guard<std::mutex> hold(g_lock);
  int device = 0;
  HIP_TRY(hipGetDevice(&device));
  Device& d = g_devices[device];
  int config = 0, splits = 1;
  // timed by the products alone (the tiled kernel's partial products; the contest's product into `values`,
  // which the real run overwrites): each way has one small kernel more, and the residual is not touched
  int status = choose_fused(
      d, 2, M, N, K, stream,
      [&](int c, int s) {
        if ((size_t)s * M * N * sizeof(float) > PARTIALS_BYTES) return Q3_ERR_UNSUPPORTED;
        return tiles::launch<bf16_t, tiles::EPI_PLAIN>(c, x, w, values, M, N, K, stream, s, d.partials,
                                                       tiles::RowScale(), true);
      },
      [&]() { return product(d, x, w, values, M, N, K, Q3_BF16, stream); }, config, splits);
  if (status) return status;
  if (config == LIBRARY) return Q3_DECLINED;
  if ((size_t)splits * M * N * sizeof(float) > PARTIALS_BYTES) return Q3_ERR_UNSUPPORTED;   // also a single share
  int used = 1;
  status = tiles::launch<bf16_t, tiles::EPI_PLAIN>(config, x, w, values, M, N, K, stream, splits, d.partials,
                                                   tiles::RowScale(), true, &used);
  if (status) return status;
  const dim3 grid(q3_tiles_residual_chunks(N), M);
  if (norm_weight_dtype == Q3_F32)
    hipLaunchKernelGGL(tiles::tiles_residual_kernel<float>, grid, dim3(256), 0, stream, d.partials, used, residual,
                       (const float*)norm_weight, (bf16_t*)values, sums, M, N);
  else
    hipLaunchKernelGGL(tiles::tiles_residual_kernel<bf16_t>, grid, dim3(256), 0, stream, d.partials, used, residual,
                       (const bf16_t*)norm_weight, (bf16_t*)values, sums, M, N);
  return q3_launch_status();
}

// The hand-written tiled kernel alone (gemm_tiles.h), tile shape `config` (0 .. q3_gemm_tiles_configs() - 1):
// x (M, K) and w (N, K) bfloat16, K a multiple of 64; `epilogue` 0: out (M, N) in `out_dtype`; 1: rows of w
// interleave gate and up, out (M, N / 2) bfloat16 = silu(gate) * up.
extern "C" int q3_gemm_tiles_configs() { return tiles::NUM_CONFIGS; }

// `splits` > 1 (plain epilogue, N a multiple of 4): K is shared out over that many blocks per tile and
// `partials` (splits * M * N floats) takes their partial products; q3_gemm_tiles_splits says how many fill the
// chip once.
extern "C" int q3_gemm_tiles_splits(int config, int M, int N, int K) {
  return tiles::takes(M, N, K) && config >= 0 && config < tiles::NUM_CONFIGS ? tiles::splits_that_fill(config, M, N, K)
                                                                            : 1;
}

extern "C" int q3_gemm_tiles(const void* x, const void* w, void* out, int M, int N, int K, int out_dtype,
                             int epilogue, int config, int splits, float* partials, void* stream_) {
  if (!x || !w || !out || !tiles::takes(M, N, K)) return Q3_ERR_BAD_ARGUMENT;
  hipStream_t stream = (hipStream_t)stream_;
  std::lock_guard<std::mutex> hold(g_lock);   // the launchers keep a per-device flag
  if (epilogue == tiles::EPI_SWIGLU) {
    if (out_dtype != Q3_BF16 || N % 2) return Q3_ERR_BAD_ARGUMENT;
    return tiles::launch<bf16_t, tiles::EPI_SWIGLU>(config, x, w, out, M, N, K, stream, splits, partials);
  }
  if (epilogue != tiles::EPI_PLAIN) return Q3_ERR_BAD_ARGUMENT;
  if (out_dtype == Q3_F32)
    return tiles::launch<float, tiles::EPI_PLAIN>(config, x, w, out, M, N, K, stream, splits, partials);
  if (out_dtype == Q3_BF16)
    return tiles::launch<bf16_t, tiles::EPI_PLAIN>(config, x, w, out, M, N, K, stream, splits, partials);
  return Q3_ERR_BAD_ARGUMENT;
}

// How many of the library's candidates are timed for a new problem size (1: take its first choice).
extern "C" int q3_matmul_set_candidates(int n) {
  if (n < 1 || n > MAX_CANDIDATES) return Q3_ERR_BAD_ARGUMENT;
  std::lock_guard<std::mutex> hold(g_lock);
  g_candidates = n;
  return 0;
}

// Which kernels enter the contest for a new size: 0 the library's and the hand-written one's (the default),
// 1 the library's alone, 2 the hand-written ones alone where they take the size. Sizes already met keep their
// choice. The products that carry a norm (q3_tiles_*) keep a choice for each of the three.
extern "C" int q3_matmul_set_kernels(int mode) {
  if (mode < KERNELS_BOTH || mode > KERNELS_OWN) return Q3_ERR_BAD_ARGUMENT;
  std::lock_guard<std::mutex> hold(g_lock);
  g_kernels = mode;
  return 0;
}

// What was chosen for a size on the current device: info[0] candidates timed, info[1] index chosen,
// info[2] microseconds of the first candidate, info[3] of the chosen one, info[4] the hand-written kernel's
// tile shape if that was chosen, else -1, info[5] over how many blocks it shares K out. Returns 1 if the size
// is known.
extern "C" int q3_matmul_plan(int M, int N, int K, int out_dtype, float* info) {
  std::lock_guard<std::mutex> hold(g_lock);
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return 0;
  auto d = g_devices.find(device);
  if (d == g_devices.end()) return 0;
  auto p = d->second.plans.find(std::make_tuple(M, N, K, out_dtype));
  if (p == d->second.plans.end()) return 0;
  info[0] = (float)p->second.candidates;
  info[1] = (float)p->second.chosen;
  info[2] = p->second.first_us;
  info[3] = p->second.best_us;
  info[4] = (float)p->second.own;
  info[5] = (float)p->second.own_splits;
  return 1;
}

extern "C" int q3_matmul(const void* x, const void* w, void* out, int M, int N, int K, int out_dtype, void* stream_) {
  if (M <= 0 || N <= 0 || K <= 0 || !x || !w || !out) return Q3_ERR_BAD_ARGUMENT;
  if (out_dtype != Q3_F32 && out_dtype != Q3_BF16) return Q3_ERR_BAD_ARGUMENT;
  std::lock_guard<std::mutex> hold(g_lock);
  int device = 0;
  HIP_TRY(hipGetDevice(&device));
  return product(g_devices[device], x, w, out, M, N, K, out_dtype, (hipStream_t)stream_);
}
