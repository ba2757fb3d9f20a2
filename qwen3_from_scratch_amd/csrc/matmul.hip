// Matrix products with many rows, out[M, N] = x[M, K] . w[N, K]^T in bfloat16
// with float32 accumulation, by the vendor library (hipBLASLt), as the
// reference's engine uses its vendor library for them
// (src/qwen3_from_scratch/models/linear.py:24-31 calls F.linear), or by the
// hand-written tiled kernel (gemm_tiles.h).
//
// Which kernel serves a size is decided without a stopwatch: the same size gets
// the same kernel in every process and on every box, so a product's bits are
// reproducible. The decision is, in this order,
//   1. an entry of the table that the caller loaded (q3_matmul_table_add): a
//      place in the library's ranked list of candidates for the size, or a tile
//      shape of the hand-written kernel with a number of shares of K; the table is
//      data made beforehand by the tuner below, keyed by (kind of product, rows
//      rounded up, N, K, output type);
//   2. a rule of thumb: the library's first candidate for a plain product; for
//      the products of 17 to 128 rows that carry a norm the 64 x 128 tiles with
//      K shared out until the chip is full, unless those tiles fit the chip badly.
// The library's list is asked for the exact size every time, so a kernel is
// never run on a size the library has not offered it for.
//
// The tuner (q3_matmul_set_mode(1), off unless asked for) is what the table is
// made with: a size first met outside a graph capture has its candidates timed
// on the caller's own operands, the library's leading ones and the tile shapes
// that fit the rows, each also with K shared out where its tiles alone would not
// fill the chip, and the fastest is kept for the life of the process
// (q3_matmul_plan and q3_matmul_fused_plan tell what it was). In the model every
// weight is read once a step, with gigabytes of other traffic in between, so a
// candidate is timed with cold caches: a kernel that reads a buffer larger than
// the last-level cache runs before each timed run.
//
// One workspace, one buffer for the tiled kernel's partial products and one
// staging buffer per device, allocated by q3_matmul_init (the engine calls it
// when a model is built) or at the first product outside a capture. Calls on one
// device share them and the plans: they are serialised by a lock and are meant to
// come from one stream at a time.

#include "common.h"
#include "gemm_tiles.h"
#include "gemm_stream.h"

#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#define Q3_ERR_LIBRARY 20000   // + the library's status
#define Q3_DECLINED 1          // q3_tiles_residual: nothing was done, the caller's other way is the one for this size

namespace {

constexpr size_t WORKSPACE_BYTES = 128u << 20;
constexpr size_t EVICT_BYTES = 512u << 20;     // twice the 256 MB last-level cache (the tuner's)
constexpr size_t PARTIALS_BYTES = 128u << 20;  // float32 partial products of the hand-written kernel's K shares
constexpr size_t STAGING_BYTES = 64u << 20;
constexpr int EVICT_BLOCKS = 2048, EVICT_THREADS = 256;
constexpr int MAX_CANDIDATES = 64;
constexpr int LIBRARY = -1;                    // a Choice's `own` when the library serves the size

// Reads the whole buffer; the store never happens (the buffer holds zeros) but keeps the loads alive.
__global__ void evict_kernel(float4* buffer, size_t count) {
  float sum = 0.f;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x) {
    const float4 v = buffer[i];
    sum += v.x + v.y + v.z + v.w;
  }
  if (sum == 12345.f) buffer[0].x = sum;
}

// The kinds of product a choice is made for.
enum { KIND_PLAIN = 0, KIND_SCALED = 1, KIND_SCALED_SWIGLU = 2, KIND_RESIDUAL = 3 };

// Who serves a size: the library's candidate number `library` (own == LIBRARY), or the hand-written kernel's
// tile shape `own` with K shared out over `splits` blocks per tile.
struct Choice {
  int library = 0;
  int own = LIBRARY;
  int splits = 1;
};

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t w = nullptr, x = nullptr, out = nullptr;
  hipblasLtMatmulAlgo_t algo;
  bool ready = false;      // the choice is made (and, for the library, its kernel found)
  bool timed = false;      // by the tuner
  Choice choice;
  int candidates = 0, chosen = 0;
  float first_us = 0.f, best_us = 0.f;
};

typedef std::tuple<int, int, int, int, int> Key;   // kind (+ 4 * which kernels, for the tuner's notes), rows, N, K, output type

struct Device {
  hipblasLtHandle_t handle = nullptr;
  void* workspace = nullptr;
  void* evict = nullptr;
  float* partials = nullptr;
  float* staging = nullptr;   // a float32 product on its way to the kernel that divides its rows (q3_tiles_scaled)
  hipEvent_t begin = nullptr, end = nullptr;
  std::map<std::tuple<int, int, int, int>, Plan> plans;   // by the exact size
  std::map<Key, Choice> noted;                            // what the tuner found, by rounded rows
};

std::mutex g_lock;
std::map<int, Device> g_devices;
std::map<Key, Choice> g_table;
int g_candidates = 16;
enum { KERNELS_BOTH = 0, KERNELS_LIBRARY = 1, KERNELS_OWN = 2 };
int g_kernels = KERNELS_BOTH;
enum { MODE_RULE = 0, MODE_TUNE = 1 };
int g_mode = MODE_RULE;

// Sizes that differ only within a step of rows share a table entry (a serving loop meets dozens of them, a
// prompt's portion plus however many requests decode): up to 64 rows, and the products that carry a norm at
// any count, in steps of 8; plain products beyond 64 rows in steps of 32.
int rows_key(int kind, int M) {
  if (kind != KIND_PLAIN || M <= 64) return (M + 7) / 8 * 8;
  return (M + 31) / 32 * 32;
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

bool capturing(hipStream_t stream, int& status) {
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  status = (int)hipStreamIsCapturing(stream, &capture);
  return capture != hipStreamCaptureStatusNone;
}

// The device's handle and buffers. Not inside a capture: it allocates.
int set_up(Device& d) {
  if (!d.workspace) HIP_TRY(hipMalloc(&d.workspace, WORKSPACE_BYTES));
  if (!d.partials) HIP_TRY(hipMalloc((void**)&d.partials, PARTIALS_BYTES));
  if (!d.staging) HIP_TRY(hipMalloc((void**)&d.staging, STAGING_BYTES));
  if (!d.handle) LT_TRY(hipblasLtCreate(&d.handle));
  return 0;
}

int ready_device(Device& d, hipStream_t stream) {
  if (d.handle && d.workspace && d.partials && d.staging) return 0;
  int status = 0;
  if (capturing(stream, status)) return (int)hipErrorStreamCaptureUnsupported;   // set-up allocates
  if (status) return status;
  return set_up(d);
}

// The tuner's own: events and the buffer that empties the caches.
int set_up_tuner(Device& d, hipStream_t stream) {
  if (!d.begin) HIP_TRY(hipEventCreate(&d.begin));
  if (!d.end) HIP_TRY(hipEventCreate(&d.end));
  if (!d.evict) {
    HIP_TRY(hipMalloc(&d.evict, EVICT_BYTES));
    HIP_TRY(hipMemsetAsync(d.evict, 0, EVICT_BYTES, stream));
  }
  return 0;
}

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

// The library's ranked candidates for the plan's exact size, at most `want` of them.
int candidates_of(Device& d, const Plan& p, int want, std::vector<hipblasLtMatmulHeuristicResult_t>& found) {
  hipblasLtMatmulPreference_t pref = nullptr;
  LT_TRY(hipblasLtMatmulPreferenceCreate(&pref));
  size_t bytes = WORKSPACE_BYTES;
  hipblasStatus_t s = hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &bytes,
                                                            sizeof(bytes));
  found.assign(want, hipblasLtMatmulHeuristicResult_t());
  int got = 0;
  if (s == HIPBLAS_STATUS_SUCCESS)
    s = hipblasLtMatmulAlgoGetHeuristic(d.handle, p.desc, p.w, p.x, p.out, p.out, pref, want, found.data(), &got);
  (void)hipblasLtMatmulPreferenceDestroy(pref);
  if (s != HIPBLAS_STATUS_SUCCESS) return Q3_ERR_LIBRARY + (int)s;
  found.resize(got);
  return got == 0 ? Q3_ERR_UNSUPPORTED : 0;
}

int run_own(Device& d, int config, int splits, const void* x, const void* w, void* out, int M, int N, int K,
            int out_dtype, hipStream_t stream) {
  if (splits > 1 && (size_t)splits * M * N * sizeof(float) > PARTIALS_BYTES) return Q3_ERR_UNSUPPORTED;
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

// ---- the rules of thumb ----------------------------------------------------------------------

// The hand-written kernel's shape for a plain product, by its rows: small tiles with three stages where the
// weights' passage bounds the product, the largest where the matrix units do; K shared out where the tiles
// alone would not fill the chip.
Choice own_by_rule(int M, int N, int K) {
  Choice c;
  c.own = M <= 256 ? 5 : (M <= 1024 ? 1 : 4);
  c.splits = M <= 1024 ? tiles::splits_that_fill(c.own, M, N, K) : 1;
  if ((size_t)c.splits * M * N * sizeof(float) > PARTIALS_BYTES) c.splits = 1;
  return c;
}

Choice plain_by_rule(int M, int N, int K) {
  if (g_kernels == KERNELS_OWN && tiles::takes(M, N, K)) return own_by_rule(M, N, K);
  if (g_kernels == KERNELS_BOTH && tiles::takes(M, N, K) && M >= 32 && M <= 640 && K >= 2 * N && N % 4 == 0) {
    // few output tiles and a long inner size (a feed-forward's way down with some hundreds of rows): the
    // library's kernels leave most of the chip idle there, the tiled kernel shares K out over the idle CUs
    // (4,096 x 12,288 at 64, 256 and 576 rows: 29, 47 and 81 us against the library's best 38, 58 and 99)
    Choice c;
    c.own = M <= 256 ? 1 : 0;
    c.splits = tiles::splits_that_fill(c.own, M, N, K);
    if (c.splits > 1 && (size_t)c.splits * M * N * sizeof(float) <= PARTIALS_BYTES) return c;
  }
  return Choice();   // the library's first candidate
}

// The products of 17 to 128 rows that carry a norm: 64 x 128 tiles in five stages (with K shared out they need
// the fewest shares to fill the chip), unless the tiles come to a little more than a whole number of rounds over
// the 256 CUs and leave most of them idle in the last one: then the library's product with the norm's work in a
// kernel behind it (for KIND_RESIDUAL: declined, the caller's plain product and the norm's own kernel).
Choice fused_by_rule(int kind, int M, int N, int K) {
  (void)kind;
  Choice c;
  if (g_kernels == KERNELS_LIBRARY) return c;
  c.own = 8;
  c.splits = tiles::splits_that_fill(8, M, N, K);
  if ((size_t)c.splits * ((M + 7) / 8 * 8) * N * sizeof(float) > PARTIALS_BYTES) c.splits = 1;
  if (g_kernels == KERNELS_BOTH && c.splits == 1) {
    const long tiles_n = (long)((M + 63) / 64) * ((N + 127) / 128);
    const long rounds = (tiles_n + 255) / 256;
    if (tiles_n < rounds * 256 * 7 / 10) return Choice();
  }
  return c;
}

// What the table or the rule says for a size.
Choice choice_for(int kind, int M, int N, int K, int out_dtype) {
  if (g_kernels == KERNELS_BOTH) {
    auto entry = g_table.find(Key(kind, rows_key(kind, M), N, K, out_dtype));
    if (entry != g_table.end()) {
      Choice c = entry->second;
      const bool fits = c.own == LIBRARY ||
                        (tiles::takes(M, N, K) && c.own < tiles::NUM_CONFIGS && c.splits >= 1 && c.splits <= K / tiles::BK &&
                         c.splits <= 64 && (c.splits == 1 || N % 4 == 0) &&
                         (size_t)c.splits * ((M + 7) / 8 * 8) * N * sizeof(float) <= PARTIALS_BYTES);
      if (fits) return c;
    }
  }
  return kind == KIND_PLAIN ? plain_by_rule(M, N, K) : fused_by_rule(kind, M, N, K);
}

// ---- the tuner ---------------------------------------------------------------------------------

// The tile shapes that enter the contest, by the product's rows (the others never won a size of the 8B, 14B
// and 32B models there). Each enters a second time with K shared out where its tiles alone would not fill the
// chip.
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

// Times the candidates for the plan's size on the caller's operands and leaves the fastest in the plan.
int tune_plain(Device& d, Plan& p, const void* x, const void* w, void* out, int M, int N, int K, int out_dtype,
               hipStream_t stream) {
  const int set = set_up_tuner(d, stream);
  if (set) return set;
  const bool own_takes = tiles::takes(M, N, K) && g_kernels != KERNELS_LIBRARY;
  std::vector<hipblasLtMatmulHeuristicResult_t> found;
  int got = 0;
  if (!(own_takes && g_kernels == KERNELS_OWN)) {
    const int status = candidates_of(d, p, g_candidates, found);
    if (status && !(status == Q3_ERR_UNSUPPORTED && own_takes)) return status;
    got = (int)found.size();
  }
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
      own_config[owns] = shapes[i];
      own_splits[owns++] = splits;
    }
  }
  const int all = got + owns;
  if (all == 0) return Q3_ERR_UNSUPPORTED;
  auto time_one = [&](int i, int reps) {
    if (i < got)
      return time_runs(d, stream, reps, [&] { return run(d, p, found[i].algo, x, w, out, stream) == HIPBLAS_STATUS_SUCCESS; });
    return time_runs(d, stream, reps, [&] {
      return run_own(d, own_config[i - got], own_splits[i - got], x, w, out, M, N, K, out_dtype, stream) == 0;
    });
  };
  // two passes: all candidates briefly (the first run of each also loads its code), then those
  // near the front again and longer
  std::vector<float> us(all, -1.f);
  float best = -1.f;
  for (int i = 0; i < all; ++i) {
    if (time_one(i, 1) < 0.f) continue;
    us[i] = time_one(i, 2);
    if (us[i] > 0.f && (best < 0.f || us[i] < best)) best = us[i];
  }
  if (best < 0.f) return Q3_ERR_UNSUPPORTED;
  for (int i = 0; i < all; ++i) {
    if (us[i] < 0.f || us[i] > 1.2f * best) continue;
    const float again = time_one(i, 5);
    if (again > 0.f && again < us[i]) us[i] = again;
  }
  int chosen = -1;
  for (int i = 0; i < all; ++i)
    if (us[i] > 0.f && (chosen < 0 || us[i] < us[chosen])) chosen = i;
  p.candidates = all;
  p.chosen = chosen;
  p.choice = Choice();
  if (chosen < got) {
    p.choice.library = chosen;
    p.algo = found[chosen].algo;
  } else {
    p.choice.own = own_config[chosen - got];
    p.choice.splits = own_splits[chosen - got];
  }
  p.first_us = us[0] > 0.f ? us[0] : us[chosen];
  p.best_us = us[chosen];
  p.ready = true;
  p.timed = true;
  return 0;
}

// The product by the plan's kernel.
int run_plan(Device& d, const Plan& p, const void* x, const void* w, void* out, int M, int N, int K, int out_dtype,
             hipStream_t stream) {
  if (p.choice.own >= 0) return run_own(d, p.choice.own, p.choice.splits, x, w, out, M, N, K, out_dtype, stream);
  const hipblasStatus_t s = run(d, p, p.algo, x, w, out, stream);
  return s == HIPBLAS_STATUS_SUCCESS ? 0 : Q3_ERR_LIBRARY + (int)s;
}

// Makes the plan ready by `c`: for the library, its candidate number c.library for this exact size (its first
// one, the rule of thumb, if it offers fewer: an entry is made at one row count and shared by its neighbours,
// whose ranked lists may be shorter, and the last of a short list is the library's worst offer; the
// hand-written kernel if the library offers none and that takes the size). q3_matmul_plan tells which it was.
int settle(Device& d, Plan& p, Choice c, int M, int N, int K) {
  p.choice = c;
  p.candidates = 1;
  p.chosen = 0;
  if (c.own < 0) {
    std::vector<hipblasLtMatmulHeuristicResult_t> found;
    const int status = candidates_of(d, p, c.library + 1, found);
    if (status == Q3_ERR_UNSUPPORTED && tiles::takes(M, N, K)) {
      p.choice = own_by_rule(M, N, K);
    } else if (status) {
      return status;
    } else {
      p.choice.library = c.library < (int)found.size() ? c.library : 0;
      p.algo = found[p.choice.library].algo;
    }
  }
  p.ready = true;
  return 0;
}

// out = x @ w^T by the kernel chosen for the size (the lock is held).
int product(Device& d, const void* x, const void* w, void* out, int M, int N, int K, int out_dtype, hipStream_t stream) {
  int status = ready_device(d, stream);
  if (status) return status;
  Plan& p = d.plans[std::make_tuple(M, N, K, out_dtype)];
  if (!p.desc) {
    status = describe(p, M, N, K, out_dtype);
    if (status) {
      forget(p);
      return status;
    }
  }
  if (g_mode == MODE_TUNE && !p.timed) {
    const bool in_capture = capturing(stream, status);
    if (status) return status;
    if (!in_capture) {
      const Key near(KIND_PLAIN + 4 * g_kernels, rows_key(KIND_PLAIN, M), N, K, out_dtype);
      auto noted = d.noted.find(near);
      if (noted != d.noted.end()) {   // a neighbour's choice, asked of the library anew for this size
        status = settle(d, p, noted->second, M, N, K);
        if (status == 0) p.timed = true;
      } else {
        status = tune_plain(d, p, x, w, out, M, N, K, out_dtype, stream);
        if (status == 0) d.noted[near] = p.choice;
      }
      if (status) {
        forget(p);
        return status;
      }
    }
  }
  if (!p.ready) {
    status = settle(d, p, choice_for(KIND_PLAIN, M, N, K, out_dtype), M, N, K);
    if (status) {
      forget(p);
      return status;
    }
  }
  return run_plan(d, p, x, w, out, M, N, K, out_dtype, stream);
}

// Tile shape and shares of K for a product of some tens of rows that carries a norm, or LIBRARY: `other()`
// then does the same work around the library's product. `launch(config, splits)` runs the tiled kernel
// without side effects and returns its status. By the table or the rule; with the tuner on, timed once per
// size with cold caches outside a graph capture.
template <typename Launch, typename Other>
int choose_fused(Device& d, int kind, int M, int N, int K, hipStream_t stream, Launch launch, Other other, Choice& c) {
  if (g_mode != MODE_TUNE) {
    c = choice_for(kind, M, N, K, Q3_BF16);
    return 0;
  }
  const Key key(kind + 4 * g_kernels, rows_key(kind, M), N, K, Q3_BF16);
  auto known = d.noted.find(key);
  if (known != d.noted.end()) {
    c = known->second;
    return 0;
  }
  int status = 0;
  if (capturing(stream, status) || status) {
    c = fused_by_rule(kind, M, N, K);
    return status;
  }
  status = set_up_tuner(d, stream);
  if (status) return status;
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
  float best = -1.f;
  c = Choice();
  // the first call of the other way holds that product's own contest: not inside a timed run, whose events it uses
  const bool other_works = g_kernels != KERNELS_OWN && other() == 0;
  for (int i = 0; i < n && !(other_works && g_kernels == KERNELS_LIBRARY); ++i) {
    auto one = [&] { return launch(configs[i], shares[i]) == 0; };
    if (time_runs(d, stream, 1, one) < 0.f) continue;   // the first run also loads the code
    const float us = time_runs(d, stream, 4, one);
    if (us > 0.f && (best < 0.f || us < best)) {
      best = us;
      c.own = configs[i];
      c.splits = shares[i];
    }
  }
  if (other_works) {
    const float us = time_runs(d, stream, 4, [&] { return other() == 0; });
    if (us > 0.f && (best < 0.f || us < best)) {
      best = us;
      c = Choice();
    }
  }
  if (best < 0.f) return Q3_ERR_UNSUPPORTED;
  d.noted[key] = c;
  return 0;
}

}  // namespace

// The device's buffers and the library's handle, once per device; the engine calls this when a bfloat16 model is
// built, so that no product in a step allocates.
extern "C" int q3_matmul_init() {
  std::lock_guard<std::mutex> hold(g_lock);
  int device = 0;
  HIP_TRY(hipGetDevice(&device));
  return set_up(g_devices[device]);
}

// Products of up to 256 rows that carry a norm, by the hand-written tiled kernel (the few-row kernel of
// gemm.hip does the same for up to 16 rows, or 64 of a small weight, and is faster there; the callers' policy decides which rows come
// here). x (M, K) and w (N, K) bfloat16, K a multiple of 64, N of 4.
//
// q3_tiles_scaled: the rows of x hold stream * norm_weight and still lack the norm's division; `sums`
// (chunks, sums_stride) float32 holds the rows' sums of squares of the stream in partial sums (row m in
// column m, sums_stride >= M), `width` the stream's width (= K). out = (x @ w^T) * rsqrt(sum / width + eps)
// row by row: epilogue 0 gives (M, N) in `out_dtype`, 1 (rows of w interleave gate and up) gives (M, N / 2)
// bfloat16 = silu(gate) * up.
extern "C" int q3_tiles_scaled(const void* x, const void* w, void* out, int M, int N, int K, int out_dtype,
                               int epilogue, const float* sums, int chunks, int sums_stride, float eps, int width,
                               void* stream_) {
  if (!x || !w || !out || !sums || M < 1 || M > 256 || N % 4 || !tiles::takes(M, N, K)) return Q3_ERR_BAD_ARGUMENT;
  if (chunks < 1 || sums_stride < M || width != K) return Q3_ERR_BAD_ARGUMENT;
  const bool swiglu = epilogue == tiles::EPI_SWIGLU;
  if (!swiglu && epilogue != tiles::EPI_PLAIN) return Q3_ERR_BAD_ARGUMENT;
  if (swiglu ? out_dtype != Q3_BF16 : (out_dtype != Q3_BF16 && out_dtype != Q3_F32)) return Q3_ERR_BAD_ARGUMENT;
  hipStream_t stream = (hipStream_t)stream_;
  std::lock_guard<std::mutex> hold(g_lock);
  int device = 0;
  HIP_TRY(hipGetDevice(&device));
  Device& d = g_devices[device];
  int status = ready_device(d, stream);
  if (status) return status;
  tiles::RowScale scale;
  scale.sums = sums;
  scale.chunks = chunks;
  scale.rows = sums_stride;
  scale.eps = eps;
  scale.inv_width = 1.f / (float)width;
  auto launch = [&](int config, int splits) {
    if (swiglu)
      return tiles::launch<bf16_t, tiles::EPI_SWIGLU>(config, x, w, out, M, N, K, stream, splits, d.partials, scale);
    if (out_dtype == Q3_F32)
      return tiles::launch<float, tiles::EPI_PLAIN>(config, x, w, out, M, N, K, stream, splits, d.partials, scale);
    return tiles::launch<bf16_t, tiles::EPI_PLAIN>(config, x, w, out, M, N, K, stream, splits, d.partials, scale);
  };
  // the other way: the library's product in float32, then the kernel that otherwise adds partial products
  // divides (and activates) its rows
  auto other = [&]() {
    if ((size_t)M * N * sizeof(float) > STAGING_BYTES) return Q3_ERR_UNSUPPORTED;
    const int product_status = product(d, x, w, d.staging, M, N, K, Q3_F32, stream);
    if (product_status) return product_status;
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
  Choice c;
  status = choose_fused(d, swiglu ? KIND_SCALED_SWIGLU : KIND_SCALED, M, N, K, stream, launch, other, c);
  if (status) return status;
  if (c.own == LIBRARY) {
    status = other();
    if (status != Q3_ERR_UNSUPPORTED) return status;
    c = fused_by_rule(KIND_SCALED, M, N, K);      // the library has nothing for the size: the tiled kernel
    if (c.own == LIBRARY) {
      c.own = 8;
      c.splits = 1;
    }
  }
  return launch(c.own, c.splits);
}

// q3_tiles_residual: residual (M, N) float32 += bfloat16(x @ w^T) in place; values (M, N) bfloat16 =
// residual * norm_weight; sums (ceil(N / 1024), sums_stride) float32 = the rows' sums of squares of the new
// residual over chunks of 1,024 columns (row m in column m): what q3_tiles_scaled takes for the next product. Returns Q3_DECLINED, and has done
// nothing, where the plain product followed by the norm's own kernel is the way for this size.
extern "C" int q3_tiles_residual_chunks(int N) { return (N + tiles::CHUNK_COLUMNS - 1) / tiles::CHUNK_COLUMNS; }

extern "C" int q3_tiles_residual(const void* x, const void* w, int M, int N, int K, float* residual,
                                 const void* norm_weight, int norm_weight_dtype, void* values, float* sums,
                                 int sums_stride, void* stream_) {
  if (!x || !w || !residual || !norm_weight || !values || !sums || sums_stride < M) return Q3_ERR_BAD_ARGUMENT;
  if (M < 1 || M > 256 || N % 4 || !tiles::takes(M, N, K)) return Q3_ERR_BAD_ARGUMENT;
  if (norm_weight_dtype != Q3_BF16 && norm_weight_dtype != Q3_F32) return Q3_ERR_BAD_ARGUMENT;
  hipStream_t stream = (hipStream_t)stream_;
  std::lock_guard<std::mutex> hold(g_lock);
  int device = 0;
  HIP_TRY(hipGetDevice(&device));
  Device& d = g_devices[device];
  int status = ready_device(d, stream);
  if (status) return status;
  Choice c;
  // the tuner times the products alone (the tiled kernel's partial products; the other product into `values`,
  // which the real run overwrites): each way has one small kernel more, and the residual is not touched
  status = choose_fused(
      d, KIND_RESIDUAL, M, N, K, stream,
      [&](int config, int splits) {
        if ((size_t)splits * M * N * sizeof(float) > PARTIALS_BYTES) return Q3_ERR_UNSUPPORTED;
        return tiles::launch<bf16_t, tiles::EPI_PLAIN>(config, x, w, values, M, N, K, stream, splits, d.partials,
                                                       tiles::RowScale(), true);
      },
      [&]() { return product(d, x, w, values, M, N, K, Q3_BF16, stream); }, c);
  if (status) return status;
  if (c.own == LIBRARY) return Q3_DECLINED;
  if ((size_t)c.splits * M * N * sizeof(float) > PARTIALS_BYTES) return Q3_ERR_UNSUPPORTED;   // also a single share
  int used = 1;
  status = tiles::launch<bf16_t, tiles::EPI_PLAIN>(c.own, x, w, values, M, N, K, stream, c.splits, d.partials,
                                                   tiles::RowScale(), true, &used);
  if (status) return status;
  const dim3 grid(q3_tiles_residual_chunks(N), M);
  if (norm_weight_dtype == Q3_F32)
    hipLaunchKernelGGL(tiles::tiles_residual_kernel<float>, grid, dim3(256), 0, stream, d.partials, used, residual,
                       (const float*)norm_weight, (bf16_t*)values, sums, sums_stride, M, N);
  else
    hipLaunchKernelGGL(tiles::tiles_residual_kernel<bf16_t>, grid, dim3(256), 0, stream, d.partials, used, residual,
                       (const bf16_t*)norm_weight, (bf16_t*)values, sums, sums_stride, M, N);
  return q3_launch_status();
}

// A product of 17 to 96 rows (and a gate/up product of 9 to 16) by the weight-streaming kernel of gemm_stream.h, from the tile-ordered copy `wt` of
// the weight (N, K): out (M, N) in `out_dtype` (`epilogue` 0) or, the weight's rows interleaving gate and up,
// out (M, N / 2) bfloat16 = silu(gate) * up (`epilogue` 1). With `sums` the rows of x still lack their norm's
// division, as for q3_tiles_scaled. Returns Q3_DECLINED, and has done nothing, where another kernel is the way:
// the caller has asked for the library's or the tiled kernel's products alone, the tuner is on (it times those),
// the size is not the kernel's, the weight is so small that other kernels serve these rows better, or its slabs
// do not fill the chip in one round of blocks.
constexpr size_t STREAM_LEAST_WEIGHT_BYTES = 24u << 20;

// The CUs of the current device (256 where it cannot be asked).
static int cu_count() {
  static int cached[16] = {};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 16) return 256;
  if (!cached[device]) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || n < 1) n = 256;
    cached[device] = n;
  }
  return cached[device];
}

// Whether the streaming kernel is the way for this product under the current settings, and with how many slabs
// per block (the lock is held): a weight of 24 MB or more whose blocks fill the chip in one round. Up to 16
// rows only a gate/up product is taken: everything else there is the few-row kernel's.
static int stream_plan_locked(int M, int N, int K, bool swiglu) {
  if (g_kernels != KERNELS_BOTH || g_mode != MODE_RULE) return 0;
  if (!stream::takes(M, N, K) || (size_t)N * K * 2 < STREAM_LEAST_WEIGHT_BYTES) return 0;
  if (M <= 16 && !swiglu) return 0;
  return stream::slabs_per_block(M, N, cu_count());
}

extern "C" int q3_stream_product(const void* x, const void* wt, void* out, int M, int N, int K, int out_dtype,
                                 int epilogue, const float* sums, int chunks, int sums_stride, float eps, int width,
                                 void* stream_) {
  if (!x || !wt || !out || M < 1 || N < 1 || K < 1) return Q3_ERR_BAD_ARGUMENT;
  const bool swiglu = epilogue == tiles::EPI_SWIGLU;
  if (!swiglu && epilogue != tiles::EPI_PLAIN) return Q3_ERR_BAD_ARGUMENT;
  if (swiglu ? out_dtype != Q3_BF16 : (out_dtype != Q3_BF16 && out_dtype != Q3_F32)) return Q3_ERR_BAD_ARGUMENT;
  if (sums && (chunks < 1 || sums_stride < M || width != K)) return Q3_ERR_BAD_ARGUMENT;
  hipStream_t stream = (hipStream_t)stream_;
  std::lock_guard<std::mutex> hold(g_lock);
  const int ws = stream_plan_locked(M, N, K, swiglu);
  if (!ws) return Q3_DECLINED;
  tiles::RowScale scale;
  if (sums) {
    scale.sums = sums;
    scale.chunks = chunks;
    scale.rows = sums_stride;
    scale.eps = eps;
    scale.inv_width = 1.f / (float)width;
  }
  if (swiglu) return stream::launch<bf16_t, tiles::EPI_SWIGLU>(ws, x, wt, out, M, N, K, stream, scale);
  if (out_dtype == Q3_F32) return stream::launch<float, tiles::EPI_PLAIN>(ws, x, wt, out, M, N, K, stream, scale);
  return stream::launch<bf16_t, tiles::EPI_PLAIN>(ws, x, wt, out, M, N, K, stream, scale);
}

// How q3_stream_product would lay a product over the chip: the slabs per block, or 0 for a size it declines
// under the current settings.
extern "C" int q3_stream_plan(int M, int N, int K, int swiglu) {
  std::lock_guard<std::mutex> hold(g_lock);
  return stream_plan_locked(M, N, K, swiglu != 0);
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

// 0: sizes get their kernels by the table and the rules (the default); 1: the tuner times the candidates of
// every size it first meets outside a capture. Sizes already settled keep their kernel.
extern "C" int q3_matmul_set_mode(int mode) {
  if (mode != MODE_RULE && mode != MODE_TUNE) return Q3_ERR_BAD_ARGUMENT;
  std::lock_guard<std::mutex> hold(g_lock);
  g_mode = mode;
  return 0;
}

// How many of the library's candidates the tuner times for a new size.
extern "C" int q3_matmul_set_candidates(int n) {
  if (n < 1 || n > MAX_CANDIDATES) return Q3_ERR_BAD_ARGUMENT;
  std::lock_guard<std::mutex> hold(g_lock);
  g_candidates = n;
  return 0;
}

// Which kernels a new size may go to: 0 the library's and the hand-written one's, by the table and the rules
// (the default), 1 the library's alone (its first candidate), 2 the hand-written ones alone where they take
// the size. The table speaks for mode 0 only. Sizes already settled are forgotten, so that the next product
// of every size follows the new setting.
extern "C" int q3_matmul_set_kernels(int mode) {
  if (mode < KERNELS_BOTH || mode > KERNELS_OWN) return Q3_ERR_BAD_ARGUMENT;
  std::lock_guard<std::mutex> hold(g_lock);
  if (mode != g_kernels) {
    for (auto& d : g_devices) {
      for (auto& p : d.second.plans) forget(p.second);
      d.second.plans.clear();
    }
  }
  g_kernels = mode;
  return 0;
}

// The table: `kind` 0 a plain product, 1 a product whose rows still lack their norm's division, 2 the same with
// the SwiGLU activation, 3 a product that is added into the residual stream; `rows` as q3_matmul_rows_key
// rounds them; `own` >= 0: the hand-written kernel's tile shape with `splits` shares of K; own < 0: the
// library's candidate number `library` (for kind 3: the caller's plain product and separate norm).
extern "C" int q3_matmul_rows_key(int kind, int M) { return rows_key(kind, M); }

extern "C" int q3_matmul_table_add(int kind, int rows, int N, int K, int out_dtype, int library, int own, int splits) {
  if (kind < KIND_PLAIN || kind > KIND_RESIDUAL || rows < 1 || N < 1 || K < 1) return Q3_ERR_BAD_ARGUMENT;
  if (library < 0 || library >= MAX_CANDIDATES || own >= tiles::NUM_CONFIGS || splits < 1 || splits > 64)
    return Q3_ERR_BAD_ARGUMENT;
  std::lock_guard<std::mutex> hold(g_lock);
  Choice c;
  c.library = library;
  c.own = own < 0 ? LIBRARY : own;
  c.splits = splits;
  g_table[Key(kind, rows, N, K, out_dtype)] = c;
  return 0;
}

extern "C" int q3_matmul_table_clear() {
  std::lock_guard<std::mutex> hold(g_lock);
  g_table.clear();
  return 0;
}

// What serves a plain product of this size on the current device: info[0] candidates timed (1 if none were),
// info[1] the one chosen among them, info[2] microseconds of the first candidate, info[3] of the chosen one
// (zero if untimed), info[4] the hand-written kernel's tile shape if that serves it, else -1, info[5] over how
// many blocks it shares K out, info[6] the library's candidate number if the library serves it. Returns 1 if
// the size has been met.
extern "C" int q3_matmul_plan(int M, int N, int K, int out_dtype, float* info) {
  std::lock_guard<std::mutex> hold(g_lock);
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return 0;
  auto d = g_devices.find(device);
  if (d == g_devices.end()) return 0;
  auto p = d->second.plans.find(std::make_tuple(M, N, K, out_dtype));
  if (p == d->second.plans.end() || !p->second.ready) return 0;
  info[0] = (float)p->second.candidates;
  info[1] = (float)p->second.chosen;
  info[2] = p->second.first_us;
  info[3] = p->second.best_us;
  info[4] = (float)p->second.choice.own;
  info[5] = (float)p->second.choice.splits;
  info[6] = (float)p->second.choice.library;
  return 1;
}

// What serves a product of 17 to 128 rows that carries a norm (`kind` 1, 2 or 3 as in the table) under the
// current settings: info[0] the tile shape or -1 (the library's product with the norm's work behind it, or
// declined), info[1] the shares of K. With the tuner on: what it found, and 0 is returned for a size it has
// not met.
extern "C" int q3_matmul_fused_plan(int kind, int M, int N, int K, int* info) {
  if (kind < KIND_SCALED || kind > KIND_RESIDUAL) return 0;
  std::lock_guard<std::mutex> hold(g_lock);
  Choice c;
  if (g_mode == MODE_TUNE) {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) return 0;
    auto d = g_devices.find(device);
    if (d == g_devices.end()) return 0;
    auto known = d->second.noted.find(Key(kind + 4 * g_kernels, rows_key(kind, M), N, K, Q3_BF16));
    if (known == d->second.noted.end()) return 0;
    c = known->second;
  } else {
    c = choice_for(kind, M, N, K, Q3_BF16);
  }
  info[0] = c.own;
  info[1] = c.splits;
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
