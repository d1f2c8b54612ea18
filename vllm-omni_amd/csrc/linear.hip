// Dense projections with fused epilogues: y = x W^T (+ bias) with, in the GEMM's own epilogue,
//   * GELU(tanh)                              (MLP up-projection: no separate activation pass)
//   * out = residual + gate * (x W^T + bias)  (attention / MLP output projections: no separate
//                                              gated-residual pass)
// The contraction itself is a genuine dense GEMM and runs on hipBLASLt's MFMA kernels; what this file
// adds is the problem set-up that lets the library's epilogue do the elementwise work (bias vector,
// activation, a per-output-feature alpha vector for the gate, beta = 1 on the residual), a per-thread
// cache of problem descriptors, and an explicit tuning call that times the library's candidate kernels
// for one problem and remembers the fastest.
//
// Row-major y[M,N] = x[M,K] W[N,K]^T is the column-major product D(N x M) = op(A) B with A = W stored
// K x N (ld = ldw, transposed), B = x stored K x M (ld = ldx): the bias and the alpha vector run along
// D's rows, i.e. along the N output features, as needed.
#include "odit_common.h"
#include "gemm_bf16.h"

#include <hipblaslt/hipblaslt.h>
#include <hipblaslt/hipblaslt-ext.hpp>

#include <algorithm>
#include <mutex>
#include <unordered_map>
#include <vector>

namespace odit {

// alpha[n] = gate[n], gbias[n] = gate[n] * bias[n], both fp32, for the gated-residual epilogue
template <typename T, typename TG>
__global__ __launch_bounds__(256) void gate_prep_kernel(const TG* __restrict__ gate, const T* __restrict__ bias,
                                                         float* __restrict__ alpha, float* __restrict__ gbias, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) {
    const float g = gate ? to_float(gate[i]) : 1.f;
    alpha[i] = g;
    gbias[i] = bias ? g * to_float(bias[i]) : 0.f;
  }
}

struct LinKey {
  int dev, m, n, k, epi, dtype;
  int64_t lda, ldb, ldc, ldd;
  bool operator==(const LinKey& o) const {
    return dev == o.dev && m == o.m && n == o.n && k == o.k && epi == o.epi && dtype == o.dtype &&
           lda == o.lda && ldb == o.ldb && ldc == o.ldc && ldd == o.ldd;
  }
};
struct LinKeyHash {
  size_t operator()(const LinKey& k) const {
    size_t h = 1469598103934665603ull;
    auto mix = [&](uint64_t v) { h = (h ^ v) * 1099511628211ull; };
    mix(k.dev); mix(k.m); mix(k.n); mix(k.k); mix(k.epi); mix(k.dtype);
    mix(static_cast<uint64_t>(k.lda)); mix(static_cast<uint64_t>(k.ldb));
    mix(static_cast<uint64_t>(k.ldc)); mix(static_cast<uint64_t>(k.ldd));
    return h;
  }
};

struct LinPlan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr, d = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t algo_ws = 0;
  bool have_algo = false;
  bool tuned = false;
};

// One hipBLASLt handle and one plan cache per host thread: plans are mutated per call (bias and
// alpha-vector pointers), so they are never shared between threads.
struct LinState {
  hipblasLtHandle_t handle[64] = {nullptr};
  std::unordered_map<LinKey, LinPlan, LinKeyHash> plans;
};
static thread_local LinState g_lin;

// Problems for which a tuning call has compared the hand-written kernel with the library: true = the
// hand-written kernel won (key: the whole problem, rows_per_gate in the lda field). Process-wide and kept
// for the life of the process: every host thread sees what any thread has measured, and the record
// outlives the per-thread descriptor cache.
static std::mutex g_engine_mu;
static std::unordered_map<LinKey, bool, LinKeyHash> g_handwritten_wins;

#define ODIT_LT(call)                                                                      \
  do {                                                                                     \
    const hipblasStatus_t st__ = (call);                                                   \
    if (st__ != HIPBLAS_STATUS_SUCCESS) {                                                  \
      set_error("odit_linear: %s failed with hipBLAS status %d", #call, static_cast<int>(st__)); \
      return ODIT_ELAUNCH;                                                                 \
    }                                                                                      \
  } while (0)

static int lin_handle(int dev, hipblasLtHandle_t* out) {
  if (dev < 0 || dev >= 64) { set_error("odit_linear: device index %d out of range", dev); return ODIT_EINVAL; }
  if (g_lin.handle[dev] == nullptr) ODIT_LT(hipblasLtCreate(&g_lin.handle[dev]));
  *out = g_lin.handle[dev];
  return ODIT_OK;
}

static hipDataType lin_type(int dtype) {
  return dtype == ODIT_BF16 ? HIP_R_16BF : (dtype == ODIT_F16 ? HIP_R_16F : HIP_R_32F);
}

static void lin_plan_release(LinPlan& p) {
  if (p.a) hipblasLtMatrixLayoutDestroy(p.a);
  if (p.b) hipblasLtMatrixLayoutDestroy(p.b);
  if (p.c) hipblasLtMatrixLayoutDestroy(p.c);
  if (p.d) hipblasLtMatrixLayoutDestroy(p.d);
  if (p.desc) hipblasLtMatmulDescDestroy(p.desc);
  p = LinPlan{};
}

static int lin_plan_build(const LinKey& key, LinPlan& p) {
  const hipDataType t = lin_type(key.dtype);
  ODIT_LT(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
  const int32_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
  ODIT_LT(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta)));
  ODIT_LT(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb)));
  // key.epi = epilogue * 4 + (bias vector in the epilogue ? 1 : 0) + (alpha vector ? 2 : 0)
  const int kind = key.epi >> 2;
  const bool has_bias = key.epi & 1, alpha_vec = key.epi & 2;
  const bool gelu = kind == ODIT_EPI_GELU_TANH || kind == ODIT_EPI_BIAS_GELU_TANH;
  const uint32_t epi = gelu ? (has_bias ? HIPBLASLT_EPILOGUE_GELU_BIAS : HIPBLASLT_EPILOGUE_GELU)
                            : (has_bias ? HIPBLASLT_EPILOGUE_BIAS : HIPBLASLT_EPILOGUE_DEFAULT);
  ODIT_LT(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epi, sizeof(epi)));
  if (alpha_vec) {
    const int32_t pm = HIPBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_HOST;
    ODIT_LT(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_POINTER_MODE, &pm, sizeof(pm)));
  }
  if (has_bias) {  // the gate-scaled bias that goes with an alpha vector is fp32
    const int32_t bt = alpha_vec ? HIP_R_32F : t;
    ODIT_LT(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bt, sizeof(bt)));
  }
  // column-major views: A = W (K x N, ld lda), B = x (K x M, ld ldb), C/D = N x M
  ODIT_LT(hipblasLtMatrixLayoutCreate(&p.a, t, key.k, key.n, key.lda));
  ODIT_LT(hipblasLtMatrixLayoutCreate(&p.b, t, key.k, key.m, key.ldb));
  ODIT_LT(hipblasLtMatrixLayoutCreate(&p.c, t, key.n, key.m, key.ldc));
  ODIT_LT(hipblasLtMatrixLayoutCreate(&p.d, t, key.n, key.m, key.ldd));
  return ODIT_OK;
}

static int lin_plan(const LinKey& key, LinPlan** out) {
  auto it = g_lin.plans.find(key);
  if (it != g_lin.plans.end()) { *out = &it->second; return ODIT_OK; }
  // A process sees a few dozen distinct problems; a caller that keeps inventing new ones (changing row
  // counts) must not grow the cache without bound: past the cap everything is rebuilt on demand.
  constexpr size_t kMaxPlans = 512;
  if (g_lin.plans.size() >= kMaxPlans) {
    for (auto& kv : g_lin.plans) lin_plan_release(kv.second);
    g_lin.plans.clear();
  }
  LinPlan p;
  const int rc = lin_plan_build(key, p);
  if (rc != ODIT_OK) {  // nothing half-built stays behind
    lin_plan_release(p);
    return rc;
  }
  auto ins = g_lin.plans.emplace(key, p);
  *out = &ins.first->second;
  return ODIT_OK;
}

// engine bits of the `flags` argument: neither = the hand-written kernel where it takes the problem and is
// expected (or was measured) to win, else the library
static int lin_engine_of(unsigned flags) {
  return (flags & ODIT_LINEAR_LIBRARY) ? 1 : ((flags & ODIT_LINEAR_HANDWRITTEN) ? 2 : 0);
}

struct LinCall {
  const void *x, *w, *bias, *residual, *gate;
  void* out;
  int M, N, K;
  int64_t ldx, ldw, ldo, ldr;
  int epilogue, gate_dtype, dtype;
  void* ws;
  size_t ws_bytes;
  hipStream_t stream;
};

static bool lin_is_residual(const LinCall& c) {
  return c.epilogue == ODIT_EPI_GATED_RESIDUAL || c.epilogue == ODIT_EPI_GATED_RESIDUAL_PRE;
}
// the gate has to be turned into fp32 alpha / gate*bias vectors by a helper launch
static bool lin_needs_prep(const LinCall& c) { return c.epilogue == ODIT_EPI_GATED_RESIDUAL && c.gate != nullptr; }

// workspace split: [0, 8N rounded to 256) gate vectors (when a helper launch makes them), the rest for
// the library
static size_t lin_gate_bytes(const LinCall& c) {
  return lin_needs_prep(c) ? ((static_cast<size_t>(c.N) * 8 + 255) / 256) * 256 : 0;
}

static int lin_prepare(const LinCall& c, hipblasLtHandle_t* h, LinPlan** plan, const void** alpha_ptr,
                       const void** c_ptr, void** lib_ws, size_t* lib_ws_bytes) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) { set_error("odit_linear: hipGetDevice failed"); return ODIT_ELAUNCH; }
  int rc = lin_handle(dev, h);
  if (rc != ODIT_OK) return rc;
  const bool gated = lin_is_residual(c);
  const bool prep = lin_needs_prep(c);
  const bool alpha_vec = gated && c.gate != nullptr;
  const bool has_bias = c.bias != nullptr;
  LinKey key{dev, c.M, c.N, c.K, c.epilogue * 4 + (has_bias ? 1 : 0) + (alpha_vec ? 2 : 0), c.dtype,
             c.ldw, c.ldx, gated ? c.ldr : c.ldo, c.ldo};
  rc = lin_plan(key, plan);
  if (rc != ODIT_OK) return rc;
  const size_t gb = lin_gate_bytes(c);
  if (gb > c.ws_bytes) {
    set_error("odit_linear: workspace of %zu bytes cannot hold the %zu bytes of gate vectors", c.ws_bytes, gb);
    return ODIT_EWORKSPACE;
  }
  *lib_ws = c.ws ? static_cast<char*>(c.ws) + gb : nullptr;
  *lib_ws_bytes = c.ws ? c.ws_bytes - gb : 0;
  static const float one = 1.f;
  *alpha_ptr = &one;
  *c_ptr = c.out;
  LinPlan& p = **plan;
  if (gated) *c_ptr = c.residual;
  if (prep) {
    float* alpha = static_cast<float*>(c.ws);
    float* gbias = alpha + c.N;
    const dim3 grid((c.N + 255) / 256);
#define ODIT_GATE_PREP(T, TG)                                                                        \
  hipLaunchKernelGGL((gate_prep_kernel<T, TG>), grid, dim3(256), 0, c.stream, static_cast<const TG*>(c.gate), \
                     static_cast<const T*>(c.bias), alpha, gbias, c.N)
    if (c.gate_dtype == ODIT_F32) {
      ODIT_DISPATCH_DTYPE(c.dtype, T, ODIT_GATE_PREP(T, float));
    } else {
      ODIT_DISPATCH_DTYPE(c.dtype, T, ODIT_GATE_PREP(T, T));
    }
#undef ODIT_GATE_PREP
    rc = check_launch("odit_linear (gate vectors)");
    if (rc != ODIT_OK) return rc;
    if (has_bias) {
      const void* bp = gbias;
      ODIT_LT(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bp, sizeof(bp)));
    }
    *alpha_ptr = alpha;
  } else {
    if (has_bias) {
      const void* bp = c.bias;
      ODIT_LT(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bp, sizeof(bp)));
    }
    if (alpha_vec) *alpha_ptr = c.gate;  // caller-made fp32 vectors
  }
  return ODIT_OK;
}

static int lin_default_algo(hipblasLtHandle_t h, LinPlan& p, size_t lib_ws_bytes) {
  hipblasLtMatmulPreference_t pref;
  ODIT_LT(hipblasLtMatmulPreferenceCreate(&pref));
  const uint64_t maxws = lib_ws_bytes;
  hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &maxws, sizeof(maxws));
  hipblasLtMatmulHeuristicResult_t res[1];
  int n = 0;
  const hipblasStatus_t st = hipblasLtMatmulAlgoGetHeuristic(h, p.desc, p.a, p.b, p.c, p.d, pref, 1, res, &n);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (st != HIPBLAS_STATUS_SUCCESS || n < 1) {
    set_error("odit_linear: hipBLASLt has no kernel for this problem (status %d)", static_cast<int>(st));
    return ODIT_ENOTSUP;
  }
  p.algo = res[0].algo;
  p.algo_ws = res[0].workspaceSize;
  p.have_algo = true;
  return ODIT_OK;
}

static int lin_check(const LinCall& c) {
  ODIT_CHECK_ARG(c.x && c.w && c.out, "odit_linear: x/w/out must not be null");
  ODIT_CHECK_ARG(c.M >= 0 && c.N > 0 && c.K > 0, "odit_linear: bad shape M=%d N=%d K=%d", c.M, c.N, c.K);
  ODIT_CHECK_ARG(c.dtype == ODIT_BF16 || c.dtype == ODIT_F16 || c.dtype == ODIT_F32, "odit_linear: bad dtype %d", c.dtype);
  ODIT_CHECK_ARG(c.epilogue >= ODIT_EPI_NONE && c.epilogue <= ODIT_EPI_GATED_RESIDUAL_PRE,
                 "odit_linear: unknown epilogue %d", c.epilogue);
  ODIT_CHECK_ARG((c.epilogue != ODIT_EPI_NONE && c.epilogue != ODIT_EPI_GELU_TANH) || c.bias == nullptr,
                 "odit_linear: this epilogue takes no bias");
  ODIT_CHECK_ARG(c.ldx >= c.K && c.ldw >= c.K && c.ldo >= c.N, "odit_linear: leading dimensions too small");
  if (c.epilogue == ODIT_EPI_BIAS || c.epilogue == ODIT_EPI_BIAS_GELU_TANH)
    ODIT_CHECK_ARG(c.bias != nullptr, "odit_linear: this epilogue needs a bias vector");
  if (lin_is_residual(c))
    ODIT_CHECK_ARG(c.residual != nullptr && c.ldr >= c.N, "odit_linear: this epilogue needs `residual` with ldr >= N");
  if (lin_needs_prep(c)) {
    ODIT_CHECK_ARG(c.ws != nullptr, "odit_linear: a gate in the tensor dtype needs a workspace for two fp32 vectors");
    ODIT_CHECK_ARG(c.gate_dtype == c.dtype || c.gate_dtype == ODIT_F32, "odit_linear: gate dtype must equal dtype or be f32");
    ODIT_CHECK_ARG((reinterpret_cast<uintptr_t>(c.ws) & 255) == 0, "odit_linear: workspace must be 256-byte aligned");
  }
  if (c.epilogue == ODIT_EPI_GATED_RESIDUAL_PRE)
    ODIT_CHECK_ARG(c.gate != nullptr && aligned16(c.gate) && aligned16(c.bias),
                   "odit_linear: the pre-scaled form needs a 16-byte aligned float32 gate (and gate*bias) vector");
  return ODIT_OK;
}

}  // namespace odit

// Workspace split: a workspace large enough starts with the hand-written kernel's scratch (tile
// counters that are zero between calls, partial-tile slots); the rest is the library's.
static void lin_split_ws(void* ws, size_t bytes, void** sk, void** lib, size_t* lib_bytes) {
  if (ws != nullptr && bytes >= odit::kGemmScratchBytes + (static_cast<size_t>(1) << 20)) {
    *sk = ws;
    *lib = static_cast<char*>(ws) + odit::kGemmScratchBytes;
    *lib_bytes = bytes - odit::kGemmScratchBytes;
  } else {
    *sk = nullptr;
    *lib = ws;
    *lib_bytes = bytes;
  }
}

static int lin_run_library(const odit::LinCall& c) {
  using namespace odit;
  hipblasLtHandle_t h;
  LinPlan* p;
  const void *alpha, *cptr;
  void* lws;
  size_t lws_bytes;
  int rc = lin_prepare(c, &h, &p, &alpha, &cptr, &lws, &lws_bytes);
  if (rc != ODIT_OK) return rc;
  if (!p->have_algo || p->algo_ws > lws_bytes) {
    rc = lin_default_algo(h, *p, lws_bytes);
    if (rc != ODIT_OK) return rc;
  }
  const float beta = lin_is_residual(c) ? 1.f : 0.f;
  ODIT_LT(hipblasLtMatmul(h, p->desc, alpha, c.w, p->a, c.x, p->b, &beta, cptr, p->c, c.out, p->d, &p->algo, lws,
                          lws_bytes, c.stream));
  return ODIT_OK;
}

static odit::GemmCall lin_gemm_call(const odit::LinCall& c, int rows_per_gate, int64_t ldg) {
  odit::GemmCall g;
  g.x = c.x; g.w = c.w; g.bias = c.bias; g.residual = c.residual; g.gate = c.gate; g.out = c.out;
  g.M = c.M; g.N = c.N; g.K = c.K;
  g.ldx = c.ldx; g.ldw = c.ldw; g.ldo = c.ldo; g.ldr = c.ldr;
  g.epilogue = c.epilogue;
  g.gate_f32 = c.gate_dtype == ODIT_F32 ? 1 : 0;
  g.rows_per_gate = rows_per_gate;
  g.ldg = ldg;
  return g;
}

// key of the whole problem for the record of which engine won a tuning run
static odit::LinKey lin_engine_key(int dev, const odit::LinCall& c, int rows_per_gate) {
  return odit::LinKey{dev, c.M, c.N, c.K, c.epilogue * 4 + (c.bias != nullptr ? 1 : 0) + (c.gate != nullptr ? 2 : 0),
                      c.dtype, rows_per_gate, c.ldx, c.ldw, c.ldo};
}

// Which hand-written kernel takes a problem: 1 = the stream-K kernel (few rows; needs its scratch), 2 = the
// tile kernel (many rows), 0 = neither.
constexpr int kTileMinRows = 1025;
static int lin_handwritten_kind(const odit::GemmCall& g, int dtype, const void* sk) {
  if (g.M >= kTileMinRows) return odit::gemm_tile_takes(g, dtype) ? 2 : 0;
  return sk != nullptr && odit::gemm_streamk_takes(g, dtype) ? 1 : 0;
}

static int lin_launch_handwritten(int kind, const odit::GemmCall& g, void* sk, hipStream_t stream) {
  if (kind == 1) return odit::launch_gemm_streamk(g, sk, stream);
  const int cus = odit::device_cus();
  if (cus <= 0) { odit::set_error("odit_linear: cannot read the device's compute-unit count"); return ODIT_ELAUNCH; }
  return odit::launch_gemm_tile(g, cus, stream);
}

// Without a tuning record: the stream-K kernel where the reduction is long against the number of output
// tiles (K >= 2 N: the library's choices split K badly there, measured 58 vs 72 us at M=512, N=3072,
// K=12288); the tile kernel for the gated form with one gate vector per group of rows, where the library
// needs a launch per group, and for the other forms where measured faster (ODIT_TILE_DEFAULT_ALL).
static bool lin_prefers_handwritten(int dev, int kind, const odit::LinCall& c, int rows_per_gate) {
  {
    std::lock_guard<std::mutex> lock(odit::g_engine_mu);
    const auto it = odit::g_handwritten_wins.find(lin_engine_key(dev, c, rows_per_gate));
    if (it != odit::g_handwritten_wins.end()) return it->second;
  }
  if (kind == 2) return false;
  return c.K >= 2 * c.N;
}

extern "C" size_t odit_linear_workspace_bytes(void) {
  return odit::kGemmScratchBytes + (static_cast<size_t>(64) << 20);
}

extern "C" int odit_linear_rows(const void* x, const void* w, const void* bias, void* out, const void* residual,
                                const void* gate, int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldo,
                                int64_t ldr, int epilogue, int gate_dtype, int dtype, int rows_per_gate,
                                int64_t gate_stride, unsigned flags, void* workspace, size_t workspace_bytes,
                                void* stream) {
  using namespace odit;
  ODIT_CHECK_ARG((flags & ~(ODIT_LINEAR_LIBRARY | ODIT_LINEAR_HANDWRITTEN)) == 0 &&
                     (flags & (ODIT_LINEAR_LIBRARY | ODIT_LINEAR_HANDWRITTEN)) != (ODIT_LINEAR_LIBRARY | ODIT_LINEAR_HANDWRITTEN),
                 "odit_linear_rows: flags may name one engine (ODIT_LINEAR_LIBRARY or ODIT_LINEAR_HANDWRITTEN), got %#x", flags);
  void *sk, *lib;
  size_t lib_bytes;
  lin_split_ws(workspace, workspace_bytes, &sk, &lib, &lib_bytes);
  LinCall c{x, w, bias, residual, gate, out, M, N, K, ldx, ldw, ldo, ldr, epilogue, gate_dtype, dtype,
            lib, lib_bytes, static_cast<hipStream_t>(stream)};
  int rc = lin_check(c);
  if (rc != ODIT_OK || M == 0) return rc;
  ODIT_CHECK_ARG(rows_per_gate >= 0 && (rows_per_gate == 0 || gate_stride >= 0),
                 "odit_linear_rows: rows_per_gate and gate_stride must not be negative");
  const bool per_rows = lin_is_residual(c) && gate != nullptr && rows_per_gate > 0 && rows_per_gate < M;
  const int engine = lin_engine_of(flags);
  const GemmCall g = lin_gemm_call(c, per_rows ? rows_per_gate : 0, per_rows ? gate_stride : 0);
  const int kind = lin_handwritten_kind(g, dtype, sk);
  if (engine == 2 && kind == 0) {
    set_error("odit_linear: no hand-written kernel takes this problem (M=%d N=%d K=%d, workspace %zu bytes)",
              M, N, K, workspace_bytes);
    return ODIT_ENOTSUP;
  }
  if (kind != 0 && engine != 1) {
    int dev = 0;
    if (engine == 2 || (hipGetDevice(&dev) == hipSuccess && lin_prefers_handwritten(dev, kind, c, g.rows_per_gate)))
      return lin_launch_handwritten(kind, g, sk, c.stream);
  }
  if (!per_rows) return lin_run_library(c);
  // the library's epilogue takes one gate vector per launch: one launch per group of rows
  const size_t esz = dtype == ODIT_F32 ? 4 : 2, gsz = gate_dtype == ODIT_F32 ? 4 : esz;
  for (int r0 = 0; r0 < M; r0 += rows_per_gate) {
    LinCall cg = c;
    const int64_t grp = r0 / rows_per_gate;
    cg.M = M - r0 < rows_per_gate ? M - r0 : rows_per_gate;
    cg.x = static_cast<const char*>(x) + static_cast<size_t>(r0) * ldx * esz;
    cg.out = static_cast<char*>(out) + static_cast<size_t>(r0) * ldo * esz;
    cg.residual = static_cast<const char*>(residual) + static_cast<size_t>(r0) * ldr * esz;
    cg.gate = static_cast<const char*>(gate) + static_cast<size_t>(grp * gate_stride) * gsz;
    if (epilogue == ODIT_EPI_GATED_RESIDUAL_PRE && bias != nullptr)
      cg.bias = static_cast<const char*>(bias) + static_cast<size_t>(grp * gate_stride) * 4;
    rc = lin_run_library(cg);
    if (rc != ODIT_OK) return rc;
  }
  return ODIT_OK;
}

extern "C" int odit_linear_rows_plan(const void* x, const void* w, const void* bias, void* out, const void* residual,
                                     const void* gate, int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldo,
                                     int64_t ldr, int epilogue, int gate_dtype, int dtype, int rows_per_gate,
                                     int64_t gate_stride, unsigned flags, void* workspace, size_t workspace_bytes,
                                     int* handwritten, int* launches) {
  using namespace odit;
  void *sk, *lib;
  size_t lib_bytes;
  lin_split_ws(workspace, workspace_bytes, &sk, &lib, &lib_bytes);
  LinCall c{x, w, bias, residual, gate, out, M, N, K, ldx, ldw, ldo, ldr, epilogue, gate_dtype, dtype,
            lib, lib_bytes, nullptr};
  int rc = lin_check(c);
  if (rc != ODIT_OK) return rc;
  ODIT_CHECK_ARG(handwritten != nullptr && launches != nullptr, "odit_linear_rows_plan: null result pointers");
  const bool per_rows = lin_is_residual(c) && gate != nullptr && rows_per_gate > 0 && rows_per_gate < M;
  const int engine = lin_engine_of(flags);
  const GemmCall g = lin_gemm_call(c, per_rows ? rows_per_gate : 0, per_rows ? gate_stride : 0);
  int dev = 0;
  (void)hipGetDevice(&dev);
  const int kind = M > 0 ? lin_handwritten_kind(g, dtype, sk) : 0;
  const bool own = kind != 0 && engine != 1 && (engine == 2 || lin_prefers_handwritten(dev, kind, c, g.rows_per_gate));
  *handwritten = own ? 1 : 0;
  *launches = M == 0 ? 0 : (own || !per_rows ? 1 : (M + rows_per_gate - 1) / rows_per_gate);
  if (!own && lin_needs_prep(c)) *launches *= 2;  // plus the [N]-sized gate-vector launch of the library form
  return ODIT_OK;
}

extern "C" int odit_linear(const void* x, const void* w, const void* bias, void* out, const void* residual,
                           const void* gate, int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldo,
                           int64_t ldr, int epilogue, int gate_dtype, int dtype, void* workspace,
                           size_t workspace_bytes, void* stream) {
  return odit_linear_rows(x, w, bias, out, residual, gate, M, N, K, ldx, ldw, ldo, ldr, epilogue, gate_dtype, dtype, 0,
                          0, 0u, workspace, workspace_bytes, stream);
}

// Times the library's kernels for problem c (cold caches before every timed launch when a flush buffer
// is given: in a model every projection has its own weights, which are never cache-resident, so
// back-to-back launches on one weight would rank the kernels wrongly) and keeps the fastest in the plan.
static int lin_tune_library(const odit::LinCall& c, int iters, void* flush, size_t flush_bytes, float* best_us) {
  using namespace odit;
  hipblasLtHandle_t h;
  LinPlan* p;
  const void *alpha, *cptr;
  void* lws;
  size_t lws_bytes;
  int rc = lin_prepare(c, &h, &p, &alpha, &cptr, &lws, &lws_bytes);
  if (rc != ODIT_OK) return rc;
  const hipDataType t = lin_type(c.dtype);
  std::vector<hipblasLtMatmulHeuristicResult_t> all;
  ODIT_LT(hipblaslt_ext::getAllAlgos(h, hipblaslt_ext::GemmType::HIPBLASLT_GEMM, HIPBLAS_OP_T, HIPBLAS_OP_N, t, t, t, t,
                                     HIPBLAS_COMPUTE_32F, all));
  const float beta = lin_is_residual(c) ? 1.f : 0.f;
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
    set_error("odit_linear_tune: hipEventCreate failed");
    return ODIT_ELAUNCH;
  }
  float best = 1e30f;
  int n_ok = 0;
  auto time_algo = [&](hipblasLtMatmulAlgo_t& algo, int reps) -> float {
    if (hipblasLtMatmul(h, p->desc, alpha, c.w, p->a, c.x, p->b, &beta, cptr, p->c, c.out, p->d, &algo, lws, lws_bytes,
                        c.stream) != HIPBLAS_STATUS_SUCCESS)
      return -1.f;
    float total = 0.f;
    for (int i = 0; i < reps; ++i) {
      if (flush != nullptr && flush_bytes > 0) (void)hipMemsetAsync(flush, i & 0xff, flush_bytes, c.stream);
      (void)hipEventRecord(e0, c.stream);
      hipblasLtMatmul(h, p->desc, alpha, c.w, p->a, c.x, p->b, &beta, cptr, p->c, c.out, p->d, &algo, lws, lws_bytes,
                      c.stream);
      (void)hipEventRecord(e1, c.stream);
      if (hipEventSynchronize(e1) != hipSuccess) return -1.f;
      float ms = 0.f;
      (void)hipEventElapsedTime(&ms, e0, e1);
      total += ms;
    }
    return total * 1e3f / reps;
  };
  // first pass: one timed launch of every kernel the library has for these types that accepts the
  // problem; second pass: the best few again with `iters` launches each
  std::vector<std::pair<float, size_t>> ranked;
  for (size_t i = 0; i < all.size(); ++i) {
    size_t need = 0;
    if (hipblaslt_ext::matmulIsAlgoSupported(h, p->desc, alpha, p->a, p->b, &beta, p->c, p->d, all[i].algo, need) !=
            HIPBLAS_STATUS_SUCCESS || need > lws_bytes)
      continue;
    all[i].workspaceSize = need;
    const float us = time_algo(all[i].algo, 2);
    if (us > 0.f) { ranked.emplace_back(us, i); ++n_ok; }
  }
  std::sort(ranked.begin(), ranked.end());
  const size_t finalists = std::min<size_t>(ranked.size(), 12);
  for (size_t r = 0; r < finalists; ++r) {
    auto& cand = all[ranked[r].second];
    const float us = time_algo(cand.algo, iters);
    if (us > 0.f && us < best) {
      best = us;
      p->algo = cand.algo;
      p->algo_ws = cand.workspaceSize;
      p->have_algo = true;
      p->tuned = true;
    }
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (n_ok == 0) {
    set_error("odit_linear_tune: none of the library's %zu kernels accepts this problem", all.size());
    return ODIT_ENOTSUP;
  }
  *best_us = best;
  return ODIT_OK;
}

static int lin_time_handwritten(int kind, const odit::GemmCall& g, void* sk, hipStream_t stream, int iters, void* flush,
                                size_t flush_bytes, float* us) {
  using namespace odit;
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
    set_error("odit_linear_tune: hipEventCreate failed");
    return ODIT_ELAUNCH;
  }
  int rc = lin_launch_handwritten(kind, g, sk, stream);
  float total = 0.f;
  for (int i = 0; i < iters && rc == ODIT_OK; ++i) {
    if (flush != nullptr && flush_bytes > 0) (void)hipMemsetAsync(flush, i & 0xff, flush_bytes, stream);
    (void)hipEventRecord(e0, stream);
    rc = lin_launch_handwritten(kind, g, sk, stream);
    (void)hipEventRecord(e1, stream);
    if (hipEventSynchronize(e1) != hipSuccess) { set_error("odit_linear_tune: hipEventSynchronize failed"); rc = ODIT_ELAUNCH; }
    float ms = 0.f;
    (void)hipEventElapsedTime(&ms, e0, e1);
    total += ms;
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  *us = total * 1e3f / iters;
  return rc;
}

extern "C" int odit_linear_rows_tune(const void* x, const void* w, const void* bias, void* out, const void* residual,
                                     const void* gate, int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldo,
                                     int64_t ldr, int epilogue, int gate_dtype, int dtype, int rows_per_gate,
                                     int64_t gate_stride, void* workspace, size_t workspace_bytes, void* stream,
                                     int iters, void* flush, size_t flush_bytes, float* best_us, int* handwritten) {
  using namespace odit;
  if (handwritten) *handwritten = 0;
  void *sk, *lib;
  size_t lib_bytes;
  lin_split_ws(workspace, workspace_bytes, &sk, &lib, &lib_bytes);
  LinCall c{x, w, bias, residual, gate, out, M, N, K, ldx, ldw, ldo, ldr, epilogue, gate_dtype, dtype,
            lib, lib_bytes, static_cast<hipStream_t>(stream)};
  int rc = lin_check(c);
  if (rc != ODIT_OK) return rc;
  ODIT_CHECK_ARG(M > 0 && iters > 0, "odit_linear_tune: needs M > 0 and iters > 0");
  ODIT_CHECK_ARG(rows_per_gate >= 0 && gate_stride >= 0, "odit_linear_tune: rows_per_gate and gate_stride must not be negative");
  const bool per_rows = lin_is_residual(c) && gate != nullptr && rows_per_gate > 0 && rows_per_gate < M;
  // the library runs one launch per group of rows: tune that launch (on the first group), and the shorter
  // launch of a last group that is not full, which is a problem of its own to the library
  LinCall cl = c;
  int launches = 1, last_rows = 0;
  if (per_rows) {
    cl.M = rows_per_gate;
    launches = M / rows_per_gate;
    last_rows = M % rows_per_gate;
  }
  float lib_us = 0.f;
  rc = lin_tune_library(cl, iters, flush, flush_bytes, &lib_us);
  if (rc != ODIT_OK) return rc;
  lib_us *= static_cast<float>(launches);
  if (last_rows > 0) {
    LinCall cr = cl;   // (timed on the first rows: only the shape matters)
    cr.M = last_rows;
    float last_us = 0.f;
    rc = lin_tune_library(cr, iters, flush, flush_bytes, &last_us);
    if (rc != ODIT_OK) return rc;
    lib_us += last_us;
  }
  float best = lib_us;
  const GemmCall g = lin_gemm_call(c, per_rows ? rows_per_gate : 0, per_rows ? gate_stride : 0);
  if (const int kind = lin_handwritten_kind(g, dtype, sk)) {
    float own_us = 0.f;
    rc = lin_time_handwritten(kind, g, sk, c.stream, iters, flush, flush_bytes, &own_us);
    if (rc != ODIT_OK) return rc;
    int dev = 0;
    (void)hipGetDevice(&dev);
    {
      std::lock_guard<std::mutex> lock(g_engine_mu);
      g_handwritten_wins[lin_engine_key(dev, c, per_rows ? rows_per_gate : 0)] = own_us < lib_us;
    }
    if (handwritten) *handwritten = own_us < lib_us ? 1 : 0;
    if (own_us < best) best = own_us;
  }
  if (best_us) *best_us = best;
  return ODIT_OK;
}

extern "C" int odit_linear_tune(const void* x, const void* w, const void* bias, void* out, const void* residual,
                                const void* gate, int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldo,
                                int64_t ldr, int epilogue, int gate_dtype, int dtype, void* workspace,
                                size_t workspace_bytes, void* stream, int iters, void* flush,
                                size_t flush_bytes, float* best_us) {
  return odit_linear_rows_tune(x, w, bias, out, residual, gate, M, N, K, ldx, ldw, ldo, ldr, epilogue, gate_dtype, dtype,
                               0, 0, workspace, workspace_bytes, stream, iters, flush, flush_bytes, best_us, nullptr);
}
