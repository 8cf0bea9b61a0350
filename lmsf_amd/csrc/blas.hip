// The BLAS library's bfloat16 matrix products, called from C++.
//
// The reference calls cuBLASLt from native code for every product of the model
// (tops/csrc/tops/tensorrt_llm/c_api/gemm.cc:43-150 sets up the descriptors and calls the wrapper,
// tops/src/cublas.rs:29-114 is its Rust face) and profiles the library's tactics per weight shape and
// bucket of rows, keeping the fastest (tops/src/cublas.rs:121-223 drives that search). Here the products of
// many rows, where the library beats this package's kernels, go to hipBLASLt through its C interface: one
// handle and one workspace per device, a plan (descriptors + algorithm) per shape kept in a table, and a search
// over the library's candidates for the shapes the caller names, timed on the caller's own weights.
//
// The library is opened at run time by its name, not linked: a process that has it loaded already (PyTorch
// links it) gets that copy, and this library still loads where hipBLASLt is absent (then lmsf_blas_init
// fails with the reason and nothing else here is callable).
#include "common.h"
#include "entry_points.h"

#include <dlfcn.h>
#include <hipblaslt/hipblaslt.h>

#include <algorithm>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>

namespace {

struct Api {
  void* lib = nullptr;
  decltype(&hipblasLtCreate) Create = nullptr;
  decltype(&hipblasLtDestroy) Destroy = nullptr;
  decltype(&hipblasLtMatrixLayoutCreate) LayoutCreate = nullptr;
  decltype(&hipblasLtMatrixLayoutDestroy) LayoutDestroy = nullptr;
  decltype(&hipblasLtMatmulDescCreate) DescCreate = nullptr;
  decltype(&hipblasLtMatmulDescDestroy) DescDestroy = nullptr;
  decltype(&hipblasLtMatmulDescSetAttribute) DescSet = nullptr;
  decltype(&hipblasLtMatmulPreferenceCreate) PrefCreate = nullptr;
  decltype(&hipblasLtMatmulPreferenceDestroy) PrefDestroy = nullptr;
  decltype(&hipblasLtMatmulPreferenceSetAttribute) PrefSet = nullptr;
  decltype(&hipblasLtMatmulAlgoGetHeuristic) Heuristic = nullptr;
  decltype(&hipblasLtMatmul) Matmul = nullptr;
};

Api g_api;
std::mutex g_mutex;

template <typename F> bool sym(void* lib, const char* name, F* out) {
  *out = reinterpret_cast<F>(dlsym(lib, name));
  if (*out == nullptr) lmsf_set_error("blas: the BLAS library has no %s", name);
  return *out != nullptr;
}

bool load_api() {
  if (g_api.lib != nullptr) return true;
  void* lib = nullptr;
  for (const char* name : {"libhipblaslt.so.1", "libhipblaslt.so"}) {
    lib = dlopen(name, RTLD_NOW | RTLD_NOLOAD);          // the copy the process already has, if any
    if (lib == nullptr) lib = dlopen(name, RTLD_NOW | RTLD_LOCAL);
    if (lib != nullptr) break;
  }
  if (lib == nullptr) {
    const char* why = dlerror();
    lmsf_set_error("blas: cannot open libhipblaslt (%s)", why ? why : "no reason given");
    return false;
  }
  Api a;
  if (!(sym(lib, "hipblasLtCreate", &a.Create) && sym(lib, "hipblasLtDestroy", &a.Destroy) &&
        sym(lib, "hipblasLtMatrixLayoutCreate", &a.LayoutCreate) &&
        sym(lib, "hipblasLtMatrixLayoutDestroy", &a.LayoutDestroy) &&
        sym(lib, "hipblasLtMatmulDescCreate", &a.DescCreate) && sym(lib, "hipblasLtMatmulDescDestroy", &a.DescDestroy) &&
        sym(lib, "hipblasLtMatmulDescSetAttribute", &a.DescSet) &&
        sym(lib, "hipblasLtMatmulPreferenceCreate", &a.PrefCreate) &&
        sym(lib, "hipblasLtMatmulPreferenceDestroy", &a.PrefDestroy) &&
        sym(lib, "hipblasLtMatmulPreferenceSetAttribute", &a.PrefSet) &&
        sym(lib, "hipblasLtMatmulAlgoGetHeuristic", &a.Heuristic) && sym(lib, "hipblasLtMatmul", &a.Matmul)))
    return false;
  a.lib = lib;
  g_api = a;
  return true;
}

// y [M, N] = x [M, K] W^T, W [N, K], all row-major. The library thinks in columns: y^T [N, M] = W . x^T, with
// A = W^T stored as a K x N column-major matrix of leading dimension ldw (transposed), B = x^T stored K x M
// with leading dimension ldx (as it is), D = y^T stored N x M with leading dimension ldy.
typedef std::tuple<int, int, int, long, long, long, int> Key;   // M, N, K, ldx, ldw, ldy, bias

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, d = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
  bool tuned = false;
};

struct Device {
  hipblasLtHandle_t handle = nullptr;
  void* workspace = nullptr;
  size_t workspace_bytes = 0;
  std::map<Key, Plan> plans;
};

const int kMaxDevices = 64;
const size_t kMaxPlans = 8192;    // per device; beyond that the untuned ones are dropped and made again on demand
Device g_devices[kMaxDevices];

void destroy_plan(Plan& p) {
  if (p.desc) g_api.DescDestroy(p.desc);
  for (hipblasLtMatrixLayout_t l : {p.a, p.b, p.d})
    if (l) g_api.LayoutDestroy(l);
  p = Plan();
}

Device* current_device() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    lmsf_set_error("blas: cannot tell the current device");
    return nullptr;
  }
  Device* d = &g_devices[dev];
  if (d->handle == nullptr) {
    lmsf_set_error("blas: lmsf_blas_init has not been called on device %d", dev);
    return nullptr;
  }
  return d;
}

// Descriptors of one shape, without an algorithm yet.
bool make_descriptors(const Key& key, Plan* p) {
  const int M = std::get<0>(key), N = std::get<1>(key), K = std::get<2>(key);
  const long ldx = std::get<3>(key), ldw = std::get<4>(key), ldy = std::get<5>(key);
  const bool bias = std::get<6>(key) != 0;
  bool ok = g_api.DescCreate(&p->desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS;
  const int32_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
  ok = ok && g_api.DescSet(p->desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta)) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && g_api.DescSet(p->desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb)) == HIPBLAS_STATUS_SUCCESS;
  if (ok && bias) {
    const uint32_t epi = HIPBLASLT_EPILOGUE_BIAS;
    const int32_t bt = HIP_R_16BF;
    ok = g_api.DescSet(p->desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epi, sizeof(epi)) == HIPBLAS_STATUS_SUCCESS &&
         g_api.DescSet(p->desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bt, sizeof(bt)) == HIPBLAS_STATUS_SUCCESS;
  }
  ok = ok && g_api.LayoutCreate(&p->a, HIP_R_16BF, K, N, ldw) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && g_api.LayoutCreate(&p->b, HIP_R_16BF, K, M, ldx) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && g_api.LayoutCreate(&p->d, HIP_R_16BF, N, M, ldy) == HIPBLAS_STATUS_SUCCESS;
  if (!ok) {
    lmsf_set_error("blas: the library refused the descriptors of a product of %d rows, %d columns over %d", M, N, K);
    destroy_plan(*p);
  }
  return ok;
}

// Up to ``want`` of the library's candidates for the plan's shape, its first choice first.
int candidates(Device* d, const Plan& p, int want, std::vector<hipblasLtMatmulHeuristicResult_t>* out) {
  hipblasLtMatmulPreference_t pref = nullptr;
  if (g_api.PrefCreate(&pref) != HIPBLAS_STATUS_SUCCESS) return 0;
  const uint64_t ws = d->workspace_bytes;
  g_api.PrefSet(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof(ws));
  out->assign(want, hipblasLtMatmulHeuristicResult_t());
  int got = 0;
  const hipblasStatus_t st = g_api.Heuristic(d->handle, p.desc, p.a, p.b, p.d, p.d, pref, want, out->data(), &got);
  g_api.PrefDestroy(pref);
  if (st != HIPBLAS_STATUS_SUCCESS) got = 0;
  out->resize(got);
  out->erase(std::remove_if(out->begin(), out->end(),
                            [&](const hipblasLtMatmulHeuristicResult_t& r) {
                              return r.state != HIPBLAS_STATUS_SUCCESS || r.workspaceSize > d->workspace_bytes;
                            }),
             out->end());
  return (int)out->size();
}

Plan* find_plan(Device* d, const Key& key) {
  auto it = d->plans.find(key);
  if (it != d->plans.end()) return &it->second;
  if (d->plans.size() >= kMaxPlans) {
    for (auto i = d->plans.begin(); i != d->plans.end();) {
      if (!i->second.tuned) {
        destroy_plan(i->second);
        i = d->plans.erase(i);
      } else {
        ++i;
      }
    }
  }
  Plan p;
  if (!make_descriptors(key, &p)) return nullptr;
  std::vector<hipblasLtMatmulHeuristicResult_t> cand;
  if (candidates(d, p, 1, &cand) < 1) {
    lmsf_set_error("blas: the library has no algorithm for a product of %d rows, %d columns over %d", std::get<0>(key),
                   std::get<1>(key), std::get<2>(key));
    destroy_plan(p);
    return nullptr;
  }
  p.algo = cand[0].algo;
  p.workspace = cand[0].workspaceSize;
  return &(d->plans[key] = p);
}

int run_plan(Device* d, Plan* p, const hipblasLtMatmulAlgo_t& algo, size_t ws, const void* x, const void* W,
             const void* bias, void* y, hipStream_t stream) {
  if (bias != nullptr &&
      g_api.DescSet(p->desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias)) != HIPBLAS_STATUS_SUCCESS) {
    lmsf_set_error("blas: the library refused the bias pointer");
    return 2;
  }
  const float one = 1.f, zero = 0.f;
  const hipblasStatus_t st = g_api.Matmul(d->handle, p->desc, &one, W, p->a, x, p->b, &zero, y, p->d, y, p->d, &algo,
                                          d->workspace, ws ? d->workspace_bytes : 0, stream);
  if (st != HIPBLAS_STATUS_SUCCESS) {
    lmsf_set_error("blas: the library's product failed with status %d", (int)st);
    return 2;
  }
  return 0;
}

bool operands_ok(const void* x, long ldx, const void* W, long ldw, const void* y, long ldy, int M, int N, int K) {
  if (!(x && W && y && M > 0 && N > 0 && K > 0 && ldx >= K && ldw >= K && ldy >= N)) {
    lmsf_set_error("blas: bad operands (M %d, N %d, K %d, strides %ld, %ld, %ld)", M, N, K, ldx, ldw, ldy);
    return false;
  }
  return true;
}

}  // namespace

// Opens the library and gives the current device its handle and a workspace of ``workspace_bytes`` (kept until
// the process ends; a later call with a larger size replaces it, which must not happen while work that uses it is
// in flight or captured). Allocates: not to be called under stream capture.
extern "C" int lmsf_blas_init(long workspace_bytes) {
  std::lock_guard<std::mutex> lock(g_mutex);
  if (!load_api()) return 1;
  int dev = 0;
  LMSF_CHECK(hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < kMaxDevices, "blas: cannot tell the current device");
  Device* d = &g_devices[dev];
  if (d->handle == nullptr) {
    LMSF_CHECK(g_api.Create(&d->handle) == HIPBLAS_STATUS_SUCCESS, "blas: hipblasLtCreate failed");
  }
  if (workspace_bytes > 0 && (size_t)workspace_bytes > d->workspace_bytes) {
    void* ws = nullptr;
    LMSF_CHECK(hipMalloc(&ws, (size_t)workspace_bytes) == hipSuccess, "blas: no memory for a workspace of %ld bytes",
               workspace_bytes);
    if (d->workspace) (void)hipFree(d->workspace);
    d->workspace = ws;
    d->workspace_bytes = (size_t)workspace_bytes;
  }
  return 0;
}

// 1 once lmsf_blas_init has succeeded on the current device.
extern "C" int lmsf_blas_ready() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
  return g_devices[dev].handle != nullptr ? 1 : 0;
}

// y [M, N] = x [M, K] W^T (+ bias), all bfloat16, sums in float32; W [N, K]; ldx, ldw, ldy are the distances
// between rows in elements. The shape's plan is made at its first call and kept.
extern "C" int lmsf_blas_linear(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, long ldy,
                                int M, int N, int K, hipStream_t stream) {
  if (!operands_ok(x, ldx, W, ldw, y, ldy, M, N, K)) return 1;
  std::lock_guard<std::mutex> lock(g_mutex);
  Device* d = current_device();
  if (d == nullptr) return 1;
  Plan* p = find_plan(d, Key(M, N, K, ldx, ldw, ldy, bias != nullptr));
  if (p == nullptr) return 1;
  return run_plan(d, p, p->algo, p->workspace, x, W, bias, y, stream);
}

// Times up to ``n_candidates`` of the library's algorithms for the shape on the given operands and keeps the
// fastest for later calls of lmsf_blas_linear with that shape. ``Ws`` holds ``n_weights`` matrices of the shape
// (the same product of several layers): the runs go round them, so that no run finds its weights in the caches
// the one before it filled. Each candidate runs once untimed and ``reps`` times timed; its time is the median.
// ``times_us`` (may be null) takes [the first choice's, the fastest's]. Synchronises the stream; not under
// capture. Returns 0, or non-zero with the reason.
extern "C" int lmsf_blas_tune(const void* x, long ldx, const void* const* Ws, int n_weights, long ldw,
                              const void* bias, void* y, long ldy, int M, int N, int K, int n_candidates, int reps,
                              float* times_us, hipStream_t stream) {
  LMSF_CHECK(Ws != nullptr && n_weights > 0 && n_candidates > 0 && reps > 0, "blas_tune: bad arguments");
  if (!operands_ok(x, ldx, Ws[0], ldw, y, ldy, M, N, K)) return 1;
  std::lock_guard<std::mutex> lock(g_mutex);
  Device* d = current_device();
  if (d == nullptr) return 1;
  const Key key(M, N, K, ldx, ldw, ldy, bias != nullptr);
  Plan* p = find_plan(d, key);
  if (p == nullptr) return 1;
  std::vector<hipblasLtMatmulHeuristicResult_t> cand;
  if (candidates(d, *p, n_candidates, &cand) < 1) return 0;   // nothing to choose from: the plan stays
  hipEvent_t e0, e1;
  LMSF_CHECK(hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess, "blas_tune: no events");
  int turn = 0, rc = 0;
  float best = -1.f, first = -1.f;
  size_t best_at = 0;
  for (size_t c = 0; c < cand.size() && rc == 0; ++c) {
    std::vector<float> ms;
    for (int r = 0; r <= reps && rc == 0; ++r) {
      const void* W = Ws[turn++ % n_weights];
      if (r > 0) (void)hipEventRecord(e0, stream);
      rc = run_plan(d, p, cand[c].algo, cand[c].workspaceSize, x, W, bias, y, stream);
      if (rc != 0) break;
      if (r > 0) {
        (void)hipEventRecord(e1, stream);
        if (hipEventSynchronize(e1) != hipSuccess) {
          lmsf_set_error("blas_tune: a candidate failed on the device");
          rc = 2;
          break;
        }
        float t = 0.f;
        (void)hipEventElapsedTime(&t, e0, e1);
        ms.push_back(t);
      }
    }
    if (rc != 0) {
      // a candidate that the library offers and then refuses to run is skipped, not an error
      if (c > 0) rc = 0;
      continue;
    }
    std::sort(ms.begin(), ms.end());
    const float med = ms[ms.size() / 2];
    if (c == 0) first = med;
    if (best < 0.f || med < best) {
      best = med;
      best_at = c;
    }
  }
  (void)hipStreamSynchronize(stream);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (rc != 0) return rc;
  if (best >= 0.f) {
    p->algo = cand[best_at].algo;
    p->workspace = cand[best_at].workspaceSize;
    p->tuned = true;
  }
  if (times_us) {
    times_us[0] = first * 1e3f;
    times_us[1] = best * 1e3f;
  }
  return 0;
}

// Plans kept for the current device (for tests and logs).
extern "C" long lmsf_blas_plans() {
  std::lock_guard<std::mutex> lock(g_mutex);
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
  return (long)g_devices[dev].plans.size();
}
