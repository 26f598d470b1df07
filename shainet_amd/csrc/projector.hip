// Row-major projections on the device and small upload helpers.  rocBLAS and
// hipBLASLt are opened with dlopen on first use so that the library does not depend
// on them for decode, where the hand-written GEMV runs.
#include <dlfcn.h>
#include <hipblaslt/hipblaslt.h>

#include <cstdlib>
#include <cstring>
#include <array>
#include <map>
#include <mutex>
#include <vector>

#include "../../include/shainet_hip_attn.h"
#include "attn_kernels.hpp"
#include "block_kernels.hpp"
#include "llama_internal.hpp"

void shainet_hip_set_error(int code, const char *msg);  // capi.hip

namespace shainet {

namespace {

typedef void *rb_handle;
typedef int (*rb_create_t)(rb_handle *);
typedef int (*rb_destroy_t)(rb_handle);
typedef int (*rb_set_stream_t)(rb_handle, hipStream_t);
typedef int (*rb_sgemm_t)(rb_handle, int, int, int, int, int, const float *, const float *, int, const float *, int,
                          const float *, float *, int);
constexpr int kRocblasOpNone = 111;

struct RocBlas {
  void *lib = nullptr;
  rb_create_t create = nullptr;
  rb_destroy_t destroy = nullptr;
  rb_set_stream_t set_stream = nullptr;
  rb_sgemm_t sgemm = nullptr;
  bool tried = false;
  std::mutex once;  // contexts on different threads may come here at the same time
  bool load() {
    std::lock_guard<std::mutex> guard(once);
    if (tried) return sgemm != nullptr;
    tried = true;
    for (const char *name : {"librocblas.so.5", "librocblas.so"}) {
      lib = dlopen(name, RTLD_LAZY | RTLD_LOCAL);
      if (lib) break;
    }
    if (!lib) return false;
    create = (rb_create_t)dlsym(lib, "rocblas_create_handle");
    destroy = (rb_destroy_t)dlsym(lib, "rocblas_destroy_handle");
    set_stream = (rb_set_stream_t)dlsym(lib, "rocblas_set_stream");
    sgemm = (rb_sgemm_t)dlsym(lib, "rocblas_sgemm");
    if (!create || !destroy || !set_stream || !sgemm) sgemm = nullptr;
    return sgemm != nullptr;
  }
};
RocBlas g_rocblas;

// hipBLASLt entry points, resolved by name
struct HipBlasLt {
  void *lib = nullptr;
  decltype(&hipblasLtCreate) create = nullptr;
  decltype(&hipblasLtDestroy) destroy = nullptr;
  decltype(&hipblasLtMatrixLayoutCreate) layout_create = nullptr;
  decltype(&hipblasLtMatrixLayoutDestroy) layout_destroy = nullptr;
  decltype(&hipblasLtMatmulDescCreate) desc_create = nullptr;
  decltype(&hipblasLtMatmulDescDestroy) desc_destroy = nullptr;
  decltype(&hipblasLtMatmulPreferenceCreate) pref_create = nullptr;
  decltype(&hipblasLtMatmulPreferenceDestroy) pref_destroy = nullptr;
  decltype(&hipblasLtMatmulPreferenceSetAttribute) pref_set = nullptr;
  decltype(&hipblasLtMatmulAlgoGetHeuristic) heuristic = nullptr;
  decltype(&hipblasLtMatmul) matmul = nullptr;
  bool tried = false, ok = false;
  std::mutex once;
  bool load() {
    std::lock_guard<std::mutex> guard(once);
    if (tried) return ok;
    tried = true;
    for (const char *name : {"libhipblaslt.so.1", "libhipblaslt.so"}) {
      lib = dlopen(name, RTLD_LAZY | RTLD_LOCAL);
      if (lib) break;
    }
    if (!lib) return false;
#define SHAINET_LT_SYM(field, sym) field = (decltype(field))dlsym(lib, #sym)
    SHAINET_LT_SYM(create, hipblasLtCreate);
    SHAINET_LT_SYM(destroy, hipblasLtDestroy);
    SHAINET_LT_SYM(layout_create, hipblasLtMatrixLayoutCreate);
    SHAINET_LT_SYM(layout_destroy, hipblasLtMatrixLayoutDestroy);
    SHAINET_LT_SYM(desc_create, hipblasLtMatmulDescCreate);
    SHAINET_LT_SYM(desc_destroy, hipblasLtMatmulDescDestroy);
    SHAINET_LT_SYM(pref_create, hipblasLtMatmulPreferenceCreate);
    SHAINET_LT_SYM(pref_destroy, hipblasLtMatmulPreferenceDestroy);
    SHAINET_LT_SYM(pref_set, hipblasLtMatmulPreferenceSetAttribute);
    SHAINET_LT_SYM(heuristic, hipblasLtMatmulAlgoGetHeuristic);
    SHAINET_LT_SYM(matmul, hipblasLtMatmul);
#undef SHAINET_LT_SYM
    ok = create && destroy && layout_create && layout_destroy && desc_create && desc_destroy && pref_create &&
         pref_destroy && pref_set && heuristic && matmul;
    return ok;
  }
};
HipBlasLt g_lt;

constexpr size_t kLtMaxWorkspace = 32u << 20;

// 0: choose by shape, 1: rocBLAS, 2: hipBLASLt (SHAINET_HIP_GEMM=rocblas|hipblaslt)
int gemm_backend_override() {
  static const int v = [] {
    const char *e = getenv("SHAINET_HIP_GEMM");
    if (e && !strcmp(e, "rocblas")) return 1;
    if (e && !strcmp(e, "hipblaslt")) return 2;
    return 0;
  }();
  return v;
}

}  // namespace

// One problem shape of the hipBLASLt path: its layouts and the algorithm the
// library's heuristic picked for it.
struct LtShape {
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
  bool usable = false;
};
struct LtState {
  hipblasLtHandle_t handle = nullptr;
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatmulPreference_t pref = nullptr;
  void *workspace = nullptr;
  size_t workspace_cap = 0;
  std::map<std::array<long long, 4>, LtShape> shapes;  // (T, K, N, stride of x)
  void drop_shapes() {
    for (auto &kv : shapes) {
      if (kv.second.a) g_lt.layout_destroy(kv.second.a);
      if (kv.second.b) g_lt.layout_destroy(kv.second.b);
      if (kv.second.c) g_lt.layout_destroy(kv.second.c);
    }
    shapes.clear();
  }
};

int llama_fail(int code, const std::string &msg) {
  shainet_hip_set_error(code, msg.c_str());
  return code;
}

bool DevF::reserve(size_t n) {
  if (n <= cap) return true;
  size_t want = cap ? cap : 1024;
  while (want < n) want *= 2;
  float *np = nullptr;
  if (hipMalloc((void **)&np, want * sizeof(float)) != hipSuccess) {
    (void)hipGetLastError();
    if (hipMalloc((void **)&np, n * sizeof(float)) != hipSuccess) return false;
    want = n;
  }
  if (p) (void)hipFree(p);
  p = np;
  cap = want;
  return true;
}

void DevF::release() {
  if (p) (void)hipFree(p);
  p = nullptr;
  cap = 0;
}

// 1 = done, 0 = not available for this shape (the caller falls back to rocBLAS), < 0 = -status
int Projector::gemm_lt(const float *x, long long x_stride, const float *w, float *y, int T, int K, int N,
                       hipStream_t stream, const float *res) {
  if (!g_lt.load()) return 0;
  if (!lt) {
    LtState *s = new LtState();
    const hipblasOperation_t op = HIPBLAS_OP_N;
    (void)op;
    bool ok = g_lt.create(&s->handle) == HIPBLAS_STATUS_SUCCESS &&
              g_lt.desc_create(&s->desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS &&
              g_lt.pref_create(&s->pref) == HIPBLAS_STATUS_SUCCESS;
    if (ok) {
      const uint64_t ws = kLtMaxWorkspace;
      ok = g_lt.pref_set(s->pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof(ws)) == HIPBLAS_STATUS_SUCCESS;
    }
    lt = s;
    if (!ok) {
      lt_broken = true;
      return 0;
    }
  }
  if (lt_broken) return 0;
  const std::array<long long, 4> key = {T, K, N, x_stride};
  if (lt->shapes.size() > 512) lt->drop_shapes();
  auto it = lt->shapes.find(key);
  if (it == lt->shapes.end()) {
    LtShape sh;
    // row-major y = x W  <=>  column-major y^T[N,T] = W^T[N,K] x^T[K,T]
    bool ok = g_lt.layout_create(&sh.a, HIP_R_32F, N, K, N) == HIPBLAS_STATUS_SUCCESS &&
              g_lt.layout_create(&sh.b, HIP_R_32F, K, T, x_stride) == HIPBLAS_STATUS_SUCCESS &&
              g_lt.layout_create(&sh.c, HIP_R_32F, N, T, N) == HIPBLAS_STATUS_SUCCESS;
    if (ok) {
      hipblasLtMatmulHeuristicResult_t res[1];
      int found = 0;
      ok = g_lt.heuristic(lt->handle, lt->desc, sh.a, sh.b, sh.c, sh.c, lt->pref, 1, res, &found) ==
               HIPBLAS_STATUS_SUCCESS &&
           found > 0 && res[0].state == HIPBLAS_STATUS_SUCCESS && res[0].workspaceSize <= kLtMaxWorkspace;
      if (ok) {
        sh.algo = res[0].algo;
        sh.workspace = res[0].workspaceSize;
      }
    }
    sh.usable = ok;
    it = lt->shapes.emplace(key, sh).first;
  }
  const LtShape &sh = it->second;
  if (!sh.usable) return 0;
  if (sh.workspace > lt->workspace_cap) {
    void *np = nullptr;
    if (hipMalloc(&np, sh.workspace) != hipSuccess) {
      (void)hipGetLastError();
      return 0;
    }
    if (lt->workspace) (void)hipFree(lt->workspace);  // hipFree waits for the device
    lt->workspace = np;
    lt->workspace_cap = sh.workspace;
  }
  // res: y = res + x W in the library's epilogue (D = A B + C): one fp32 add per element, as in
  // the separate add kernel
  const float one = 1.0f, zero = 0.0f;
  const hipblasStatus_t st = g_lt.matmul(lt->handle, lt->desc, &one, w, sh.a, x, sh.b, res ? &one : &zero,
                                         res ? res : y, sh.c, y, sh.c, &sh.algo, lt->workspace, sh.workspace, stream);
  return st == HIPBLAS_STATUS_SUCCESS ? 1 : -(int)st;
}

// hipBLASLt where its kernels are the faster ones on this device: many rows, or a large
// weight matrix (rocBLAS picks slow kernels for long K with few rows)
static bool wants_lt(int T, int K, int N) {
  const int force = gemm_backend_override();
  return force == 2 || (force == 0 && (T >= 256 || (long long)K * N > (8ll << 20)));
}

int Projector::gemm(const float *x, long long x_stride, const float *w, float *y, int T, int K, int N,
                    hipStream_t stream) {
  const int force = gemm_backend_override();
  const bool want_lt = wants_lt(T, K, N);
  if (want_lt) {
    const int r = gemm_lt(x, x_stride, w, y, T, K, N, stream);
    if (r == 1) return SHAINET_HIP_OK;
    if (r < 0) return llama_fail(SHAINET_HIP_ERR_RUNTIME, "hipblasLtMatmul failed with status " + std::to_string(-r));
    if (force == 2)
      return llama_fail(SHAINET_HIP_ERR_RUNTIME, "hipBLASLt is not available for this projection GEMM");
  }
  if (!g_rocblas.load())
    return llama_fail(SHAINET_HIP_ERR_RUNTIME, "librocblas.so.5 could not be opened for a projection GEMM");
  if (!blas && g_rocblas.create(&blas) != 0)
    return llama_fail(SHAINET_HIP_ERR_RUNTIME, "rocblas_create_handle failed");
  if (g_rocblas.set_stream(blas, stream) != 0) return llama_fail(SHAINET_HIP_ERR_RUNTIME, "rocblas_set_stream failed");
  // row-major y = x W  <=>  column-major y^T[N,T] = W^T[N,K] x^T[K,T]
  const float one = 1.0f, zero = 0.0f;
  const int st = g_rocblas.sgemm(blas, kRocblasOpNone, kRocblasOpNone, N, T, K, &one, w, N, x, (int)x_stride, &zero, y, N);
  if (st != 0) return llama_fail(SHAINET_HIP_ERR_RUNTIME, "rocblas_sgemm failed with status " + std::to_string(st));
  return SHAINET_HIP_OK;
}

int Projector::project(const float *x, long long x_stride, const float *w, float *y, int T, int K, int N,
                       hipStream_t stream, const Fused &f) {
  const bool swiglu = f.epilogue == kGemvSwiglu;
  if (f.epilogue == kGemvQkvPrep && (!f.prep || T > 16 || (N & 3)))
    return llama_fail(SHAINET_HIP_ERR_ARGUMENT, "the fused q | k | v epilogue takes at most 16 rows");
  if (T <= 16 && (N & 3) == 0) {
    const float *xin = x;
    long long xs = x_stride;
    bool norm = f.norm;
    if (norm && T > 4) {  // every workgroup would redo the sums of squares of all rows: norm them once instead
      if (!normed.reserve((size_t)T * K)) return llama_fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
      hipError_t e = launch_rmsnorm(x, x_stride, f.gamma, normed.p, T, K, f.eps, stream);
      if (e != hipSuccess) return llama_fail(SHAINET_HIP_ERR_RUNTIME, std::string("rmsnorm launch: ") + hipGetErrorString(e));
      xin = normed.p;
      xs = K;
      norm = false;
    }
    const GemvPlan p = plan_gemv(T, K, N, f.epilogue, f.prep ? f.prep->hd : 0);
    if (!scratch.reserve(p.partial_floats)) return llama_fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
    const size_t n_flags = (size_t)p.col_tiles * p.splits;
    if (p.splits > 1 && n_flags > flags_cap) {
      size_t want = flags_cap ? flags_cap : 4096;
      while (want < n_flags) want *= 2;
      unsigned *np = nullptr;
      if (hipMalloc((void **)&np, want * sizeof(unsigned)) != hipSuccess) return llama_fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
      if (hipMemsetAsync(np, 0, want * sizeof(unsigned), stream) != hipSuccess) {
        (void)hipFree(np);
        return llama_fail(SHAINET_HIP_ERR_RUNTIME, "hipMemsetAsync(flags) failed");
      }
      if (flags) (void)hipFree(flags);  // hipFree waits for the device
      flags = np;
      flags_cap = want;
    }
    if (p.splits > 1 && !error) return llama_fail(SHAINET_HIP_ERR_RUNTIME, "the projector has no error word");
    GemvArgs a = {};
    a.x = xin;
    a.x_stride = xs;
    a.norm = norm ? 1 : 0;
    a.gamma = f.gamma;
    a.eps = f.eps;
    a.w = w;
    a.res = f.res;
    a.y = y;
    a.partials = scratch.p;
    a.flags = flags;
    a.error = error;
    a.T = T;
    a.K = K;
    a.N = N;
    a.epilogue = f.epilogue;
    if (f.prep) a.prep = *f.prep;
    hipError_t e = launch_gemv(a, p, stream);
    if (e != hipSuccess)
      return llama_fail(SHAINET_HIP_ERR_RUNTIME, std::string("gemv launch: ") + hipGetErrorString(e));
    return SHAINET_HIP_OK;
  }
  // many rows: norm kernel, library GEMM, epilogue kernel
  const float *xin = x;
  long long xs = x_stride;
  hipError_t e = hipSuccess;
  if (f.norm) {
    if (!normed.reserve((size_t)T * K)) return llama_fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
    e = launch_rmsnorm(x, x_stride, f.gamma, normed.p, T, K, f.eps, stream);
    if (e != hipSuccess) return llama_fail(SHAINET_HIP_ERR_RUNTIME, std::string("rmsnorm launch: ") + hipGetErrorString(e));
    xin = normed.p;
    xs = K;
  }
  if (swiglu) {
    if (!wide.reserve((size_t)T * 2 * N)) return llama_fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
    int rc = gemm(xin, xs, w, wide.p, T, K, 2 * N, stream);
    if (rc) return rc;
    e = launch_swiglu_act(wide.p, y, T, N, stream);
  } else if (f.epilogue == kGemvResidual) {
    if (f.res != y && wants_lt(T, K, N)) {  // the library adds the residual in its epilogue
      const int r = gemm_lt(xin, xs, w, y, T, K, N, stream, f.res);
      if (r == 1) return SHAINET_HIP_OK;
      if (r < 0) return llama_fail(SHAINET_HIP_ERR_RUNTIME, "hipblasLtMatmul failed with status " + std::to_string(-r));
    }
    if (!wide.reserve((size_t)T * N)) return llama_fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
    int rc = gemm(xin, xs, w, wide.p, T, K, N, stream);
    if (rc) return rc;
    e = launch_add(f.res, wide.p, y, (long long)T * N, stream);
  } else {
    return gemm(xin, xs, w, y, T, K, N, stream);
  }
  if (e != hipSuccess) return llama_fail(SHAINET_HIP_ERR_RUNTIME, std::string("epilogue launch: ") + hipGetErrorString(e));
  return SHAINET_HIP_OK;
}

void Projector::release() {
  if (blas && g_rocblas.destroy) g_rocblas.destroy(blas);
  blas = nullptr;
  if (lt) {
    lt->drop_shapes();
    if (lt->pref) g_lt.pref_destroy(lt->pref);
    if (lt->desc) g_lt.desc_destroy(lt->desc);
    if (lt->handle) g_lt.destroy(lt->handle);
    if (lt->workspace) (void)hipFree(lt->workspace);
    delete lt;
    lt = nullptr;
  }
  lt_broken = false;
  scratch.release();
  normed.release();
  wide.release();
  if (flags) (void)hipFree(flags);
  flags = nullptr;
  flags_cap = 0;
}

int upload_floats(float **dst, const float *src, size_t n) {
  if (*dst) (void)hipFree(*dst);
  *dst = nullptr;
  if (hipMalloc((void **)dst, n * sizeof(float)) != hipSuccess) return llama_fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
  if (hipMemcpy(*dst, src, n * sizeof(float), hipMemcpyHostToDevice) != hipSuccess)
    return llama_fail(SHAINET_HIP_ERR_RUNTIME, "hipMemcpy of a weight matrix failed");
  return SHAINET_HIP_OK;
}

int upload_side_by_side(float **dst, const float *const *mats, const int *widths, int count, int rows) {
  if (*dst) (void)hipFree(*dst);
  *dst = nullptr;
  size_t total = 0;
  for (int i = 0; i < count; ++i) total += (size_t)widths[i];
  if (hipMalloc((void **)dst, (size_t)rows * total * sizeof(float)) != hipSuccess)
    return llama_fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
  const size_t pitch = total * sizeof(float);
  size_t off = 0;
  for (int i = 0; i < count; ++i) {
    const size_t wb = (size_t)widths[i] * sizeof(float);
    if (hipMemcpy2D(*dst + off, pitch, mats[i], wb, wb, rows, hipMemcpyHostToDevice) != hipSuccess)
      return llama_fail(SHAINET_HIP_ERR_RUNTIME, "hipMemcpy2D of a weight matrix failed");
    off += (size_t)widths[i];
  }
  return SHAINET_HIP_OK;
}

}  // namespace shainet
