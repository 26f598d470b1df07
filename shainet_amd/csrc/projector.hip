// Row-major projections on the device and small upload helpers.  rocBLAS is
// opened with dlopen on first use so that the library does not depend on it for
// decode, where the hand-written GEMV runs.
#include <dlfcn.h>

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
  bool load() {
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

}  // namespace

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

int Projector::gemm(const float *x, long long x_stride, const float *w, float *y, int T, int K, int N,
                    hipStream_t stream) {
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
    const GemvPlan p = plan_gemv(T, K, N, f.epilogue);
    if (!scratch.reserve(p.partial_floats)) return llama_fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
    if ((size_t)p.col_tiles > counters_cap) {
      size_t want = counters_cap ? counters_cap : 1024;
      while (want < (size_t)p.col_tiles) want *= 2;
      int *np = nullptr;
      if (hipMalloc((void **)&np, want * sizeof(int)) != hipSuccess) return llama_fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
      if (hipMemsetAsync(np, 0, want * sizeof(int), stream) != hipSuccess) {
        (void)hipFree(np);
        return llama_fail(SHAINET_HIP_ERR_RUNTIME, "hipMemsetAsync(counters) failed");
      }
      if (counters) (void)hipFree(counters);  // hipFree waits for the device
      counters = np;
      counters_cap = want;
    }
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
    a.counters = counters;
    a.T = T;
    a.K = K;
    a.N = N;
    a.epilogue = f.epilogue;
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
  scratch.release();
  normed.release();
  wide.release();
  if (counters) (void)hipFree(counters);
  counters = nullptr;
  counters_cap = 0;
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
