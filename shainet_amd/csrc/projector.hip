// Row-major projections on the device and small upload helpers.  rocBLAS is
// opened with dlopen on first use so that the library does not depend on it for
// decode, where the hand-written GEMV runs.
#include <dlfcn.h>

#include <vector>

#include "../../include/shainet_hip_attn.h"
#include "attn_kernels.hpp"
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

int Projector::project(const float *x, const float *w, float *y, int T, int K, int N, hipStream_t stream) {
  if (T <= 16 && (N & 3) == 0) {
    const GemvPlan p = plan_gemv(T, K, N);
    if (!scratch.reserve(p.partial_floats)) return llama_fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
    hipError_t e = launch_gemv(x, w, y, scratch.p, T, K, N, p, stream);
    if (e != hipSuccess)
      return llama_fail(SHAINET_HIP_ERR_RUNTIME, std::string("gemv launch: ") + hipGetErrorString(e));
    return SHAINET_HIP_OK;
  }
  if (!g_rocblas.load())
    return llama_fail(SHAINET_HIP_ERR_RUNTIME, "librocblas.so.5 could not be opened for a projection GEMM");
  if (!blas && g_rocblas.create(&blas) != 0)
    return llama_fail(SHAINET_HIP_ERR_RUNTIME, "rocblas_create_handle failed");
  if (g_rocblas.set_stream(blas, stream) != 0) return llama_fail(SHAINET_HIP_ERR_RUNTIME, "rocblas_set_stream failed");
  // row-major y = x W  <=>  column-major y^T[N,T] = W^T[N,K] x^T[K,T]
  const float one = 1.0f, zero = 0.0f;
  const int st = g_rocblas.sgemm(blas, kRocblasOpNone, kRocblasOpNone, N, T, K, &one, w, N, x, K, &zero, y, N);
  if (st != 0) return llama_fail(SHAINET_HIP_ERR_RUNTIME, "rocblas_sgemm failed with status " + std::to_string(st));
  return SHAINET_HIP_OK;
}

void Projector::release() {
  if (blas && g_rocblas.destroy) g_rocblas.destroy(blas);
  blas = nullptr;
  scratch.release();
}

int upload_floats(float **dst, const float *src, size_t n) {
  if (*dst) (void)hipFree(*dst);
  *dst = nullptr;
  if (hipMalloc((void **)dst, n * sizeof(float)) != hipSuccess) return llama_fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
  if (hipMemcpy(*dst, src, n * sizeof(float), hipMemcpyHostToDevice) != hipSuccess)
    return llama_fail(SHAINET_HIP_ERR_RUNTIME, "hipMemcpy of a weight matrix failed");
  return SHAINET_HIP_OK;
}

int upload_side_by_side(float **dst, const float *a, int n_a, const float *b, int n_b, int rows) {
  if (*dst) (void)hipFree(*dst);
  *dst = nullptr;
  const size_t n = (size_t)rows * (n_a + n_b);
  if (hipMalloc((void **)dst, n * sizeof(float)) != hipSuccess) return llama_fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
  const size_t pitch = (size_t)(n_a + n_b) * sizeof(float);
  if (hipMemcpy2D(*dst, pitch, a, (size_t)n_a * sizeof(float), (size_t)n_a * sizeof(float), rows,
                  hipMemcpyHostToDevice) != hipSuccess ||
      hipMemcpy2D(*dst + n_a, pitch, b, (size_t)n_b * sizeof(float), (size_t)n_b * sizeof(float), rows,
                  hipMemcpyHostToDevice) != hipSuccess)
    return llama_fail(SHAINET_HIP_ERR_RUNTIME, "hipMemcpy2D of a weight matrix failed");
  return SHAINET_HIP_OK;
}

}  // namespace shainet
