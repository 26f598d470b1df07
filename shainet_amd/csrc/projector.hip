// Row-major projections on the device and small upload helpers.
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <vector>

#include "../../include/shainet_hip_attn.h"
#include "attn_kernels.hpp"
#include "block_kernels.hpp"
#include "gemm_kernel.hpp"
#include "llama_internal.hpp"

void shainet_hip_set_error(int code, const char *msg);  // capi.hip

namespace shainet {

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

bool PinnedF::reserve(size_t n) {
  if (n <= cap) return true;
  size_t want = cap ? cap : 4096;
  while (want < n) want *= 2;
  float *np = nullptr;
  if (hipHostMalloc((void **)&np, want * sizeof(float), hipHostMallocDefault) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  if (p) (void)hipHostFree(p);
  p = np;
  cap = want;
  return true;
}

void PinnedF::release() {
  if (p) (void)hipHostFree(p);
  p = nullptr;
  cap = 0;
}

void DevF::release() {
  if (p) (void)hipFree(p);
  p = nullptr;
  cap = 0;
}

// SHAINET_HIP_NO_TRANSPOSED_WEIGHTS: no second, transposed copy of q | k | v, W_o, gate | up and down (the
// products of a single row then run as the split GEMV over the [in, out] matrices, like the rest)
bool transposed_twins_wanted() {
  static const bool wanted = getenv("SHAINET_HIP_NO_TRANSPOSED_WEIGHTS") == nullptr;
  return wanted;
}

// *twin = src transposed (src: [rows, cols] on the device), allocated on first use.  Returns the
// twin, or null when there is no memory for it (the caller then goes without).
const float *transposed_twin(float **twin, bool *stale, const float *src, int rows, int cols, hipStream_t stream,
                             const float *row_scale) {
  if (!transposed_twins_wanted() || !src) return nullptr;
  if (!*twin) {
    if (hipMalloc((void **)twin, (size_t)rows * cols * sizeof(float)) != hipSuccess) {
      (void)hipGetLastError();
      *twin = nullptr;
      return nullptr;
    }
    *stale = true;
  }
  if (*stale) {
    // (waited for, once per set of weights: the copy may next be read on another stream)
    if (launch_transpose(src, *twin, rows, cols, stream, row_scale) != hipSuccess || hipStreamSynchronize(stream) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    *stale = false;
  }
  return *twin;
}

// The flag words are shared by all kernels of this projector: each leaves them zero, and the
// launches of one projector follow each other on one stream.
int Projector::reserve_flags(size_t n_flags, hipStream_t stream) {
  if (n_flags <= flags_cap) return SHAINET_HIP_OK;
  if (!flags) lose_marks = getenv("SHAINET_HIP_TEST_LOSE_PARTIAL_MARKS") != nullptr;
  size_t want = flags_cap ? flags_cap : 4096;
  while (want < n_flags) want *= 2;
  unsigned *np = nullptr;
  // (twice the words: the second half is where the marks go in the test of the give-up path)
  if (hipMalloc((void **)&np, 2 * want * sizeof(unsigned)) != hipSuccess) return llama_fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
  if (hipMemsetAsync(np, 0, 2 * want * sizeof(unsigned), stream) != hipSuccess) {
    (void)hipFree(np);
    return llama_fail(SHAINET_HIP_ERR_RUNTIME, "hipMemsetAsync(flags) failed");
  }
  if (flags) (void)hipFree(flags);  // hipFree waits for the device
  flags = np;
  flags_cap = want;
  return SHAINET_HIP_OK;
}

// y = (res +) x W with the library's own MFMA kernel; res == y is allowed.
int Projector::gemm(const float *x, long long x_stride, const float *w, float *y, int T, int K, int N,
                    hipStream_t stream, const float *res) {
  const GemmPlan p = plan_gemm(T, K, N, x_stride);
  if (!scratch.reserve(p.partial_floats)) return llama_fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
  if (int rc = reserve_flags(p.flag_words, stream)) return rc;
  if (p.flag_words && !error) return llama_fail(SHAINET_HIP_ERR_RUNTIME, "the projector has no error word");
  hipError_t e = launch_gemm(x, x_stride, w, y, res, scratch.p, flags, error, T, K, N, p, stream,
                             lose_marks ? flags + flags_cap : nullptr, lose_marks ? 2000 : 0);
  if (e != hipSuccess) return llama_fail(SHAINET_HIP_ERR_RUNTIME, std::string("gemm launch: ") + hipGetErrorString(e));
  return SHAINET_HIP_OK;
}

int Projector::project(const float *x, long long x_stride, const float *w, float *y, int T, int K, int N,
                       hipStream_t stream, const Fused &f) {
  const bool swiglu = f.epilogue == kGemvSwiglu;
  if (f.epilogue == kGemvQkvPrep && (!f.prep || T > 16 || (N & 3)))
    return llama_fail(SHAINET_HIP_ERR_ARGUMENT, "the fused q | k | v epilogue takes at most 16 rows");
  if (f.w_t && gemvt_takes(T, K, N, f.epilogue, f.norm, f.prep) && !(((uintptr_t)x | (uintptr_t)f.gamma) & 15)) {
    GemvArgs a = {};
    a.x = x;
    a.x_stride = x_stride;
    a.norm = f.norm ? 1 : 0;
    a.gamma = f.w_t_has_gamma ? nullptr : f.gamma;
    a.eps = f.eps;
    a.w = f.w_t;
    a.res = f.res;
    a.y = y;
    a.T = T;
    a.K = K;
    a.N = N;
    a.epilogue = f.epilogue;
    if (f.prep) a.prep = *f.prep;
    hipError_t e = launch_gemvt(a, stream);
    if (e != hipSuccess)
      return llama_fail(SHAINET_HIP_ERR_RUNTIME, std::string("gemv launch: ") + hipGetErrorString(e));
    return SHAINET_HIP_OK;
  }
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
    if (p.splits > 1)
      if (int rc = reserve_flags((size_t)p.col_tiles * p.splits, stream)) return rc;
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
    a.flag_set = lose_marks ? flags + flags_cap : nullptr;
    a.spin_limit = lose_marks ? 2000 : 0;
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
  // many rows: norm kernel, MFMA product (the residual rides in its epilogue), activation kernel
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
    if (e != hipSuccess) return llama_fail(SHAINET_HIP_ERR_RUNTIME, std::string("epilogue launch: ") + hipGetErrorString(e));
    return SHAINET_HIP_OK;
  }
  return gemm(xin, xs, w, y, T, K, N, stream, f.epilogue == kGemvResidual ? f.res : nullptr);
}

void Projector::release() {
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

// ---- the product by itself ---------------------------------------------------------------
namespace {
std::mutex g_matmul_lock;
// Grow-only scratch of the handle-less calls (partial products of split shapes, their flag words, the
// error word their kernels report into), one set per stream: calls on different streams may overlap
// on the device and must not share partial products.  Never freed, like the reference's class-level scratch.
std::map<hipStream_t, shainet::Projector> g_matmul;
}  // namespace

extern "C" int shainet_hip_matmul_f32(const float *x, long long x_stride, const float *w, const float *res, float *y,
                                      int rows, int k, int n, void *stream) {
  using namespace shainet;
  if (!x || !w || !y || rows < 1 || k < 1 || n < 1 || x_stride < k)
    return llama_fail(SHAINET_HIP_ERR_ARGUMENT, "invalid matmul arguments");
  if (!shainet_hip_available()) return llama_fail(SHAINET_HIP_ERR_RUNTIME, "no gfx950 device available");
  std::lock_guard<std::mutex> guard(g_matmul_lock);
  Projector &p = g_matmul[(hipStream_t)stream];
  if (!p.error) p.error = alloc_error_word();
  // what a kernel of an earlier call on this stream reported (a given-up wait for partial sums)
  // is said by the next call, which does nothing else then
  if (int rc = check_error_word(p.error)) return rc;
  Fused f;
  if (res) {
    f.epilogue = kGemvResidual;
    f.res = res;
  }
  return p.project(x, x_stride, w, y, rows, k, n, (hipStream_t)stream, f);
}
