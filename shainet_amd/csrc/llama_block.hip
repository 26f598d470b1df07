// Host mirror of the attention half of SHAInet's LlamaBlock
// (src/shainet/transformer/llama_block.cr): the state the reference keeps per
// block (weights in [in, out] layout, optional biases, QK-norm weights, RoPE
// parameters, the KV cache and @cache_len) and attention_cached_cpu (246-299)
// with every step on the device: Q/K/V projections, bias, QK-norm, RoPE,
// append, causal GQA attention, output projection.  Activations stay in HBM
// between the steps; only x comes in and the [T, d_model] result goes out.
//
// Projections: a hand-written split GEMV for up to 16 rows (decode), rocBLAS
// SGEMM (the counterpart of the reference's cuBLAS SGEMM, cuda.cr:237-247) for
// more.  rocBLAS is opened with dlopen on first use so that the library does not
// depend on it for decode.
#include <dlfcn.h>
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdio.h>
#include <string.h>

#include <new>
#include <string>
#include <vector>

#include "../../include/shainet_hip_attn.h"
#include "attn_kernels.hpp"

using namespace shainet;

void shainet_hip_set_error(int code, const char *msg);  // capi.hip

namespace {

// ---- rocBLAS through dlopen -------------------------------------------------
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

struct DevF {
  float *p = nullptr;
  size_t cap = 0;
  bool reserve(size_t n) {
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
  void release() {
    if (p) (void)hipFree(p);
    p = nullptr;
    cap = 0;
  }
};

int fail(int code, const std::string &msg) {
  shainet_hip_set_error(code, msg.c_str());
  return code;
}

}  // namespace

struct shainet_llama_attn {
  // llama_block.cr:10-28
  int d_model, num_heads, num_kv_heads, head_dim, q_dim, kv_dim;
  double qk_norm_eps, rope_theta;
  std::vector<float> rope_freqs, q_norm, k_norm, b_q, b_k, b_v;
  bool has_rope_freqs = false, has_q_norm = false, has_k_norm = false, has_bq = false, has_bk = false, has_bv = false;
  bool params_dirty = true;  // setters may run after construction (hf_loader.cr:319-373)
  float *w_q = nullptr, *w_k = nullptr, *w_v = nullptr, *w_o = nullptr;  // device, [in, out]
  shainet_attn_ctx *ctx = nullptr;
  shainet_kv_cache *cache = nullptr;
  int cache_len = 0;  // @cache_len
  rb_handle blas = nullptr;
  DevF x, q, k, v, attn, out, gemv_scratch;
};

namespace {

constexpr int kInitialCapacity = 256;  // llama_block.cr:500

void drop_context(shainet_llama_attn *l) {
  if (l->cache) shainet_kv_cache_destroy(l->cache);
  if (l->ctx) shainet_attn_destroy(l->ctx);
  l->cache = nullptr;
  l->ctx = nullptr;
}

// Build (or rebuild after a setter ran) the attention context; the cache is
// cleared by a rebuild, which only happens between conversations in practice.
int ensure_context(shainet_llama_attn *l) {
  if (l->ctx && !l->params_dirty) return SHAINET_HIP_OK;
  drop_context(l);
  l->cache_len = 0;
  int rc = shainet_attn_create(&l->ctx, l->num_heads, l->num_kv_heads, l->head_dim, l->rope_theta,
                               l->has_rope_freqs ? l->rope_freqs.data() : nullptr,
                               l->has_q_norm ? l->q_norm.data() : nullptr, (int)l->q_norm.size(),
                               l->has_k_norm ? l->k_norm.data() : nullptr, (int)l->k_norm.size(), l->qk_norm_eps,
                               kInitialCapacity);
  if (rc) return rc;
  rc = shainet_attn_set_bias(l->ctx, l->has_bq ? l->b_q.data() : nullptr, (int)l->b_q.size(),
                             l->has_bk ? l->b_k.data() : nullptr, (int)l->b_k.size(),
                             l->has_bv ? l->b_v.data() : nullptr, (int)l->b_v.size());
  if (!rc) rc = shainet_kv_cache_create(&l->cache, l->ctx, 1, kInitialCapacity);
  if (rc) {
    drop_context(l);
    return rc;
  }
  l->params_dirty = false;
  return SHAINET_HIP_OK;
}

// y[T,N] = x[T,K] * W[K,N], all row-major on the device.
int project(shainet_llama_attn *l, const float *x, const float *w, float *y, int T, int K, int N,
            hipStream_t stream) {
  if (T <= 16 && (N & 3) == 0) {
    const GemvPlan p = plan_gemv(T, K, N);
    if (!l->gemv_scratch.reserve(p.partial_floats)) return fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
    hipError_t e = launch_gemv(x, w, y, l->gemv_scratch.p, T, K, N, p, stream);
    if (e != hipSuccess) return fail(SHAINET_HIP_ERR_RUNTIME, std::string("gemv launch: ") + hipGetErrorString(e));
    return SHAINET_HIP_OK;
  }
  if (!g_rocblas.load()) return fail(SHAINET_HIP_ERR_RUNTIME, "librocblas.so.5 could not be opened for a projection GEMM");
  if (!l->blas && g_rocblas.create(&l->blas) != 0) return fail(SHAINET_HIP_ERR_RUNTIME, "rocblas_create_handle failed");
  if (g_rocblas.set_stream(l->blas, stream) != 0) return fail(SHAINET_HIP_ERR_RUNTIME, "rocblas_set_stream failed");
  // row-major y = x W  <=>  column-major y^T[N,T] = W^T[N,K] x^T[K,T]
  const float one = 1.0f, zero = 0.0f;
  const int st = g_rocblas.sgemm(l->blas, kRocblasOpNone, kRocblasOpNone, N, T, K, &one, w, N, x, K, &zero, y, N);
  if (st != 0) return fail(SHAINET_HIP_ERR_RUNTIME, "rocblas_sgemm failed with status " + std::to_string(st));
  return SHAINET_HIP_OK;
}

int upload_weight(float **dst, const float *src, size_t n) {
  if (*dst) (void)hipFree(*dst);
  *dst = nullptr;
  if (hipMalloc((void **)dst, n * sizeof(float)) != hipSuccess) return fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
  if (hipMemcpy(*dst, src, n * sizeof(float), hipMemcpyHostToDevice) != hipSuccess)
    return fail(SHAINET_HIP_ERR_RUNTIME, "hipMemcpy of a weight matrix failed");
  return SHAINET_HIP_OK;
}

void set_vec(std::vector<float> &v, bool &has, const float *src, int n) {
  has = src != nullptr;
  v.assign(src ? src : nullptr, src ? src + (n > 0 ? n : 0) : nullptr);
}

}  // namespace

extern "C" {

int shainet_llama_attn_create(shainet_llama_attn **out, int d_model, int num_heads, int num_kv_heads, int head_dim,
                              double eps, double rope_theta) {
  if (!out) return fail(SHAINET_HIP_ERR_ARGUMENT, "out is null");
  *out = nullptr;
  // llama_block.cr:80-89
  if (!(num_kv_heads > 0 && num_heads > 0 && num_heads % num_kv_heads == 0))
    return fail(SHAINET_HIP_ERR_ARGUMENT, "num_heads must be divisible by num_kv_heads");
  if (head_dim < 0) return fail(SHAINET_HIP_ERR_ARGUMENT, "head_dim must be positive");
  if (head_dim == 0) {
    if (d_model <= 0 || d_model % num_heads != 0)
      return fail(SHAINET_HIP_ERR_ARGUMENT, "d_model must be divisible by num_heads");
    head_dim = d_model / num_heads;
  }
  shainet_llama_attn *l = new (std::nothrow) shainet_llama_attn();
  if (!l) return fail(SHAINET_HIP_ERR_ALLOC, "out of host memory");
  l->d_model = d_model;
  l->num_heads = num_heads;
  l->num_kv_heads = num_kv_heads;
  l->head_dim = head_dim;
  l->q_dim = num_heads * head_dim;
  l->kv_dim = num_kv_heads * head_dim;
  l->qk_norm_eps = eps;
  l->rope_theta = rope_theta;
  *out = l;
  return SHAINET_HIP_OK;
}

int shainet_llama_attn_destroy(shainet_llama_attn *l) {
  if (!l) return SHAINET_HIP_OK;
  drop_context(l);
  if (l->blas && g_rocblas.destroy) g_rocblas.destroy(l->blas);
  for (float *p : {l->w_q, l->w_k, l->w_v, l->w_o})
    if (p) (void)hipFree(p);
  for (DevF *b : {&l->x, &l->q, &l->k, &l->v, &l->attn, &l->out, &l->gemv_scratch}) b->release();
  delete l;
  return SHAINET_HIP_OK;
}

int shainet_llama_attn_set_rope(shainet_llama_attn *l, double rope_theta, const float *rope_freqs) {
  if (!l) return fail(SHAINET_HIP_ERR_ARGUMENT, "layer is null");
  l->rope_theta = rope_theta;
  set_vec(l->rope_freqs, l->has_rope_freqs, rope_freqs, l->head_dim / 2);
  l->params_dirty = true;
  return SHAINET_HIP_OK;
}

int shainet_llama_attn_set_qk_norm(shainet_llama_attn *l, const float *q_norm, int q_len, const float *k_norm,
                                   int k_len) {
  if (!l) return fail(SHAINET_HIP_ERR_ARGUMENT, "layer is null");
  set_vec(l->q_norm, l->has_q_norm, q_norm, q_len);
  set_vec(l->k_norm, l->has_k_norm, k_norm, k_len);
  l->params_dirty = true;
  return SHAINET_HIP_OK;
}

int shainet_llama_attn_set_bias(shainet_llama_attn *l, const float *b_q, int q_len, const float *b_k, int k_len,
                                const float *b_v, int v_len) {
  if (!l) return fail(SHAINET_HIP_ERR_ARGUMENT, "layer is null");
  set_vec(l->b_q, l->has_bq, b_q, q_len);
  set_vec(l->b_k, l->has_bk, b_k, k_len);
  set_vec(l->b_v, l->has_bv, b_v, v_len);
  l->params_dirty = true;
  return SHAINET_HIP_OK;
}

int shainet_llama_attn_set_weights(shainet_llama_attn *l, const float *w_q, const float *w_k, const float *w_v,
                                   const float *w_o) {
  if (!l || !w_q || !w_k || !w_v || !w_o) return fail(SHAINET_HIP_ERR_ARGUMENT, "null argument");
  if (!shainet_hip_available()) return fail(SHAINET_HIP_ERR_RUNTIME, "no gfx950 device available");
  int rc = upload_weight(&l->w_q, w_q, (size_t)l->d_model * l->q_dim);
  if (!rc) rc = upload_weight(&l->w_k, w_k, (size_t)l->d_model * l->kv_dim);
  if (!rc) rc = upload_weight(&l->w_v, w_v, (size_t)l->d_model * l->kv_dim);
  if (!rc) rc = upload_weight(&l->w_o, w_o, (size_t)l->q_dim * l->d_model);
  return rc;
}

int shainet_llama_attn_clear_cache(shainet_llama_attn *l) {
  if (!l) return fail(SHAINET_HIP_ERR_ARGUMENT, "layer is null");
  l->cache_len = 0;
  return l->cache ? shainet_kv_cache_clear(l->cache, -1) : SHAINET_HIP_OK;
}

int shainet_llama_attn_cache_len(const shainet_llama_attn *l) { return l ? l->cache_len : -1; }

int shainet_llama_attn_forward_cached(shainet_llama_attn *l, const float *x, int new_tokens, float *out) {
  if (!l || !x || !out || new_tokens < 1) return fail(SHAINET_HIP_ERR_ARGUMENT, "invalid arguments");
  if (!l->w_q) return fail(SHAINET_HIP_ERR_ARGUMENT, "weights not set");
  int rc = ensure_context(l);  // raises what add_bias! / apply_head_rmsnorm! raise (llama_block.cr:587, 618)
  if (rc) return rc;
  const int T = new_tokens;
  const int total_len = l->cache_len + T;
  const int cap = shainet_kv_cache_capacity(l->cache);
  if (total_len > cap) {  // ensure_gpu_cache! (llama_block.cr:497-520): grow by doubling, contents stay on the device
    rc = shainet_kv_cache_reserve(l->cache, total_len > 2 * cap ? total_len : 2 * cap);
    if (rc) return rc;
  }
  const size_t xd = (size_t)T * l->d_model, qd = (size_t)T * l->q_dim, kd = (size_t)T * l->kv_dim;
  if (!l->x.reserve(xd) || !l->q.reserve(qd) || !l->k.reserve(kd) || !l->v.reserve(kd) || !l->attn.reserve(qd) ||
      !l->out.reserve(xd))
    return fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
  hipStream_t stream = (hipStream_t)shainet_attn_stream(l->ctx);
  if (hipMemcpyAsync(l->x.p, x, xd * sizeof(float), hipMemcpyHostToDevice, stream) != hipSuccess)
    return fail(SHAINET_HIP_ERR_RUNTIME, "hipMemcpyAsync(x) failed");
  if ((rc = project(l, l->x.p, l->w_q, l->q.p, T, l->d_model, l->q_dim, stream))) return rc;  // llama_block.cr:253
  if ((rc = project(l, l->x.p, l->w_k, l->k.p, T, l->d_model, l->kv_dim, stream))) return rc;  // 254
  if ((rc = project(l, l->x.p, l->w_v, l->v.p, T, l->d_model, l->kv_dim, stream))) return rc;  // 255
  rc = shainet_attn_forward(l->ctx, l->cache, nullptr, &T, 1, l->q.p, l->k.p, l->v.p, l->attn.p,
                            SHAINET_HIP_MEM_DEVICE);  // 256-296
  if (rc) return rc;
  l->cache_len = total_len;
  if ((rc = project(l, l->attn.p, l->w_o, l->out.p, T, l->q_dim, l->d_model, stream))) return rc;  // 298
  if (hipMemcpyAsync(out, l->out.p, xd * sizeof(float), hipMemcpyDeviceToHost, stream) != hipSuccess ||
      hipStreamSynchronize(stream) != hipSuccess)
    return fail(SHAINET_HIP_ERR_RUNTIME, "copying the result back failed");
  return SHAINET_HIP_OK;
}

}  // extern "C"
