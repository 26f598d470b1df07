// Host mirror of the attention half of SHAInet's LlamaBlock
// (src/shainet/transformer/llama_block.cr): the state the reference keeps per
// block (weights in [in, out] layout, optional biases, QK-norm weights, RoPE
// parameters, the KV cache and @cache_len) and attention_cached_cpu (246-299)
// with every step on the device: Q/K/V projections, bias, QK-norm, RoPE,
// append, causal GQA attention, output projection.  Activations stay in HBM
// between the steps; only x comes in and the [T, d_model] result goes out.
//
// The second half of this file adds what LlamaBlock#forward_cached
// (llama_block.cr:189-196) does around attention: the two RMSNorms, the two
// residual adds and the dense SwiGLU feed-forward, again all on the device.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <new>
#include <string>
#include <vector>

#include "../../include/shainet_hip_attn.h"
#include "attn_kernels.hpp"
#include "block_kernels.hpp"
#include "llama_internal.hpp"
#include "step_kernel.hpp"

using namespace shainet;

namespace {
int fail(int code, const std::string &msg) { return llama_fail(code, msg); }
}  // namespace

struct shainet_llama_attn {
  // llama_block.cr:10-28
  int d_model, num_heads, num_kv_heads, head_dim, q_dim, kv_dim;
  double qk_norm_eps, rope_theta;
  std::vector<float> rope_freqs, q_norm, k_norm, b_q, b_k, b_v;
  bool has_rope_freqs = false, has_q_norm = false, has_k_norm = false, has_bq = false, has_bk = false, has_bv = false;
  bool params_dirty = true;  // setters may run after construction (hf_loader.cr:319-373)
  float *w_qkv = nullptr, *w_o = nullptr;  // device, [in, out]; w_q | w_k | w_v side by side in one matrix
  // w_o once more, transposed ([d_model, q_dim]), for the product of a single row (launch_gemvt):
  // made on the device when such a call first needs it, made again after the weights change
  // (and q | k | v, [q_dim + 2 kv_dim, d_model], for layers without QK-norm)
  float *w_o_t = nullptr, *w_qkv_t = nullptr;
  bool w_o_t_stale = true, w_qkv_t_stale = true;
  // the norm weights multiplied into the rows of w_qkv_t (null: none), and whether any were
  const float *w_qkv_t_gamma = nullptr;
  shainet_attn_ctx *ctx = nullptr;
  shainet_kv_cache *cache = nullptr;
  shainet_kv_cache *scratch_cache = nullptr;  // rows of a no-cache forward call; empty between calls
  int cache_len = 0;  // @cache_len
  int *shared_error = nullptr;  // the error word of the model that owns this block, if one does
  Projector proj;
  DevF x, qkv, attn, out;
  PinnedF x_pin, out_pin;  // host-pointer calls stage their rows here
};

namespace {

constexpr int kInitialCapacity = 256;  // llama_block.cr:500

void drop_context(shainet_llama_attn *l) {
  if (l->scratch_cache) shainet_kv_cache_destroy(l->scratch_cache);
  l->scratch_cache = nullptr;
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
  if (l->shared_error) shainet_attn_adopt_error_word(l->ctx, l->shared_error);
  l->proj.error = shainet_attn_error_word(l->ctx);
  return SHAINET_HIP_OK;
}

void set_vec(std::vector<float> &v, bool &has, const float *src, int n) {
  has = src != nullptr;
  v.assign(src ? src : nullptr, src ? src + (n > 0 ? n : 0) : nullptr);
}

// attention_cached_cpu (llama_block.cr:246-299) with x and out on the device,
// asynchronous on the layer's stream.  pre: an RMSNorm to apply to x on its way
// into the projections; residual: rows to add to the result of the output
// projection (both are what LlamaBlock#forward_cached does around attention).
//
// no_cache: attention_full_cpu (209-243) instead: the same arithmetic from
// position 0 over the rows of this call alone; they go through a scratch cache
// that is empty again afterwards, and the block's own cache is not touched.
struct AheadRows {  // the transposed gate | up weights ([2 n, k]) the block's next product but one will read
  const float *wt;
  int k, n;
};
int attn_forward_device(shainet_llama_attn *l, const float *x, int T, float *out, const Fused &pre = Fused(),
                        const float *residual = nullptr, bool no_cache = false, const AheadRows *ahead = nullptr) {
  if (!l->w_qkv) return fail(SHAINET_HIP_ERR_ARGUMENT, "weights not set");
  int rc = ensure_context(l);
  if (rc) return rc;
  shainet_kv_cache *cache = l->cache;
  if (no_cache) {
    if (!l->scratch_cache && (rc = shainet_kv_cache_create(&l->scratch_cache, l->ctx, 1, T > kInitialCapacity ? T : kInitialCapacity)))
      return rc;
    cache = l->scratch_cache;
    if ((rc = shainet_kv_cache_clear(cache, -1))) return rc;
  }
  const int total_len = (no_cache ? 0 : l->cache_len) + T;
  const int cap = shainet_kv_cache_capacity(cache);
  if (total_len > cap) {  // ensure_gpu_cache! (llama_block.cr:497-520): grow by doubling, contents stay on the device
    rc = shainet_kv_cache_reserve(cache, total_len > 2 * cap ? total_len : 2 * cap);
    if (rc) return rc;
  }
  const int wide = l->q_dim + 2 * l->kv_dim;
  if (!l->qkv.reserve((size_t)T * wide) || !l->attn.reserve((size_t)T * l->q_dim))
    return fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
  hipStream_t stream = (hipStream_t)shainet_attn_stream(l->ctx);
  // q_full, k_new, v_new (llama_block.cr:253-255) as the three column blocks of one product
  const int hd = l->head_dim;
  static const bool fuse_off = getenv("SHAINET_HIP_NO_FUSED_PREP") != nullptr;
  if (!fuse_off && T <= 16 && (wide & 3) == 0 && hd >= 2 && hd <= 128 && (hd & (hd - 1)) == 0) {
    // few rows: bias, QK-norm, RoPE and the cache append (256-286, 332-344) happen where the
    // product's head rows are summed up; the attention kernel follows directly
    GemvPrep where;
    if ((rc = shainet_attn_begin_prepared(l->ctx, cache, T, &where))) return rc;
    Fused qkv = pre;
    qkv.epilogue = kGemvQkvPrep;
    qkv.prep = &where;
    if (gemvt_takes(T, l->d_model, wide, qkv.epilogue, qkv.norm, &where)) {
      // the copy carries the weights of the norm this product follows (a layer used with another
      // norm, or with none, gets its copy made again)
      const float *gamma = qkv.norm ? qkv.gamma : nullptr;
      if (gamma != l->w_qkv_t_gamma) l->w_qkv_t_stale = true;
      qkv.w_t = transposed_twin(&l->w_qkv_t, &l->w_qkv_t_stale, l->w_qkv, l->d_model, wide, stream, gamma);
      l->w_qkv_t_gamma = qkv.w_t ? gamma : nullptr;
      qkv.w_t_has_gamma = qkv.w_t && gamma;
    }
    if ((rc = l->proj.project(x, l->d_model, l->w_qkv, nullptr, T, l->d_model, wide, stream, qkv))) return rc;
    // One row: the attention launch leaves the memory system idle while it waits on its chain of
    // dependent loads, and takes along workgroups that read the first rows of the gate | up
    // weights into the L2s (8 MB: 1134 -> 1120 us per token of the 1B shape; 17 MB and more
    // slow the attention's own chain down by more than the product gains)
    static const int ahead_wgs = getenv("SHAINET_HIP_READ_AHEAD_WGS") ? atoi(getenv("SHAINET_HIP_READ_AHEAD_WGS")) : 128;
    if (ahead && ahead->wt && ahead_wgs > 0 && T == 1) shainet_attn_read_ahead(l->ctx, ahead->wt, ahead->k, ahead->n, ahead_wgs);
    rc = shainet_attn_finish_prepared(l->ctx, cache, T, l->attn.p);  // 287-296
  } else {
    if ((rc = l->proj.project(x, l->d_model, l->w_qkv, l->qkv.p, T, l->d_model, wide, stream, pre))) return rc;
    rc = shainet_attn_forward_strided(l->ctx, cache, nullptr, &T, 1, l->qkv.p, l->qkv.p + l->q_dim,
                                      l->qkv.p + l->q_dim + l->kv_dim, wide, wide, wide, l->attn.p,
                                      SHAINET_HIP_MEM_DEVICE);  // 256-296
  }
  if (rc) return rc;
  if (no_cache) {
    if ((rc = shainet_kv_cache_clear(cache, -1))) return rc;
  } else {
    l->cache_len = total_len;
  }
  Fused post;
  if (residual) {
    post.epilogue = kGemvResidual;
    post.res = residual;
  }
  if (gemvt_takes(T, l->q_dim, l->d_model, post.epilogue, false)) post.w_t = transposed_twin(&l->w_o_t, &l->w_o_t_stale, l->w_o, l->q_dim, l->d_model, stream);
  return l->proj.project(l->attn.p, l->q_dim, l->w_o, out, T, l->q_dim, l->d_model, stream, post);  // 298
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
  l->proj.release();
  for (float *p : {l->w_qkv, l->w_o, l->w_o_t, l->w_qkv_t})
    if (p) (void)hipFree(p);
  for (DevF *b : {&l->x, &l->qkv, &l->attn, &l->out}) b->release();
  l->x_pin.release();
  l->out_pin.release();
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
  const float *mats[3] = {w_q, w_k, w_v};
  const int widths[3] = {l->q_dim, l->kv_dim, l->kv_dim};
  int rc = upload_side_by_side(&l->w_qkv, mats, widths, 3, l->d_model);
  if (!rc) rc = upload_floats(&l->w_o, w_o, (size_t)l->q_dim * l->d_model);
  l->w_o_t_stale = l->w_qkv_t_stale = true;
  return rc;
}

int shainet_llama_attn_clear_cache(shainet_llama_attn *l) {
  if (!l) return fail(SHAINET_HIP_ERR_ARGUMENT, "layer is null");
  l->cache_len = 0;
  return l->cache ? shainet_kv_cache_clear(l->cache, -1) : SHAINET_HIP_OK;
}

int shainet_llama_attn_cache_len(const shainet_llama_attn *l) { return l ? l->cache_len : -1; }

static int attn_forward_host(shainet_llama_attn *l, const float *x, int new_tokens, float *out, bool no_cache);

int shainet_llama_attn_forward_cached(shainet_llama_attn *l, const float *x, int new_tokens, float *out) {
  return attn_forward_host(l, x, new_tokens, out, false);
}

int shainet_llama_attn_forward_full(shainet_llama_attn *l, const float *x, int seq_len, float *out) {
  return attn_forward_host(l, x, seq_len, out, true);
}

static int attn_forward_host(shainet_llama_attn *l, const float *x, int new_tokens, float *out, bool no_cache) {
  if (!l || !x || !out || new_tokens < 1) return fail(SHAINET_HIP_ERR_ARGUMENT, "invalid arguments");
  if (!l->w_qkv) return fail(SHAINET_HIP_ERR_ARGUMENT, "weights not set");
  int rc = ensure_context(l);  // raises what add_bias! / apply_head_rmsnorm! raise (llama_block.cr:587, 618)
  if (rc) return rc;
  const size_t xd = (size_t)new_tokens * l->d_model;
  if (!l->x.reserve(xd) || !l->out.reserve(xd) || !l->x_pin.reserve(xd) || !l->out_pin.reserve(xd))
    return fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
  hipStream_t stream = (hipStream_t)shainet_attn_stream(l->ctx);
  memcpy(l->x_pin.p, x, xd * sizeof(float));  // the last call's copies are done: every host-pointer call ends with a wait
  if (hipMemcpyAsync(l->x.p, l->x_pin.p, xd * sizeof(float), hipMemcpyHostToDevice, stream) != hipSuccess)
    return fail(SHAINET_HIP_ERR_RUNTIME, "hipMemcpyAsync(x) failed");
  if ((rc = attn_forward_device(l, l->x.p, new_tokens, l->out.p, Fused(), nullptr, no_cache))) {
    (void)hipStreamSynchronize(stream);  // the copy out of the pinned staging buffer may still run
    return rc;
  }
  if (hipMemcpyAsync(l->out_pin.p, l->out.p, xd * sizeof(float), hipMemcpyDeviceToHost, stream) != hipSuccess ||
      hipStreamSynchronize(stream) != hipSuccess)
    return fail(SHAINET_HIP_ERR_RUNTIME, "copying the result back failed");
  memcpy(out, l->out_pin.p, xd * sizeof(float));
  return check_error_word(shainet_attn_error_word(l->ctx));
}

}  // extern "C"

// ---------------------------------------------------------------------------
// The whole block: LlamaBlock#forward_cached (llama_block.cr:189-196) with a dense
// SwiGLU feed-forward (swiglu_ff.cr:76-91).
struct shainet_llama_block {
  shainet_llama_attn *attn = nullptr;
  int d_model = 0, ff_hidden = 0;
  double eps = 1e-6;                                // RMSNorm eps of @norm1 / @norm2 (llama_block.cr:93-94)
  float *norm1 = nullptr, *norm2 = nullptr;         // device gamma [d_model]; null = ones (rms_norm.cr:10)
  float *gate_up = nullptr, *down = nullptr;        // device [d_model, 2*ff] (gate | up) and [ff, d_model]
  float *gate_up_t = nullptr, *down_t = nullptr;    // the same transposed ([2*ff, d_model], [d_model, ff]), like w_o_t
  bool gate_up_t_stale = true, down_t_stale = true;
  DevF x, h, hidden, out;
  PinnedF x_pin, out_pin;  // host-pointer calls stage their rows here
};

namespace {

// x and out on the device; asynchronous on the block's stream.
int block_forward_device(shainet_llama_block *b, const float *x, int T, float *out, bool no_cache = false) {
  if (!b->gate_up || !b->down) return fail(SHAINET_HIP_ERR_ARGUMENT, "feed-forward weights not set");
  shainet_llama_attn *l = b->attn;
  int rc = ensure_context(l);
  if (rc) return rc;
  hipStream_t stream = (hipStream_t)shainet_attn_stream(l->ctx);
  const int d = b->d_model, ff = b->ff_hidden;
  if (!b->h.reserve((size_t)T * d) || !b->hidden.reserve((size_t)T * ff))
    return fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
  // h = x + attention_cached_cpu(@norm1.forward(x))
  Fused n1;
  n1.norm = true;
  n1.gamma = b->norm1;
  n1.eps = b->eps;
  Fused gate;
  gate.norm = true;
  gate.gamma = b->norm2;
  gate.eps = b->eps;
  gate.epilogue = kGemvSwiglu;
  if (gemvt_takes(T, d, ff, gate.epilogue, true)) {
    gate.w_t = transposed_twin(&b->gate_up_t, &b->gate_up_t_stale, b->gate_up, d, 2 * ff, stream, b->norm2);
    gate.w_t_has_gamma = gate.w_t && b->norm2;
  }
  const AheadRows ahead = {gate.w_t, d, ff};
  if ((rc = attn_forward_device(l, x, T, b->h.p, n1, x, no_cache, &ahead))) return rc;
  // hidden = silu(normed2 * gate_proj) * (normed2 * up_proj), normed2 = @norm2.forward(h)
  if ((rc = l->proj.project(b->h.p, d, b->gate_up, b->hidden.p, T, d, ff, stream, gate))) return rc;
  // out = h + hidden * down_proj
  Fused down;
  down.epilogue = kGemvResidual;
  down.res = b->h.p;
  if (gemvt_takes(T, ff, d, down.epilogue, false)) down.w_t = transposed_twin(&b->down_t, &b->down_t_stale, b->down, ff, d, stream);
  return l->proj.project(b->hidden.p, ff, b->down, out, T, ff, d, stream, down);
}

}  // namespace

// used by the model (llama_model.hip)
int shainet_llama_block_forward_device(shainet_llama_block *b, const float *x, int T, float *out, bool no_cache) {
  return block_forward_device(b, x, T, out, no_cache);
}
int shainet_llama_block_buffers(shainet_llama_block *b, LlamaBlockBuffers *out) {
  shainet_llama_attn *l = b->attn;
  const size_t d = (size_t)b->d_model, ff = (size_t)b->ff_hidden;
  struct Want {
    float **p;
    size_t n;
  } wants[] = {{&l->w_qkv, d * (size_t)(l->q_dim + 2 * l->kv_dim)}, {&l->w_o, (size_t)l->q_dim * d},
               {&b->gate_up, d * 2 * ff},                            {&b->down, ff * d},
               {&b->norm1, d},                                       {&b->norm2, d}};
  for (const Want &w : wants)
    if (!*w.p && hipMalloc((void **)w.p, w.n * sizeof(float)) != hipSuccess) {
      *w.p = nullptr;
      return fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
    }
  // (whoever asks for the buffers is about to write the weights: the transposed copies are made again)
  l->w_o_t_stale = l->w_qkv_t_stale = b->gate_up_t_stale = b->down_t_stale = true;
  *out = LlamaBlockBuffers{l->w_qkv, l->w_o, b->gate_up, b->down, b->norm1, b->norm2,
                           b->d_model, l->q_dim, l->kv_dim, b->ff_hidden};
  return SHAINET_HIP_OK;
}

// One decode step of the whole stack in one launch (step_kernel.hip): where this block's weights,
// parameters and cache are, with room for one more row made first (ensure_gpu_cache!,
// llama_block.cr:497-520); *pos = rows cached so far.  The step's kernel appends the row;
// shainet_llama_block_step_commit counts it afterwards.
int shainet_llama_block_step_begin(shainet_llama_block *b, StepLayer *out, int *pos) {
  shainet_llama_attn *l = b->attn;
  if (!l->w_qkv || !l->w_o || !b->gate_up || !b->down) return fail(SHAINET_HIP_ERR_ARGUMENT, "weights not set");
  int rc = ensure_context(l);
  if (rc) return rc;
  const int cap = shainet_kv_cache_capacity(l->cache);
  if (l->cache_len + 1 > cap && (rc = shainet_kv_cache_reserve(l->cache, 2 * cap))) return rc;
  GemvPrep where;
  if ((rc = shainet_attn_begin_prepared(l->ctx, l->cache, 1, &where))) return rc;
  out->w_qkv = l->w_qkv;
  out->w_o = l->w_o;
  out->w_gu = b->gate_up;
  out->w_down = b->down;
  out->norm1 = b->norm1;
  out->norm2 = b->norm2;
  out->b_q = where.b_q;
  out->b_k = where.b_k;
  out->b_v = where.b_v;
  out->q_norm = where.q_norm;
  out->k_norm = where.k_norm;
  out->rope_tab = where.rope_tab;
  out->kc = where.kc;
  out->vc = where.vc;
  out->cap = where.cap;
  out->pad_ = 0;
  *pos = where.start_pos;
  return SHAINET_HIP_OK;
}
void shainet_llama_block_step_commit(shainet_llama_block *b) {
  shainet_llama_attn *l = b->attn;
  shainet_attn_commit_prepared(l->ctx, l->cache, 1);
  l->cache_len += 1;
}
// The block's geometry, for the planner of the step kernel.
void shainet_llama_block_geometry(const shainet_llama_block *b, int *H, int *KV, int *hd, int *ff, double *qk_eps) {
  *H = b->attn->num_heads;
  *KV = b->attn->num_kv_heads;
  *hd = b->attn->head_dim;
  *ff = b->ff_hidden;
  *qk_eps = b->attn->qk_norm_eps;
}

// Forget the cached rows past `len` (generation that ran ahead of a stop token).
int shainet_llama_block_truncate(shainet_llama_block *b, int len) {
  shainet_llama_attn *l = b->attn;
  if (len < 0 || len > l->cache_len) return fail(SHAINET_HIP_ERR_ARGUMENT, "truncate beyond the cached length");
  if (l->cache) {
    int rc = shainet_kv_cache_truncate(l->cache, 0, len);
    if (rc) return rc;
  }
  l->cache_len = len;
  return SHAINET_HIP_OK;
}
// The model's kernels and its blocks' report a given-up wait into one word, the model's.
void shainet_llama_block_share_error_word(shainet_llama_block *b, int *word) {
  shainet_llama_attn *l = b->attn;
  l->shared_error = word;
  if (l->ctx) {
    shainet_attn_adopt_error_word(l->ctx, word);
    l->proj.error = shainet_attn_error_word(l->ctx);
  }
}
int shainet_llama_block_set_stream(shainet_llama_block *b, hipStream_t stream) {
  int rc = ensure_context(b->attn);
  if (rc) return rc;
  return shainet_attn_set_stream(b->attn->ctx, (void *)stream);
}

extern "C" {

int shainet_llama_block_create(shainet_llama_block **out, int d_model, int num_heads, int ff_hidden, double eps,
                               double rope_theta, int num_kv_heads, int head_dim) {
  if (!out) return fail(SHAINET_HIP_ERR_ARGUMENT, "out is null");
  *out = nullptr;
  if (ff_hidden < 1) return fail(SHAINET_HIP_ERR_ARGUMENT, "ff_hidden must be positive");
  if (num_kv_heads == 0) num_kv_heads = num_heads;  // @num_kv_heads = @num_heads (llama_block.cr:73)
  shainet_llama_attn *a = nullptr;
  int rc = shainet_llama_attn_create(&a, d_model, num_heads, num_kv_heads, head_dim, eps, rope_theta);
  if (rc) return rc;
  shainet_llama_block *b = new (std::nothrow) shainet_llama_block();
  if (!b) {
    shainet_llama_attn_destroy(a);
    return fail(SHAINET_HIP_ERR_ALLOC, "out of host memory");
  }
  b->attn = a;
  b->d_model = d_model;
  b->ff_hidden = ff_hidden;
  b->eps = eps;
  *out = b;
  return SHAINET_HIP_OK;
}

int shainet_llama_block_destroy(shainet_llama_block *b) {
  if (!b) return SHAINET_HIP_OK;
  shainet_llama_attn_destroy(b->attn);
  for (float *p : {b->norm1, b->norm2, b->gate_up, b->down, b->gate_up_t, b->down_t})
    if (p) (void)hipFree(p);
  for (DevF *f : {&b->x, &b->h, &b->hidden, &b->out}) f->release();
  b->x_pin.release();
  b->out_pin.release();
  delete b;
  return SHAINET_HIP_OK;
}

shainet_llama_attn *shainet_llama_block_attn(shainet_llama_block *b) { return b ? b->attn : nullptr; }

int shainet_llama_block_set_norms(shainet_llama_block *b, const float *norm1, const float *norm2) {
  if (!b) return fail(SHAINET_HIP_ERR_ARGUMENT, "block is null");
  if (!shainet_hip_available()) return fail(SHAINET_HIP_ERR_RUNTIME, "no gfx950 device available");
  int rc = SHAINET_HIP_OK;
  float **dst[2] = {&b->norm1, &b->norm2};
  const float *src[2] = {norm1, norm2};
  for (int i = 0; i < 2 && !rc; ++i) {
    if (src[i]) {
      rc = upload_floats(dst[i], src[i], (size_t)b->d_model);
    } else if (*dst[i]) {
      (void)hipFree(*dst[i]);
      *dst[i] = nullptr;
    }
  }
  // (the transposed copies of q | k | v and gate | up carry the norm weights)
  b->attn->w_qkv_t_stale = b->gate_up_t_stale = true;
  b->attn->w_qkv_t_gamma = nullptr;
  return rc;
}

int shainet_llama_block_set_ffn(shainet_llama_block *b, const float *gate, const float *up, const float *down) {
  if (!b || !gate || !up || !down) return fail(SHAINET_HIP_ERR_ARGUMENT, "null argument");
  if (!shainet_hip_available()) return fail(SHAINET_HIP_ERR_RUNTIME, "no gfx950 device available");
  const float *mats[2] = {gate, up};
  const int widths[2] = {b->ff_hidden, b->ff_hidden};
  int rc = upload_side_by_side(&b->gate_up, mats, widths, 2, b->d_model);
  if (!rc) rc = upload_floats(&b->down, down, (size_t)b->ff_hidden * b->d_model);
  b->gate_up_t_stale = b->down_t_stale = true;
  return rc;
}

int shainet_llama_block_clear_cache(shainet_llama_block *b) {
  if (!b) return fail(SHAINET_HIP_ERR_ARGUMENT, "block is null");
  return shainet_llama_attn_clear_cache(b->attn);
}

int shainet_llama_block_cache_len(const shainet_llama_block *b) { return b ? b->attn->cache_len : -1; }

static int block_forward_any(shainet_llama_block *b, const float *x, int new_tokens, float *out, int mem, bool no_cache);

int shainet_llama_block_forward_cached(shainet_llama_block *b, const float *x, int new_tokens, float *out, int mem) {
  return block_forward_any(b, x, new_tokens, out, mem, false);
}

int shainet_llama_block_forward(shainet_llama_block *b, const float *x, int seq_len, float *out, int mem) {
  return block_forward_any(b, x, seq_len, out, mem, true);
}

static int block_forward_any(shainet_llama_block *b, const float *x, int new_tokens, float *out, int mem, bool no_cache) {
  if (!b || !x || !out || new_tokens < 1) return fail(SHAINET_HIP_ERR_ARGUMENT, "invalid arguments");
  if (mem != SHAINET_HIP_MEM_HOST && mem != SHAINET_HIP_MEM_DEVICE)
    return fail(SHAINET_HIP_ERR_ARGUMENT, "mem must be SHAINET_HIP_MEM_HOST or SHAINET_HIP_MEM_DEVICE");
  if (mem == SHAINET_HIP_MEM_DEVICE) return block_forward_device(b, x, new_tokens, out, no_cache);
  int rc = ensure_context(b->attn);
  if (rc) return rc;
  const size_t xd = (size_t)new_tokens * b->d_model;
  if (!b->x.reserve(xd) || !b->out.reserve(xd) || !b->x_pin.reserve(xd) || !b->out_pin.reserve(xd))
    return fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
  hipStream_t stream = (hipStream_t)shainet_attn_stream(b->attn->ctx);
  memcpy(b->x_pin.p, x, xd * sizeof(float));
  if (hipMemcpyAsync(b->x.p, b->x_pin.p, xd * sizeof(float), hipMemcpyHostToDevice, stream) != hipSuccess)
    return fail(SHAINET_HIP_ERR_RUNTIME, "hipMemcpyAsync(x) failed");
  if ((rc = block_forward_device(b, b->x.p, new_tokens, b->out.p, no_cache))) {
    (void)hipStreamSynchronize(stream);  // the copy out of the pinned staging buffer may still run
    return rc;
  }
  if (hipMemcpyAsync(b->out_pin.p, b->out.p, xd * sizeof(float), hipMemcpyDeviceToHost, stream) != hipSuccess ||
      hipStreamSynchronize(stream) != hipSuccess)
    return fail(SHAINET_HIP_ERR_RUNTIME, "copying the result back failed");
  memcpy(out, b->out_pin.p, xd * sizeof(float));
  return check_error_word(shainet_attn_error_word(b->attn->ctx));
}

}  // extern "C"
