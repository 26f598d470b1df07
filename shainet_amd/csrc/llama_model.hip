// Host mirror of the decoder-only model around the blocks, as Network#run walks it
// with use_kv_cache (src/shainet/basic/network_run.cr:185-226): embedding lookup
// (text/embedding_layer.cr:129-153) -> LlamaBlock#forward_cached per layer ->
// final RMSNorm over all rows -> last row times the lm_head matrix
// [d_model, vocab] (1390-1404) -> bias.  The activations never leave the device;
// the logits stay there too, so that greedy argmax, the repetition penalty and the
// top-k selection of text/sampler.cr run on them without a copy of the vocab row.
#include <hip/hip_runtime.h>

#include <math.h>
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

// llama_block.hip
int shainet_llama_block_forward_device(shainet_llama_block *b, const float *x, int T, float *out, bool no_cache);
int shainet_llama_block_set_stream(shainet_llama_block *b, hipStream_t stream);
int shainet_llama_block_truncate(shainet_llama_block *b, int len);
void shainet_llama_block_share_error_word(shainet_llama_block *b, int *word);
int shainet_llama_block_step_begin(shainet_llama_block *b, shainet::StepLayer *out, int *pos);
void shainet_llama_block_step_commit(shainet_llama_block *b);
void shainet_llama_block_geometry(const shainet_llama_block *b, int *H, int *KV, int *hd, int *ff, double *qk_eps);

// What the one-launch decode step (step_kernel.hip) keeps between steps.
struct ModelStep {
  int mode = 0;          // SHAINET_HIP_DECODE_*: 0 auto, 1 one launch per product, 2 one launch per step or an error
  bool planned = false;  // plan holds the answer for this model's geometry
  StepPlan plan = {};
  int n_wgs = 0;
  int H = 0, KV = 0, hd = 0, ff = 0;
  double qk_eps = 0.0;
  StepLayer *d_layers = nullptr;
  std::vector<StepLayer> layers;  // what d_layers holds
  float *parts = nullptr;         // the five partial areas, one allocation
  unsigned *bar = nullptr;        // the barrier's words, then as many more where the give-up test sends arrivals
  unsigned epoch = 0;
  bool lose_marks = false;
  long long *trace = nullptr;     // device, [n_wgs][1 + kStepTraceSlots layers]; SHAINET_HIP_STEP_TRACE only
  void release() {
    if (d_layers) (void)hipFree(d_layers);
    if (parts) (void)hipFree(parts);
    if (bar) (void)hipFree(bar);
    if (trace) (void)hipFree(trace);
    d_layers = nullptr;
    parts = nullptr;
    bar = nullptr;
    trace = nullptr;
    layers.clear();
    planned = false;
  }
};

struct shainet_llama_model {
  int vocab = 0, d_model = 0;
  double eps = 1e-6;
  std::vector<shainet_llama_block *> blocks;
  float *embedding = nullptr;   // device [vocab, d_model]
  float *final_norm = nullptr;  // device [d_model]; has_final_norm says whether the step exists (@final_norm)
  bool has_final_norm = false;
  float *lm_head = nullptr;     // device [d_model, vocab]
  // lm_head transposed ([vocab, d_model]) for the product of a single row: the embedding table
  // itself where the two are tied (compared on the device, bit for bit, the first time it is
  // needed), else a copy of its own
  const float *lm_head_t = nullptr;
  float *lm_head_t_own = nullptr;
  bool lm_head_t_stale = true;
  float *lm_bias = nullptr;     // device [vocab] or null
  hipStream_t stream = nullptr;
  int *error = nullptr;  // pinned host word: set by any kernel of the model that gave up a bounded wait
  Projector proj;
  DevF act[2], logits;
  int *d_tokens = nullptr;
  size_t d_tokens_cap = 0;
  bool have_logits = false;
  // sampler scratch
  void *topk_scratch = nullptr;
  size_t topk_scratch_cap = 0;
  int *d_ids = nullptr;    // kMaxTopK ids, then the count
  float *d_vals = nullptr;
  int *d_gen = nullptr;    // generated ids of one chunk of shainet_llama_model_generate_greedy
  ModelStep step;
};

namespace {

int fail(int code, const std::string &msg) { return llama_fail(code, msg); }

}  // namespace

int shainet_llama_model_buffers(shainet_llama_model *m, LlamaModelBuffers *out) {
  struct Want {
    float **p;
    size_t n;
  } wants[] = {{&m->embedding, (size_t)m->vocab * m->d_model},
               {&m->final_norm, (size_t)m->d_model},
               {&m->lm_head, (size_t)m->d_model * m->vocab}};
  for (const Want &w : wants)
    if (!*w.p && hipMalloc((void **)w.p, w.n * sizeof(float)) != hipSuccess) {
      *w.p = nullptr;
      return fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
    }
  m->has_final_norm = true;
  m->lm_head_t_stale = true;  // (whoever asks for the buffers is about to write them)
  if (m->lm_bias) (void)hipFree(m->lm_bias);  // the loader's output bias is all zeros (hf_loader.cr:404)
  m->lm_bias = nullptr;
  *out = LlamaModelBuffers{m->embedding, m->final_norm, m->lm_head};
  return SHAINET_HIP_OK;
}

namespace {

// lm_head transposed, or null (see the struct).  The comparison with the embedding table waits
// for the stream once, when the weights are new.
const float *lm_head_twin(shainet_llama_model *m) {
  if (!transposed_twins_wanted() || !m->lm_head) return nullptr;
  if (!m->lm_head_t_stale) return m->lm_head_t;
  m->lm_head_t = nullptr;
  m->lm_head_t_stale = false;
  if (m->embedding) {
    int *differ = nullptr, host = 1;
    if (hipMalloc((void **)&differ, sizeof(int)) == hipSuccess) {
      bool ok = hipMemsetAsync(differ, 0, sizeof(int), m->stream) == hipSuccess &&
                launch_transposed_differ(m->lm_head, m->embedding, m->d_model, m->vocab, differ, m->stream) == hipSuccess &&
                hipMemcpyAsync(&host, differ, sizeof(int), hipMemcpyDeviceToHost, m->stream) == hipSuccess &&
                hipStreamSynchronize(m->stream) == hipSuccess;
      (void)hipFree(differ);
      if (ok && host == 0) {
        if (m->lm_head_t_own) (void)hipFree(m->lm_head_t_own);
        m->lm_head_t_own = nullptr;
        return m->lm_head_t = m->embedding;
      }
    }
    (void)hipGetLastError();
  }
  bool stale = true;
  return m->lm_head_t = transposed_twin(&m->lm_head_t_own, &stale, m->lm_head, m->d_model, m->vocab, m->stream);
}

int reserve_ints(int **p, size_t *cap, size_t n) {
  if (n <= *cap) return SHAINET_HIP_OK;
  size_t want = *cap ? *cap : 256;
  while (want < n) want *= 2;
  int *np = nullptr;
  if (hipMalloc((void **)&np, want * sizeof(int)) != hipSuccess) return fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
  if (*p) (void)hipFree(*p);
  *p = np;
  *cap = want;
  return SHAINET_HIP_OK;
}

int run_topk(shainet_llama_model *m, int k, bool finite_only, int *ids, float *vals, int *count) {
  if (!m->have_logits) return fail(SHAINET_HIP_ERR_ARGUMENT, "no logits: call shainet_llama_model_run first");
  if (k < 1 || k > kMaxTopK) return fail(SHAINET_HIP_ERR_ARGUMENT, "k must be in [1, 256]");
  const size_t need = topk_scratch_bytes(m->vocab, k);
  if (need > m->topk_scratch_cap) {
    if (m->topk_scratch) (void)hipFree(m->topk_scratch);
    m->topk_scratch = nullptr;
    m->topk_scratch_cap = 0;
    if (hipMalloc(&m->topk_scratch, need) != hipSuccess) return fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
    m->topk_scratch_cap = need;
  }
  if (!m->d_ids) {
    if (hipMalloc((void **)&m->d_ids, (kMaxTopK + 2) * sizeof(int)) != hipSuccess ||
        hipMalloc((void **)&m->d_vals, kMaxTopK * sizeof(float)) != hipSuccess)
      return fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
  }
  hipError_t e = launch_topk(m->logits.p, m->vocab, k, finite_only, m->topk_scratch, m->d_ids, m->d_vals,
                             m->d_ids + kMaxTopK, m->stream);
  if (e != hipSuccess) return fail(SHAINET_HIP_ERR_RUNTIME, std::string("top-k launch: ") + hipGetErrorString(e));
  int host_ids[kMaxTopK + 1];
  if (hipMemcpyAsync(host_ids, m->d_ids, (kMaxTopK + 1) * sizeof(int), hipMemcpyDeviceToHost, m->stream) !=
          hipSuccess ||
      (vals && hipMemcpyAsync(vals, m->d_vals, k * sizeof(float), hipMemcpyDeviceToHost, m->stream) != hipSuccess) ||
      hipStreamSynchronize(m->stream) != hipSuccess)
    return fail(SHAINET_HIP_ERR_RUNTIME, "copying the selection back failed");
  if (int rc = check_error_word(m->error)) return rc;
  *count = host_ids[kMaxTopK];
  for (int i = 0; i < k; ++i) ids[i] = host_ids[i];
  return SHAINET_HIP_OK;
}

// Decides once per model whether its decode steps can run as one launch.
void plan_model_step(shainet_llama_model *m) {
  ModelStep &st = m->step;
  st.planned = true;
  st.plan.ok = false;
  // AUTO: one launch per product.  Measured on the 16-block, d_model 2048 shape at 512 cached positions:
  // 1.31 ms per token with one launch per product, 1.36 ms with the single launch (its five barriers
  // per block and the sums of partial results after them cost what the launches did); the variable
  // SHAINET_HIP_PERSISTENT_STEP makes AUTO take the single launch where the geometry fits.
  static const bool auto_persistent = getenv("SHAINET_HIP_PERSISTENT_STEP") != nullptr;
  if (st.mode == SHAINET_HIP_DECODE_PER_PRODUCT || (st.mode == SHAINET_HIP_DECODE_AUTO && !auto_persistent)) return;
  hipDeviceProp_t prop;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return;
  st.n_wgs = prop.multiProcessorCount;  // one workgroup per compute unit, all resident at once
  if (const char *env = getenv("SHAINET_HIP_STEP_WGS")) {  // tuning knob; never more than the compute units
    const int v = atoi(env);
    if (v >= 1 && v < st.n_wgs) st.n_wgs = v;
  }
  shainet_llama_block_geometry(m->blocks[0], &st.H, &st.KV, &st.hd, &st.ff, &st.qk_eps);
  for (shainet_llama_block *b : m->blocks) {
    int H, KV, hd, ff;
    double qe;
    shainet_llama_block_geometry(b, &H, &KV, &hd, &ff, &qe);
    if (H != st.H || KV != st.KV || hd != st.hd || ff != st.ff || qe != st.qk_eps) return;
  }
  const StepPlan p = plan_step(m->d_model, st.H, st.KV, st.hd, st.ff, st.n_wgs);
  if (!p.ok) return;
  const size_t floats = p.qkv_floats + p.attn_floats + p.o_floats + p.gu_floats + p.down_floats;
  const size_t n_layers = m->blocks.size();
  st.lose_marks = getenv("SHAINET_HIP_TEST_LOSE_PARTIAL_MARKS") != nullptr;
  const bool want_trace = getenv("SHAINET_HIP_STEP_TRACE") != nullptr;
  const size_t trace_bytes = (size_t)st.n_wgs * (1 + kStepTraceSlots * n_layers) * sizeof(long long);
  if (hipMalloc((void **)&st.d_layers, n_layers * sizeof(StepLayer)) != hipSuccess ||
      hipMalloc((void **)&st.parts, floats * sizeof(float)) != hipSuccess ||
      hipMalloc((void **)&st.bar, 2 * step_barrier_words(st.n_wgs) * sizeof(unsigned)) != hipSuccess ||
      hipMemset(st.bar, 0, 2 * step_barrier_words(st.n_wgs) * sizeof(unsigned)) != hipSuccess ||
      hipMemset(st.parts, 0, floats * sizeof(float)) != hipSuccess ||
      (want_trace && (hipMalloc((void **)&st.trace, trace_bytes) != hipSuccess ||
                      hipMemset(st.trace, 0, trace_bytes) != hipSuccess))) {
    (void)hipGetLastError();
    st.release();
    st.planned = true;
    return;
  }
  st.epoch = 0;
  st.plan = p;
}

// One new token through all blocks in one launch; m->act[0] receives the last block's output row.
// Returns -1 when this step has to take the launch-per-product path instead.
int run_step(shainet_llama_model *m, const int *d_token) {
  ModelStep &st = m->step;
  if (!st.planned) plan_model_step(m);
  if (!st.plan.ok) return -1;
  const size_t n_layers = m->blocks.size();
  std::vector<StepLayer> now(n_layers);
  int pos = -1, rc;
  for (size_t i = 0; i < n_layers; ++i) {
    int p = 0;
    if ((rc = shainet_llama_block_set_stream(m->blocks[i], m->stream))) return rc;
    if ((rc = shainet_llama_block_step_begin(m->blocks[i], &now[i], &p))) return rc;
    if (i == 0) pos = p;
    if (p != pos) return -1;  // blocks that were driven one by one hold different lengths
  }
  if (st.layers.size() != n_layers || memcmp(st.layers.data(), now.data(), n_layers * sizeof(StepLayer)) != 0) {
    // pageable source: the copy has left `now` when the call returns; ordered on the stream
    // behind the steps that still read the old table
    if (hipMemcpyAsync(st.d_layers, now.data(), n_layers * sizeof(StepLayer), hipMemcpyHostToDevice, m->stream) !=
        hipSuccess)
      return fail(SHAINET_HIP_ERR_RUNTIME, "hipMemcpyAsync(layer table) failed");
    st.layers = now;
  }
  const StepPlan &p = st.plan;
  StepArgs a = {};
  a.layers = st.d_layers;
  a.n_layers = (int)n_layers;
  a.d = m->d_model;
  a.H = st.H;
  a.KV = st.KV;
  a.hd = st.hd;
  a.ff = st.ff;
  a.eps = m->eps;
  a.qk_eps = st.qk_eps;
  a.scale = (float)(1.0 / sqrt((double)st.hd));  // llama_block.cr:249
  a.qkv = p.qkv;
  a.wo = p.wo;
  a.gu = p.gu;
  a.down = p.down;
  a.attn_chunks = p.attn_chunks;
  a.attn_ck = step_keys_per_chunk(p, pos);
  a.embedding = m->embedding;
  a.token = d_token;
  a.pos = pos;
  a.x_out = m->act[0].p;
  a.qkv_part = st.parts;
  a.attn_part = a.qkv_part + p.qkv_floats;
  a.o_part = a.attn_part + p.attn_floats;
  a.gu_part = a.o_part + p.o_floats;
  a.down_part = a.gu_part + p.gu_floats;
  a.bar = st.bar;
  a.bar_set = st.lose_marks ? st.bar + step_barrier_words(st.n_wgs) : st.bar;
  a.epoch0 = st.epoch;
  a.spin_limit = st.lose_marks ? 200 : (1 << 22);
  a.error = m->error;
  a.trace = st.trace;
  const hipError_t e = launch_step(a, st.n_wgs, p.lds_bytes, m->stream);
  if (e != hipSuccess) return fail(SHAINET_HIP_ERR_RUNTIME, std::string("step launch: ") + hipGetErrorString(e));
  st.epoch += (unsigned)kStepBarriersPerLayer * (unsigned)n_layers;
  for (shainet_llama_block *b : m->blocks) shainet_llama_block_step_commit(b);
  return SHAINET_HIP_OK;
}

// Network#run on token ids that already sit in device memory; asynchronous.  no_cache: every block's
// LlamaBlock#forward instead of forward_cached (network_run.cr:199-204 with use_kv_cache off): the
// rows attend among themselves from position 0 and the caches stay as they are.
int run_device_tokens(shainet_llama_model *m, const int *d_tokens, int T, bool no_cache = false) {
  const int d = m->d_model;
  if (!m->act[0].reserve((size_t)T * d) || !m->act[1].reserve((size_t)T * d) || !m->logits.reserve((size_t)m->vocab))
    return fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
  m->have_logits = false;
  int cur = 0, rc = -1;
  if (T == 1 && !no_cache) {
    rc = run_step(m, d_tokens);
    if (rc > 0) return rc;
    if (rc < 0 && m->step.mode == SHAINET_HIP_DECODE_PERSISTENT)
      return fail(SHAINET_HIP_ERR_ARGUMENT, "this model's geometry does not fit the one-launch decode step");
  }
  if (rc < 0) {
    hipError_t e = launch_embed(m->embedding, d_tokens, m->act[0].p, T, d, m->stream);
    if (e != hipSuccess) return fail(SHAINET_HIP_ERR_RUNTIME, std::string("embedding launch: ") + hipGetErrorString(e));
    for (shainet_llama_block *b : m->blocks) {
      if ((rc = shainet_llama_block_set_stream(b, m->stream))) return rc;
      if ((rc = shainet_llama_block_forward_device(b, m->act[cur].p, T, m->act[cur ^ 1].p, no_cache))) return rc;
      cur ^= 1;
    }
  }
  hipError_t e = hipSuccess;
  // the final norm runs over every row in the reference; only the last one is used afterwards
  const float *last = m->act[cur].p + (size_t)(T - 1) * d;
  Fused fin;
  fin.norm = m->has_final_norm;
  fin.gamma = m->final_norm;
  fin.eps = m->eps;
  if (gemvt_takes(1, d, m->vocab, fin.epilogue, fin.norm)) fin.w_t = lm_head_twin(m);
  if ((rc = m->proj.project(last, d, m->lm_head, m->logits.p, 1, d, m->vocab, m->stream, fin))) return rc;
  if (m->lm_bias) {
    e = launch_add_bias_row(m->logits.p, m->lm_bias, m->vocab, m->stream);
    if (e != hipSuccess) return fail(SHAINET_HIP_ERR_RUNTIME, std::string("bias launch: ") + hipGetErrorString(e));
  }
  m->have_logits = true;
  return SHAINET_HIP_OK;
}

}  // namespace

extern "C" {

int shainet_llama_model_create(shainet_llama_model **out, int vocab, int d_model, int n_layers, int num_heads,
                               int num_kv_heads, int head_dim, int ff_hidden, double eps, double rope_theta) {
  if (!out) return fail(SHAINET_HIP_ERR_ARGUMENT, "out is null");
  *out = nullptr;
  if (vocab < 1 || d_model < 1 || n_layers < 1) return fail(SHAINET_HIP_ERR_ARGUMENT, "vocab, d_model and n_layers must be positive");
  shainet_llama_model *m = new (std::nothrow) shainet_llama_model();
  if (!m) return fail(SHAINET_HIP_ERR_ALLOC, "out of host memory");
  m->vocab = vocab;
  m->d_model = d_model;
  m->eps = eps;
  m->error = alloc_error_word();  // null without a device: said by the first call that needs one
  m->proj.error = m->error;
  for (int i = 0; i < n_layers; ++i) {
    shainet_llama_block *b = nullptr;
    int rc = shainet_llama_block_create(&b, d_model, num_heads, ff_hidden, eps, rope_theta, num_kv_heads, head_dim);
    if (rc) {
      shainet_llama_model_destroy(m);
      return rc;
    }
    shainet_llama_block_share_error_word(b, m->error);
    m->blocks.push_back(b);
  }
  *out = m;
  return SHAINET_HIP_OK;
}

int shainet_llama_model_destroy(shainet_llama_model *m) {
  if (!m) return SHAINET_HIP_OK;
  for (shainet_llama_block *b : m->blocks) shainet_llama_block_destroy(b);
  for (float *p : {m->embedding, m->final_norm, m->lm_head, m->lm_bias, m->d_vals, m->lm_head_t_own})
    if (p) (void)hipFree(p);
  if (m->d_tokens) (void)hipFree(m->d_tokens);
  if (m->d_ids) (void)hipFree(m->d_ids);
  if (m->d_gen) (void)hipFree(m->d_gen);
  if (m->topk_scratch) (void)hipFree(m->topk_scratch);
  m->proj.release();
  m->step.release();
  for (DevF *f : {&m->act[0], &m->act[1], &m->logits}) f->release();
  if (m->stream) (void)hipStreamDestroy(m->stream);
  free_error_word(m->error);
  delete m;
  return SHAINET_HIP_OK;
}

int shainet_llama_model_layers(const shainet_llama_model *m) { return m ? (int)m->blocks.size() : -1; }

shainet_llama_block *shainet_llama_model_block(shainet_llama_model *m, int i) {
  if (!m || i < 0 || i >= (int)m->blocks.size()) return nullptr;
  return m->blocks[i];
}

int shainet_llama_model_set_embedding(shainet_llama_model *m, const float *table) {
  if (!m || !table) return fail(SHAINET_HIP_ERR_ARGUMENT, "null argument");
  if (!shainet_hip_available()) return fail(SHAINET_HIP_ERR_RUNTIME, "no gfx950 device available");
  m->lm_head_t_stale = true;
  return upload_floats(&m->embedding, table, (size_t)m->vocab * m->d_model);
}

int shainet_llama_model_set_final_norm(shainet_llama_model *m, const float *gamma) {
  if (!m) return fail(SHAINET_HIP_ERR_ARGUMENT, "model is null");
  m->has_final_norm = gamma != nullptr;
  if (!gamma) return SHAINET_HIP_OK;
  if (!shainet_hip_available()) return fail(SHAINET_HIP_ERR_RUNTIME, "no gfx950 device available");
  return upload_floats(&m->final_norm, gamma, (size_t)m->d_model);
}

int shainet_llama_model_set_lm_head(shainet_llama_model *m, const float *w, const float *bias) {
  if (!m || !w) return fail(SHAINET_HIP_ERR_ARGUMENT, "null argument");
  if (!shainet_hip_available()) return fail(SHAINET_HIP_ERR_RUNTIME, "no gfx950 device available");
  m->lm_head_t_stale = true;
  int rc = upload_floats(&m->lm_head, w, (size_t)m->d_model * m->vocab);
  if (rc) return rc;
  if (bias) return upload_floats(&m->lm_bias, bias, (size_t)m->vocab);
  if (m->lm_bias) (void)hipFree(m->lm_bias);
  m->lm_bias = nullptr;
  return SHAINET_HIP_OK;
}

int shainet_llama_model_clear_cache(shainet_llama_model *m) {
  if (!m) return fail(SHAINET_HIP_ERR_ARGUMENT, "model is null");
  for (shainet_llama_block *b : m->blocks) {
    int rc = shainet_llama_block_clear_cache(b);
    if (rc) return rc;
  }
  return SHAINET_HIP_OK;
}

int shainet_llama_model_cache_len(const shainet_llama_model *m) {
  return m && !m->blocks.empty() ? shainet_llama_block_cache_len(m->blocks[0]) : -1;
}

static int model_run(shainet_llama_model *m, const int *tokens, int n_tokens, float *logits, bool no_cache);

int shainet_llama_model_run(shainet_llama_model *m, const int *tokens, int n_tokens, float *logits) {
  return model_run(m, tokens, n_tokens, logits, false);
}

int shainet_llama_model_run_full(shainet_llama_model *m, const int *tokens, int n_tokens, float *logits) {
  return model_run(m, tokens, n_tokens, logits, true);
}

static int model_run(shainet_llama_model *m, const int *tokens, int n_tokens, float *logits, bool no_cache) {
  if (!m || !tokens || n_tokens < 1) return fail(SHAINET_HIP_ERR_ARGUMENT, "invalid arguments");
  if (!m->embedding || !m->lm_head) return fail(SHAINET_HIP_ERR_ARGUMENT, "embedding or lm_head not set");
  for (int i = 0; i < n_tokens; ++i)  // an id outside the table raises IndexError in the reference
    if (tokens[i] < 0 || tokens[i] >= m->vocab) return fail(SHAINET_HIP_ERR_ARGUMENT, "token id outside the vocabulary");
  if (!m->stream && hipStreamCreateWithFlags(&m->stream, hipStreamNonBlocking) != hipSuccess)
    return fail(SHAINET_HIP_ERR_RUNTIME, "hipStreamCreate failed");
  int rc = reserve_ints(&m->d_tokens, &m->d_tokens_cap, (size_t)n_tokens);
  if (rc) return rc;
  m->have_logits = false;
  // pageable source: the copy has left the host buffer when the call returns
  if (hipMemcpyAsync(m->d_tokens, tokens, (size_t)n_tokens * sizeof(int), hipMemcpyHostToDevice, m->stream) !=
      hipSuccess)
    return fail(SHAINET_HIP_ERR_RUNTIME, "hipMemcpyAsync(tokens) failed");
  if ((rc = run_device_tokens(m, m->d_tokens, n_tokens, no_cache))) return rc;
  if (logits) {
    if (hipMemcpyAsync(logits, m->logits.p, (size_t)m->vocab * sizeof(float), hipMemcpyDeviceToHost, m->stream) !=
            hipSuccess ||
        hipStreamSynchronize(m->stream) != hipSuccess)
      return fail(SHAINET_HIP_ERR_RUNTIME, "copying the logits back failed");
    return check_error_word(m->error);
  }
  return SHAINET_HIP_OK;
}

int shainet_llama_model_generate_greedy(shainet_llama_model *m, int max_tokens, const int *stop_ids, int n_stop,
                                        int *out, int *n_out) {
  if (!m || !out || !n_out || max_tokens < 0 || (n_stop > 0 && !stop_ids))
    return fail(SHAINET_HIP_ERR_ARGUMENT, "invalid arguments");
  *n_out = 0;
  if (!m->have_logits) return fail(SHAINET_HIP_ERR_ARGUMENT, "no logits: call shainet_llama_model_run first");
  constexpr int kChunk = 16;  // steps queued between two looks at the generated ids
  if (!m->d_gen && hipMalloc((void **)&m->d_gen, kChunk * sizeof(int)) != hipSuccess)
    return fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
  const size_t need = topk_scratch_bytes(m->vocab, 1);
  if (need > m->topk_scratch_cap) {
    if (m->topk_scratch) (void)hipFree(m->topk_scratch);
    m->topk_scratch = nullptr;
    m->topk_scratch_cap = 0;
    if (hipMalloc(&m->topk_scratch, need) != hipSuccess) return fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
    m->topk_scratch_cap = need;
  }
  int host_ids[kChunk];
  while (*n_out < max_tokens) {
    const int steps = max_tokens - *n_out < kChunk ? max_tokens - *n_out : kChunk;
    const int len0 = shainet_llama_model_cache_len(m);
    for (int i = 0; i < steps; ++i) {
      // best_id = Sampler.greedy(logits) into d_gen[i]; then net.run([best_id]) reading it from there
      hipError_t e = launch_topk(m->logits.p, m->vocab, 1, true, m->topk_scratch, m->d_gen + i, nullptr, nullptr,
                                 m->stream, 0);
      if (e != hipSuccess) return fail(SHAINET_HIP_ERR_RUNTIME, std::string("argmax launch: ") + hipGetErrorString(e));
      int rc = run_device_tokens(m, m->d_gen + i, 1);
      if (rc) return rc;
    }
    if (hipMemcpyAsync(host_ids, m->d_gen, steps * sizeof(int), hipMemcpyDeviceToHost, m->stream) != hipSuccess ||
        hipStreamSynchronize(m->stream) != hipSuccess)
      return fail(SHAINET_HIP_ERR_RUNTIME, "copying the generated ids back failed");
    if (int rc = check_error_word(m->error)) return rc;
    for (int i = 0; i < steps; ++i) {
      bool stop = false;
      for (int j = 0; j < n_stop; ++j) stop = stop || host_ids[i] == stop_ids[j];
      if (stop) {
        // the device ran ahead: the caches keep the rows of the i tokens before the stop token
        for (shainet_llama_block *b : m->blocks) {
          int rc = shainet_llama_block_truncate(b, len0 + i);
          if (rc) return rc;
        }
        m->have_logits = false;  // the row on the device belongs to a later position
        return SHAINET_HIP_OK;
      }
      out[(*n_out)++] = host_ids[i];
    }
  }
  return SHAINET_HIP_OK;
}

int shainet_llama_model_set_decode_mode(shainet_llama_model *m, int mode) {
  if (!m) return fail(SHAINET_HIP_ERR_ARGUMENT, "model is null");
  if (mode != SHAINET_HIP_DECODE_AUTO && mode != SHAINET_HIP_DECODE_PER_PRODUCT && mode != SHAINET_HIP_DECODE_PERSISTENT)
    return fail(SHAINET_HIP_ERR_ARGUMENT, "mode must be one of SHAINET_HIP_DECODE_*");
  if (m->stream && hipStreamSynchronize(m->stream) != hipSuccess)
    return fail(SHAINET_HIP_ERR_RUNTIME, "hipStreamSynchronize failed");
  m->step.release();
  m->step.mode = mode;
  return SHAINET_HIP_OK;
}

int shainet_llama_model_decode_mode_in_use(shainet_llama_model *m) {
  if (!m || m->blocks.empty()) return -1;
  if (!m->step.planned) plan_model_step(m);
  return m->step.plan.ok ? SHAINET_HIP_DECODE_PERSISTENT : SHAINET_HIP_DECODE_PER_PRODUCT;
}

int shainet_llama_model_step_trace(shainet_llama_model *m, long long *out, int capacity, int *workgroups, int *per_workgroup) {
  if (!m || !workgroups || !per_workgroup) return fail(SHAINET_HIP_ERR_ARGUMENT, "null argument");
  *workgroups = m->step.n_wgs;
  *per_workgroup = 1 + kStepTraceSlots * (int)m->blocks.size();
  if (!m->step.trace) return fail(SHAINET_HIP_ERR_ARGUMENT, "no trace: set SHAINET_HIP_STEP_TRACE before the model's first decode step");
  const long long n = (long long)*workgroups * *per_workgroup;
  if (!out || capacity < n) return fail(SHAINET_HIP_ERR_CAPACITY, "the trace holds " + std::to_string(n) + " readings");
  if ((m->stream && hipStreamSynchronize(m->stream) != hipSuccess) ||
      hipMemcpy(out, m->step.trace, (size_t)n * sizeof(long long), hipMemcpyDeviceToHost) != hipSuccess)
    return fail(SHAINET_HIP_ERR_RUNTIME, "copying the trace failed");
  return SHAINET_HIP_OK;
}

int shainet_llama_model_sync(shainet_llama_model *m) {
  if (!m) return fail(SHAINET_HIP_ERR_ARGUMENT, "model is null");
  if (m->stream && hipStreamSynchronize(m->stream) != hipSuccess)
    return fail(SHAINET_HIP_ERR_RUNTIME, "hipStreamSynchronize failed");
  return check_error_word(m->error);
}

int shainet_llama_model_greedy(shainet_llama_model *m, int *token) {
  if (!m || !token) return fail(SHAINET_HIP_ERR_ARGUMENT, "null argument");
  int id = 0, count = 0;
  int rc = run_topk(m, 1, true, &id, nullptr, &count);
  if (rc) return rc;
  *token = count > 0 ? id : 0;  // best_id starts at 0 (sampler.cr:41)
  return SHAINET_HIP_OK;
}

int shainet_llama_model_repetition_penalty(shainet_llama_model *m, const int *recent_ids, int n, double penalty) {
  if (!m || (n > 0 && !recent_ids)) return fail(SHAINET_HIP_ERR_ARGUMENT, "null argument");
  if (!m->have_logits) return fail(SHAINET_HIP_ERR_ARGUMENT, "no logits: call shainet_llama_model_run first");
  if (penalty == 1.0 || n < 1) return SHAINET_HIP_OK;  // sampler.cr:64
  int rc = reserve_ints(&m->d_tokens, &m->d_tokens_cap, (size_t)n);
  if (rc) return rc;
  if (hipMemcpyAsync(m->d_tokens, recent_ids, (size_t)n * sizeof(int), hipMemcpyHostToDevice, m->stream) != hipSuccess)
    return fail(SHAINET_HIP_ERR_RUNTIME, "hipMemcpyAsync(ids) failed");
  hipError_t e = launch_repetition_penalty(m->logits.p, m->vocab, m->d_tokens, n, penalty, m->stream);
  if (e != hipSuccess) return fail(SHAINET_HIP_ERR_RUNTIME, std::string("penalty launch: ") + hipGetErrorString(e));
  return SHAINET_HIP_OK;
}

int shainet_llama_model_topk(shainet_llama_model *m, int k, int *ids, float *vals, int *count) {
  if (!m || !ids || !vals || !count) return fail(SHAINET_HIP_ERR_ARGUMENT, "null argument");
  return run_topk(m, k, false, ids, vals, count);
}

int shainet_llama_model_sample(shainet_llama_model *m, int k, double temperature, double r, int *token) {
  if (!m || !token) return fail(SHAINET_HIP_ERR_ARGUMENT, "null argument");
  if (!m->have_logits) return fail(SHAINET_HIP_ERR_ARGUMENT, "no logits: call shainet_llama_model_run first");
  if (k < 1 || k > kMaxTopK) return fail(SHAINET_HIP_ERR_ARGUMENT, "top_k must be in [1, 256]");  // sampler.cr:24
  if (!(temperature > 0.0)) return fail(SHAINET_HIP_ERR_ARGUMENT, "temperature must be > 0");     // sampler.cr:25
  const size_t need = topk_scratch_bytes(m->vocab, k);
  if (need > m->topk_scratch_cap) {
    if (m->topk_scratch) (void)hipFree(m->topk_scratch);
    m->topk_scratch = nullptr;
    m->topk_scratch_cap = 0;
    if (hipMalloc(&m->topk_scratch, need) != hipSuccess) return fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
    m->topk_scratch_cap = need;
  }
  if (!m->d_ids) {
    if (hipMalloc((void **)&m->d_ids, (kMaxTopK + 2) * sizeof(int)) != hipSuccess ||
        hipMalloc((void **)&m->d_vals, kMaxTopK * sizeof(float)) != hipSuccess)
      return fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
  }
  // dividing by a positive temperature keeps the order of the logits: the selection over v / t
  // (sampler.cr:100-115) is the selection over v
  hipError_t e = launch_topk(m->logits.p, m->vocab, k, false, m->topk_scratch, m->d_ids, m->d_vals,
                             m->d_ids + kMaxTopK, m->stream);
  if (e == hipSuccess)
    e = launch_sample_pick(m->d_ids, m->d_vals, m->d_ids + kMaxTopK, temperature, r, m->d_ids + kMaxTopK + 1, m->stream);
  if (e != hipSuccess) return fail(SHAINET_HIP_ERR_RUNTIME, std::string("sample launch: ") + hipGetErrorString(e));
  if (hipMemcpyAsync(token, m->d_ids + kMaxTopK + 1, sizeof(int), hipMemcpyDeviceToHost, m->stream) != hipSuccess ||
      hipStreamSynchronize(m->stream) != hipSuccess)
    return fail(SHAINET_HIP_ERR_RUNTIME, "copying the sampled id back failed");
  return check_error_word(m->error);
}

int shainet_llama_model_write_logits(shainet_llama_model *m, const float *logits) {
  if (!m || !logits) return fail(SHAINET_HIP_ERR_ARGUMENT, "null argument");
  if (!shainet_hip_available()) return fail(SHAINET_HIP_ERR_RUNTIME, "no gfx950 device available");
  if (!m->stream && hipStreamCreateWithFlags(&m->stream, hipStreamNonBlocking) != hipSuccess)
    return fail(SHAINET_HIP_ERR_RUNTIME, "hipStreamCreate failed");
  if (!m->logits.reserve((size_t)m->vocab)) return fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
  if (hipMemcpyAsync(m->logits.p, logits, (size_t)m->vocab * sizeof(float), hipMemcpyHostToDevice, m->stream) !=
          hipSuccess ||
      hipStreamSynchronize(m->stream) != hipSuccess)
    return fail(SHAINET_HIP_ERR_RUNTIME, "copying the logits failed");
  m->have_logits = true;
  return SHAINET_HIP_OK;
}

int shainet_llama_model_read_logits(shainet_llama_model *m, float *logits) {
  if (!m || !logits) return fail(SHAINET_HIP_ERR_ARGUMENT, "null argument");
  if (!m->have_logits) return fail(SHAINET_HIP_ERR_ARGUMENT, "no logits: call shainet_llama_model_run first");
  if (hipMemcpyAsync(logits, m->logits.p, (size_t)m->vocab * sizeof(float), hipMemcpyDeviceToHost, m->stream) !=
          hipSuccess ||
      hipStreamSynchronize(m->stream) != hipSuccess)
    return fail(SHAINET_HIP_ERR_RUNTIME, "copying the logits back failed");
  return check_error_word(m->error);
}

}  // extern "C"
