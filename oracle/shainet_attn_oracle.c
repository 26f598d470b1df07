/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement of SHAInet's LLaMA/Qwen attention
 * path, used as the parity checker for the HIP kernels and as the timed CPU
 * baseline.  Nothing in the product library links, loads or calls this file.
 *
 * Every function follows one reference routine line by line and keeps that
 * routine's number types and evaluation order:
 *   - fp32 storage everywhere, no FMA contraction (build with
 *     -ffp-contract=off -fno-fast-math);
 *   - scale, inv_freq and the QK-norm factor are computed in fp64 and rounded
 *     once to fp32;
 *   - the RoPE angle is an fp32 product, cosf/sinf of that fp32 angle;
 *   - dot products and softmax sums are fp32, sequential, ascending index;
 *   - exp is evaluated in fp64 on the fp32 difference and rounded to fp32;
 *   - the cached path normalises each softmax weight before the V sum.
 *
 * Pinning (what each function is checked against, see tests/test_oracle_*.py):
 *   orc_rope_apply           reference known answers: identity at pos 0 and
 *                            (cos 1, sin 1) for hd=4,pos=1 (spec/rope_kv_cache_spec.cr:5-26);
 *                            pair-norm preservation; relative-position property.
 *   orc_inv_freq / llama3    closed form theta^(-2i/hd); transformers' rope
 *                            init fixtures (tests/golden).
 *   orc_head_rmsnorm         RMSNorm closed form in fp64; unit RMS for w=1;
 *                            Qwen3 attention fixture from transformers.
 *   orc_add_bias             nil bias == zero bias; size mismatch is an error
 *                            (spec/llama_qkv_bias_spec.cr:8-72).
 *   K-RoPE + append          cache invariants (length, row index = position,
 *                            V stored un-rotated), clear + re-run is bit-identical,
 *                            chunking invariance.
 *   orc_attention_heads_cpu  brute-force fp64 softmax attention; closed-form
 *                            special cases; torch SDPA; cached == full recompute
 *                            (spec/rope_kv_cache_spec.cr:29-59); LLaMA/Qwen3
 *                            attention fixtures from transformers.
 *   orc_attention_full       same fixtures and cached == full.
 *   orc_matmul / orc_rmsnorm / orc_swiglu   numpy fp64 closed forms; tiny-llama
 *                            end-to-end hidden states from transformers.
 *   orc_embed / orc_logits_last   row gather and numpy fp64 closed forms; tiny-llama
 *                            end-to-end logits from transformers.
 *   orc_greedy / orc_repetition_penalty / orc_topk / orc_sample
 *                            every known answer of spec/sampler_spec.cr; brute force
 *                            (numpy sort) on random rows with ties, NaN and infinities;
 *                            the empirical distribution of orc_sample against the
 *                            temperature softmax.
 * The bit patterns of the sequential fp32 sums and of libm's cosf/sinf/exp/pow
 * as Crystal links them can only be pinned by running the reference, which is
 * not possible without a Crystal compiler; they are restated in the same order
 * with the same libm calls and asserted against the invariants above.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define ORC_OK 0
#define ORC_ERR_ARGUMENT 1 /* the reference raises ArgumentError */
#define ORC_ERR_STATE 2

static char g_err[256];
const char *orc_last_error(void) { return g_err; }
static int fail(int code, const char *msg) {
  snprintf(g_err, sizeof g_err, "%s", msg);
  return code;
}

/* ------------------------------------------------------------------ */
/* SimpleMatrix#* : fp64 accumulate of exact fp32xfp32 products, ascending k,
 * rounded once to fp32.  src/shainet/math/simple_matrix.cr:61-74 (with
 * [] returning Float64, 27-29, and []= rounding to fp32, 35-37). */
void orc_matmul(const float *a, const float *b, float *c, int m, int k, int n) {
  for (int i = 0; i < m; ++i)
    for (int j = 0; j < n; ++j) {
      double sum = 0.0;
      for (int p = 0; p < k; ++p)
        sum += (double)a[(size_t)i * k + p] * (double)b[(size_t)p * n + j];
      c[(size_t)i * n + j] = (float)sum;
    }
}

/* RMSNorm#forward : src/shainet/transformer/rms_norm.cr:18-37. */
void orc_rmsnorm(const float *x, const float *gamma, float *out, int rows, int cols, double eps) {
  for (int i = 0; i < rows; ++i) {
    double sq = 0.0;
    for (int j = 0; j < cols; ++j) {
      double v = (double)x[(size_t)i * cols + j];
      sq += v * v;
    }
    double rms = sqrt(sq / (double)cols + eps);
    for (int j = 0; j < cols; ++j)
      out[(size_t)i * cols + j] = (float)(((double)x[(size_t)i * cols + j] / rms) * (double)gamma[j]);
  }
}

/* SwiGLUFF#forward(SimpleMatrix) : src/shainet/transformer/swiglu_ff.cr:76-91. */
void orc_swiglu(const float *x, const float *gate_w, const float *up_w, const float *down_w,
                float *out, int rows, int d, int hidden) {
  float *gate = malloc(sizeof(float) * (size_t)rows * hidden);
  float *up = malloc(sizeof(float) * (size_t)rows * hidden);
  orc_matmul(x, gate_w, gate, rows, d, hidden);
  orc_matmul(x, up_w, up, rows, d, hidden);
  for (size_t i = 0; i < (size_t)rows * hidden; ++i) {
    double g = (double)gate[i];
    gate[i] = (float)((g / (1.0 + exp(-g))) * (double)up[i]);
  }
  orc_matmul(gate, down_w, out, rows, hidden, d);
  free(gate);
  free(up);
}

/* RoPE.apply : src/shainet/transformer/rope.cr:7-33.  All fp64, stored fp32;
 * an odd trailing column is copied through. */
void orc_rope_apply(const float *x, float *out, int seq_len, int head_dim, int start_pos, double theta) {
  int half = head_dim / 2;
  for (int pos = 0; pos < seq_len; ++pos) {
    int actual = pos + start_pos;
    for (int i = 0; i < half; ++i) {
      double freq = 1.0 / pow(theta, 2.0 * i / head_dim);
      double angle = actual * freq;
      double c = cos(angle), s = sin(angle);
      double x0 = (double)x[(size_t)pos * head_dim + i];
      double x1 = (double)x[(size_t)pos * head_dim + i + half];
      out[(size_t)pos * head_dim + i] = (float)(x0 * c - x1 * s);
      out[(size_t)pos * head_dim + i + half] = (float)(x1 * c + x0 * s);
    }
    if (head_dim & 1) out[(size_t)pos * head_dim + head_dim - 1] = x[(size_t)pos * head_dim + head_dim - 1];
  }
}

/* HFLoader.compute_rope_freqs, llama3 branch : src/shainet/hf_loader.cr:235-265. */
void orc_llama3_rope_freqs(double theta, int head_dim, double factor, double low_freq_factor,
                           double high_freq_factor, double old_ctx, float *out) {
  double low_freq_wavelen = old_ctx / low_freq_factor;
  double high_freq_wavelen = old_ctx / high_freq_factor;
  int half = head_dim / 2;
  for (int i = 0; i < half; ++i) {
    double inv = 1.0 / pow(theta, 2.0 * i / head_dim);
    double wavelen = 2.0 * M_PI / inv;
    double new_inv;
    if (wavelen < high_freq_wavelen)
      new_inv = inv;
    else if (wavelen > low_freq_wavelen)
      new_inv = inv / factor;
    else {
      double smooth = (old_ctx / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor);
      new_inv = (1.0 - smooth) * inv / factor + smooth * inv;
    }
    out[i] = (float)new_inv;
  }
}

/* ------------------------------------------------------------------ */
/* LlamaBlock state that the attention path reads: llama_block.cr:7-48, 73-108. */
typedef struct {
  int d_model, num_heads, num_kv_heads, head_dim, q_dim, kv_dim;
  double rope_theta;
  double qk_norm_eps;
  float *rope_freqs;        /* nil or [head_dim/2] */
  float *q_norm, *k_norm;   /* nil or [head_dim]; *_len is the array's size */
  int q_norm_len, k_norm_len;
  float *w_q, *w_k, *w_v, *w_o; /* [d_model,q_dim] [d_model,kv_dim] x2 [q_dim,d_model] */
  float *b_q, *b_k, *b_v;
  int b_q_len, b_k_len, b_v_len;
  float **k_cache, **v_cache; /* [num_kv_heads][cache_len*head_dim], growing */
  int cache_len;
  size_t cache_cap; /* floats allocated per kv head */
} OrcBlock;

/* LlamaBlock#initialize : llama_block.cr:73-108 (argument checks 80-89). */
OrcBlock *orc_block_new(int d_model, int num_heads, int num_kv_heads, int head_dim /*0 = nil*/,
                        double eps, double rope_theta) {
  if (!(num_kv_heads > 0 && num_heads % num_kv_heads == 0)) {
    fail(ORC_ERR_ARGUMENT, "num_heads must be divisible by num_kv_heads");
    return NULL;
  }
  if (head_dim < 0) {
    fail(ORC_ERR_ARGUMENT, "head_dim must be positive");
    return NULL;
  }
  if (head_dim == 0) {
    if (d_model % num_heads != 0) {
      fail(ORC_ERR_ARGUMENT, "d_model must be divisible by num_heads");
      return NULL;
    }
    head_dim = d_model / num_heads;
  }
  OrcBlock *b = calloc(1, sizeof *b);
  b->d_model = d_model;
  b->num_heads = num_heads;
  b->num_kv_heads = num_kv_heads;
  b->head_dim = head_dim;
  b->q_dim = num_heads * head_dim;
  b->kv_dim = num_kv_heads * head_dim;
  b->rope_theta = rope_theta;
  b->qk_norm_eps = eps;
  b->k_cache = calloc((size_t)num_kv_heads, sizeof(float *));
  b->v_cache = calloc((size_t)num_kv_heads, sizeof(float *));
  return b;
}

static void set_vec(float **dst, int *len, const float *src, int n) {
  free(*dst);
  *dst = NULL;
  if (len) *len = 0;
  if (src && n >= 0) {
    *dst = malloc(sizeof(float) * (size_t)(n > 0 ? n : 1));
    memcpy(*dst, src, sizeof(float) * (size_t)n);
    if (len) *len = n;
  }
}

void orc_block_free(OrcBlock *b) {
  if (!b) return;
  for (int c = 0; c < b->num_kv_heads; ++c) {
    free(b->k_cache[c]);
    free(b->v_cache[c]);
  }
  free(b->k_cache); free(b->v_cache);
  free(b->rope_freqs); free(b->q_norm); free(b->k_norm);
  free(b->w_q); free(b->w_k); free(b->w_v); free(b->w_o);
  free(b->b_q); free(b->b_k); free(b->b_v);
  free(b);
}

void orc_block_set_rope(OrcBlock *b, double theta, const float *freqs /*nil or [hd/2]*/) {
  b->rope_theta = theta;
  set_vec(&b->rope_freqs, NULL, freqs, b->head_dim / 2);
}
void orc_block_set_qk_norm(OrcBlock *b, const float *qn, int qn_len, const float *kn, int kn_len) {
  set_vec(&b->q_norm, &b->q_norm_len, qn, qn_len);
  set_vec(&b->k_norm, &b->k_norm_len, kn, kn_len);
}
void orc_block_set_bias(OrcBlock *b, const float *bq, int bq_len, const float *bk, int bk_len,
                        const float *bv, int bv_len) {
  set_vec(&b->b_q, &b->b_q_len, bq, bq_len);
  set_vec(&b->b_k, &b->b_k_len, bk, bk_len);
  set_vec(&b->b_v, &b->b_v_len, bv, bv_len);
}
void orc_block_set_weights(OrcBlock *b, const float *wq, const float *wk, const float *wv, const float *wo) {
  set_vec(&b->w_q, NULL, wq, b->d_model * b->q_dim);
  set_vec(&b->w_k, NULL, wk, b->d_model * b->kv_dim);
  set_vec(&b->w_v, NULL, wv, b->d_model * b->kv_dim);
  set_vec(&b->w_o, NULL, wo, b->q_dim * b->d_model);
}

/* LlamaBlock#clear_cache! : llama_block.cr:116-122. */
void orc_block_clear_cache(OrcBlock *b) { b->cache_len = 0; }
int orc_block_cache_len(const OrcBlock *b) { return b->cache_len; }
/* Read access for tests: row-major [cache_len, head_dim] of one kv head. */
const float *orc_block_k_cache(const OrcBlock *b, int kv_h) { return b->k_cache[kv_h]; }
const float *orc_block_v_cache(const OrcBlock *b, int kv_h) { return b->v_cache[kv_h]; }

static void cache_reserve(OrcBlock *b, int total_len) {
  size_t need = (size_t)total_len * b->head_dim;
  if (need <= b->cache_cap) return;
  size_t cap = b->cache_cap ? b->cache_cap : 1024;
  while (cap < need) cap *= 2;
  for (int c = 0; c < b->num_kv_heads; ++c) {
    b->k_cache[c] = realloc(b->k_cache[c], cap * sizeof(float));
    b->v_cache[c] = realloc(b->v_cache[c], cap * sizeof(float));
  }
  b->cache_cap = cap;
}

/* Test-only: put `n` already-rotated K rows and V rows ([num_kv_heads][n][hd])
 * straight into the cache, replacing its contents.  The reference's cache is
 * private state with no setter (llama_block.cr:46-48); benchmark configurations
 * that start from a pre-filled cache need one. */
void orc_block_fill_cache(OrcBlock *b, const float *k_rows, const float *v_rows, int n) {
  cache_reserve(b, n);
  size_t row = (size_t)n * b->head_dim;
  for (int c = 0; c < b->num_kv_heads; ++c) {
    memcpy(b->k_cache[c], k_rows + c * row, row * sizeof(float));
    memcpy(b->v_cache[c], v_rows + c * row, row * sizeof(float));
  }
  b->cache_len = n;
}

/* inv_freq : llama_block.cr:669-675. */
static inline float inv_freq(const OrcBlock *b, int i) {
  if (b->rope_freqs) return b->rope_freqs[i];
  return (float)(1.0 / pow(b->rope_theta, 2.0 * i / b->head_dim));
}
void orc_inv_freq(const OrcBlock *b, float *out) {
  for (int i = 0; i < b->head_dim / 2; ++i) out[i] = inv_freq(b, i);
}

/* add_bias! : llama_block.cr:585-601. */
static int add_bias(float *m, int rows, int cols, const float *bias, int bias_len) {
  if (!bias) return ORC_OK;
  if (bias_len != cols) return fail(ORC_ERR_ARGUMENT, "bias size does not match matrix cols");
  for (int r = 0; r < rows; ++r)
    for (int c = 0; c < cols; ++c) m[(size_t)r * cols + c] += bias[c];
  return ORC_OK;
}

/* apply_head_rmsnorm! : llama_block.cr:615-641. */
static int head_rmsnorm(const OrcBlock *b, float *m, int rows, int cols, int nheads, const float *w, int w_len) {
  if (!w) return ORC_OK;
  int hd = b->head_dim;
  if (w_len != hd) return fail(ORC_ERR_ARGUMENT, "qk_norm weight size != head_dim");
  double eps = b->qk_norm_eps;
  for (int r = 0; r < rows; ++r)
    for (int h = 0; h < nheads; ++h) {
      float *p = m + (size_t)r * cols + (size_t)h * hd;
      float ss = 0.0f;
      for (int d = 0; d < hd; ++d) {
        float v = p[d];
        ss += v * v;
      }
      float mean = ss / (float)hd;                          /* Float32 / Int32 -> Float32 */
      float inv = (float)(1.0 / sqrt((double)mean + eps));  /* Float32 + Float64 -> Float64 */
      for (int d = 0; d < hd; ++d) p[d] = p[d] * inv * w[d];
    }
  return ORC_OK;
}
int orc_head_rmsnorm(const OrcBlock *b, float *m, int rows, int nheads, const float *w, int w_len) {
  return head_rmsnorm(b, m, rows, nheads * b->head_dim, nheads, w, w_len);
}

/* K RoPE + append : llama_block.cr:266-289. */
static void rope_append(OrcBlock *b, const float *k_new, const float *v_new, int new_tokens) {
  int hd = b->head_dim, half = hd / 2, start_pos = b->cache_len;
  cache_reserve(b, start_pos + new_tokens);
  for (int kv_h = 0; kv_h < b->num_kv_heads; ++kv_h) {
    int kv_col = kv_h * hd;
    for (int t = 0; t < new_tokens; ++t) {
      int pos = start_pos + t;
      float *krow = b->k_cache[kv_h] + (size_t)pos * hd;
      float *vrow = b->v_cache[kv_h] + (size_t)pos * hd;
      for (int d = 0; d < hd; ++d) krow[d] = 0.0f; /* Array.new(head_dim, 0.0): an odd last slot stays 0 */
      for (int i = 0; i < half; ++i) {
        float freq = inv_freq(b, i);
        float angle = (float)pos * freq;
        float c = cosf(angle), s = sinf(angle);
        float x0 = k_new[(size_t)t * b->kv_dim + kv_col + i];
        float x1 = k_new[(size_t)t * b->kv_dim + kv_col + i + half];
        krow[i] = x0 * c - x1 * s;
        krow[i + half] = x1 * c + x0 * s;
      }
      for (int d = 0; d < hd; ++d) vrow[d] = v_new[(size_t)t * b->kv_dim + kv_col + d];
    }
  }
  b->cache_len = start_pos + new_tokens;
}

/* attention_heads_cpu for query heads [h0, h1) : llama_block.cr:302-401.
 * Heads are independent, so a caller may run disjoint head ranges on several
 * threads without changing any result. */
void orc_attention_heads_cpu(const OrcBlock *b, const float *q_full, float *output, int new_tokens,
                             int start_pos, int total_len, float scale, int h0, int h1) {
  int hd = b->head_dim, half = hd / 2, dm = b->q_dim;
  int heads_per_kv = b->num_heads / b->num_kv_heads;
  float *q_rot = calloc((size_t)hd, sizeof(float)); /* zero-filled: odd last slot stays 0 */
  float *scores = malloc(sizeof(float) * (size_t)(total_len > 0 ? total_len : 1));
  float *out = malloc(sizeof(float) * (size_t)hd);
  for (int h = h0; h < h1; ++h) {
    int q_col = h * hd;
    const float *kptr = b->k_cache[h / heads_per_kv];
    const float *vptr = b->v_cache[h / heads_per_kv];
    for (int i = 0; i < new_tokens; ++i) {
      int pos = start_pos + i;
      size_t qrow = (size_t)i * dm + q_col;
      for (int idx = 0; idx < half; ++idx) {
        float freq = inv_freq(b, idx);
        float angle = (float)pos * freq;
        float c = cosf(angle), s = sinf(angle);
        float x0 = q_full[qrow + idx], x1 = q_full[qrow + idx + half];
        q_rot[idx] = x0 * c - x1 * s;
        q_rot[idx + half] = x1 * c + x0 * s;
      }
      int visible = start_pos + i + 1;
      float max_val = -INFINITY;
      for (int j = 0; j < visible; ++j) {
        const float *k = kptr + (size_t)j * hd;
        float dot = 0.0f;
        for (int d = 0; d < hd; ++d) dot += q_rot[d] * k[d];
        float sv = dot * scale;
        scores[j] = sv;
        if (sv > max_val) max_val = sv;
      }
      float exp_sum = 0.0f;
      for (int j = 0; j < visible; ++j) {
        float e = (float)exp((double)(scores[j] - max_val));
        scores[j] = e;
        exp_sum += e;
      }
      float inv_sum = 1.0f / exp_sum;
      for (int d = 0; d < hd; ++d) out[d] = 0.0f;
      for (int j = 0; j < visible; ++j) {
        float w = scores[j] * inv_sum;
        const float *v = vptr + (size_t)j * hd;
        for (int d = 0; d < hd; ++d) out[d] += w * v[d];
      }
      for (int d = 0; d < hd; ++d) output[(size_t)i * dm + q_col + d] = out[d];
    }
  }
  free(q_rot); free(scores); free(out);
}

/* The query rotation alone (llama_block.cr:332-344), for every head and row of
 * q_full [T,q_dim] (after bias and QK-norm): lets a test compare the device's
 * rotated rows bit for bit. */
void orc_rotate_q(const OrcBlock *b, const float *q_full, float *q_rot, int new_tokens, int start_pos) {
  int hd = b->head_dim, half = hd / 2, dm = b->q_dim;
  memset(q_rot, 0, sizeof(float) * (size_t)new_tokens * dm);
  for (int h = 0; h < b->num_heads; ++h)
    for (int i = 0; i < new_tokens; ++i) {
      int pos = start_pos + i;
      size_t qrow = (size_t)i * dm + (size_t)h * hd;
      for (int idx = 0; idx < half; ++idx) {
        float freq = inv_freq(b, idx);
        float angle = (float)pos * freq;
        float c = cosf(angle), s = sinf(angle);
        float x0 = q_full[qrow + idx], x1 = q_full[qrow + idx + half];
        q_rot[qrow + idx] = x0 * c - x1 * s;
        q_rot[qrow + idx + half] = x1 * c + x0 * s;
      }
    }
}

/* scale : llama_block.cr:249. */
float orc_scale(const OrcBlock *b) { return (float)(1.0 / sqrt((double)b->head_dim)); }

/* Steps 256-289 of attention_cached_cpu on already projected rows: bias, QK-norm,
 * K RoPE + append.  q_full [T,q_dim], k_new/v_new [T,kv_dim] are modified in
 * place exactly as the reference modifies them.  Returns start_pos in *start_pos. */
int orc_block_prepare_append(OrcBlock *b, float *q_full, float *k_new, float *v_new, int new_tokens,
                             int *start_pos) {
  int rc;
  if ((rc = add_bias(q_full, new_tokens, b->q_dim, b->b_q, b->b_q_len))) return rc;
  if ((rc = add_bias(k_new, new_tokens, b->kv_dim, b->b_k, b->b_k_len))) return rc;
  if ((rc = add_bias(v_new, new_tokens, b->kv_dim, b->b_v, b->b_v_len))) return rc;
  if ((rc = head_rmsnorm(b, q_full, new_tokens, b->q_dim, b->num_heads, b->q_norm, b->q_norm_len))) return rc;
  if ((rc = head_rmsnorm(b, k_new, new_tokens, b->kv_dim, b->num_kv_heads, b->k_norm, b->k_norm_len))) return rc;
  *start_pos = b->cache_len;
  rope_append(b, k_new, v_new, new_tokens);
  return ORC_OK;
}

/* attention_cached_cpu from the projections' outputs to the head loop's output
 * (llama_block.cr:256-296) on one thread.  output is [T, q_dim]. */
int orc_block_attention_cached_qkv(OrcBlock *b, float *q_full, float *k_new, float *v_new,
                                   int new_tokens, float *output) {
  int start_pos, rc;
  if ((rc = orc_block_prepare_append(b, q_full, k_new, v_new, new_tokens, &start_pos))) return rc;
  orc_attention_heads_cpu(b, q_full, output, new_tokens, start_pos, b->cache_len, orc_scale(b), 0, b->num_heads);
  return ORC_OK;
}

/* attention_cached_cpu, whole : llama_block.cr:246-299.  x [T,d_model] -> out [T,d_model]. */
int orc_block_attention_cached(OrcBlock *b, const float *x, int new_tokens, float *out) {
  if (!b->w_q) return fail(ORC_ERR_STATE, "weights not set");
  size_t T = (size_t)new_tokens;
  float *q = malloc(sizeof(float) * T * b->q_dim), *k = malloc(sizeof(float) * T * b->kv_dim);
  float *v = malloc(sizeof(float) * T * b->kv_dim), *o = malloc(sizeof(float) * T * b->q_dim);
  orc_matmul(x, b->w_q, q, new_tokens, b->d_model, b->q_dim);
  orc_matmul(x, b->w_k, k, new_tokens, b->d_model, b->kv_dim);
  orc_matmul(x, b->w_v, v, new_tokens, b->d_model, b->kv_dim);
  int rc = orc_block_attention_cached_qkv(b, q, k, v, new_tokens, o);
  if (!rc) orc_matmul(o, b->w_o, out, new_tokens, b->q_dim, b->d_model);
  free(q); free(k); free(v); free(o);
  return rc;
}

/* apply_rope! : llama_block.cr:678-693, on a [rows, head_dim] head slice. */
static void apply_rope(const OrcBlock *b, float *m, int rows, int start_pos) {
  int hd = b->head_dim, half = hd / 2;
  for (int pos = 0; pos < rows; ++pos) {
    int actual = pos + start_pos;
    for (int i = 0; i < half; ++i) {
      float freq = inv_freq(b, i);
      float angle = (float)actual * freq;
      float c = cosf(angle), s = sinf(angle);
      float x0 = m[(size_t)pos * hd + i], x1 = m[(size_t)pos * hd + i + half];
      m[(size_t)pos * hd + i] = x0 * c - x1 * s;
      m[(size_t)pos * hd + i + half] = x1 * c + x0 * s;
    }
  }
}

/* attention_full_cpu from the projections' outputs to `output` [T,q_dim]:
 * llama_block.cr:217-240 with extract_head 662-666 and causal_attention! 696-716.
 * The [T,T] score product and the weights x V product accumulate in fp64
 * (SimpleMatrix#*), including the masked upper triangle (whose weights are 0). */
int orc_block_attention_full_qkv(const OrcBlock *b, float *q_full, float *k_full, float *v_full,
                                 int seq_len, float *output) {
  int rc, hd = b->head_dim;
  if ((rc = add_bias(q_full, seq_len, b->q_dim, b->b_q, b->b_q_len))) return rc;
  if ((rc = add_bias(k_full, seq_len, b->kv_dim, b->b_k, b->b_k_len))) return rc;
  if ((rc = add_bias(v_full, seq_len, b->kv_dim, b->b_v, b->b_v_len))) return rc;
  if ((rc = head_rmsnorm(b, q_full, seq_len, b->q_dim, b->num_heads, b->q_norm, b->q_norm_len))) return rc;
  if ((rc = head_rmsnorm(b, k_full, seq_len, b->kv_dim, b->num_kv_heads, b->k_norm, b->k_norm_len))) return rc;
  float scale = (float)(1.0 / sqrt((double)hd));
  int heads_per_kv = b->num_heads / b->num_kv_heads;
  size_t T = (size_t)seq_len;
  float *q_h = malloc(sizeof(float) * T * hd), *k_h = malloc(sizeof(float) * T * hd);
  float *v_h = malloc(sizeof(float) * T * hd), *k_t = malloc(sizeof(float) * T * hd);
  float *scores = malloc(sizeof(float) * T * T), *w = calloc(T * T, sizeof(float));
  float *attn_out = malloc(sizeof(float) * T * hd);
  for (int h = 0; h < b->num_heads; ++h) {
    int q_col = h * hd, kv_col = (h / heads_per_kv) * hd;
    for (int r = 0; r < seq_len; ++r)
      for (int c = 0; c < hd; ++c) {
        q_h[(size_t)r * hd + c] = q_full[(size_t)r * b->q_dim + q_col + c];
        k_h[(size_t)r * hd + c] = k_full[(size_t)r * b->kv_dim + kv_col + c];
        v_h[(size_t)r * hd + c] = v_full[(size_t)r * b->kv_dim + kv_col + c];
      }
    apply_rope(b, q_h, seq_len, 0);
    apply_rope(b, k_h, seq_len, 0);
    for (int r = 0; r < seq_len; ++r)
      for (int c = 0; c < hd; ++c) k_t[(size_t)c * T + r] = k_h[(size_t)r * hd + c];
    orc_matmul(q_h, k_t, scores, seq_len, hd, seq_len);
    memset(w, 0, sizeof(float) * T * T);
    for (int i = 0; i < seq_len; ++i) {
      float max_val = -INFINITY;
      for (int j = 0; j <= i; ++j) {
        float sv = scores[(size_t)i * T + j] * scale;
        if (sv > max_val) max_val = sv;
      }
      float exp_sum = 0.0f;
      for (int j = 0; j <= i; ++j) {
        float e = (float)exp((double)(scores[(size_t)i * T + j] * scale - max_val));
        w[(size_t)i * T + j] = e;
        exp_sum += e;
      }
      for (int j = 0; j <= i; ++j) w[(size_t)i * T + j] = w[(size_t)i * T + j] / exp_sum;
    }
    orc_matmul(w, v_h, attn_out, seq_len, seq_len, hd);
    for (int s = 0; s < seq_len; ++s)
      for (int d = 0; d < hd; ++d) output[(size_t)s * b->q_dim + q_col + d] = attn_out[(size_t)s * hd + d];
  }
  free(q_h); free(k_h); free(v_h); free(k_t); free(scores); free(w); free(attn_out);
  return ORC_OK;
}

/* attention_full_cpu, whole : llama_block.cr:209-243. */
int orc_block_attention_full(const OrcBlock *b, const float *x, int seq_len, float *out) {
  if (!b->w_q) return fail(ORC_ERR_STATE, "weights not set");
  size_t T = (size_t)seq_len;
  float *q = malloc(sizeof(float) * T * b->q_dim), *k = malloc(sizeof(float) * T * b->kv_dim);
  float *v = malloc(sizeof(float) * T * b->kv_dim), *o = malloc(sizeof(float) * T * b->q_dim);
  orc_matmul(x, b->w_q, q, seq_len, b->d_model, b->q_dim);
  orc_matmul(x, b->w_k, k, seq_len, b->d_model, b->kv_dim);
  orc_matmul(x, b->w_v, v, seq_len, b->d_model, b->kv_dim);
  int rc = orc_block_attention_full_qkv(b, q, k, v, seq_len, o);
  if (!rc) orc_matmul(o, b->w_o, out, seq_len, b->q_dim, b->d_model);
  free(q); free(k); free(v); free(o);
  return rc;
}

/* LlamaBlock#forward_cached / #forward with a dense SwiGLU FFN :
 * llama_block.cr:179-196.  `+` on SimpleMatrix adds in fp64 and rounds
 * (simple_matrix.cr:39-48).  cached != 0 selects forward_cached. */
int orc_block_forward(OrcBlock *b, const float *x, int rows, const float *norm1, const float *norm2,
                      double norm_eps, const float *gate_w, const float *up_w, const float *down_w,
                      int ff_hidden, int cached, float *out) {
  int d = b->d_model;
  size_t n = (size_t)rows * d;
  float *normed = malloc(sizeof(float) * n), *attn = malloc(sizeof(float) * n);
  float *h = malloc(sizeof(float) * n), *ff = malloc(sizeof(float) * n);
  orc_rmsnorm(x, norm1, normed, rows, d, norm_eps);
  int rc = cached ? orc_block_attention_cached(b, normed, rows, attn) : orc_block_attention_full(b, normed, rows, attn);
  if (!rc) {
    for (size_t i = 0; i < n; ++i) h[i] = (float)((double)x[i] + (double)attn[i]);
    orc_rmsnorm(h, norm2, normed, rows, d, norm_eps);
    orc_swiglu(normed, gate_w, up_w, down_w, ff, rows, d, ff_hidden);
    for (size_t i = 0; i < n; ++i) out[i] = (float)((double)h[i] + (double)ff[i]);
  }
  free(normed); free(attn); free(h); free(ff);
  return rc;
}

/* ------------------------------------------------------------------ */
/* After the last block: Network#run, src/shainet/basic/network_run.cr:185-226,
 * and Sampler, src/shainet/text/sampler.cr. */

/* EmbeddingLayer#embed_cpu : src/shainet/text/embedding_layer.cr:129-153. */
int orc_embed(const float *table, int vocab, const int *ids, int n, int d, float *out) {
  for (int r = 0; r < n; ++r) {
    if (ids[r] < 0 || ids[r] >= vocab) return fail(ORC_ERR_ARGUMENT, "token id outside the table (IndexError)");
    memcpy(out + (size_t)r * d, table + (size_t)ids[r] * d, sizeof(float) * (size_t)d);
  }
  return ORC_OK;
}

/* network_run.cr:205-226 : final norm over all rows (when the network has one),
 * last row times the [d, vocab] output matrix (safe_output_transform, 1390-1404,
 * SimpleMatrix#*), then matrix[i, j] += b[0, j] through the fp64 accessors. */
void orc_logits_last(const float *h, int rows, int d, const float *final_gamma, double eps, const float *w,
                     int vocab, const float *bias, float *logits) {
  float *normed = malloc(sizeof(float) * (size_t)rows * d);
  const float *src = h;
  if (final_gamma) {
    orc_rmsnorm(h, final_gamma, normed, rows, d, eps);
    src = normed;
  }
  orc_matmul(src + (size_t)(rows - 1) * d, w, logits, 1, d, vocab);
  if (bias)
    for (int j = 0; j < vocab; ++j) logits[j] = (float)((double)logits[j] + (double)bias[j]);
  free(normed);
}

/* Sampler.greedy : sampler.cr:38-53. */
int orc_greedy(const float *logits, int cols) {
  int best_id = 0;
  float best = -INFINITY;
  for (int j = 0; j < cols; ++j) {
    float v = logits[j];
    if (isfinite(v) && v > best) {
      best = v;
      best_id = j;
    }
  }
  return best_id;
}

/* Sampler#apply_repetition_penalty! : sampler.cr:59-81.  window < 0 = all ids. */
void orc_repetition_penalty(float *logits, int cols, const int *ids, int n, int window, double p) {
  if (p == 1.0) return;
  int start = window < 0 ? 0 : n - window;
  if (start < 0) start = 0;
  for (int i = start; i < n; ++i) {
    int id = ids[i];
    if (0 <= id && id < cols) {
      float v = logits[id];
      logits[id] = (float)(v > 0 ? (double)v / p : (double)v * p);
    }
  }
}

/* The selection loop of Sampler#sample : sampler.cr:88-116.  A sorted buffer of
 * at most k (value / temperature, id) pairs, descending; bsearch_index { |x| x < v }
 * is the first slot holding a smaller value, so equal values keep arrival order.
 * Returns the number of survivors. */
int orc_topk(const float *logits, int cols, int k, double t, int *ids, double *vals) {
  int sz = 0;
  for (int j = 0; j < cols; ++j) {
    double v = (double)logits[j] / t;
    if (isnan(v)) continue;
    if (sz == k && !(v > vals[k - 1])) continue;
    int lo = 0, hi = sz; /* first index with vals[i] < v, or sz */
    while (lo < hi) {
      int mid = (lo + hi) / 2;
      if (vals[mid] < v) hi = mid; else lo = mid + 1;
    }
    int last = sz < k ? sz : k - 1; /* insert at lo, dropping the tail when full */
    for (int i = last; i > lo; --i) {
      vals[i] = vals[i - 1];
      ids[i] = ids[i - 1];
    }
    vals[lo] = v;
    ids[lo] = j;
    if (sz < k) ++sz;
  }
  return sz;
}

/* Sampler#sample : sampler.cr:88-150, with the uniform draw r handed in. */
int orc_sample(const float *logits, int cols, int k, double t, double r) {
  int *ids = malloc(sizeof(int) * (size_t)k);
  double *vals = malloc(sizeof(double) * (size_t)k);
  int szk = orc_topk(logits, cols, k, t, ids, vals);
  int best_id = 0;
  if (szk > 0) {
    double max_val = vals[0], sum = 0.0;
    for (int i = 0; i < szk; ++i) {
      vals[i] = exp(vals[i] - max_val);
      sum += vals[i];
    }
    double inv_sum = 1.0 / sum, cumulative = 0.0;
    best_id = ids[szk - 1];
    for (int i = 0; i < szk; ++i) {
      cumulative += vals[i] * inv_sum;
      if (r <= cumulative) {
        best_id = ids[i];
        break;
      }
    }
  }
  free(ids);
  free(vals);
  return best_id;
}
