// C ABI of libshainet_hip_kernels.so (declared in include/shainet_hip_attn.h).
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>
#include <new>
#include <vector>

#include "../../include/shainet_hip_attn.h"
#include "attn_kernels.hpp"
#include "block_kernels.hpp"

using namespace shainet;

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof g_err, fmt, ap);
  va_end(ap);
  return code;
}

}  // namespace

// for the other translation units of the library
void shainet_hip_set_error(int code, const char *msg) { fail(code, "%s", msg); }

namespace shainet {

int *alloc_error_word() {
  int *p = nullptr;
  if (hipHostMalloc((void **)&p, sizeof(int), hipHostMallocPortable) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  *p = 0;
  return p;
}

void free_error_word(int *w) {
  if (w) (void)hipHostFree(w);
}

int check_error_word(int *w) {
  if (!w || *(volatile int *)w == 0) return SHAINET_HIP_OK;
  const int what = *(volatile int *)w;
  *(volatile int *)w = 0;
  if (what == 2)
    return fail(SHAINET_HIP_ERR_CAPACITY,
                "a decode step found a sequence at the capacity of its cache or at the end of the context's "
                "cos/sin table: that step and the steps after it appended nothing and wrote no output");
  return fail(SHAINET_HIP_ERR_RUNTIME, "a kernel gave up waiting for the partial results of other workgroups; the results of the calls on this handle since its last wait are invalid and it must be destroyed");
}

}  // namespace shainet

namespace {

int scratch_on_current_device(unsigned char **out);  // below, with the static scratch of the entry point that allocates nothing

int hip_fail(hipError_t e, const char *what) {
  return fail(e == hipErrorOutOfMemory ? SHAINET_HIP_ERR_ALLOC : SHAINET_HIP_ERR_RUNTIME, "%s: %s", what,
              hipGetErrorString(e));
}

#define HIP_TRY(expr)                                  \
  do {                                                 \
    hipError_t e_ = (expr);                            \
    if (e_ != hipSuccess) return hip_fail(e_, #expr);  \
  } while (0)

// Grow-only device buffer.
struct DevBuf {
  float *p = nullptr;
  size_t cap = 0;  // floats
  int reserve(size_t n) {
    if (n <= cap) return SHAINET_HIP_OK;
    size_t want = cap ? cap : 1024;
    while (want < n) want *= 2;
    float *np = nullptr;
    hipError_t e = hipMalloc((void **)&np, want * sizeof(float));
    if (e != hipSuccess) {  // try the exact size before giving up
      want = n;
      e = hipMalloc((void **)&np, want * sizeof(float));
    }
    if (e != hipSuccess) return hip_fail(e, "hipMalloc");
    if (p) (void)hipFree(p);
    p = np;
    cap = want;
    return SHAINET_HIP_OK;
  }
  void release() {
    if (p) (void)hipFree(p);
    p = nullptr;
    cap = 0;
  }
};

// Grow-only pinned host buffer: host-pointer calls stage their rows through it, so that each
// copy to or from the device is one asynchronous DMA instead of the runtime's staged copy of
// pageable memory.
struct PinBuf {
  float *p = nullptr;
  size_t cap = 0;  // floats
  int reserve(size_t n) {
    if (n <= cap) return SHAINET_HIP_OK;
    size_t want = cap ? cap : 4096;
    while (want < n) want *= 2;
    float *np = nullptr;
    hipError_t e = hipHostMalloc((void **)&np, want * sizeof(float), hipHostMallocDefault);
    if (e != hipSuccess) return hip_fail(e, "hipHostMalloc");
    if (p) (void)hipHostFree(p);
    p = np;
    cap = want;
    return SHAINET_HIP_OK;
  }
  void release() {
    if (p) (void)hipHostFree(p);
    p = nullptr;
    cap = 0;
  }
};

}  // namespace

struct shainet_attn_ctx {
  int H, KV, g, hd;
  double eps;
  float scale;  // (float)(1.0 / sqrt((double)hd)), llama_block.cr:249
  std::vector<float> inv_freq;
  float *d_q_norm = nullptr, *d_k_norm = nullptr;
  float *d_bq = nullptr, *d_bk = nullptr, *d_bv = nullptr;
  float2 *d_rope = nullptr;
  int rope_positions = 0;
  // DecodeArgs::ahead_* of the next decode launch (shainet_attn_read_ahead); forgotten after it
  const float *ahead_w = nullptr;
  int ahead_k = 0, ahead_n = 0, ahead_wgs = 0;
  hipStream_t stream = nullptr;      // where work is issued
  hipStream_t own_stream = nullptr;  // created with the context, destroyed with it
  DevBuf q_rot, partials, in_q, in_k, in_v, out;
  PinBuf pin_in, pin_out;  // host-pointer calls: q | k | v rows on their way in, the result on its way out
  // decode split: a word per partial slot that says when it is complete (zero between launches)
  unsigned *part_flag = nullptr;
  size_t part_flag_cap = 0;
  bool test_lose_marks = false;  // SHAINET_HIP_TEST_LOSE_PARTIAL_MARKS: exercises the give-up path
  // pinned host word this context's kernels set when they give up a bounded wait; `error` is
  // the one in use: the context's own, or the one of the block or model that owns the context
  int *error = nullptr, *own_error = nullptr;
  int last_rows = 0;
  int decode_wgs_override = 0;  // 0 = default workgroup count of the decode split
  int prefill_wgs_per_cu = 0;   // 0 = default occupancy of the prefill kernel
  int prefill_splits_override = 0;  // 0 = default number of key splits of the prefill kernel
  int prefill_groups_override = 0;  // 0 = default number of wavefront groups of the prefill kernel
  bool profiling = false;
  std::vector<hipEvent_t> prof_events;  // start, stop, start, stop, ...
};

// What shainet_attn_decode_step works with: all of it allocated by shainet_kv_cache_lengths_to_device,
// none of it by the step.
struct StepState {
  int *d_len = nullptr;               // [batch] cached rows per slot, as the device counts them
  int *pin_len = nullptr;             // [batch] pinned staging for both directions
  DecodeDevicePlan *d_plan = nullptr; // rewritten by every step
  float *q_rot = nullptr;             // [batch, H, hd]
  float *partials = nullptr;          // device_plan_slots(batch, KV) slots of g columns
  unsigned *flags = nullptr;          // zero between launches
  int cap = 0;                        // the capacity the buffers above were laid out for
  // Between shainet_kv_cache_lengths_to_device and _from_device the device's lengths are the ones that count
  // (decode steps advance only those): every entry point that reads or writes the host's copy is refused.
  bool lengths_on_device = false;
};

static void release_step_state(StepState &s) {
  if (s.d_len) (void)hipFree(s.d_len);
  if (s.pin_len) (void)hipHostFree(s.pin_len);
  if (s.d_plan) (void)hipFree(s.d_plan);
  if (s.q_rot) (void)hipFree(s.q_rot);
  if (s.partials) (void)hipFree(s.partials);
  if (s.flags) (void)hipFree(s.flags);
  s = StepState();
}

struct shainet_kv_cache {
  shainet_attn_ctx *ctx;
  int batch, cap;
  float *k = nullptr, *v = nullptr;
  std::vector<int> len;
  StepState step;
};

namespace {
int refuse_while_lengths_on_device(const shainet_kv_cache *kc, const char *what) {
  if (!kc->step.lengths_on_device) return SHAINET_HIP_OK;
  return fail(SHAINET_HIP_ERR_ARGUMENT,
              "%s: the cached lengths are on the device (shainet_kv_cache_lengths_to_device); call "
              "shainet_kv_cache_lengths_from_device first", what);
}
}  // namespace

namespace {

int upload(float **dst, const float *src, size_t n) {
  if (*dst) (void)hipFree(*dst);
  *dst = nullptr;
  if (!src) return SHAINET_HIP_OK;
  HIP_TRY(hipMalloc((void **)dst, (n ? n : 1) * sizeof(float)));
  HIP_TRY(hipMemcpy(*dst, src, n * sizeof(float), hipMemcpyHostToDevice));
  return SHAINET_HIP_OK;
}

// cos/sin of (float)pos * inv_freq[i], computed with the host's libm exactly as
// llama_block.cr:274-277 does, for pos in [0, positions).
int ensure_rope_table(shainet_attn_ctx *c, int positions) {
  if (positions <= c->rope_positions) return SHAINET_HIP_OK;
  int want = c->rope_positions ? c->rope_positions : 1024;
  while (want < positions) want *= 2;
  const int half = c->hd / 2;
  if (half == 0) {
    c->rope_positions = want;
    return SHAINET_HIP_OK;
  }
  std::vector<float2> tab((size_t)want * half);
  for (int pos = 0; pos < want; ++pos)
    for (int i = 0; i < half; ++i) {
      const float angle = (float)pos * c->inv_freq[i];
      tab[(size_t)pos * half + i] = float2{cosf(angle), sinf(angle)};
    }
  float2 *np = nullptr;
  HIP_TRY(hipMalloc((void **)&np, tab.size() * sizeof(float2)));
  hipError_t e = hipMemcpy(np, tab.data(), tab.size() * sizeof(float2), hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    (void)hipFree(np);
    return hip_fail(e, "hipMemcpy(rope table)");
  }
  if (c->d_rope) {
    // kernels already queued may still read the old table
    (void)hipStreamSynchronize(c->stream);
    (void)hipFree(c->d_rope);
  }
  c->d_rope = np;
  c->rope_positions = want;
  return SHAINET_HIP_OK;
}

Shape shape_of(const shainet_attn_ctx *c, int cap) {
  Shape sh;
  sh.H = c->H;
  sh.KV = c->KV;
  sh.g = c->g;
  sh.hd = c->hd;
  sh.cap = cap;
  sh.seq_stride = (long long)c->KV * cap * c->hd;
  return sh;
}

// Zero-initialised flag words of the decode split.
int ensure_decode_flags(shainet_attn_ctx *c, size_t n, hipStream_t stream) {
  if (!c->error) {  // the handle-less context of the reference-named entry points gets its word here
    c->error = c->own_error = alloc_error_word();
    if (!c->error) return fail(SHAINET_HIP_ERR_ALLOC, "hipHostMalloc failed");
  }
  if (n <= c->part_flag_cap) return SHAINET_HIP_OK;
  size_t want = c->part_flag_cap ? c->part_flag_cap : 1024;
  while (want < n) want *= 2;
  unsigned *np = nullptr;
  const size_t words = c->test_lose_marks ? 2 * want : want;  // second half: where lost marks go
  HIP_TRY(hipMalloc((void **)&np, words * sizeof(unsigned)));
  hipError_t e = hipMemsetAsync(np, 0, words * sizeof(unsigned), stream);
  if (e != hipSuccess) {
    (void)hipFree(np);
    return hip_fail(e, "hipMemsetAsync(partial flags)");
  }
  if (c->part_flag) (void)hipFree(c->part_flag);  // hipFree waits for the device
  c->part_flag = np;
  c->part_flag_cap = want;
  return SHAINET_HIP_OK;
}

// Device memory a forward call's kernels use beyond its inputs and outputs, when the caller of
// run_attention brings it along instead of letting the context allocate it on demand.
struct Workspace {
  float *q_rot;
  size_t q_rot_floats;
  float *partials;
  size_t partial_floats;
  unsigned *flags;  // zero at launch
  size_t flag_words;
  unsigned *lost_marks;  // flag_words words: where the test of the give-up path sends the marks
};

// Attention over a cache: shared by the fused entry point and by attention_kv_f32.
// prep != nullptr: the rows are raw projection outputs; the prep kernel does bias,
// QK-norm, RoPE and the append first.  prep == nullptr: q_rot holds rotated
// queries and the cache already holds the new rows.
// ws != nullptr: nothing is allocated; the split-K decode path only.
int run_attention(shainet_attn_ctx *c, const float *q_rot, float *kc, float *vc, float *out, SeqTable &st,
                  const Shape &sh, int total_tokens, float scale, hipStream_t stream, const PrepArgs *prep,
                  const Workspace *ws = nullptr) {
  const Path path = choose_path(st, sh);
  if (ws && path != Path::kDecodeSplitK)
    return fail(SHAINET_HIP_ERR_ARGUMENT,
                "the entry point that allocates nothing takes decode calls only: at most %d new rows per sequence "
                "with this head geometry (head_dim a multiple of 4 up to 256)", 32 / (sh.g < 1 ? 1 : sh.g));
  // the MFMA prefill kernels address the rows of a (sequence, kv head) by a 32-bit byte offset;
  // said before anything is written to the cache
  if (path == Path::kPrefillMfma && (long long)sh.cap * sh.hd * 4 > 0xffffffffLL)
    return fail(SHAINET_HIP_ERR_ARGUMENT,
                "capacity %d x head_dim %d x 4 bytes is 4 GiB or more: not supported for more than 16/g new rows",
                sh.cap, sh.hd);
  hipError_t e;
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  if (c->profiling && !ws) {
    if (hipEventCreate(&ev0) != hipSuccess || hipEventCreate(&ev1) != hipSuccess)
      return fail(SHAINET_HIP_ERR_RUNTIME, "hipEventCreate failed");
    c->prof_events.push_back(ev0);
    c->prof_events.push_back(ev1);
  }
  if (path == Path::kDecodeSplitK) {
    SeqTable att;  // the attention kernel's view: long runs of new rows as two entries
    if (!decode_entries(st, sh, att)) return fail(SHAINET_HIP_ERR_RUNTIME, "decode entries do not fit");
    const DecodePlan plan = plan_decode(att, sh, c->decode_wgs_override);
    DecodeArgs d;
    if (ws) {
      if (decode_partial_floats(sh, plan) > ws->partial_floats || decode_flag_words(plan) > ws->flag_words)
        return fail(SHAINET_HIP_ERR_CAPACITY,
                    "this call needs %zu floats of partial results and %zu flag words; the static scratch holds "
                    "%zu and %zu", decode_partial_floats(sh, plan), decode_flag_words(plan), ws->partial_floats,
                    ws->flag_words);
      d.partials = ws->partials;
      d.part_flag = ws->flags;
      d.flag_set = c->test_lose_marks ? ws->lost_marks : nullptr;
    } else {
      int rc = c->partials.reserve(decode_partial_floats(sh, plan));
      if (!rc) rc = ensure_decode_flags(c, decode_flag_words(plan), stream);
      if (rc) return rc;
      d.partials = c->partials.p;
      d.part_flag = c->part_flag;
      d.flag_set = c->test_lose_marks ? c->part_flag + c->part_flag_cap : nullptr;
    }
    d.q_rot = q_rot;
    d.kc = kc;
    d.vc = vc;
    d.out = out;
    d.error = c->error;
    d.spin_limit = c->test_lose_marks ? 2000 : 0;
    if (!ws) {  // (asked for by the caller of this one launch)
      d.ahead_w = c->ahead_w;
      d.ahead_k = c->ahead_k;
      d.ahead_n = c->ahead_n;
      d.ahead_wgs = c->ahead_wgs;
    }
    c->ahead_w = nullptr;
    if (prep) {
      e = launch_prep(*prep, st, sh, total_tokens, stream);
      if (e != hipSuccess) return hip_fail(e, "prep launch");
    }
    e = launch_decode(d, att, sh, plan, scale, stream, ev0, ev1);
  } else {
    if (prep) {
      e = launch_prep(*prep, st, sh, total_tokens, stream);
      if (e != hipSuccess) return hip_fail(e, "prep launch");
    }
    if (path == Path::kPrefillMfma) {
      const int items = plan_work(st, sh, path);
      int ns = c->prefill_splits_override > 0 ? c->prefill_splits_override : prefill_key_splits(st, sh, items);
      int rc = c->partials.reserve(prefill_partial_floats(sh, items, ns));
      if (rc) return rc;
      e = launch_prefill(q_rot, kc, vc, out, c->partials.p, st, sh, items, ns, scale, stream,
                         c->prefill_wgs_per_cu, c->prefill_groups_override, ev0, ev1);
    } else {
      plan_work(st, sh, path);
      if (ev0) (void)hipEventRecord(ev0, stream);
      e = launch_generic(q_rot, kc, vc, out, st, sh, total_tokens, scale, stream);
      if (ev1) (void)hipEventRecord(ev1, stream);
    }
  }
  if (e != hipSuccess) return hip_fail(e, "attention launch");
  return SHAINET_HIP_OK;
}

// Context behind the two reference-named entry points: they carry no handle, so
// they share one grow-only scratch set, as the reference's class-level scratch
// does (llama_block.cr:57-68).
shainet_attn_ctx *legacy_ctx() {
  static shainet_attn_ctx *c = [] {
    shainet_attn_ctx *n = new (std::nothrow) shainet_attn_ctx();
    if (n) n->test_lose_marks = getenv("SHAINET_HIP_TEST_LOSE_PARTIAL_MARKS") != nullptr;
    return n;
  }();
  return c;
}

}  // namespace

int shainet_attn_forward_strided(shainet_attn_ctx *c, shainet_kv_cache *kc, const int *seq_ids,
                                 const int *new_tokens, int n_seqs, const float *q, const float *k, const float *v,
                                 long long q_stride, long long k_stride, long long v_stride, float *out, int mem);

extern "C" {

const char *shainet_hip_last_error(void) { return g_err; }

int shainet_hip_available(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n < 1) {
    (void)hipGetLastError();
    return 0;
  }
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, 0) != hipSuccess) return 0;
  return strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : 0;
}

void kv_cache_append_f32(const float *staging, float *kc, float *vc, int new_tokens, int start_pos,
                         int num_kv_heads, int head_dim, int capacity) {
  hipError_t e = launch_legacy_append(staging, kc, vc, new_tokens, start_pos, num_kv_heads, head_dim, capacity,
                                      nullptr);
  if (e != hipSuccess) {
    hip_fail(e, "kv_cache_append_f32");
    fprintf(stderr, "HIP Error in kv_cache_append_f32: %s\n", hipGetErrorString(e));
  }
}

void attention_kv_f32(const float *q, const float *kc, const float *vc, float *out, float *ws, int new_tokens,
                      int start_pos, int num_heads, int heads_per_kv, int head_dim, int capacity, float scale) {
  (void)ws;
  shainet_attn_ctx *c = legacy_ctx();
  if (!c || new_tokens < 1 || start_pos < 0 || heads_per_kv < 1 || num_heads % heads_per_kv != 0 ||
      head_dim < 1 || head_dim > 256 || start_pos + new_tokens > capacity) {
    fail(SHAINET_HIP_ERR_ARGUMENT, "attention_kv_f32: invalid arguments");
    fprintf(stderr, "HIP Error in attention_kv_f32: invalid arguments\n");
    return;
  }
  // The calls are asynchronous and return nothing: what an earlier call's kernel reported (a given-up
  // wait for partial results) is said here, the way the reference prints the launch error of every
  // call (cuda_kernels.cu:821-824).
  if (check_error_word(c->error)) fprintf(stderr, "HIP Error in attention_kv_f32 (an earlier call): %s\n", g_err);
  c->H = num_heads;
  c->KV = num_heads / heads_per_kv;
  c->g = heads_per_kv;
  c->hd = head_dim;
  SeqTable st;
  memset(&st, 0, sizeof st);
  st.n_seqs = 1;
  st.start_pos[0] = start_pos;
  st.n_new[0] = new_tokens;
  st.tok_off[1] = new_tokens;
  Shape sh = shape_of(c, capacity);
  // the cache is only read on this path
  int rc = run_attention(c, q, const_cast<float *>(kc), const_cast<float *>(vc), out, st, sh, new_tokens, scale,
                         nullptr, nullptr);
  if (rc) fprintf(stderr, "HIP Error in attention_kv_f32: %s\n", g_err);
}

int shainet_attn_create(shainet_attn_ctx **out, int num_heads, int num_kv_heads, int head_dim,
                        double rope_theta, const float *rope_freqs, const float *q_norm, int q_norm_len,
                        const float *k_norm, int k_norm_len, double qk_norm_eps, int max_positions) {
  if (!out) return fail(SHAINET_HIP_ERR_ARGUMENT, "out is null");
  *out = nullptr;
  if (!(num_kv_heads > 0 && num_heads > 0 && num_heads % num_kv_heads == 0))
    return fail(SHAINET_HIP_ERR_ARGUMENT, "num_heads must be divisible by num_kv_heads");
  if (head_dim <= 0) return fail(SHAINET_HIP_ERR_ARGUMENT, "head_dim must be positive");
  if (head_dim > 256) return fail(SHAINET_HIP_ERR_ARGUMENT, "head_dim above 256 is not supported");
  if (q_norm && q_norm_len != head_dim)
    return fail(SHAINET_HIP_ERR_ARGUMENT, "qk_norm weight size %d != head_dim %d", q_norm_len, head_dim);
  if (k_norm && k_norm_len != head_dim)
    return fail(SHAINET_HIP_ERR_ARGUMENT, "qk_norm weight size %d != head_dim %d", k_norm_len, head_dim);
  if (!shainet_hip_available()) return fail(SHAINET_HIP_ERR_RUNTIME, "no gfx950 device available");
  shainet_attn_ctx *c = new (std::nothrow) shainet_attn_ctx();
  if (!c) return fail(SHAINET_HIP_ERR_ALLOC, "out of host memory");
  c->H = num_heads;
  c->KV = num_kv_heads;
  c->g = num_heads / num_kv_heads;
  c->hd = head_dim;
  c->eps = qk_norm_eps;
  c->scale = (float)(1.0 / sqrt((double)head_dim));
  c->inv_freq.resize(head_dim / 2);
  for (int i = 0; i < head_dim / 2; ++i)  // llama_block.cr:669-675
    c->inv_freq[i] = rope_freqs ? rope_freqs[i] : (float)(1.0 / pow(rope_theta, 2.0 * i / head_dim));
  if (const char *env = getenv("SHAINET_HIP_DECODE_WGS")) {  // tuning knob: workgroups of the decode split
    int v = atoi(env);
    if (v >= 1 && v <= 65536) c->decode_wgs_override = v;
  }
  c->test_lose_marks = getenv("SHAINET_HIP_TEST_LOSE_PARTIAL_MARKS") != nullptr;
  if (const char *env = getenv("SHAINET_HIP_PREFILL_WGS_PER_CU")) c->prefill_wgs_per_cu = atoi(env);
  if (const char *env = getenv("SHAINET_HIP_PREFILL_SPLITS")) c->prefill_splits_override = atoi(env);
  if (const char *env = getenv("SHAINET_HIP_PREFILL_GROUPS")) c->prefill_groups_override = atoi(env);
  int rc = SHAINET_HIP_OK;
  hipError_t e = hipStreamCreateWithFlags(&c->own_stream, hipStreamNonBlocking);
  if (e != hipSuccess) rc = hip_fail(e, "hipStreamCreate");
  c->stream = c->own_stream;
  c->error = c->own_error = alloc_error_word();
  if (!rc && !c->error) rc = fail(SHAINET_HIP_ERR_ALLOC, "hipHostMalloc failed");
  if (!rc) rc = upload(&c->d_q_norm, q_norm, head_dim);
  if (!rc) rc = upload(&c->d_k_norm, k_norm, head_dim);
  if (!rc) rc = ensure_rope_table(c, max_positions > 0 ? max_positions : 1024);
  // the address of the static scratch of shainet_attn_forward_noalloc on this device: asked for here,
  // once per device, so that the call itself (which may run under stream capture) only looks it up
  unsigned char *scratch_base = nullptr;
  if (!rc) rc = scratch_on_current_device(&scratch_base);
  if (rc) {
    shainet_attn_destroy(c);
    return rc;
  }
  *out = c;
  return SHAINET_HIP_OK;
}

int shainet_attn_set_bias(shainet_attn_ctx *c, const float *b_q, int b_q_len, const float *b_k, int b_k_len,
                          const float *b_v, int b_v_len) {
  if (!c) return fail(SHAINET_HIP_ERR_ARGUMENT, "ctx is null");
  const int q_dim = c->H * c->hd, kv_dim = c->KV * c->hd;
  if (b_q && b_q_len != q_dim)
    return fail(SHAINET_HIP_ERR_ARGUMENT, "bias size %d does not match matrix cols %d", b_q_len, q_dim);
  if (b_k && b_k_len != kv_dim)
    return fail(SHAINET_HIP_ERR_ARGUMENT, "bias size %d does not match matrix cols %d", b_k_len, kv_dim);
  if (b_v && b_v_len != kv_dim)
    return fail(SHAINET_HIP_ERR_ARGUMENT, "bias size %d does not match matrix cols %d", b_v_len, kv_dim);
  HIP_TRY(hipStreamSynchronize(c->stream));
  int rc = upload(&c->d_bq, b_q, q_dim);
  if (!rc) rc = upload(&c->d_bk, b_k, kv_dim);
  if (!rc) rc = upload(&c->d_bv, b_v, kv_dim);
  return rc;
}

int shainet_attn_destroy(shainet_attn_ctx *c) {
  if (!c) return SHAINET_HIP_OK;
  (void)hipStreamSynchronize(c->stream);
  if (c->own_stream) {
    (void)hipStreamSynchronize(c->own_stream);
    (void)hipStreamDestroy(c->own_stream);
  }
  for (float *p : {c->d_q_norm, c->d_k_norm, c->d_bq, c->d_bk, c->d_bv})
    if (p) (void)hipFree(p);
  if (c->d_rope) (void)hipFree(c->d_rope);
  if (c->part_flag) (void)hipFree(c->part_flag);
  for (hipEvent_t ev : c->prof_events) (void)hipEventDestroy(ev);
  for (DevBuf *b : {&c->q_rot, &c->partials, &c->in_q, &c->in_k, &c->in_v, &c->out}) b->release();
  c->pin_in.release();
  c->pin_out.release();
  free_error_word(c->own_error);
  delete c;
  return SHAINET_HIP_OK;
}

int shainet_attn_sync(shainet_attn_ctx *c) {
  if (!c) return fail(SHAINET_HIP_ERR_ARGUMENT, "ctx is null");
  HIP_TRY(hipStreamSynchronize(c->stream));
  return check_error_word(c->error);
}

void *shainet_attn_stream(shainet_attn_ctx *c) { return c ? (void *)c->stream : nullptr; }

int shainet_attn_set_stream(shainet_attn_ctx *c, void *stream) {
  if (!c) return fail(SHAINET_HIP_ERR_ARGUMENT, "ctx is null");
  if ((hipStream_t)stream == c->stream) return SHAINET_HIP_OK;  // nothing changes: no reason to drain the queue
  HIP_TRY(hipStreamSynchronize(c->stream));  // nothing of ours may still run on the old one
  c->stream = (hipStream_t)stream;
  return SHAINET_HIP_OK;
}

int shainet_attn_inv_freq(shainet_attn_ctx *c, float *out) {
  if (!c || !out) return fail(SHAINET_HIP_ERR_ARGUMENT, "null argument");
  memcpy(out, c->inv_freq.data(), c->inv_freq.size() * sizeof(float));
  return SHAINET_HIP_OK;
}

int shainet_kv_cache_create(shainet_kv_cache **out, shainet_attn_ctx *ctx, int batch, int capacity) {
  if (!out) return fail(SHAINET_HIP_ERR_ARGUMENT, "out is null");
  *out = nullptr;
  if (!ctx || batch < 1 || capacity < 1) return fail(SHAINET_HIP_ERR_ARGUMENT, "invalid cache geometry");
  shainet_kv_cache *kc = new (std::nothrow) shainet_kv_cache();
  if (!kc) return fail(SHAINET_HIP_ERR_ALLOC, "out of host memory");
  kc->ctx = ctx;
  kc->batch = batch;
  kc->cap = capacity;
  kc->len.assign(batch, 0);
  const size_t bytes = (size_t)batch * ctx->KV * capacity * ctx->hd * sizeof(float);
  hipError_t e = hipMalloc((void **)&kc->k, bytes);
  if (e == hipSuccess) e = hipMalloc((void **)&kc->v, bytes);
  // zero-fill: rows never appended must hold finite values.  On the context's stream and
  // waited for: a fill on the null stream is not ordered with the kernels that append rows
  // (the stream is non-blocking) and could wipe rows written right after this call.
  if (e == hipSuccess) e = hipMemsetAsync(kc->k, 0, bytes, ctx->stream);
  if (e == hipSuccess) e = hipMemsetAsync(kc->v, 0, bytes, ctx->stream);
  if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
  if (e != hipSuccess) {
    int rc = hip_fail(e, "kv cache allocation");
    shainet_kv_cache_destroy(kc);
    return rc;
  }
  *out = kc;
  return SHAINET_HIP_OK;
}

int shainet_kv_cache_destroy(shainet_kv_cache *kc) {
  if (!kc) return SHAINET_HIP_OK;
  if (kc->ctx) (void)hipStreamSynchronize(kc->ctx->stream);
  release_step_state(kc->step);
  if (kc->k) (void)hipFree(kc->k);
  if (kc->v) (void)hipFree(kc->v);
  delete kc;
  return SHAINET_HIP_OK;
}

int shainet_kv_cache_clear(shainet_kv_cache *kc, int seq) {
  if (!kc || seq >= kc->batch) return fail(SHAINET_HIP_ERR_ARGUMENT, "invalid sequence");
  if (int rc = refuse_while_lengths_on_device(kc, "shainet_kv_cache_clear")) return rc;
  if (seq < 0)
    kc->len.assign(kc->batch, 0);
  else
    kc->len[seq] = 0;
  return SHAINET_HIP_OK;
}

int shainet_kv_cache_truncate(shainet_kv_cache *kc, int seq, int len) {
  if (!kc || seq < 0 || seq >= kc->batch) return fail(SHAINET_HIP_ERR_ARGUMENT, "invalid sequence");
  if (int rc = refuse_while_lengths_on_device(kc, "shainet_kv_cache_truncate")) return rc;
  if (len < 0 || len > kc->len[seq])
    return fail(SHAINET_HIP_ERR_ARGUMENT, "truncate to %d outside 0..%d", len, kc->len[seq]);
  kc->len[seq] = len;
  return SHAINET_HIP_OK;
}

int shainet_kv_cache_len(const shainet_kv_cache *kc, int seq) {
  if (!kc || seq < 0 || seq >= kc->batch) return -1;
  if (refuse_while_lengths_on_device(kc, "shainet_kv_cache_len")) return -1;
  return kc->len[seq];
}

int shainet_kv_cache_capacity(const shainet_kv_cache *kc) { return kc ? kc->cap : -1; }

float *shainet_kv_cache_k(shainet_kv_cache *kc) { return kc ? kc->k : nullptr; }
float *shainet_kv_cache_v(shainet_kv_cache *kc) { return kc ? kc->v : nullptr; }

int shainet_kv_cache_reserve(shainet_kv_cache *kc, int capacity) {
  if (!kc) return fail(SHAINET_HIP_ERR_ARGUMENT, "cache is null");
  if (capacity <= kc->cap) return SHAINET_HIP_OK;
  if (int rc = refuse_while_lengths_on_device(kc, "shainet_kv_cache_reserve")) return rc;  // growth copies len rows
  shainet_attn_ctx *c = kc->ctx;
  const size_t row = (size_t)c->hd * sizeof(float);
  const size_t bytes = (size_t)kc->batch * c->KV * capacity * row;
  float *nk = nullptr, *nv = nullptr;
  hipError_t e = hipMalloc((void **)&nk, bytes);
  if (e == hipSuccess) e = hipMalloc((void **)&nv, bytes);
  if (e == hipSuccess) e = hipMemsetAsync(nk, 0, bytes, c->stream);
  if (e == hipSuccess) e = hipMemsetAsync(nv, 0, bytes, c->stream);
  // one strided copy per tensor: [batch*KV] runs of cap rows into runs of capacity rows
  if (e == hipSuccess)
    e = hipMemcpy2DAsync(nk, (size_t)capacity * row, kc->k, (size_t)kc->cap * row, (size_t)kc->cap * row,
                         (size_t)kc->batch * c->KV, hipMemcpyDeviceToDevice, c->stream);
  if (e == hipSuccess)
    e = hipMemcpy2DAsync(nv, (size_t)capacity * row, kc->v, (size_t)kc->cap * row, (size_t)kc->cap * row,
                         (size_t)kc->batch * c->KV, hipMemcpyDeviceToDevice, c->stream);
  if (e == hipSuccess) e = hipStreamSynchronize(c->stream);
  if (e != hipSuccess) {
    if (nk) (void)hipFree(nk);
    if (nv) (void)hipFree(nv);
    return hip_fail(e, "kv cache growth");
  }
  (void)hipFree(kc->k);
  (void)hipFree(kc->v);
  kc->k = nk;
  kc->v = nv;
  kc->cap = capacity;
  return SHAINET_HIP_OK;
}

int shainet_kv_cache_fill(shainet_kv_cache *kc, int seq, const float *k_rows, const float *v_rows, int n, int mem) {
  if (!kc || seq < 0 || seq >= kc->batch || n < 0 || !k_rows || !v_rows)
    return fail(SHAINET_HIP_ERR_ARGUMENT, "invalid fill arguments");
  if (int rc = refuse_while_lengths_on_device(kc, "shainet_kv_cache_fill")) return rc;
  if (n > kc->cap) return fail(SHAINET_HIP_ERR_CAPACITY, "fill of %d rows exceeds capacity %d", n, kc->cap);
  shainet_attn_ctx *c = kc->ctx;
  const size_t row = (size_t)c->hd * sizeof(float);
  const hipMemcpyKind kind = mem == SHAINET_HIP_MEM_HOST ? hipMemcpyHostToDevice : hipMemcpyDeviceToDevice;
  if (n > 0) {
    float *dk = kc->k + (size_t)seq * c->KV * kc->cap * c->hd;
    float *dv = kc->v + (size_t)seq * c->KV * kc->cap * c->hd;
    HIP_TRY(hipMemcpy2DAsync(dk, (size_t)kc->cap * row, k_rows, (size_t)n * row, (size_t)n * row, c->KV, kind,
                             c->stream));
    HIP_TRY(hipMemcpy2DAsync(dv, (size_t)kc->cap * row, v_rows, (size_t)n * row, (size_t)n * row, c->KV, kind,
                             c->stream));
    HIP_TRY(hipStreamSynchronize(c->stream));
  }
  kc->len[seq] = n;
  return ensure_rope_table(c, n + 1);
}

int shainet_kv_cache_read(shainet_kv_cache *kc, int seq, int kv_head, int pos0, int n, float *k_out, float *v_out) {
  if (!kc || seq < 0 || seq >= kc->batch || kv_head < 0 || kv_head >= kc->ctx->KV || pos0 < 0 || n < 0 ||
      pos0 + n > kc->cap)
    return fail(SHAINET_HIP_ERR_ARGUMENT, "invalid read arguments");
  shainet_attn_ctx *c = kc->ctx;
  const size_t off = (((size_t)seq * c->KV + kv_head) * kc->cap + pos0) * c->hd;
  HIP_TRY(hipStreamSynchronize(c->stream));
  if (k_out && n) HIP_TRY(hipMemcpy(k_out, kc->k + off, (size_t)n * c->hd * sizeof(float), hipMemcpyDeviceToHost));
  if (v_out && n) HIP_TRY(hipMemcpy(v_out, kc->v + off, (size_t)n * c->hd * sizeof(float), hipMemcpyDeviceToHost));
  return SHAINET_HIP_OK;
}

int shainet_attn_forward(shainet_attn_ctx *c, shainet_kv_cache *kc, const int *seq_ids, const int *new_tokens,
                         int n_seqs, const float *q, const float *k, const float *v, float *out, int mem) {
  if (!c) return fail(SHAINET_HIP_ERR_ARGUMENT, "context and cache do not belong together");
  return shainet_attn_forward_strided(c, kc, seq_ids, new_tokens, n_seqs, q, k, v, (long long)c->H * c->hd,
                                      (long long)c->KV * c->hd, (long long)c->KV * c->hd, out, mem);
}

}  // extern "C"

// The same with the rows of q, k and v at given strides (device pointers): lets a
// caller hand over the three column blocks of one fused projection output.
namespace {
int forward_core(shainet_attn_ctx *c, shainet_kv_cache *kc, const int *seq_ids, const int *new_tokens, int n_seqs,
                 const float *q, const float *k, const float *v, long long q_stride, long long k_stride,
                 long long v_stride, float *out, int mem, const Workspace *ws);
}

int shainet_attn_forward_strided(shainet_attn_ctx *c, shainet_kv_cache *kc, const int *seq_ids,
                                 const int *new_tokens, int n_seqs, const float *q, const float *k, const float *v,
                                 long long q_stride, long long k_stride, long long v_stride, float *out, int mem) {
  return forward_core(c, kc, seq_ids, new_tokens, n_seqs, q, k, v, q_stride, k_stride, v_stride, out, mem, nullptr);
}

namespace {

// ws != nullptr: device pointers only, and nothing is allocated: what the context would grow on
// demand (cos/sin table, rotated-query rows, split-K partials and their flags) must already be
// large enough or come with ws.
int forward_core(shainet_attn_ctx *c, shainet_kv_cache *kc, const int *seq_ids, const int *new_tokens, int n_seqs,
                 const float *q, const float *k, const float *v, long long q_stride, long long k_stride,
                 long long v_stride, float *out, int mem, const Workspace *ws) {
  if (!c || !kc || kc->ctx != c) return fail(SHAINET_HIP_ERR_ARGUMENT, "context and cache do not belong together");
  if (int rc = refuse_while_lengths_on_device(kc, "shainet_attn_forward")) return rc;
  if (ws && mem != SHAINET_HIP_MEM_DEVICE)
    return fail(SHAINET_HIP_ERR_ARGUMENT, "the entry point that allocates nothing takes device pointers only");
  if (!new_tokens || !q || !k || !v || !out) return fail(SHAINET_HIP_ERR_ARGUMENT, "null argument");
  if (n_seqs < 1 || n_seqs > SHAINET_HIP_MAX_BATCH)
    return fail(SHAINET_HIP_ERR_ARGUMENT, "n_seqs must be in 1..%d", SHAINET_HIP_MAX_BATCH);
  if (mem == SHAINET_HIP_MEM_DEVICE &&
      (q_stride < (long long)c->H * c->hd || k_stride < (long long)c->KV * c->hd || v_stride < (long long)c->KV * c->hd))
    return fail(SHAINET_HIP_ERR_ARGUMENT, "row strides must be at least the row widths %d and %d", c->H * c->hd,
                c->KV * c->hd);
  SeqTable st;
  memset(&st, 0, sizeof st);
  st.n_seqs = n_seqs;
  long long total = 0;
  int max_pos = 0;
  for (int s = 0; s < n_seqs; ++s) {
    const int slot = seq_ids ? seq_ids[s] : s;
    if (slot < 0 || slot >= kc->batch) return fail(SHAINET_HIP_ERR_ARGUMENT, "sequence id %d out of range", slot);
    for (int t = 0; t < s; ++t)
      if (st.slot[t] == slot) return fail(SHAINET_HIP_ERR_ARGUMENT, "sequence id %d appears twice", slot);
    if (new_tokens[s] < 1) return fail(SHAINET_HIP_ERR_ARGUMENT, "new_tokens must be positive");
    if ((long long)kc->len[slot] + new_tokens[s] > kc->cap)
      return fail(SHAINET_HIP_ERR_CAPACITY, "sequence %d: %d cached + %d new rows exceed capacity %d", slot,
                  kc->len[slot], new_tokens[s], kc->cap);
    st.slot[s] = slot;
    st.start_pos[s] = kc->len[slot];
    st.n_new[s] = new_tokens[s];
    st.tok_off[s] = (int)total;
    total += new_tokens[s];
    if (total > 0x3fffffff) return fail(SHAINET_HIP_ERR_ARGUMENT, "too many rows in one call");
    max_pos = max_pos > kc->len[slot] + new_tokens[s] ? max_pos : kc->len[slot] + new_tokens[s];
  }
  st.tok_off[n_seqs] = (int)total;
  const int rows = (int)total;
  const size_t q_floats = (size_t)rows * c->H * c->hd, kv_floats = (size_t)rows * c->KV * c->hd;
  int rc = SHAINET_HIP_OK;
  float *q_rot = nullptr;
  if (ws) {
    if (max_pos > c->rope_positions)
      return fail(SHAINET_HIP_ERR_CAPACITY,
                  "position %d is beyond the %d positions of the context's cos/sin table: create the context "
                  "with max_positions of at least the cache capacity", max_pos - 1, c->rope_positions);
    if (q_floats > ws->q_rot_floats)
      return fail(SHAINET_HIP_ERR_CAPACITY, "%d rows of %d query floats exceed the %zu floats of static scratch "
                  "for rotated queries", rows, c->H * c->hd, ws->q_rot_floats);
    q_rot = ws->q_rot;
  } else {
    rc = ensure_rope_table(c, max_pos);
    if (!rc) rc = c->q_rot.reserve(q_floats);
    if (rc) return rc;
    q_rot = c->q_rot.p;
  }

  const float *dq = q, *dk = k, *dv = v;
  float *dout = out;
  if (mem == SHAINET_HIP_MEM_HOST) {
    if ((rc = c->in_q.reserve(q_floats)) || (rc = c->in_k.reserve(kv_floats)) ||
        (rc = c->in_v.reserve(kv_floats)) || (rc = c->out.reserve(q_floats)) ||
        (rc = c->pin_in.reserve(q_floats + 2 * kv_floats)) || (rc = c->pin_out.reserve(q_floats)))
      return rc;
    // (the last call's copies are done: every host-pointer call ends with a wait)
    float *pq = c->pin_in.p, *pk = pq + q_floats, *pv = pk + kv_floats;
    memcpy(pq, q, q_floats * sizeof(float));
    memcpy(pk, k, kv_floats * sizeof(float));
    memcpy(pv, v, kv_floats * sizeof(float));
    hipError_t ce = hipMemcpyAsync(c->in_q.p, pq, q_floats * sizeof(float), hipMemcpyHostToDevice, c->stream);
    if (ce == hipSuccess) ce = hipMemcpyAsync(c->in_k.p, pk, kv_floats * sizeof(float), hipMemcpyHostToDevice, c->stream);
    if (ce == hipSuccess) ce = hipMemcpyAsync(c->in_v.p, pv, kv_floats * sizeof(float), hipMemcpyHostToDevice, c->stream);
    if (ce != hipSuccess) {
      (void)hipStreamSynchronize(c->stream);  // a copy already queued may still read the staging buffer
      return hip_fail(ce, "hipMemcpyAsync(q, k, v)");
    }
    dq = c->in_q.p;
    dk = c->in_k.p;
    dv = c->in_v.p;
    dout = c->out.p;
  } else if (mem != SHAINET_HIP_MEM_DEVICE) {
    return fail(SHAINET_HIP_ERR_ARGUMENT, "mem must be SHAINET_HIP_MEM_HOST or SHAINET_HIP_MEM_DEVICE");
  }

  Shape sh = shape_of(c, kc->cap);
  PrepArgs pa;
  pa.q = dq;
  pa.k = dk;
  pa.v = dv;
  pa.q_stride = mem == SHAINET_HIP_MEM_HOST ? (long long)c->H * c->hd : q_stride;
  pa.k_stride = mem == SHAINET_HIP_MEM_HOST ? (long long)c->KV * c->hd : k_stride;
  pa.v_stride = mem == SHAINET_HIP_MEM_HOST ? (long long)c->KV * c->hd : v_stride;
  pa.b_q = c->d_bq;
  pa.b_k = c->d_bk;
  pa.b_v = c->d_bv;
  pa.q_norm = c->d_q_norm;
  pa.k_norm = c->d_k_norm;
  pa.eps = c->eps;
  pa.rope_tab = c->d_rope;
  pa.q_rot = q_rot;
  pa.kc = kc->k;
  pa.vc = kc->v;
  rc = run_attention(c, q_rot, kc->k, kc->v, dout, st, sh, rows, c->scale, c->stream, &pa, ws);
  if (rc) {
    // the copies out of the pinned staging buffer may still run: the next call overwrites it
    if (mem == SHAINET_HIP_MEM_HOST) (void)hipStreamSynchronize(c->stream);
    return rc;  // the cached lengths stay as they were: the call did not happen
  }
  // the rows are in the cache once this call's kernels have run: @cache_len = total_len (llama_block.cr:288-289)
  for (int s = 0; s < n_seqs; ++s) kc->len[st.slot[s]] += st.n_new[s];
  c->last_rows = ws ? 0 : rows;  // shainet_attn_last_q_rot reads the context's own buffer
  if (mem == SHAINET_HIP_MEM_HOST) {
    const hipError_t ce = hipMemcpyAsync(c->pin_out.p, dout, q_floats * sizeof(float), hipMemcpyDeviceToHost, c->stream);
    const hipError_t se = hipStreamSynchronize(c->stream);  // also when the copy could not be queued
    if (ce != hipSuccess) return hip_fail(ce, "hipMemcpyAsync(out)");
    if (se != hipSuccess) return hip_fail(se, "hipStreamSynchronize");
    memcpy(out, c->pin_out.p, q_floats * sizeof(float));
    return check_error_word(c->error);
  }
  return SHAINET_HIP_OK;
}

// ---- the entry point that allocates nothing ------------------------------------------------
//
// Static device memory for what shainet_attn_forward's decode path otherwise allocates on demand:
// the flag words of the split (zero at launch), the rotated query rows and the partial results.
// Every GPU the library runs on holds its own copy of the array at its own address until the
// process ends; all calls on a GPU share it, so two such calls that overlap on one GPU race.
constexpr size_t kScratchFlagWords = 8192;              // 32 KiB of flags + 32 KiB for the give-up test's lost marks
constexpr size_t kScratchQRotFloats = 512 * 1024;       // 2 MiB: e.g. 128 rows of 32 heads x 128
constexpr size_t kScratchPartialFloats = 1536 * 1024;   // 6 MiB: e.g. 776 slots x 16 columns x (128 + 2)
constexpr size_t kScratchBytes =
    2 * kScratchFlagWords * sizeof(unsigned) + (kScratchQRotFloats + kScratchPartialFloats) * sizeof(float);
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
void *g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each device, once asked for
std::mutex g_scratch_lock;

// The address of this device's copy of `scratch` (the array's name is a host-side stand-in, not
// a device address: only hipGetSymbolAddress tells where the array lives on the current device).
int scratch_on_current_device(unsigned char **out) {
  int dev = -1;
  HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(SHAINET_HIP_ERR_RUNTIME, "device index %d out of range", dev);
  std::lock_guard<std::mutex> guard(g_scratch_lock);
  if (!g_scratch_ptr[dev]) {
    void *p = nullptr;
    HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return fail(SHAINET_HIP_ERR_RUNTIME, "hipGetSymbolAddress returned a null address");
    g_scratch_ptr[dev] = p;
  }
  *out = (unsigned char *)g_scratch_ptr[dev];
  return SHAINET_HIP_OK;
}

__global__ void fill_words_kernel(unsigned *p, unsigned value, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = value;
}

}  // namespace

extern "C" int shainet_attn_forward_noalloc(shainet_attn_ctx *c, shainet_kv_cache *kc, const int *seq_ids,
                                            const int *new_tokens, int n_seqs, const float *q, const float *k,
                                            const float *v, float *out) {
  if (!c) return fail(SHAINET_HIP_ERR_ARGUMENT, "context and cache do not belong together");
  unsigned char *base = nullptr;
  if (int rc = scratch_on_current_device(&base)) return rc;
  Workspace ws;
  ws.flags = (unsigned *)base;
  ws.flag_words = kScratchFlagWords;
  ws.lost_marks = ws.flags + kScratchFlagWords;
  ws.q_rot = (float *)(base + 2 * kScratchFlagWords * sizeof(unsigned));
  ws.q_rot_floats = kScratchQRotFloats;
  ws.partials = ws.q_rot + kScratchQRotFloats;
  ws.partial_floats = kScratchPartialFloats;
  // The array keeps what the last call on this GPU left in it.  The flag words must be zero at
  // launch; a launch leaves them so unless a wait was given up, so they are cleared every time, with
  // a fill kernel (a caller may be capturing the stream into a graph, where memset nodes are unsafe).
  hipLaunchKernelGGL(fill_words_kernel, dim3((unsigned)((kScratchFlagWords + 255) / 256)), dim3(256), 0, c->stream,
                     ws.flags, 0u, kScratchFlagWords);
  HIP_TRY(hipGetLastError());
  return forward_core(c, kc, seq_ids, new_tokens, n_seqs, q, k, v, (long long)c->H * c->hd, (long long)c->KV * c->hd,
                      (long long)c->KV * c->hd, out, SHAINET_HIP_MEM_DEVICE, &ws);
}

// ---- decode steps whose launches never change ------------------------------------------------

namespace {
DecodePlan step_launch_plan(const shainet_attn_ctx *c, int n_seqs) {
  DecodePlan p;
  memset(&p, 0, sizeof p);
  p.n_wgs = kDevicePlanWorkgroups;
  p.n_slots = device_plan_slots(n_seqs, c->KV);
  p.cols = c->g;
  return p;
}
}  // namespace

extern "C" int shainet_kv_cache_lengths_to_device(shainet_kv_cache *kc) {
  if (!kc) return fail(SHAINET_HIP_ERR_ARGUMENT, "cache is null");
  shainet_attn_ctx *c = kc->ctx;
  if (!decode_tile_head_dim(c->hd) || c->hd > 128 || c->g > 16)  // (the step's prep kernel: a wavefront per row of at most 128)
    return fail(SHAINET_HIP_ERR_ARGUMENT,
                "decode steps need a head_dim that is a multiple of 4 up to 128 and at most 16 query heads per kv head");
  if (kc->batch > SHAINET_HIP_MAX_BATCH)
    return fail(SHAINET_HIP_ERR_ARGUMENT, "decode steps take caches of at most %d sequences", SHAINET_HIP_MAX_BATCH);
  StepState &st = kc->step;
  if (int rc = refuse_while_lengths_on_device(kc, "shainet_kv_cache_lengths_to_device")) return rc;
  if (!st.d_len) {
    // all of it or none: a state with some buffers missing must never reach a launch
    const DecodePlan p = step_launch_plan(c, kc->batch);
    const size_t flag_words = decode_flag_words(p);
    StepState n;
    hipError_t e = hipMalloc((void **)&n.d_len, kc->batch * sizeof(int));
    if (e == hipSuccess) e = hipHostMalloc((void **)&n.pin_len, kc->batch * sizeof(int), hipHostMallocDefault);
    if (e == hipSuccess) e = hipMalloc((void **)&n.d_plan, sizeof(DecodeDevicePlan));
    if (e == hipSuccess) e = hipMalloc((void **)&n.q_rot, (size_t)kc->batch * c->H * c->hd * sizeof(float));
    if (e == hipSuccess)
      e = hipMalloc((void **)&n.partials, decode_partial_floats(shape_of(c, kc->cap), p) * sizeof(float));
    if (e == hipSuccess) e = hipMalloc((void **)&n.flags, flag_words * sizeof(unsigned));
    if (e == hipSuccess) e = hipMemsetAsync(n.d_plan, 0, sizeof(DecodeDevicePlan), c->stream);
    if (e == hipSuccess) e = hipMemsetAsync(n.flags, 0, flag_words * sizeof(unsigned), c->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(c->stream);
    if (e == hipSuccess && !c->error) {
      c->error = c->own_error = alloc_error_word();
      if (!c->error) e = hipErrorOutOfMemory;
    }
    if (e != hipSuccess) {
      release_step_state(n);
      return hip_fail(e, "allocation of the decode step's buffers");
    }
    st = n;
  }
  // the cos/sin table must reach as far as the cache: a step cannot grow it
  if (int rc = ensure_rope_table(c, kc->cap)) return rc;
  for (int s = 0; s < kc->batch; ++s) st.pin_len[s] = kc->len[s];
  HIP_TRY(hipMemcpyAsync(st.d_len, st.pin_len, kc->batch * sizeof(int), hipMemcpyHostToDevice, c->stream));
  HIP_TRY(hipStreamSynchronize(c->stream));
  st.cap = kc->cap;
  st.lengths_on_device = true;
  return SHAINET_HIP_OK;
}

extern "C" int shainet_kv_cache_lengths_from_device(shainet_kv_cache *kc) {
  if (!kc) return fail(SHAINET_HIP_ERR_ARGUMENT, "cache is null");
  StepState &st = kc->step;
  if (!st.d_len) return fail(SHAINET_HIP_ERR_ARGUMENT, "shainet_kv_cache_lengths_to_device has not been called");
  shainet_attn_ctx *c = kc->ctx;
  HIP_TRY(hipMemcpyAsync(st.pin_len, st.d_len, kc->batch * sizeof(int), hipMemcpyDeviceToHost, c->stream));
  HIP_TRY(hipStreamSynchronize(c->stream));
  for (int s = 0; s < kc->batch; ++s) {
    if (st.pin_len[s] < 0 || st.pin_len[s] > kc->cap)
      return fail(SHAINET_HIP_ERR_RUNTIME, "the device holds length %d for sequence %d of a cache of capacity %d",
                  st.pin_len[s], s, kc->cap);
    kc->len[s] = st.pin_len[s];
  }
  st.lengths_on_device = false;
  return check_error_word(c->error);
}

extern "C" int shainet_attn_decode_step(shainet_attn_ctx *c, shainet_kv_cache *kc, int n_seqs, const float *q,
                                        const float *k, const float *v, float *out) {
  if (!c || !kc || kc->ctx != c) return fail(SHAINET_HIP_ERR_ARGUMENT, "context and cache do not belong together");
  if (!q || !k || !v || !out) return fail(SHAINET_HIP_ERR_ARGUMENT, "null argument");
  if (n_seqs < 1 || n_seqs > kc->batch) return fail(SHAINET_HIP_ERR_ARGUMENT, "n_seqs must be in 1..%d", kc->batch);
  StepState &ss = kc->step;
  if (!ss.d_len || !ss.lengths_on_device)
    return fail(SHAINET_HIP_ERR_ARGUMENT,
                "shainet_kv_cache_lengths_to_device has not been called (again) since the lengths last came back to the host");
  if (ss.cap != kc->cap)  // cannot happen while the lengths are on the device: reserve is refused then
    return fail(SHAINET_HIP_ERR_ARGUMENT, "the cache has grown since shainet_kv_cache_lengths_to_device: call it again");
  const Shape sh = shape_of(c, kc->cap);
  hipError_t e = launch_decode_plan(ss.d_len, n_seqs, sh, c->rope_positions, ss.d_plan, c->error, c->stream);
  if (e != hipSuccess) return hip_fail(e, "plan launch");
  SeqTable st;
  memset(&st, 0, sizeof st);
  st.n_seqs = n_seqs;
  PrepArgs pa;
  pa.q = q;
  pa.k = k;
  pa.v = v;
  pa.q_stride = (long long)c->H * c->hd;
  pa.k_stride = pa.v_stride = (long long)c->KV * c->hd;
  pa.b_q = c->d_bq;
  pa.b_k = c->d_bk;
  pa.b_v = c->d_bv;
  pa.q_norm = c->d_q_norm;
  pa.k_norm = c->d_k_norm;
  pa.eps = c->eps;
  pa.rope_tab = c->d_rope;
  pa.q_rot = ss.q_rot;
  pa.kc = kc->k;
  pa.vc = kc->v;
  e = launch_prep(pa, st, sh, n_seqs, c->stream, ss.d_plan);
  if (e != hipSuccess) return hip_fail(e, "prep launch");
  DecodeArgs d;
  d.q_rot = ss.q_rot;
  d.kc = kc->k;
  d.vc = kc->v;
  d.out = out;
  d.partials = ss.partials;
  d.part_flag = ss.flags;
  d.flag_set = nullptr;
  d.error = c->error;
  d.spin_limit = 0;
  // (the buffers are sized for the whole cache; a step of fewer sequences uses the front of them)
  DecodePlan p = step_launch_plan(c, n_seqs);
  e = launch_decode(d, st, sh, p, c->scale, c->stream, nullptr, nullptr, ss.d_plan);
  if (e != hipSuccess) return hip_fail(e, "attention launch");
  c->last_rows = 0;
  return SHAINET_HIP_OK;
}

// The owner of a context (a block, a model) makes the context's kernels report into the owner's
// word, so that the owner's wait sees what any of its kernels gave up on; null = back to its own.
void shainet_attn_adopt_error_word(shainet_attn_ctx *c, int *word) {
  if (c) c->error = word ? word : c->own_error;
}
int *shainet_attn_error_word(shainet_attn_ctx *c) { return c ? c->error : nullptr; }

int shainet_attn_begin_prepared(shainet_attn_ctx *c, shainet_kv_cache *kc, int new_tokens, GemvPrep *where) {
  if (!c || !kc || kc->ctx != c || !where)
    return fail(SHAINET_HIP_ERR_ARGUMENT, "context and cache do not belong together");
  if (new_tokens < 1) return fail(SHAINET_HIP_ERR_ARGUMENT, "new_tokens must be positive");
  if ((long long)kc->len[0] + new_tokens > kc->cap)
    return fail(SHAINET_HIP_ERR_CAPACITY, "sequence 0: %d cached + %d new rows exceed capacity %d", kc->len[0],
                new_tokens, kc->cap);
  int rc = ensure_rope_table(c, kc->len[0] + new_tokens);
  if (!rc) rc = c->q_rot.reserve((size_t)new_tokens * c->H * c->hd);
  if (rc) return rc;
  where->b_q = c->d_bq;
  where->b_k = c->d_bk;
  where->b_v = c->d_bv;
  where->q_norm = c->d_q_norm;
  where->k_norm = c->d_k_norm;
  where->eps = c->eps;
  where->rope_tab = c->d_rope;
  where->q_rot = c->q_rot.p;
  where->kc = kc->k;
  where->vc = kc->v;
  where->H = c->H;
  where->KV = c->KV;
  where->hd = c->hd;
  where->cap = kc->cap;
  where->start_pos = kc->len[0];
  return SHAINET_HIP_OK;
}

// The rows shainet_attn_begin_prepared made room for are in the cache (a kernel of the caller's
// appended them and did the attention over them): count them.
void shainet_attn_commit_prepared(shainet_attn_ctx *c, shainet_kv_cache *kc, int new_tokens) {
  kc->len[0] += new_tokens;
  c->last_rows = 0;
}

void shainet_attn_read_ahead(shainet_attn_ctx *c, const float *w, int k, int n, int wgs) {
  if (!c) return;
  c->ahead_w = w;
  c->ahead_k = k;
  c->ahead_n = n;
  c->ahead_wgs = wgs;
}

int shainet_attn_finish_prepared(shainet_attn_ctx *c, shainet_kv_cache *kc, int new_tokens, float *out) {
  if (!c || !kc || kc->ctx != c || !out)
    return fail(SHAINET_HIP_ERR_ARGUMENT, "context and cache do not belong together");
  if (new_tokens < 1 || (long long)kc->len[0] + new_tokens > kc->cap)
    return fail(SHAINET_HIP_ERR_CAPACITY, "sequence 0: %d cached + %d new rows exceed capacity %d", kc->len[0],
                new_tokens, kc->cap);
  SeqTable st;
  memset(&st, 0, sizeof st);
  st.n_seqs = 1;
  st.start_pos[0] = kc->len[0];
  st.n_new[0] = new_tokens;
  st.tok_off[1] = new_tokens;
  Shape sh = shape_of(c, kc->cap);
  const int rc = run_attention(c, c->q_rot.p, kc->k, kc->v, out, st, sh, new_tokens, c->scale, c->stream, nullptr);
  if (rc) return rc;
  kc->len[0] += new_tokens;
  c->last_rows = new_tokens;
  return SHAINET_HIP_OK;
}

extern "C" {

int shainet_rope_apply(const float *x, float *out, int seq_len, int head_dim, int start_pos, double theta, int mem) {
  if (!x || !out || seq_len < 0 || head_dim < 1) return fail(SHAINET_HIP_ERR_ARGUMENT, "invalid arguments");
  if (mem != SHAINET_HIP_MEM_HOST && mem != SHAINET_HIP_MEM_DEVICE)
    return fail(SHAINET_HIP_ERR_ARGUMENT, "mem must be SHAINET_HIP_MEM_HOST or SHAINET_HIP_MEM_DEVICE");
  if (seq_len == 0) return SHAINET_HIP_OK;
  if (!shainet_hip_available()) return fail(SHAINET_HIP_ERR_RUNTIME, "no gfx950 device available");
  if (mem == SHAINET_HIP_MEM_DEVICE) {
    const hipError_t e = launch_rope_apply(x, out, seq_len, head_dim, start_pos, theta, nullptr);
    return e == hipSuccess ? SHAINET_HIP_OK : hip_fail(e, "rope launch");
  }
  const size_t bytes = (size_t)seq_len * head_dim * sizeof(float);
  float *dx = nullptr, *dy = nullptr;
  hipError_t e = hipMalloc((void **)&dx, bytes);
  if (e == hipSuccess) e = hipMalloc((void **)&dy, bytes);
  if (e == hipSuccess) e = hipMemcpy(dx, x, bytes, hipMemcpyHostToDevice);
  if (e == hipSuccess) e = launch_rope_apply(dx, dy, seq_len, head_dim, start_pos, theta, nullptr);
  if (e == hipSuccess) e = hipMemcpy(out, dy, bytes, hipMemcpyDeviceToHost);  // waits for the kernel
  if (dx) (void)hipFree(dx);
  if (dy) (void)hipFree(dy);
  return e == hipSuccess ? SHAINET_HIP_OK : hip_fail(e, "shainet_rope_apply");
}

int shainet_attn_describe_plan(int num_heads, int num_kv_heads, int head_dim, int n_seqs, const int *start_pos,
                               const int *new_tokens, int plan[8]) {
  if (!start_pos || !new_tokens || !plan) return fail(SHAINET_HIP_ERR_ARGUMENT, "null argument");
  if (!(num_kv_heads > 0 && num_heads > 0 && num_heads % num_kv_heads == 0) || head_dim < 1 || head_dim > 256)
    return fail(SHAINET_HIP_ERR_ARGUMENT, "invalid head geometry");
  if (n_seqs < 1 || n_seqs > SHAINET_HIP_MAX_BATCH)
    return fail(SHAINET_HIP_ERR_ARGUMENT, "n_seqs must be in 1..%d", SHAINET_HIP_MAX_BATCH);
  SeqTable st;
  memset(&st, 0, sizeof st);
  st.n_seqs = n_seqs;
  int total = 0, cap = 1;
  for (int s = 0; s < n_seqs; ++s) {
    if (start_pos[s] < 0 || new_tokens[s] < 1) return fail(SHAINET_HIP_ERR_ARGUMENT, "invalid sequence");
    st.slot[s] = s;
    st.start_pos[s] = start_pos[s];
    st.n_new[s] = new_tokens[s];
    st.tok_off[s] = total;
    total += new_tokens[s];
    cap = cap > start_pos[s] + new_tokens[s] ? cap : start_pos[s] + new_tokens[s];
  }
  st.tok_off[n_seqs] = total;
  Shape sh;
  sh.H = num_heads;
  sh.KV = num_kv_heads;
  sh.g = num_heads / num_kv_heads;
  sh.hd = head_dim;
  sh.cap = cap;
  sh.seq_stride = (long long)num_kv_heads * cap * head_dim;
  for (int i = 0; i < 8; ++i) plan[i] = 0;
  const Path path = choose_path(st, sh);
  plan[1] = head_dim;
  if (path == Path::kDecodeSplitK) {
    SeqTable att;
    if (!decode_entries(st, sh, att)) return fail(SHAINET_HIP_ERR_RUNTIME, "decode entries do not fit");
    const DecodePlan p = plan_decode(att, sh, 0);
    plan[0] = 0;
    plan[1] = decode_tile_head_dim(head_dim);
    plan[2] = 1;
    plan[3] = 1;
    plan[5] = p.n_wgs;
    plan[6] = p.tiles_per_wg;
    plan[7] = 1;
  } else if (path == Path::kPrefillMfma) {
    const int items = plan_work(st, sh, path);
    const int ns = prefill_key_splits(st, sh, items);
    const PrefillLaunch p = plan_prefill_launch(sh, items, ns, 0, 0);
    plan[0] = 1;
    plan[1] = prefill_tile_head_dim(head_dim);
    plan[2] = ns;
    plan[3] = p.groups;
    plan[4] = p.turns;
    plan[5] = (int)(p.turns ? (p.n_wgs + p.turns - 1) / p.turns : p.n_wgs);
    plan[6] = items;
    plan[7] = p.wgs_per_cu;
  } else {
    plan[0] = 2;
    plan[2] = 1;
    plan[3] = 1;
    plan[5] = total * num_heads;
  }
  return SHAINET_HIP_OK;
}

int shainet_attn_profile(shainet_attn_ctx *c, int enable) {
  if (!c) return fail(SHAINET_HIP_ERR_ARGUMENT, "ctx is null");
  c->profiling = enable != 0;
  return SHAINET_HIP_OK;
}

int shainet_attn_profile_samples(shainet_attn_ctx *c, float *ms_out, int capacity, int *launches) {
  if (!c || !launches || capacity < 0 || (capacity > 0 && !ms_out)) return fail(SHAINET_HIP_ERR_ARGUMENT, "null argument");
  HIP_TRY(hipStreamSynchronize(c->stream));
  int n = 0;
  for (size_t i = 0; i + 1 < c->prof_events.size(); i += 2) {
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, c->prof_events[i], c->prof_events[i + 1]) == hipSuccess) {
      if (n < capacity) ms_out[n] = ms;
      ++n;
    }
    (void)hipEventDestroy(c->prof_events[i]);
    (void)hipEventDestroy(c->prof_events[i + 1]);
  }
  (void)hipGetLastError();
  c->prof_events.clear();
  *launches = n;
  return SHAINET_HIP_OK;
}

int shainet_attn_profile_read(shainet_attn_ctx *c, double *total_ms, int *launches) {
  if (!c || !total_ms || !launches) return fail(SHAINET_HIP_ERR_ARGUMENT, "null argument");
  std::vector<float> ms(c->prof_events.size() / 2 + 1);
  int n = 0;
  const int rc = shainet_attn_profile_samples(c, ms.data(), (int)ms.size(), &n);
  if (rc) return rc;
  double sum = 0.0;
  for (int i = 0; i < n && i < (int)ms.size(); ++i) sum += ms[i];
  *total_ms = sum;
  *launches = n;
  return SHAINET_HIP_OK;
}

int shainet_attn_last_q_rot(shainet_attn_ctx *c, float *out, int rows) {
  if (!c || !out || rows < 0 || rows > c->last_rows) return fail(SHAINET_HIP_ERR_ARGUMENT, "invalid arguments");
  HIP_TRY(hipStreamSynchronize(c->stream));
  HIP_TRY(hipMemcpy(out, c->q_rot.p, (size_t)rows * c->H * c->hd * sizeof(float), hipMemcpyDeviceToHost));
  return SHAINET_HIP_OK;
}

}  // extern "C"
