// Shared by the host mirrors of LlamaBlock and of the model around it: grow-only
// device buffers and the row-major projection y = x W.
#pragma once
#include <hip/hip_runtime.h>

#include <string>

#include "../../include/shainet_hip_attn.h"

// capi.hip: shainet_attn_forward with the rows of q, k and v at given strides
int shainet_attn_forward_strided(shainet_attn_ctx *c, shainet_kv_cache *kc, const int *seq_ids,
                                 const int *new_tokens, int n_seqs, const float *q, const float *k, const float *v,
                                 long long q_stride, long long k_stride, long long v_stride, float *out, int mem);

// capi.hip: the two halves of shainet_attn_forward for one sequence (slot 0 of the
// cache) when the kernel that produces q | k | v also does the bias / QK-norm / RoPE /
// append step (the kGemvQkvPrep epilogue).  begin checks the capacity and says where
// the prepared rows go; finish runs the attention kernel over them and counts the rows
// into the cache.  Both are asynchronous on the context's stream.
namespace shainet {
struct GemvPrep;
}
int shainet_attn_begin_prepared(shainet_attn_ctx *c, shainet_kv_cache *kc, int new_tokens, shainet::GemvPrep *where);
int shainet_attn_finish_prepared(shainet_attn_ctx *c, shainet_kv_cache *kc, int new_tokens, float *out);
// capi.hip: the next decode launch of the context (finish_prepared for a few rows) also reads, in
// workgroups of its own, what the first `wgs` workgroups of the one-row SwiGLU product over the
// transposed weights w ([2 n, k]) will read, into the L2s (DecodeArgs::ahead_w)
void shainet_attn_read_ahead(shainet_attn_ctx *c, const float *w, int k, int n, int wgs);
// capi.hip: instead of finish, when the caller's own kernel appended the rows and attended over them
void shainet_attn_commit_prepared(shainet_attn_ctx *c, shainet_kv_cache *kc, int new_tokens);
// capi.hip: the pinned host word a context's kernels report a given-up wait into; a block or a
// model that owns the context makes it the owner's word (null = back to the context's own)
void shainet_attn_adopt_error_word(shainet_attn_ctx *c, int *word);
int *shainet_attn_error_word(shainet_attn_ctx *c);

// Device weight buffers of a block / a model, allocated on first request, for a loader
// that fills them on the device (llama_block.hip, llama_model.hip).
struct LlamaBlockBuffers {
  float *w_qkv, *w_o, *gate_up, *down, *norm1, *norm2;
  int d_model, q_dim, kv_dim, ff_hidden;
};
int shainet_llama_block_buffers(shainet_llama_block *b, LlamaBlockBuffers *out);
struct LlamaModelBuffers {
  float *embedding, *final_norm, *lm_head;
};
int shainet_llama_model_buffers(shainet_llama_model *m, LlamaModelBuffers *out);

namespace shainet {

struct DevF {
  float *p = nullptr;
  size_t cap = 0;
  bool reserve(size_t n);
  void release();
};

// Grow-only pinned host buffer: host-pointer calls stage their rows through it, so that the
// copies to and from the device run as one asynchronous DMA each instead of the runtime's
// staged copy of pageable memory.
struct PinnedF {
  float *p = nullptr;
  size_t cap = 0;
  bool reserve(size_t n);
  void release();
};

// What rides along with a projection y = x W.
struct Fused {
  int epilogue = 0;            // kGemvPlain, kGemvResidual (y = res + x W) or kGemvSwiglu (W = gate | up, [K, 2N])
  const float *res = nullptr;  // [T, N]
  bool norm = false;           // RMSNorm the rows of x first
  const float *gamma = nullptr;
  double eps = 0.0;
  const GemvPrep *prep = nullptr;  // kGemvQkvPrep: where the head rows go (y may be null); at most 16 rows
  // the same weights transposed ([N, K]; kGemvSwiglu: [2N, K]) or null: one row of x then takes the
  // product that gives a wavefront whole outputs (launch_gemvt) where its shapes allow
  const float *w_t = nullptr;
  bool w_t_has_gamma = false;  // the rows of w_t were made with gamma multiplied in: the norm's factor 1 / rms is all that is left to apply
};

// y[T,N] = epilogue(norm(x)[T,K] * W), all row-major on the device.  Up to 16 rows
// (decode) run as one hand-written split GEMV with the norm and the epilogue
// inside; more rows run as the MFMA product of gemm_kernel.hip (the counterpart of
// the reference's cuBLAS SGEMM, cuda.cr:237-247) after the separate norm kernel,
// with the residual add in its epilogue and the SwiGLU activation as a kernel of its own.
struct Projector {
  DevF scratch, normed, wide;
  // split products: a word per partial that says when it is complete (zero between launches)
  unsigned *flags = nullptr;
  size_t flags_cap = 0;
  // SHAINET_HIP_TEST_LOSE_PARTIAL_MARKS (read when the flag words are first allocated): the marks
  // go to a second set of words nobody reads and waits end after 2000 polls, so that the report
  // of a given-up wait can be exercised without hanging anything
  bool lose_marks = false;
  // where the split products' kernels report a given-up wait: the owner's pinned host word
  int *error = nullptr;
  // returns a SHAINET_HIP_* status; the message is left for shainet_hip_last_error
  int project(const float *x, long long x_stride, const float *w, float *y, int T, int K, int N, hipStream_t stream,
              const Fused &f = Fused());
  void release();

 private:
  int reserve_flags(size_t n_flags, hipStream_t stream);
  // res != nullptr: y = res + x W
  int gemm(const float *x, long long x_stride, const float *w, float *y, int T, int K, int N, hipStream_t stream,
           const float *res = nullptr);
};

// Replace *dst (device, hipMalloc'ed or null) by a copy of n host floats.
int upload_floats(float **dst, const float *src, size_t n);
// Host matrices [rows, n_i] side by side into one device matrix [rows, sum n_i].
int upload_side_by_side(float **dst, const float *const *mats, const int *widths, int count, int rows);

int llama_fail(int code, const std::string &msg);

// Second copies of weight matrices, transposed, for the product of a single row (launch_gemvt).
// SHAINET_HIP_NO_TRANSPOSED_WEIGHTS turns them off.  transposed_twin: *twin = src ([rows, cols] on
// the device) transposed, allocated on first use and made again when *stale; returns the twin, or
// null when they are turned off or there is no memory for one (the caller then goes without).
bool transposed_twins_wanted();
// row_scale (nullable): a factor per row of src, i.e. per input of the product: the RMSNorm weights
// gamma of the norm the product always follows, so that (x gamma) W = x (diag(gamma) W) needs no gamma.
const float *transposed_twin(float **twin, bool *stale, const float *src, int rows, int cols, hipStream_t stream,
                             const float *row_scale = nullptr);

}  // namespace shainet
