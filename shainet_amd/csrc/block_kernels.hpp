// Launchers of the kernels around attention in a LlamaBlock and after the last
// block: RMSNorm, residual add, SwiGLU activation, embedding lookup, logits bias,
// repetition penalty, greedy argmax and top-k selection.  Device pointers only.
#pragma once
#include <hip/hip_runtime.h>

namespace shainet {

// out[r, :] = x[r, :] / sqrt(mean(x[r, :]^2) + eps) * gamma   (gamma == nullptr: ones);
// the rows of x are x_stride floats apart, those of out are dense
hipError_t launch_rmsnorm(const float *x, long long x_stride, const float *gamma, float *out, int rows, int cols,
                          double eps, hipStream_t stream);
// dst[c, r] = src[r, c]: src is [rows, cols], dst [cols, rows], both dense
hipError_t launch_transpose(const float *src, float *dst, int rows, int cols, hipStream_t stream,
                            const float *row_scale = nullptr);
// *differ (a device int the caller has set to 0) becomes 1 when a [rows, cols] is not, bit for bit,
// the transpose of b [cols, rows]
hipError_t launch_transposed_differ(const float *a, const float *b, int rows, int cols, int *differ, hipStream_t stream);
// out = a + b, n floats
hipError_t launch_add(const float *a, const float *b, float *out, long long n, hipStream_t stream);
// hidden[r, j] = silu(gate_up[r, j]) * gate_up[r, ff + j];  gate_up is [rows, 2*ff]
hipError_t launch_swiglu_act(const float *gate_up, float *hidden, int rows, int ff, hipStream_t stream);
// out[t, :] = table[tokens[t], :];  the caller has checked 0 <= tokens[t] < vocab
hipError_t launch_embed(const float *table, const int *tokens, float *out, int n_tokens, int d_model,
                        hipStream_t stream);
// logits[j] += bias[j]
hipError_t launch_add_bias_row(float *logits, const float *bias, int n, hipStream_t stream);
// Sampler#apply_repetition_penalty! : ids in order, duplicates penalised once per occurrence
hipError_t launch_repetition_penalty(float *logits, int vocab, const int *ids, int n, double penalty,
                                     hipStream_t stream);

// RoPE.apply (rope.cr:7-33) on [seq_len, head_dim] rows: half-split rotation by
// (row + start_pos) * theta^(-2i/head_dim), frequency, angle, cosine, sine and the products in
// fp64, one rounding to fp32; an odd trailing column is copied through.
hipError_t launch_rope_apply(const float *x, float *out, int seq_len, int head_dim, int start_pos, double theta,
                             hipStream_t stream);

// Top-k of a logits row, descending by value, ties by ascending index, NaN never
// selected (Sampler#sample's selection); with finite_only also +-inf are skipped
// (Sampler.greedy).  scratch: topk_scratch_bytes(vocab, k) bytes.  out_ids /
// out_vals: k entries; *out_count = entries found (< k when the row has fewer
// eligible values); the unused ids are set to fallback_id.  out_vals and out_count
// may be null.
constexpr int kMaxTopK = 256;
size_t topk_scratch_bytes(int vocab, int k);
hipError_t launch_topk(const float *logits, int vocab, int k, bool finite_only, void *scratch, int *out_ids,
                       float *out_vals, int *out_count, hipStream_t stream, int fallback_id = -1);

// The rest of Sampler#sample (text/sampler.cr:118-150) on a selection launch_topk made: softmax of
// vals / temperature over the *count survivors and the pick for the uniform draw r in [0, 1);
// *out = the chosen id (0 when nothing was eligible).
hipError_t launch_sample_pick(const int *ids, const float *vals, const int *count, double temperature, double r,
                              int *out, hipStream_t stream);

}  // namespace shainet
