// One decode step (one new token, one sequence) of a whole stack of LlamaBlocks as a
// single persistent launch: see step_kernel.hip.
#pragma once
#include <hip/hip_runtime.h>

namespace shainet {

// One block of the stack, read by the kernel from device memory.
struct StepLayer {
  const float *w_qkv;   // [d, q_dim + 2 kv_dim] = w_q | w_k | w_v
  const float *w_o;     // [q_dim, d]
  const float *w_gu;    // [d, 2 ff] = gate_proj | up_proj
  const float *w_down;  // [ff, d]
  const float *norm1, *norm2;                       // [d] or null (= ones)
  const float *b_q, *b_k, *b_v, *q_norm, *k_norm;   // nullable
  const float2 *rope_tab;                           // [positions][hd / 2] (cos, sin)
  float *kc, *vc;                                   // this block's cache of sequence 0: [KV, cap, hd]
  int cap;
  int pad_;
};

constexpr int kStepThreads = 512;
constexpr int kStepMaxSplits = 16;
constexpr int kStepTraceSlots = 24;  // clock readings per block in StepArgs::trace
constexpr int kStepBarGroup = 16;  // workgroups per first-level arrival counter of the barrier
// 32-bit words of barrier state for n_wgs workgroups (zero when allocated, never reset)
inline size_t step_barrier_words(int n_wgs) { return 64 * (size_t)((n_wgs + kStepBarGroup - 1) / kStepBarGroup + 1); }
constexpr int kStepMaxSlice = 4096;  // most rows of W a workgroup takes in one product
constexpr int kStepSlicePad = 3328;  // zeros kept behind the x slice in LDS

// How one product y = x W is cut over the workgroups: column tiles of 4 F floats, `splits`
// workgroups along K per tile.  Without split_fast workgroup w takes tile w % col_tiles and
// split w / col_tiles (none when that is >= splits).
struct StepProduct {
  int K, N, ldw;  // ldw: floats between two rows of W
  int F, col_tiles, splits;
  // Split s takes rows [bound[s], bound[s + 1]) of W.  With split_fast, workgroup w takes split
  // w % splits and tile w / splits: workgroups go to the eight XCDs round-robin by index, so a
  // split then stays on the same XCDs and its share of the rows can follow their speed.
  int split_fast;
  int bound[kStepMaxSplits + 1];
};

struct StepArgs {
  const StepLayer *layers;
  int n_layers;
  int d, H, KV, hd, ff;
  double eps, qk_eps;  // RMSNorm of the blocks, QK-norm
  float scale;
  StepProduct qkv, wo, gu, down;
  int attn_chunks;  // key chunks per kv head the partial area is laid out for (<= workgroups / KV)
  int attn_ck;      // keys per chunk in this launch
  const float *embedding;  // [vocab, d]
  const int *token;        // device: the id of the new token
  int pos;                 // its position = rows cached before this step
  float *x_out;            // [d]: the last block's output row
  float *qkv_part, *attn_part, *o_part, *gu_part, *down_part;
  unsigned *bar;      // step_barrier_words() words: arrival counters and release words
  unsigned *bar_set;  // where arrivals and releases are written: `bar`, or elsewhere in the test of the give-up path
  unsigned epoch0;    // barriers since `bar` was zeroed; a launch has kStepBarriersPerLayer * n_layers of them
  int spin_limit;     // polls before a wait for the other workgroups is given up
  int *error;         // set to 1 then
  long long *trace;   // null, or [workgroups][1 + kStepTraceSlots * n_layers] clock readings (tuning aid)
};

struct StepPlan {
  bool ok;  // false: this geometry does not fit the kernel; use one launch per product
  StepProduct qkv, wo, gu, down;
  int attn_chunks;
  size_t lds_bytes;
  size_t qkv_floats, attn_floats, o_floats, gu_floats, down_floats;
};
// n_wgs: workgroups of the launch = compute units of the device (all must be resident at once).
StepPlan plan_step(int d, int H, int KV, int hd, int ff, int n_wgs);
constexpr int kStepBarriersPerLayer = 5;
// Keys per chunk for a step at position pos (pos + 1 keys).
int step_keys_per_chunk(const StepPlan &p, int pos);
hipError_t launch_step(const StepArgs &a, int n_wgs, size_t lds_bytes, hipStream_t stream);

}  // namespace shainet
