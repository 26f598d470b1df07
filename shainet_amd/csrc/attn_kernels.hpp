// Launchers of the gfx950 attention kernels.  Device pointers only; every
// launcher validates the shapes its kernel assumes and returns a hipError_t.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

// A kernel launch that hands the kernel's own first and last clock reading to two events when
// there are any (hipExtLaunchKernel), and is a plain launch, as a caller's stream capture may
// need it, when there are none.
#define SHAINET_LAUNCH_TIMED(kernel, grid, block, lds, stream, before, after, ...)                         \
  do {                                                                                                   \
    if ((before) || (after))                                                                             \
      hipExtLaunchKernelGGL(kernel, grid, block, lds, stream, before, after, 0, __VA_ARGS__);            \
    else                                                                                                 \
      hipLaunchKernelGGL(kernel, grid, block, lds, stream, __VA_ARGS__);                                 \
  } while (0)

namespace shainet {

constexpr int kMaxSeqs = 64;

// Per-call description of the sequences taking part, passed to kernels by value
// (it lives in the kernel-argument segment, so no copy to the device is needed).
struct SeqTable {
  int n_seqs;
  int slot[kMaxSeqs];          // cache slot of sequence s
  int start_pos[kMaxSeqs];     // cached positions before this call
  int n_new[kMaxSeqs];         // rows appended by this call
  int tok_off[kMaxSeqs + 1];   // prefix sums of n_new
  int work_off[kMaxSeqs + 1];  // per-path work description (see plan_work / plan_decode)
  int ord[kMaxSeqs];           // prefill: sequences by descending number of row blocks
};

struct Shape {
  int H, KV, g, hd;
  int cap;               // positions per (sequence, kv head)
  long long seq_stride;  // floats between two sequences' caches = KV*cap*hd
};

struct PrepArgs {
  const float *q, *k, *v;           // [tokens, H*hd], [tokens, KV*hd] x2: projection outputs
  long long q_stride, k_stride, v_stride;  // floats between the rows of two tokens (>= the row width)
  const float *b_q, *b_k, *b_v;     // nullable
  const float *q_norm, *k_norm;     // nullable, [hd]
  double eps;
  const float2 *rope_tab;           // [positions][hd/2] (cos, sin)
  float *q_rot;                     // [tokens, H*hd]
  float *kc, *vc;
};

struct DecodeDevicePlan;
// bias -> QK-norm -> RoPE -> append (K rotated, V as is); rotated Q to q_rot.
// dev != nullptr: one new row for each of st.n_seqs sequences, their positions read from
// *dev (device memory) instead of st.
hipError_t launch_prep(const PrepArgs &a, const SeqTable &st, const Shape &sh, int total_tokens,
                       hipStream_t stream, const DecodeDevicePlan *dev = nullptr);

// Which attention kernel a call uses.
enum class Path { kDecodeSplitK, kPrefillMfma, kGeneric };
Path choose_path(const SeqTable &st, const Shape &sh);
// The sequences as the split-K decode kernel takes them: one entry per sequence with up to
// 16 / g new rows, two entries (the first 16 / g rows, then the rest, which see the first ones
// as cached) with up to twice as many.  False when some sequence has more or the entries
// do not fit a table.
bool decode_entries(const SeqTable &st, const Shape &sh, SeqTable &out);

// Fills st.work_off for the prefill or generic path and returns the number of work items.
int plan_work(SeqTable &st, const Shape &sh, Path path);

// Where the spans of eight consecutive workgroups begin within their 8 * tiles_per_wg tiles.
struct SpanTable {
  int off[9];
};
// Decode work split (a few new rows per sequence: rows x group size <= 16, the columns of one
// MFMA tile): the 16-key tiles of all (sequence, kv head) pairs laid end to
// end (st.work_off = per-sequence prefix sums) and cut into spans.
struct DecodePlan {
  int total_tiles;
  int tiles_per_wg;
  SpanTable spans;
  int n_wgs;
  int n_slots;  // partial slots: workgroup index + pair index is unique per segment
  int cols;     // columns (new rows x heads of a group) per partial: the most any sequence has, at most 16
};
// wg_target: 0 = default
DecodePlan plan_decode(SeqTable &st, const Shape &sh, int wg_target);

// The same plan made on the device, for decode steps whose launches must not change from step to
// step (a captured graph that is replayed): a step of one new row for each of the first n_seqs
// slots of a cache.  decode_plan_kernel reads the cached lengths from device memory, writes
// this record (also device memory) for the prep and decode kernels of the step, and adds the
// step's rows to the lengths.  The launches then depend on nothing but the number of
// sequences and the head geometry: a fixed 256 workgroups, kDevicePlanSlots(...) partial slots.
struct DecodeDevicePlan {
  SeqTable st;
  int tiles_per_wg;
  SpanTable spans;
  int total_tiles;
  int skip;  // a sequence would outgrow the cache or the cos/sin table: the step's kernels do nothing
};
constexpr int kDevicePlanWorkgroups = 256;
inline int device_plan_slots(int n_seqs, int KV) { return kDevicePlanWorkgroups + n_seqs * KV; }
// lens: cached length per slot (device); rope_positions: positions the cos/sin table covers;
// error: set to 2 when the step is skipped.
hipError_t launch_decode_plan(int *lens, int n_seqs, const Shape &sh, int rope_positions, DecodeDevicePlan *out,
                              int *error, hipStream_t stream);
size_t decode_partial_floats(const Shape &sh, const DecodePlan &p);
// The head dimension the split-K decode kernel lays its tiles out for when the data's is hd: 64,
// 128 or 256, the first that holds hd (a multiple of 4; the rest of a tile is padding that costs
// no memory traffic); 0 when none does.
int decode_tile_head_dim(int hd);
size_t decode_flag_words(const DecodePlan &p);

// q_rot: rotated queries [rows][H*hd]; the cache already holds the new rows.
// before / after (here and in launch_prefill; nullable): events that receive the first clock
// reading of the first kernel and the last one of the last kernel of the launch.
// part_flag: decode_flag_words() words of device memory, zero when allocated; the kernel
// leaves them zero.  error: an int the device can write (pinned host memory will do), set
// to 1 when a workgroup gave up waiting for the partials of others.
struct DecodeArgs {
  const float *q_rot;
  const float *kc, *vc;
  float *out;
  float *partials;
  unsigned *part_flag;
  int *error;
  // for the test of the give-up path only: marks go to flag_set (decode_flag_words() words)
  // instead of part_flag, and waiting ends after spin_limit polls; null / 0 otherwise
  unsigned *flag_set;
  int spin_limit;
  // Rows of another kernel's weights to read into the L2s meanwhile (null: none): extra workgroups
  // behind the attention's own read what the first ahead_wgs workgroups of the product
  // gemvt_kernel<K / 256, 2, 1, false> over ahead_w ([2 ahead_n, ahead_k]) will read, from the
  // same indices modulo 8 and so on the same XCDs.  Host-planned launches of head_dim 64 or 128 only.
  const float *ahead_w = nullptr;
  int ahead_k = 0, ahead_n = 0, ahead_wgs = 0;
};
// dev != nullptr: st gives the number of sequences only, p the grid (kDevicePlanWorkgroups), the
// slots and the columns; everything that depends on the cached lengths is read from *dev.
hipError_t launch_decode(const DecodeArgs &d, const SeqTable &st, const Shape &sh, const DecodePlan &p, float scale,
                         hipStream_t stream, hipEvent_t before = nullptr, hipEvent_t after = nullptr,
                         const DecodeDevicePlan *dev = nullptr);
// Key splits of a prefill launch: 1 when the row blocks alone fill the chip, more
// when they do not (few new rows on a long cached prefix); each split leaves
// partial rows in `partials` (prefill_partial_floats) and a second kernel merges.
int prefill_key_splits(const SeqTable &st, const Shape &sh, int items);
size_t prefill_partial_floats(const Shape &sh, int items, int ns);
// The head dimension the MFMA prefill kernel lays its tiles out for when the data's is hd: 64 or
// 128, the first that holds hd (a multiple of 4); 0 when neither does.
int prefill_tile_head_dim(int hd);
// wgs_per_cu: 0 = default; 1..3 pads the kernel's LDS so that at most that many
// workgroups share a compute unit (a tuning knob).
// groups: 0 = default; 1 or 2 forces the number of wavefront groups per workgroup (a tuning knob).
hipError_t launch_prefill(const float *q_rot, const float *kc, const float *vc, float *out, float *partials,
                          const SeqTable &st, const Shape &sh, int items, int ns, float scale,
                          hipStream_t stream, int wgs_per_cu = 0, int groups = 0, hipEvent_t before = nullptr,
                          hipEvent_t after = nullptr);
// Which instantiation a prefill launch uses and how it is laid out; launch_prefill follows it.
struct PrefillLaunch {
  long long n_wgs;   // row blocks x kv heads x key chunks
  int groups;        // 1: four wavefronts per workgroup; 2: eight
  int turns;         // 0: one workgroup per row block and chunk; 2 or 3: prefill_turns_kernel with that many blocks per workgroup
  int wgs_per_cu;    // 0: as the kernel's registers and LDS allow; 1..3: LDS padded to that occupancy
  size_t pad;        // bytes of dynamic LDS that enforce wgs_per_cu
};
PrefillLaunch plan_prefill_launch(const Shape &sh, int items, int ns, int wgs_per_cu, int groups);
hipError_t launch_generic(const float *q_rot, const float *kc, const float *vc, float *out,
                          const SeqTable &st, const Shape &sh, int total_tokens, float scale,
                          hipStream_t stream);

// y[T,N] = epilogue(norm(x)[T,K] * W[K,N]), T <= 16, N % 4 == 0: the projections of a
// decode step with what surrounds them fused in.
enum { kGemvPlain = 0, kGemvResidual = 1, kGemvSwiglu = 2, kGemvQkvPrep = 3 };
// kGemvQkvPrep: W = W_q | W_k | W_v and the product's rows never go to memory as
// they are: each head row gets its bias, QK-norm and rotation where it is summed up
// and lands in q_rot (query heads) or in the cache of one sequence at positions
// start_pos + row (key heads rotated, value heads as they are), exactly as
// launch_prep would have left it.  head_dim: a power of two, at most 128.
struct GemvPrep {
  const float *b_q, *b_k, *b_v;  // nullable
  const float *q_norm, *k_norm;  // nullable, [hd]
  double eps;
  const float2 *rope_tab;        // [positions][hd/2] (cos, sin)
  float *q_rot;                  // [T, H*hd]
  float *kc, *vc;                // the sequence's cache: [KV, cap, hd]
  int H, KV, hd, cap, start_pos;
};
struct GemvArgs {
  const float *x;        // [T, K], rows x_stride floats apart
  long long x_stride;
  int norm;              // != 0: RMSNorm the rows of x first (gamma may be null = ones)
  const float *gamma;    // [K]
  double eps;
  const float *w;        // [K, N]; kGemvSwiglu: [K, 2N] = gate_proj | up_proj
  const float *res;      // kGemvResidual: [T, N], y = res + x W
  float *y;              // [T, N]; kGemvSwiglu: silu(x W_gate) * (x W_up)
  float *partials;       // GemvPlan::partial_floats floats when the plan has splits > 1
  unsigned *flags;       // GemvPlan::col_tiles * splits words, zero when allocated; left zero
  unsigned *flag_set;    // null, or where partials are marked complete instead of in `flags` (the test of the give-up path)
  int spin_limit;        // 0, or the polls after which a wait is given up (that test)
  int *error;            // device-writable int, set to 1 when a wait for partials was given up
  int T, K, N;
  int epilogue;
  int rows_per_wave;     // filled in by launch_gemv
  GemvPrep prep;         // kGemvQkvPrep only (y is not written then)
};
struct GemvPlan {
  int rows_per_instr;     // 1: 256-column tiles; 4: 64-column tiles, four rows of W per load instruction
  int rows_per_wave;
  int splits;             // workgroups along K; partial sums are added in a fixed order
  int col_tiles;
  size_t partial_floats;  // scratch the launch needs
};
// head_dim: kGemvQkvPrep only (a column tile must hold whole heads)
GemvPlan plan_gemv(int T, int K, int N, int epilogue, int head_dim = 0);
hipError_t launch_gemv(const GemvArgs &a, const GemvPlan &p, hipStream_t stream);
// The same product for one row of x against weights kept transposed (a.w: [N, K], or [2N, K] =
// gate | up for kGemvSwiglu): a wavefront per output, nothing shared between wavefronts.
// gemvt_takes: what it serves (one row; K 1024, 2048, 4096, or 8192 without norm and SwiGLU; the
// kGemvQkvPrep epilogue, a.w: [(H + 2 KV) hd, K], where *prep asks for no QK-norm).
bool gemvt_takes(int T, int K, int N, int epilogue, bool norm, const GemvPrep *prep = nullptr);
hipError_t launch_gemvt(const GemvArgs &a, hipStream_t stream);

// A pinned host int per context (block, model) that its kernels set when they give up a
// bounded wait for other workgroups (null when it cannot be allocated); check_error_word,
// called after a wait for the handle's stream, turns a set word into SHAINET_HIP_ERR_RUNTIME
// and clears it: the give-up is reported by the handle whose kernel gave up.
int *alloc_error_word();
void free_error_word(int *w);
int check_error_word(int *w);

hipError_t launch_legacy_append(const float *staging, float *kc, float *vc, int new_tokens, int start_pos,
                                int num_kv_heads, int head_dim, int capacity, hipStream_t stream);

}  // namespace shainet
