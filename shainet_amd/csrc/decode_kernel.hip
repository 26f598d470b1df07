// Split-K (flash-decoding) attention of one new row per sequence over the device
// KV cache, for gfx950.  Replaces the T = 1 case of attention_heads_cpu
// (llama_block.cr:302-401) and of the reference's attention_kv_kernel
// (cuda_kernels.cu:734-806), which launches one block per query head and walks
// the keys serially.
//
// Work split.  The key ranges of all (sequence, kv head) pairs are laid end to
// end in units of 16-key tiles and cut into equal contiguous spans, one per
// workgroup, so every workgroup streams the same number of bytes whatever the
// sequence lengths are.  A span that crosses a pair boundary is processed as two
// segments.  The four wavefronts of a workgroup take the tiles of the span
// round-robin (across segments), each keeping its own online softmax per segment,
// and merge through LDS into one partial (max, sum, O) per segment; the workgroup
// that holds the end of a pair waits, once its own span is done, for the partials
// of the workgroups that hold the pair's earlier parts (flag words say when a
// partial is complete; the merging workgroup clears them again), merges them in a
// fixed order and writes the output row, so a decode step is one launch.  Nothing
// a workgroup does between two segments waits for another workgroup or for memory:
// a wavefront's first tile of the next segment is fetched during its last tile of
// this one, and a partial is marked complete one tile later.
//
// Per 16-key tile a wavefront
//   * copies the K tile (16 contiguous rows) from HBM straight into LDS with
//     global_load_lds_dwordx4, 1 KiB per instruction, fully coalesced, with the
//     16-byte pieces of each row XOR-swizzled so that the later ds_read_b128 of
//     MFMA operands is bank-conflict free;
//   * loads the V tile into registers (256 contiguous bytes per 16 lanes);
//   * computes S^T = K Q^T with v_mfma_f32_16x16x4_f32: rows = keys, columns =
//     the g query heads of the GQA group, so K and V are read once per group;
//   * updates the online softmax with wavefront shuffles, and accumulates
//     O^T += V^T P^T with the probabilities taken directly from the S^T
//     accumulator registers (they already have the B-operand layout).
// The loads of tile t+1 are issued before the arithmetic of tile t.
//
// MFMA 16x16x4 operand layout (lane l): A[m = l%16][k = l/16], B[k = l/16][n = l%16],
// D[m = 4*(l/16) + r][n = l%16] for accumulator register r = 0..3.  The
// contraction index may be visited in any order as long as A and B agree:
//   scores: k-step s of lane group j = l/16 covers d = 16*(s/4) + 4*j + s%4;
//   output: tile t, row m is d = 64*(t/4) + 4*m + t%4; k-step r of lane group j is
//           key 4*j + r of the tile, where accumulator register r of S^T lives.
#include "attn_kernels.hpp"

#include <math.h>
#include <stdint.h>
#include <stdlib.h>

namespace shainet {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Split-K partials cross workgroups that may sit on different XCDs, whose L2
// caches are not kept coherent with each other for ordinary accesses.  Relaxed
// atomic accesses at agent scope compile to write-through stores and cache-
// bypassing loads, which is all that is needed for data published through a
// flag word written after them.
__device__ __forceinline__ void coherent_store(float *p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void coherent_store4(float *p, f32x4 v) {  // the same, 16 bytes at a time
  asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ float coherent_load(const float *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

#define LDS_PTR(p) ((__attribute__((address_space(3))) void *)(uintptr_t)(p))
#define GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void *)(p))

template <int HD>
struct DecodeCfg {
  static constexpr int NT = HD / 16;         // float4 of K per lane per tile; d tiles of the output
  static constexpr int PPR = HD / 4;         // 16-byte pieces per row
  static constexpr int ROW_BYTES = HD * 4;
  static constexpr int TILE_BYTES = 16 * ROW_BYTES;
  static constexpr int NKI = TILE_BYTES / 1024;  // global_load_lds instructions per K tile
  static constexpr int NVU = HD / 64;            // float4 of a V row per lane
};

// K and V rows are read once per launch and there are far more of them than the caches hold:
// they are loaded with the non-temporal hint (`nt`), which tells the caches not to keep them.
// Measured on the batch of 16 sequences of 2048 to 8192 keys: 112.2 -> 102.5 us per launch, and
// 181 -> 162 us with every sequence at 8192; the cache-scope bits on top of it change nothing.
constexpr int kNonTemporal = 2;  // the nt bit of the cache-policy operand

// PAD: the head dimension hd of the data is any multiple of 4 up to HD, the head dimension the
// tiles are laid out for.  The query's elements beyond hd are zeros, so whatever stands in for
// the keys' there does not reach the scores, and output elements beyond hd are never stored;
// the pieces of a tile beyond hd repeat the row's first piece (a cache hit, no HBM traffic).
// Without PAD hd == HD and no instruction is spent on any of this.
//
// Issue the asynchronous copy of the K tile starting at row `kb` into `lds`.
template <int HD, bool PAD>
__device__ __forceinline__ void issue_k_tile(const float *kbase, int kb, int last_row, char *lds, int lane, int hd) {
  using C = DecodeCfg<HD>;
#pragma unroll
  for (int u = 0; u < C::NKI; ++u) {
    const int slot = u * 64 + lane;
    const int row = slot / C::PPR, q = slot % C::PPR;
    int piece = q ^ row;  // row < 16 only touches the low four bits
    if (PAD) piece = 4 * piece < hd ? piece : 0;
    const float *src = kbase + (long long)min(kb + row, last_row) * (PAD ? hd : HD) + 4 * piece;
    __builtin_amdgcn_global_load_lds(GLOBAL_PTR(src), LDS_PTR(lds + u * 1024), 16, 0, kNonTemporal);
  }
}

template <int HD, bool PAD>
__device__ __forceinline__ void load_v_tile(const float *vbase, int kb, int last_row, int col, int j,
                                            f32x4 (&v)[4][DecodeCfg<HD>::NVU], int hd) {
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const float *vp = vbase + (long long)min(kb + 4 * j + r, last_row) * (PAD ? hd : HD);
#pragma unroll
    for (int u = 0; u < DecodeCfg<HD>::NVU; ++u) {
      int d = 4 * col + 64 * u;
      if (PAD) d = d < hd ? d : 0;
      v[r][u] = __builtin_nontemporal_load((const f32x4 *)(vp + d));
    }
  }
}

// Spans: eight consecutive workgroups share 8 * tiles_per_wg tiles of the stream, workgroup
// 8k + r taking tiles [off[r], off[r + 1]) of them (SpanTable, made by plan_decode).  Workgroups
// go to the eight XCDs round-robin by index, and the XCDs of the machines measured do not
// stream equally fast (see plan_decode), so equal spans would not end together.
__device__ __forceinline__ int span_begin(int w, int tiles_per_wg, const SpanTable &sp) {
  return (w >> 3) * 8 * tiles_per_wg + sp.off[w & 7];
}
__device__ __forceinline__ int workgroup_of_tile(int t, int tiles_per_wg, const SpanTable &sp) {
  const int k = t / (8 * tiles_per_wg), rel = t - k * 8 * tiles_per_wg;
  int r = 0;
#pragma unroll
  for (int i = 1; i < 8; ++i) r += rel >= sp.off[i] ? 1 : 0;
  return 8 * k + r;
}

// One segment of a workgroup's span: tiles [tile0, tile1) of one (sequence, kv head) pair.
struct Segment {
  int s, kvh, R, L, n_s, tile0, tile1, token;  // R new rows; L keys visible to the last of them
  int rot;  // the segment's tiles are visited from tile0 + rot on, wrapping round to tile0 + rot - 1
  const float *kbase, *vbase;
};

// Where a workgroup starts within a segment.  Workgroups that all walk their spans from the first
// tile on move through memory in step, a fixed number of bytes apart, and for some distances
// (129 or 145 tiles of 8 KiB, for one) their requests pile up on a few memory channels: a plain
// read kernel laid out that way drops from 6.1 to 5.2 and 4.8 TB/s, and keeps 6.0 TB/s at every
// distance when each workgroup starts at a different place of its range.  The order of the keys
// does not matter to an online softmax.
__device__ __forceinline__ int segment_rotation(int n_tiles, unsigned rotate) {
  if (!rotate || n_tiles < 2) return 0;
  return (int)(((blockIdx.x * 2654435761u) >> 12) % min((unsigned)n_tiles, rotate));
}

// The segment that starts at tile t of the stream; s: a sequence at or before t's, moved up to it.
__device__ __forceinline__ Segment segment_at(int t, int t_end, int &s, const SeqTable &st, const Shape &sh, int hd,
                                              const float *kc, const float *vc, unsigned rotate) {
  while (s + 1 < st.n_seqs && t >= st.work_off[s + 1]) ++s;
  Segment g;
  g.s = s;
  g.R = st.n_new[s];
  g.L = st.start_pos[s] + g.R;  // visible keys of the last new row
  g.n_s = (g.L + 15) >> 4;    // tiles per kv head of this sequence
  const int rel = t - st.work_off[s];
  g.kvh = rel / g.n_s;
  g.tile0 = rel - g.kvh * g.n_s;
  g.tile1 = g.tile0 + min(g.n_s - g.tile0, t_end - t);
  g.rot = __builtin_amdgcn_readfirstlane(segment_rotation(g.tile1 - g.tile0, rotate));
  const long long head_base = (long long)st.slot[s] * sh.seq_stride + (long long)g.kvh * sh.cap * hd;
  g.kbase = kc + head_base;
  g.vbase = vc + head_base;
  g.token = st.tok_off[s];
  return g;
}

constexpr int kFlagSpinLimit = 1 << 21;  // polls of about a microsecond each: seconds

// part_flag: NW words per partial slot, zero between launches: each wavefront sets its word of
// a partial once its share is in memory, the workgroup that merges the pair clears the words it waited for
// (so a launch may be replayed as it is).  error: set when the wait for other workgroups'
// partials was given up, after spin_limit polls.  flag_set: where the marks are written; the
// same as part_flag except in the test of that give-up, which sends them elsewhere.
// DEV: the sequence table and the spans come from *dev (device memory, written by
// decode_plan_kernel earlier on the stream) instead of from the kernel arguments.
struct ReadAhead {
  const float *w;  // [2 n, k]
  int k, n, first_wg;
};
// AHEAD: workgroups from ah.first_wg on (a multiple of 8) do not attend: workgroup first_wg + j
// reads the rows 4 j .. 4 j + 3 and n + the same of ah.w with ordinary loads and drops them, so
// that the launch that needs them next finds them in its XCD's L2 (a decode step of one sequence
// leaves the memory system idle while it waits on its chain of dependent loads).
template <int HD, int NW, bool DEV, bool PAD, bool AHEAD = false>
__global__ __launch_bounds__(64 * NW, NW == 4 && HD <= 128 ? 2 : 1) void decode_splitk_kernel(
    const float *__restrict__ q_rot, const float *__restrict__ kc, const float *__restrict__ vc,
    float *__restrict__ out, float *part_o, float *part_ml, unsigned *part_flag, unsigned *flag_set,
    int spin_limit, int *error, SeqTable st_arg, Shape sh, int tiles_per_wg_arg, SpanTable sp_arg, int total_tiles_arg,
    int n_slots, int pstride, float c, unsigned rotate, const DecodeDevicePlan *__restrict__ dev, ReadAhead ah) {
  if constexpr (AHEAD) {
    if ((int)blockIdx.x >= ah.first_wg) {
      const int row = 4 * ((int)blockIdx.x - ah.first_wg) + (int)(threadIdx.x >> 6);
      if (row >= ah.n) return;
      const int pieces = ah.k >> 8;  // 16-byte pieces per lane and row
      for (int half = 0; half < 2; ++half) {
        const float *p = ah.w + ((long long)half * ah.n + row) * ah.k + 4 * (threadIdx.x & 63);
        for (int i0 = 0; i0 < pieces; i0 += 8) {
          f32x4 v[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) v[u] = *(const f32x4 *)(p + 256 * min(i0 + u, pieces - 1));
#pragma unroll
          for (int u = 0; u < 8; ++u) asm volatile("" : : "v"(v[u]));
        }
      }
      return;
    }
  }
  using C = DecodeCfg<HD>;
  const SeqTable &st = DEV ? dev->st : st_arg;
  const SpanTable &sp = DEV ? dev->spans : sp_arg;
  const int tiles_per_wg = DEV ? dev->tiles_per_wg : tiles_per_wg_arg;
  const int total_tiles = DEV ? dev->total_tiles : total_tiles_arg;
  constexpr int NT = C::NT;
  // per wavefront two K tile buffers; after a segment's last tile the wavefront parks its O
  // rows [g][HD] in one while the other already receives the next segment's first tile
  __shared__ __attribute__((aligned(1024))) char k_lds[NW][2][C::TILE_BYTES];
  __shared__ float sm_m[NW][16], sm_l[NW][16];  // per wavefront and head: running max, sum
  __shared__ int sm_park[NW];                   // where each wavefront parked its O rows
  constexpr int TILE_FLOATS = C::TILE_BYTES / 4;
  constexpr int WAVE_LDS_FLOATS = 2 * TILE_FLOATS;  // floats between two wavefronts' areas

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // uniform: tile numbers stay in scalar registers
  const int col = lane & 15, j = lane >> 4;
  const int g = sh.g;
  const int hd = PAD ? sh.hd : HD;  // floats between two rows of q, K, V and the output
  const int t_begin = span_begin(blockIdx.x, tiles_per_wg, sp);
  const int t_end = min(total_tiles, span_begin(blockIdx.x + 1, tiles_per_wg, sp));
  if (t_begin >= t_end) return;  // unequal spans can leave the last workgroup without tiles
  char *my_lds = &k_lds[wave][0][0];

  int t = t_begin;
  // The sequence the span starts in: every lane looks at one entry of the prefix sums (a walk
  // along them with dependent scalar loads took 2.5 us for a workgroup in the middle of 16
  // sequences).
  int s = (int)__popcll(__ballot(lane + 1 < st.n_seqs && t_begin >= st.work_off[lane + 1 < kMaxSeqs ? lane + 1 : kMaxSeqs]));
  Segment seg = segment_at(t, t_end, s, st, sh, hd, kc, vc, rotate);

  f32x4 v_next[4][C::NVU];
  float qr[HD / 4];
  // columns beyond the last repeat column 0: their results are never stored, and leaving the
  // loaded values untouched here keeps the wait for them out of this place
  // MFMA column c of a segment is new row c / g, head c % g of the group (R * g <= 16 columns)
  auto load_q = [&](const Segment &sg) {
    const int cq = col < sg.R * g ? col : 0, row = cq / g;
    const float *qp = q_rot + ((long long)(sg.token + row) * sh.H + sg.kvh * g + (cq - row * g)) * hd + 4 * j;
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      f32x4 x = {0.f, 0.f, 0.f, 0.f};
      if (!PAD || 16 * i + 4 * j < hd) x = *(const f32x4 *)(qp + 16 * i);
      qr[4 * i + 0] = x.x;
      qr[4 * i + 1] = x.y;
      qr[4 * i + 2] = x.z;
      qr[4 * i + 3] = x.w;
    }
  };
  // `par`: the one of this wavefront's two buffers that holds (or is receiving) its next K tile.
  // A segment's first tile is fetched while the segment before it is still being worked on.
  int par = 0;
  // The tiles of the span go to the wavefronts round-robin as one sequence, whatever segments
  // they fall into (a fresh start per segment would leave one wavefront with a tile more than
  // its share in every segment): this wavefront's first place in the visiting order of the
  // segment at stream position ts, and the tile at place i of that order.
  auto first_place = [&](int ts) { return (wave - (ts - t_begin)) & (NW - 1); };
  auto tile_at = [&](const Segment &sg, int i) {
    const int n = sg.tile1 - sg.tile0, k = i + sg.rot;
    return sg.tile0 + (k < n ? k : k - n);
  };
  static_assert((NW & (NW - 1)) == 0, "round-robin by masking");
  // start fetching the tile at key row `row` into buffer `which`
  auto fetch = [&](int which, const float *kb_, const float *vb_, int row, int last_row) {
    issue_k_tile<HD, PAD>(kb_, row, last_row, my_lds + which * C::TILE_BYTES, lane, hd);
    load_v_tile<HD, PAD>(vb_, row, last_row, col, j, v_next, hd);
  };
  if (first_place(t) < seg.tile1 - seg.tile0) fetch(0, seg.kbase, seg.vbase, tile_at(seg, first_place(t)) * 16, seg.L - 1);
  load_q(seg);

  // the pair whose last segment this workgroup holds without holding all of it: merged at the
  // end of the span (only a span's first segment can start inside a pair, so there is one at most)
  bool have_merge = false;
  Segment mseg = seg;
  // this wavefront's share of a partial is written but not yet marked complete (slot, or -1):
  // the mark follows the next wait for loads, which then also covers those stores
  int pending = -1;
  auto mark_pending = [&]() {
    if (pending >= 0) {
      if (lane == 0)
        __hip_atomic_store(&flag_set[NW * pending + wave], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      pending = -1;
    }
  };

  for (;;) {
    const int L = seg.L, tile1 = seg.tile1;
    const float *kbase = seg.kbase, *vbase = seg.vbase;
    const int nc = seg.R * g;                                   // columns in use
    const int Lc = L - (seg.R - 1 - (col < nc ? col : 0) / g);  // keys visible to this lane's column
    // the segment after this one, if the span has one
    const int t_next = t + (tile1 - seg.tile0);
    const bool more = t_next < t_end;
    Segment nseg = seg;
    if (more) nseg = segment_at(t_next, t_end, s, st, sh, hd, kc, vc, rotate);
    const int nplace = first_place(t_next);
    const bool nhave = more && nplace < nseg.tile1 - nseg.tile0;
    const int ntile = nhave ? tile_at(nseg, nplace) : 0;
    const int n_here = tile1 - seg.tile0;

    float m = -INFINITY, l = 0.f;
    f32x4 o[NT];
#pragma unroll
    for (int i = 0; i < NT; ++i) o[i] = f32x4{0.f, 0.f, 0.f, 0.f};

    int place = first_place(t);
    // no tile of this segment for this wavefront: on to the next one's
    if (place >= n_here && nhave) fetch(par, nseg.kbase, nseg.vbase, ntile * 16, nseg.L - 1);
    for (; place < n_here; place += NW) {
      const int kb = tile_at(seg, place) * 16;
      const char *buf = my_lds + par * C::TILE_BYTES;
      par ^= 1;
      // everything issued so far (this tile's K copy and V loads) has landed:
      // s_waitcnt vmcnt(0) (expcnt and lgkmcnt fields left at their maxima), then a
      // compiler barrier so that no LDS read of the tile is scheduled above it
      __builtin_amdgcn_s_waitcnt(0x0F70);
      asm volatile("" ::: "memory");
      mark_pending();
      f32x4 v_cur[4][C::NVU];
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int u = 0; u < C::NVU; ++u) v_cur[r][u] = v_next[r][u];
      if (place + NW < n_here)
        fetch(par, kbase, vbase, tile_at(seg, place + NW) * 16, L - 1);
      else if (nhave)
        fetch(par, nseg.kbase, nseg.vbase, ntile * 16, nseg.L - 1);

      f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
      const char *krow = buf + col * C::ROW_BYTES;
#pragma unroll
      for (int i = 0; i < NT; ++i) {
        const f32x4 kk = *(const f32x4 *)(krow + (((4 * i + j) ^ col) << 4));
        s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(kk.x, qr[4 * i + 0], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(kk.y, qr[4 * i + 1], s1, 0, 0, 0);
        s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(kk.z, qr[4 * i + 2], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(kk.w, qr[4 * i + 3], s1, 0, 0, 0);
      }
      float sv[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) sv[r] = (kb + 4 * j + r < Lc) ? s0[r] + s1[r] : -INFINITY;
      float mx = fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3]));
      mx = fmaxf(mx, __shfl_xor(mx, 16));
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      const float mnew = fmaxf(m, mx);
      // with several new rows a column may not see any key of a late tile (-inf so far: 0 stands in)
      const float mref = mnew == -INFINITY ? 0.f : mnew;
      const float alpha = fast_exp2((m - mref) * c);
      float p[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) p[r] = fast_exp2((sv[r] - mref) * c);
      l = l * alpha + ((p[0] + p[1]) + (p[2] + p[3]));
      m = mnew;
#pragma unroll
      for (int i = 0; i < NT; ++i) o[i] *= alpha;
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int u = 0; u < C::NVU; ++u) {
          o[4 * u + 0] = __builtin_amdgcn_mfma_f32_16x16x4f32(v_cur[r][u].x, p[r], o[4 * u + 0], 0, 0, 0);
          o[4 * u + 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(v_cur[r][u].y, p[r], o[4 * u + 1], 0, 0, 0);
          o[4 * u + 2] = __builtin_amdgcn_mfma_f32_16x16x4f32(v_cur[r][u].z, p[r], o[4 * u + 2], 0, 0, 0);
          o[4 * u + 3] = __builtin_amdgcn_mfma_f32_16x16x4f32(v_cur[r][u].w, p[r], o[4 * u + 3], 0, 0, 0);
        }
    }
    // the next segment's query rows (this one's are not needed any more)
    if (more) load_q(nseg);

    // merge the wavefronts through LDS: the wavefront parks its O rows [g][HD] in the one of
    // its two buffers that does not hold (or receive) its next tile
    l += __shfl_xor(l, 16);
    l += __shfl_xor(l, 32);
    float *sm_o = (float *)&k_lds[0][0][0];
    if (col < nc) {
      float *dst = sm_o + wave * WAVE_LDS_FLOATS + (par ^ 1) * TILE_FLOATS + col * HD;
#pragma unroll
      for (int i = 0; i < NT; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) dst[64 * (i >> 2) + 4 * (4 * j + r) + (i & 3)] = o[i][r];
      if (j == 0) {
        sm_m[wave][col] = m;
        sm_l[wave][col] = l;
      }
    }
    if (lane == 0) sm_park[wave] = (par ^ 1) * TILE_FLOATS;
    // a share of an earlier partial that is still unmarked (a wavefront that had no tile since)
    if (pending >= 0) {
      __builtin_amdgcn_s_waitcnt(0x0F70);
      mark_pending();
    }
    __syncthreads();
    const bool whole_pair = seg.tile0 == 0 && tile1 == seg.n_s;
    const int pair = seg.s * sh.KV + seg.kvh;
    const int slot = blockIdx.x + pair;  // unique: both terms only grow along the tile stream
    int park[NW];
#pragma unroll
    for (int w = 0; w < NW; ++w) park[w] = w * WAVE_LDS_FLOATS + sm_park[w];
    for (int idx = threadIdx.x; idx < nc * HD; idx += 64 * NW) {
      const int cc = idx / HD, d = idx - cc * HD;
      float mm = sm_m[0][cc];
#pragma unroll
      for (int w = 1; w < NW; ++w) mm = fmaxf(mm, sm_m[w][cc]);
      const float mref = mm == -INFINITY ? 0.f : mm;  // no key of the segment visible to this column
      float acc = 0.f, ls = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const float f = fast_exp2((sm_m[w][cc] - mref) * c);  // 0 for a wavefront that saw no visible key
        acc += f * sm_o[park[w] + cc * HD + d];
        ls += f * sm_l[w][cc];
      }
      if (whole_pair) {
        const int row = cc / g;
        if (!PAD || d < hd) out[((long long)(seg.token + row) * sh.H + seg.kvh * g + (cc - row * g)) * hd + d] = acc / ls;
      } else if (slot < n_slots) {
        const long long pi = (long long)slot * pstride + cc;
        coherent_store(&part_o[pi * HD + d], acc);
        if (d == 0) {
          coherent_store(&part_ml[2 * pi], mm);
          coherent_store(&part_ml[2 * pi + 1], ls);
        }
      }
    }
    const bool pair_end = !whole_pair && tile1 == seg.n_s;
    if (pair_end) {
      have_merge = true;
      mseg = seg;
    }
    // Partials are written through to device-coherent memory (coherent_store).  Each
    // wavefront marks its share complete in a word of its own once its stores are
    // acknowledged, which the next wait for a tile tells (the barrier alone does not).
    // The partial of a pair's end is read by this workgroup only.
    if (!whole_pair && !pair_end && slot < n_slots) pending = slot;
    // the parked rows are read: the next tiles may land there (with a copy into LDS in flight
    // the barriers here also wait for this wavefront's loads: the compiler's rule, which is
    // what a boundary inside a span still costs)
    __syncthreads();
    if (!more) break;
    seg = nseg;
    t = t_next;
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // this wavefront's last stores are acknowledged
  mark_pending();

  if (have_merge) {
    // This workgroup holds the end of a pair that others began: they have lower indices, were
    // started before this one and wait for nobody, so waiting for their partials is safe.
    const int a = st.work_off[mseg.s] + mseg.kvh * mseg.n_s;  // the pair's tiles are [a, a + n_s)
    const int w_lo = workgroup_of_tile(a, tiles_per_wg, sp);
    const int n_part = (int)blockIdx.x - w_lo + 1;
    const int pair = mseg.s * sh.KV + mseg.kvh;
    if (wave == 0) {
      // NW words per partial; the last of the n_part partials is this workgroup's own
      unsigned *fl = part_flag + NW * (w_lo + pair);
      for (int spins = 0;; ++spins) {
        bool ok = true;
        for (int i = lane; i < NW * (n_part - 1); i += 64)
          ok = ok && __hip_atomic_load(fl + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u;
        if (__all(ok)) {
          for (int i = lane; i < NW * (n_part - 1); i += 64)
            __hip_atomic_store(fl + i, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
        if (spins >= spin_limit) {
          if (lane == 0) *error = 1;
          break;
        }
        __builtin_amdgcn_s_sleep(2);
      }
    }
    __syncthreads();
    // every partial of the pair is in memory: drop whatever this XCD's caches
    // still hold of those addresses, then read them with ordinary wide loads
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    constexpr int LPR = HD / 4;       // lanes that cover one row with float4
    constexpr int GROUPS = 64 / LPR;  // partials handled side by side
    const int d4 = lane % LPR, grp = lane / LPR;
    const long long base = (long long)(w_lo + pair) * pstride;  // partial of workgroup w, column cc: base + (w - w_lo) * pstride + cc
    for (int cc = wave; cc < mseg.R * g; cc += NW) {
      const long long first = base + cc;
      // the largest of the partials' maxima: from a pass of its own over them, or, when one
      // round of loads covers all partials, from that round (one memory round trip less)
      const bool one_round = n_part <= 8 * GROUPS;
      float mm = -INFINITY;
      if (!one_round) {
        for (int i = lane; i < n_part; i += 64) mm = fmaxf(mm, part_ml[2 * (first + (long long)i * pstride)]);
        for (int o2 = 32; o2 > 0; o2 >>= 1) mm = fmaxf(mm, __shfl_xor(mm, o2));
      }
      float ls = 0.f;
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
      for (int i0 = 0; i0 < n_part; i0 += 8 * GROUPS) {  // eight rows in flight per lane
        f32x4 x[8];
        float f[8], lp[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int i = i0 + u * GROUPS + grp;
          const long long pi = first + (long long)min(i, n_part - 1) * pstride;
          x[u] = *(const f32x4 *)&part_o[pi * HD + 4 * d4];
          f[u] = part_ml[2 * pi];
          lp[u] = part_ml[2 * pi + 1];
        }
        if (one_round) {
#pragma unroll
          for (int u = 0; u < 8; ++u)
            if (u * GROUPS + grp < n_part) mm = fmaxf(mm, f[u]);
#pragma unroll
          for (int o2 = LPR; o2 < 64; o2 <<= 1) mm = fmaxf(mm, __shfl_xor(mm, o2));  // over the lanes of one d4
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int i = i0 + u * GROUPS + grp;
          const float w = i < n_part ? fast_exp2((f[u] - mm) * c) : 0.f;
          acc += w * x[u];
          ls += w * lp[u];
        }
      }
#pragma unroll
      for (int o2 = LPR; o2 < 64; o2 <<= 1) {
        acc.x += __shfl_xor(acc.x, o2);
        acc.y += __shfl_xor(acc.y, o2);
        acc.z += __shfl_xor(acc.z, o2);
        acc.w += __shfl_xor(acc.w, o2);
        ls += __shfl_xor(ls, o2);
      }
      if (grp == 0 && (!PAD || 4 * d4 < hd)) {
        const float inv = 1.0f / ls;
        const int row = cc / g;
        *(f32x4 *)&out[((long long)(mseg.token + row) * sh.H + mseg.kvh * g + (cc - row * g)) * hd + 4 * d4] = acc * inv;
      }
    }
  }
}

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kDecodeWaves = 4;  // wavefronts per workgroup (eight measured 4 % slower)

// Share of each of eight consecutive spans, in thousandths of an equal share, by the XCD the
// workgroup lands on (index mod 8).  With equal spans the workgroups on odd XCDs finished
// streaming about 5 % after those on even XCDs on every box traced (3 and 5 last, 0 and 6
// first; the finer pattern differs from box to box).  SHAINET_HIP_DECODE_SHARES: eight
// numbers, or "0" for equal spans.  Not worth it for short spans.
struct Shares {
  int v[8] = {1050, 950, 1050, 950, 1050, 950, 1050, 950};
  Shares() {
    const char *env = getenv("SHAINET_HIP_DECODE_SHARES");
    if (!env) return;
    int w[8], n = 0;
    for (const char *c = env; *c && n < 8;) {
      char *end;
      const long x = strtol(c, &end, 10);
      if (end == c) break;
      w[n++] = (int)x;
      c = *end ? end + 1 : end;
    }
    for (int i = 0; i < 8; ++i) v[i] = n == 8 && w[i] >= 500 && w[i] <= 1500 ? w[i] : 1000;
  }
};
const Shares &span_shares() {
  static const Shares shares;
  return shares;
}

// Where the spans of eight consecutive workgroups begin within their 8 q tiles, from their shares.
__host__ __device__ inline void spans_from_shares(const int (&share)[8], int q, SpanTable &spans) {
  long long sum = 0, acc = 0;
  for (int i = 0; i < 8; ++i) sum += share[i];
  for (int i = 0; i <= 8; ++i) {
    spans.off[i] = q >= 32 ? (int)(acc * 8 * q / sum) : i * q;
    if (i < 8) acc += share[i];
  }
}

struct ShareArg {
  int v[8];
};

// plan_decode on the device for one new row per sequence: one wavefront, lane s looks after
// sequence s.  Reads the cached lengths, writes the record the step's prep and decode kernels
// read, and adds the step's rows to the lengths.
__global__ __launch_bounds__(64) void decode_plan_kernel(int *__restrict__ lens, int n_seqs, Shape sh, int rope_positions,
                                                         ShareArg shares, DecodeDevicePlan *__restrict__ out,
                                                         int *error) {
  const int s = threadIdx.x;
  const bool mine = s < n_seqs;
  const int start = mine ? lens[s] : 0;
  const bool fits = !mine || (start >= 0 && start + 1 <= sh.cap && start + 1 <= rope_positions);
  if (!__all(fits)) {  // nothing is appended: the lengths stay as they are
    if (s == 0) {
      out->st.n_seqs = n_seqs;
      out->tiles_per_wg = 0;
      out->total_tiles = 0;
      out->skip = 1;
      spans_from_shares(shares.v, 0, out->spans);  // all zero: no workgroup finds tiles
      if (*error == 0) *error = 2;  // a pending 1 (a given-up wait) is the graver report and stays
    }
    return;
  }
  const int tiles = mine ? sh.KV * ((start + 1 + 15) >> 4) : 0;
  int incl = tiles;  // inclusive prefix sum over the lanes
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int up = __shfl_up(incl, o);
    if (s >= o) incl += up;
  }
  const int total = __shfl(incl, 63);
  if (mine) {
    out->st.slot[s] = s;
    out->st.start_pos[s] = start;
    out->st.n_new[s] = 1;
    out->st.tok_off[s] = s;
    out->st.work_off[s] = incl - tiles;
    lens[s] = start + 1;
  }
  if (s == 0) {
    out->st.n_seqs = n_seqs;
    out->st.tok_off[n_seqs] = n_seqs;
    out->st.work_off[n_seqs] = total;
    int q = (total + kDevicePlanWorkgroups - 1) / kDevicePlanWorkgroups;
    if (q < kDecodeWaves) q = kDecodeWaves;
    out->tiles_per_wg = q;
    out->total_tiles = total;
    out->skip = 0;
    spans_from_shares(shares.v, q, out->spans);
  }
}

}  // namespace

DecodePlan plan_decode(SeqTable &st, const Shape &sh, int wg_target) {
  DecodePlan p;
  st.work_off[0] = 0;
  for (int s = 0; s < st.n_seqs; ++s)
    st.work_off[s + 1] = st.work_off[s] + sh.KV * ((st.start_pos[s] + st.n_new[s] + 15) / 16);
  p.total_tiles = st.work_off[st.n_seqs];
  // One workgroup on each of the 256 compute units.  Its four wavefronts keep 64 KiB
  // of K and V in flight, 16 MiB over the chip, which saturates HBM; twice as many
  // workgroups only double the partials to merge and the arrivals at each pair's
  // counter (measured: 4 to 10 % slower from batch 1 x 4096 to batch 4 x 32768).
  if (wg_target < 1) wg_target = 256;
  // at least one tile per wavefront
  int q = (p.total_tiles + wg_target - 1) / wg_target;
  if (q < kDecodeWaves) q = kDecodeWaves;
  p.tiles_per_wg = q;
  spans_from_shares(span_shares().v, q, p.spans);
  // the first workgroup count whose spans cover the stream
  p.n_wgs = (p.total_tiles + q - 1) / q;
  auto begin_of = [&](int w) { return (w >> 3) * 8 * q + p.spans.off[w & 7]; };
  while (p.n_wgs > 1 && begin_of(p.n_wgs - 1) >= p.total_tiles) --p.n_wgs;
  while (begin_of(p.n_wgs) < p.total_tiles) ++p.n_wgs;
  p.n_slots = p.n_wgs + st.n_seqs * sh.KV;
  p.cols = 0;
  for (int s = 0; s < st.n_seqs; ++s) p.cols = st.n_new[s] * sh.g > p.cols ? st.n_new[s] * sh.g : p.cols;
  return p;
}

size_t decode_flag_words(const DecodePlan &p) { return (size_t)p.n_slots * kDecodeWaves; }

// The head dimension the split-K kernel's tiles are laid out for: 64, 128 or 256 (0: none fits).
int decode_tile_head_dim(int hd) {
  if (hd < 4 || (hd & 3) || hd > 256) return 0;
  return hd <= 64 ? 64 : hd <= 128 ? 128 : 256;
}

size_t decode_partial_floats(const Shape &sh, const DecodePlan &p) {
  return (size_t)p.n_slots * p.cols * (decode_tile_head_dim(sh.hd) + 2);
}

hipError_t launch_decode_plan(int *lens, int n_seqs, const Shape &sh, int rope_positions, DecodeDevicePlan *out,
                              int *error, hipStream_t stream) {
  if (!lens || !out || !error || n_seqs < 1 || n_seqs > kMaxSeqs) return hipErrorInvalidValue;
  ShareArg shares;
  for (int i = 0; i < 8; ++i) shares.v[i] = span_shares().v[i];
  hipLaunchKernelGGL(decode_plan_kernel, dim3(1), dim3(64), 0, stream, lens, n_seqs, sh, rope_positions, shares, out,
                     error);
  return hipGetLastError();
}

hipError_t launch_decode(const DecodeArgs &d, const SeqTable &st, const Shape &sh, const DecodePlan &p, float scale,
                         hipStream_t stream, hipEvent_t before, hipEvent_t after, const DecodeDevicePlan *dev) {
  if (st.n_seqs < 1 || st.n_seqs > kMaxSeqs || sh.g < 1 || sh.g > 16 || sh.H != sh.KV * sh.g ||
      !decode_tile_head_dim(sh.hd) || p.n_wgs < 1 || !d.partials || !d.part_flag || !d.error)
    return hipErrorInvalidValue;
  if (dev) {
    if (p.n_wgs != kDevicePlanWorkgroups || p.n_slots != device_plan_slots(st.n_seqs, sh.KV) || p.cols < sh.g)
      return hipErrorInvalidValue;
  } else {
    if (p.tiles_per_wg < 1) return hipErrorInvalidValue;
    for (int s = 0; s < st.n_seqs; ++s)
      if (st.n_new[s] < 1 || st.n_new[s] * sh.g > 16 || st.n_new[s] * sh.g > p.cols || st.start_pos[s] < 0 ||
          st.start_pos[s] + st.n_new[s] > sh.cap || st.slot[s] < 0)
        return hipErrorInvalidValue;
  }
  if (!d.q_rot) return hipErrorInvalidValue;
  unsigned *flag_set = d.flag_set ? d.flag_set : d.part_flag;
  const int spin_limit = d.spin_limit > 0 ? d.spin_limit : kFlagSpinLimit;
  float *part_o = d.partials;
  const int tile_hd = decode_tile_head_dim(sh.hd);
  float *part_ml = d.partials + (size_t)p.n_slots * p.cols * tile_hd;
  const float c = scale * kLog2e;
  // before / after (nullable) receive the kernel's own first and last clock reading, not the
  // time at which the stream reached them: what is between two kernels stays out
  dim3 grid((unsigned)p.n_wgs), block(64 * kDecodeWaves);
  ReadAhead ah = {nullptr, 0, 0, 0};
  if (d.ahead_w && d.ahead_wgs > 0 && !dev && !before && !after && (sh.hd == 64 || sh.hd == 128) && d.ahead_k >= 256 &&
      (d.ahead_k & 255) == 0 && d.ahead_n > 0) {
    ah.w = d.ahead_w;
    ah.k = d.ahead_k;
    ah.n = d.ahead_n;
    ah.first_wg = (p.n_wgs + 7) / 8 * 8;
    const int most = (d.ahead_n + 3) / 4;
    grid.x = (unsigned)(ah.first_wg + (d.ahead_wgs < most ? d.ahead_wgs : most));
  }
  // SHAINET_HIP_DECODE_NO_ROTATE: every workgroup walks its segments from their first tile (for
  // comparison); SHAINET_HIP_DECODE_ROTATE=n: starts spread over the first n tiles only
  static const unsigned rotate = getenv("SHAINET_HIP_DECODE_NO_ROTATE") ? 0u
                                 : getenv("SHAINET_HIP_DECODE_ROTATE")
                                     ? (unsigned)atoi(getenv("SHAINET_HIP_DECODE_ROTATE"))
                                     : 0x7fffffffu;
#define SHAINET_DECODE_LAUNCH(HD_, DEV_, PAD_)                                                                      \
  SHAINET_LAUNCH_TIMED((decode_splitk_kernel<HD_, kDecodeWaves, DEV_, PAD_>), grid, block, 0, stream, before,      \
                       after, d.q_rot, d.kc, d.vc, d.out, part_o, part_ml, d.part_flag, flag_set, spin_limit,       \
                       d.error, st, sh, p.tiles_per_wg, p.spans, p.total_tiles, p.n_slots, p.cols, c, rotate, dev, ah)
#define SHAINET_DECODE_LAUNCH_HD(HD_, PAD_) \
  do {                                      \
    if (dev)                                \
      SHAINET_DECODE_LAUNCH(HD_, true, PAD_);  \
    else                                    \
      SHAINET_DECODE_LAUNCH(HD_, false, PAD_); \
  } while (0)
  if (ah.w && sh.hd == 64)
    hipLaunchKernelGGL((decode_splitk_kernel<64, kDecodeWaves, false, false, true>), grid, block, 0, stream, d.q_rot, d.kc,
                       d.vc, d.out, part_o, part_ml, d.part_flag, flag_set, spin_limit, d.error, st, sh, p.tiles_per_wg,
                       p.spans, p.total_tiles, p.n_slots, p.cols, c, rotate, dev, ah);
  else if (ah.w)
    hipLaunchKernelGGL((decode_splitk_kernel<128, kDecodeWaves, false, false, true>), grid, block, 0, stream, d.q_rot, d.kc,
                       d.vc, d.out, part_o, part_ml, d.part_flag, flag_set, spin_limit, d.error, st, sh, p.tiles_per_wg,
                       p.spans, p.total_tiles, p.n_slots, p.cols, c, rotate, dev, ah);
  else if (sh.hd == 64)
    SHAINET_DECODE_LAUNCH_HD(64, false);
  else if (sh.hd == 128)
    SHAINET_DECODE_LAUNCH_HD(128, false);
  else if (tile_hd == 64)
    SHAINET_DECODE_LAUNCH_HD(64, true);
  else if (tile_hd == 128)
    SHAINET_DECODE_LAUNCH_HD(128, true);
  else
    SHAINET_DECODE_LAUNCH_HD(256, true);
#undef SHAINET_DECODE_LAUNCH_HD
#undef SHAINET_DECODE_LAUNCH
  return hipGetLastError();
}

}  // namespace shainet
