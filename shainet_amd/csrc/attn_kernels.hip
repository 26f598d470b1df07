// Causal grouped-query attention over the device KV cache for gfx950 (CDNA4).
//
// Together with decode_kernel.hip (one new row per sequence) these kernels replace
// attention_heads_cpu (llama_block.cr:302-401) and the reference's
// attention_kv_kernel (cuda_kernels.cu:734-806):
//
//   prefill_mfma_kernel   many new rows.  Query rows and the heads of a group
//       are flattened into "virtual rows"; a wavefront owns 32 of them, a
//       workgroup 128.  K/V tiles of 32 keys are staged through LDS (double
//       buffered) and consumed by v_mfma_f32_32x32x2_f32.
//   generic_attn_kernel   any head_dim; one wavefront per (row, head).  Used for
//       head dims other than 64 and 128.
//
// The MFMA kernels compute S^T = K Q^T so that the probabilities come out of the MFMA
// accumulator already laid out as the B operand of O^T = V^T P^T: no transpose,
// no LDS round trip for P.  The contraction index of an MFMA may be visited in
// any order as long as A and B agree, which lets every lane fetch 16-byte
// pieces of K rows.
#include "attn_kernels.hpp"

#include <math.h>
#include <stdlib.h>
#include <string.h>

namespace shainet {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Scheduling fence that scalar and vector ALU instructions may cross but LDS,
// MFMA and global-memory instructions may not: keeps operand fetches ahead of the
// MFMAs that use them, where the source puts them, instead of next to them.
#define ORDER_LDS_AND_MFMA() __builtin_amdgcn_sched_barrier(0x7)

__device__ __forceinline__ int find_seq(const SeqTable &st, int item, const int *off) {
  int s = 0;
  while (s + 1 < st.n_seqs && item >= off[s + 1]) ++s;
  return s;
}

// ---------------------------------------------------------------------------
// Prefill: MFMA 32x32x2, K/V tiles staged through LDS.
//
// Virtual row v of a (sequence, kv head): query row v / g, head kvh*g + v % g.
// MFMA 32x32x2 layout (lane l): A[m = l%32][k = l/32], B[k = l/32][n = l%32],
// D[m = 8*(r/4) + 4*(l/32) + r%4][n = l%32] for accumulator register r = 0..15.
//   scores:  m = key within the tile, n = virtual row; k-step s of lane half
//            j = l/32 covers d = 8*(s/4) + 4*j + s%4 (float4 pieces of a K row).
//   output:  tile t, m = d index (d = NT*m + t), contraction over the tile's keys in
//            the order the score accumulator holds them.
// Row block number `rank` in dispatch order -> (sequence, block).  Level 0 is every
// sequence's last block (the longest key range), level 1 the one before, and so
// on.  st.work_off[s] = row blocks of sequence s, st.ord = sequences by descending
// block count.
__device__ __forceinline__ void locate_block(const SeqTable &st, int rank, int &s, int &vb) {
  s = 0;
  int level = 0;
  for (int b = st.n_seqs - 1; b >= 0; --b) {  // levels [n_{b+1}, n_b) have b+1 active sequences
    const int lo = b + 1 < st.n_seqs ? st.work_off[st.ord[b + 1]] : 0;
    const int cnt = (st.work_off[st.ord[b]] - lo) * (b + 1);
    if (rank < cnt) {
      level = lo + rank / (b + 1);
      s = st.ord[rank % (b + 1)];
      break;
    }
    rank -= cnt;
  }
  vb = st.work_off[s] - 1 - level;
}

// G = 1: four wavefronts, each with 32 virtual rows, walk the key tiles together.
// G = 2: eight wavefronts; wavefronts 4..7 own the same rows as 0..3 and take every
// second key tile, so that each SIMD holds two wavefronts of one workgroup and the
// waits of one (barrier, LDS and memory latencies) hide behind the work of the other
// even when a launch puts a single workgroup on a compute unit (vector instructions
// do not hide: fp32 MFMAs and vector instructions share the SIMD's lanes).  The two
// halves merge through LDS.
// One workgroup's work: the row block (and key chunk) number `bid` of the launch.
// PAD: the head dimension of the data (sh.hd, a multiple of 4) is smaller than HD, the one the
// tiles are laid out for: query elements beyond it are zeros (whatever stands in for the keys'
// there does not reach the scores), output elements beyond it are not stored, and a tile's
// pieces beyond it repeat the row's first piece (a cache hit, no HBM traffic).
template <int HD, bool SPLIT, int G, bool PAD>
__device__ __forceinline__ void prefill_block(const int bid, const float *__restrict__ q_rot,
                                              const float *__restrict__ kc, const float *__restrict__ vc,
                                              float *__restrict__ out, float *__restrict__ part_o,
                                              float *__restrict__ part_ml, const SeqTable &st, const Shape &sh,
                                              int ns, float c) {
  constexpr int NK4 = HD / 8;   // float4 pieces of a K row per lane
  constexpr int NT = HD / 32;   // d tiles of the output
  constexpr int KSTR = HD + 4;  // padded K row stride in LDS: conflict-free 16-byte reads down a column
  constexpr int LD4 = HD / 32;  // float4 per thread to stage the G K (or V) tiles of one step
  constexpr int NTHREADS = 256 * G;
  constexpr int TILE4 = 32 * (HD / 4);  // float4 per tile
  __shared__ float Ks[2][G][32 * KSTR];
  __shared__ float Vs[2][G][32 * HD];

  // Workgroups are numbered so that the hardware dispatcher, which hands them out in
  // index order, starts the row blocks with the longest key ranges first; the kv
  // head is the fastest index, so with 8 kv heads each XCD (index % 8) keeps to one
  // head and its K/V stay in that XCD's L2.  When a launch has too few row blocks to
  // fill the chip, each block's key range is cut into ns chunks that run as separate
  // workgroups and leave partial (max, sum, O) rows for prefill_combine_kernel.
  const int kvh = bid % sh.KV;
  const int chunk = SPLIT ? (bid / sh.KV) % ns : 0;
  const int item = SPLIT ? bid / sh.KV / ns : bid / sh.KV;
  int s, vb;
  locate_block(st, item, s, vb);
  // These are the same for all lanes of a wavefront, which the compiler cannot see: said so,
  // tile counts, loop conditions and address bases live in scalar registers and their
  // arithmetic leaves the vector ALU, which the MFMAs need
  auto uniform = [](int x) { return __builtin_amdgcn_readfirstlane(x); };
  s = uniform(s);
  vb = uniform(vb);
  const int g = sh.g, T = st.n_new[s], S = st.start_pos[s];
  const int L = S + T, VR = T * g;
  const int lane = threadIdx.x & 63;
  const int wave = uniform((threadIdx.x >> 6) & 3);  // which 32 virtual rows of the block
  const int gidx = uniform(threadIdx.x >> 8);        // which share of the key tiles (always 0 for G = 1)
  const int n = lane & 31, j = lane >> 5;
  const int v0 = vb * 128 + wave * 32;
  const bool wave_active = v0 < VR;
  const int my_v = v0 + n;
  const bool valid = my_v < VR;
  const int row = valid ? my_v / g : T - 1;
  const int hg = valid ? my_v - row * g : 0;
  const int lim = S + row;                                            // last visible key of this lane's row
  const int wave_lo = S + (wave_active ? v0 / g : 0);                 // smallest lim in the wavefront
  const int wave_hi = wave_active ? S + min(v0 + 31, VR - 1) / g : -1;  // largest
  const int wg_hi = S + min(vb * 128 + 127, VR - 1) / g;
  const int n_tiles = wg_hi / 32 + 1;
  const int tiles_per_chunk = SPLIT ? (n_tiles + ns - 1) / ns : n_tiles;
  const int kt0 = chunk * tiles_per_chunk, kt1 = min(n_tiles, kt0 + tiles_per_chunk);
  const int hd = PAD ? uniform(sh.hd) : HD;  // floats between two rows of q, K, V and the output
  const long long head_base = (long long)st.slot[s] * sh.seq_stride + (long long)kvh * sh.cap * hd;
  const float *kbase = kc + head_base;
  const float *vbase = vc + head_base;
  const long long qo_off = ((long long)(st.tok_off[s] + row) * sh.H + kvh * g + hg) * hd;

  float qr[HD / 2];
  {
    const float *qp = q_rot + qo_off + 4 * j;
#pragma unroll
    for (int i = 0; i < NK4; ++i) {
      // (lanes past the last virtual row repeat the last row: their results are never used,
      // and not touching the loaded values here lets the first K and V loads go out behind
      // these instead of after their arrival)
      f32x4 t = {0.f, 0.f, 0.f, 0.f};
      if (!PAD || 8 * i + 4 * j < hd) t = *(const f32x4 *)(qp + 8 * i);
      qr[4 * i + 0] = t.x;
      qr[4 * i + 1] = t.y;
      qr[4 * i + 2] = t.z;
      qr[4 * i + 3] = t.w;
    }
  }

  // Online softmax against a reference value per virtual row instead of the running maximum.
  // The fp32 MFMAs run on the lanes of the vector ALU (a wavefront's vector instructions and
  // MFMAs, its own or its SIMD neighbour's, never overlap: measured, 6 cycles per fma and 12
  // per exp2 added to a stream of 64-cycle MFMAs), so every vector instruction of the tile loop
  // is paid in matrix throughput.  Hence:
  //   * the query rows are scaled by scale * log2(e) once, so scores come out in log2 units;
  //   * the score accumulator starts at -m_ref instead of 0, so the MFMAs deliver s - m_ref;
  //   * m_ref is only moved (and l, O rescaled) when a score exceeds it by more than kTau, or
  //     for a row's first visible key; probabilities are then at most 2^kTau, no overflow.
  // A tile on the common path costs a maximum, 16 exp2 and 16 adds per lane.
  constexpr float kTau = 8.f;
  float m_ref = 0.f, l = 0.f;
  float thr = -INFINITY;  // a row's scores move m_ref when above this: anything finite until its first key, kTau after
  // -m_ref as the score MFMAs' initial accumulator: sixteen registers that hold it, or, where
  // registers are short (head_dim 128), one more MFMA per tile that multiplies it by a column
  // of ones
  constexpr bool kRefByMfma = HD == 128;
  f32x16 neg_m;
#pragma unroll
  for (int r = 0; r < 16; ++r) neg_m[r] = 0.f;
  const float ones_col = j == 0 ? 1.f : 0.f;  // A[key][k]: 1 for k = 0
  f32x16 o[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[t][r] = 0.f;

  // Staging registers: the G tiles of a step (tiles kt0 + G*sp .. + G-1, one per
  // group of wavefronts) travel global memory -> registers during one iteration and
  // registers -> LDS at the start of the next.
  f32x4 stage_k[LD4], stage_v[LD4];
  // what a thread fetches of a step's G tiles does not change from step to step: row
  // row_in_step[u] of the step's 32 G rows, columns col4 .. col4 + 3
  int row_in_step[LD4];
#pragma unroll
  for (int u = 0; u < LD4; ++u) {
    const int idx = threadIdx.x + NTHREADS * u;
    const int ts = idx / TILE4, rem = idx - ts * TILE4;
    row_in_step[u] = ts * 32 + rem / (HD / 4);
  }
  // NTHREADS is a multiple of HD / 4
  const unsigned col_bytes = PAD && 4 * (threadIdx.x % (HD / 4)) >= (unsigned)hd ? 0u : 16u * (threadIdx.x % (HD / 4));
  static_assert(NTHREADS % (HD / 4) == 0, "a thread keeps its columns");
  // a scalar base and a 32-bit byte offset per lane (a head's rows span less than 4 GiB: checked
  // at launch); rows past the last one repeat it
  auto load_tiles = [&](f32x4 (&dst)[LD4], const float *base, int sp) {
    const int first_row = (kt0 + G * sp) * 32;
#pragma unroll
    for (int u = 0; u < LD4; ++u) {
      const unsigned off = (unsigned)min(first_row + row_in_step[u], L - 1) * (unsigned)(hd * 4) + col_bytes;
      dst[u] = *(const f32x4 *)((const char *)base + off);
    }
  };
  auto park_k = [&](const f32x4 (&src)[LD4], int buf) {
#pragma unroll
    for (int u = 0; u < LD4; ++u) {
      const int idx = threadIdx.x + NTHREADS * u;
      const int ts = idx / TILE4, rem = idx - ts * TILE4;
      const int r = rem / (HD / 4), c4 = rem - r * (HD / 4);
      *(f32x4 *)&Ks[buf][ts][r * KSTR + 4 * c4] = src[u];
    }
  };
  auto park_v = [&](const f32x4 (&src)[LD4], int buf) {
#pragma unroll
    for (int u = 0; u < LD4; ++u) {
      const int idx = threadIdx.x + NTHREADS * u;
      const int ts = idx / TILE4, rem = idx - ts * TILE4;
      const int r = rem / (HD / 4), c4 = rem - r * (HD / 4);
      *(f32x4 *)&Vs[buf][ts][r * HD + 4 * c4] = src[u];
    }
  };
  auto load_k = [&](int sp) { load_tiles(stage_k, kbase, sp); };
  auto load_v = [&](int sp) { load_tiles(stage_v, vbase, sp); };
  auto store_k = [&](int buf) { park_k(stage_k, buf); };
  auto store_v = [&](int buf) { park_v(stage_v, buf); };

  // S^T of one key tile: 32 keys x 32 virtual rows, K from LDS stage `buf`
  // MFMA operands come from LDS; every fetch is issued PF steps before the MFMAs
  // that use it, so that the matrix pipe never waits for an LDS round trip.
  auto scores = [&](int buf) {
    constexpr int PF = 2;
    f32x16 sacc;
    if constexpr (kRefByMfma) {
#pragma unroll
      for (int r = 0; r < 16; ++r) sacc[r] = 0.f;
      sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(ones_col, -m_ref, sacc, 0, 0, 0);
    } else {
      sacc = neg_m;
    }
    const float *kl = &Ks[buf][gidx][n * KSTR + 4 * j];
    f32x4 kv[NK4];
#pragma unroll
    for (int i = 0; i < PF && i < NK4; ++i) kv[i] = *(const f32x4 *)(kl + 8 * i);
#pragma unroll
    for (int i = 0; i < NK4; ++i) {
      if (i + PF < NK4) kv[i + PF] = *(const f32x4 *)(kl + 8 * (i + PF));
      ORDER_LDS_AND_MFMA();
      sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[i].x, qr[4 * i + 0], sacc, 0, 0, 0);
      sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[i].y, qr[4 * i + 1], sacc, 0, 0, 0);
      sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[i].z, qr[4 * i + 2], sacc, 0, 0, 0);
      sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[i].w, qr[4 * i + 3], sacc, 0, 0, 0);
      ORDER_LDS_AND_MFMA();
    }
    return sacc;
  };

  // Software pipeline over the key tiles, in steps of G tiles (one per group of
  // wavefronts; below "tile sp" is this group's tile of step sp).  Step sp issues the
  // MFMAs of S^T(sp+1) before the softmax arithmetic of tile sp (its scores are then a
  // step old and certainly there), then O^T += V^T(sp) P^T(sp).  K runs two steps ahead of V:
  //   LDS at the start of step sp:  K(sp+1) in Ks[(sp+1)&1], V(sp) in Vs[sp&1];
  //   registers:                     K(sp+2), V(sp+1), fetched during step sp-1.
  // The step first parks those registers in the two LDS stages nobody reads any
  // more (Ks[sp&1] held K(sp), Vs[(sp+1)&1] held V(sp-1); both were last read in
  // step sp-1), then fetches K(sp+3) and V(sp+2).  One barrier per step, at its
  // end, orders all of this.
  const int n_sp = kt0 < kt1 ? (kt1 - kt0 + G - 1) / G : 0;
  f32x16 s_cur, s_next;
#pragma unroll
  for (int r = 0; r < 16; ++r) s_cur[r] = s_next[r] = 0.f;
  if (n_sp > 0) {
    // everything the first step needs is requested at once, with registers of its own for
    // the tiles that go to LDS right away: one memory round trip before the first MFMA
    // instead of three
    f32x4 k0[LD4], v0[LD4], k1[LD4];
    load_tiles(k0, kbase, 0);
    load_tiles(v0, vbase, 0);
    if (n_sp > 1) {
      load_tiles(k1, kbase, 1);
      load_v(1);
    }
    if (n_sp > 2) load_k(2);
    park_k(k0, 0);
    park_v(v0, 0);
    if (n_sp > 1) park_k(k1, 1);
  }
#pragma unroll
  for (int i = 0; i < HD / 2; ++i) qr[i] *= c;
  __syncthreads();
  if (kt0 + gidx < kt1 && (kt0 + gidx) * 32 <= wave_hi) s_cur = scores(0);
  __syncthreads();  // step 0 overwrites Ks[0]

  // O^T += V^T P^T of one tile; the probabilities are the registers of `p`
  auto accumulate = [&](const f32x16 &p, int buf) {
    constexpr int PF = NT == 2 ? 4 : 2;
    const float *vl = &Vs[buf][gidx][4 * j * HD + NT * n];
    typedef float vrow_t __attribute__((ext_vector_type(NT)));
    vrow_t vv[16];
#pragma unroll
    for (int r = 0; r < PF; ++r) vv[r] = *(const vrow_t *)(vl + (8 * (r >> 2) + (r & 3)) * HD);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      if (r + PF < 16) vv[r + PF] = *(const vrow_t *)(vl + (8 * ((r + PF) >> 2) + ((r + PF) & 3)) * HD);
      ORDER_LDS_AND_MFMA();
#pragma unroll
      for (int t = 0; t < NT; ++t) o[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv[r][t], p[r], o[t], 0, 0, 0);
      ORDER_LDS_AND_MFMA();
    }
  };

  // One step; `cur` holds this step's scores, `nxt` receives the next step's.  The loop below
  // calls it with the two register sets swapping roles, so that nothing is copied between
  // steps (T = 2048: 161 -> 154 us).
  auto step = [&](const int sp, f32x16 &cur, f32x16 &nxt) {
    const int buf = sp & 1;
    const int kt = kt0 + G * sp + gidx, kt_next = kt + G;  // this group's tile now and in the next step
    if (sp + 2 < n_sp) store_k(buf);
    if (sp + 1 < n_sp) store_v(buf ^ 1);
    if (sp + 3 < n_sp) load_k(sp + 3);
    if (sp + 2 < n_sp) load_v(sp + 2);
    const bool have_next = kt_next < kt1 && kt_next * 32 <= wave_hi;
    const bool have_cur = kt < kt1 && kt * 32 <= wave_hi;
    if (have_next) nxt = scores(buf ^ 1);
    if (have_cur) {
      f32x16 &sacc = cur;            // scores of tile kt minus m_ref, log2 units; not needed after this step
      if (kt * 32 + 31 > wave_lo) {  // tile crosses the diagonal for some row of this wavefront
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = kt * 32 + 8 * (r >> 2) + 4 * j + (r & 3);
          if (key > lim) sacc[r] = -INFINITY;
        }
      }
      float mx = fmaxf(fmaxf(sacc[0], sacc[1]), sacc[2]);
#pragma unroll
      for (int r = 3; r < 15; r += 2) mx = fmaxf(fmaxf(mx, sacc[r]), sacc[r + 1]);
      mx = fmaxf(mx, sacc[15]);
      // mx covers this lane's half of the row's keys in the tile; the row's maximum is above thr
      // exactly when one of the two halves' is (never for a row without a visible key here:
      // -inf), so the halves only exchange their maxima once a move is certain
      if (__builtin_amdgcn_ballot_w64(mx > thr) != 0) {
        // rare after a row's first tiles: move the reference to this tile's maximum
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const bool move = mx > thr;
        const float delta = move ? mx : 0.f;
        const float alpha = (move && thr != -INFINITY) ? fast_exp2(-delta) : 1.f;  // nothing to rescale before a row's first key
        m_ref += delta;
        l *= alpha;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[t][r] *= alpha;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          sacc[r] -= delta;
          nxt[r] -= delta;     // computed against the old reference (unused if there is no next tile)
          if constexpr (!kRefByMfma) neg_m[r] = -m_ref;
        }
        if (move) thr = kTau;
      }
      float psum = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        sacc[r] = fast_exp2(sacc[r]);
        psum += sacc[r];
      }
      l += psum;
      accumulate(sacc, buf);
    }
    __syncthreads();
  };
  for (int sp = 0; sp < n_sp; sp += 2) {
    step(sp, s_cur, s_next);
    if (sp + 1 < n_sp) step(sp + 1, s_next, s_cur);
  }

  l += __shfl_xor(l, 32);
  // what the merges below call the maximum: the reference the sums are relative to, in log2
  // units, or -inf for a row that saw no key (its l and O are 0)
  float m = thr == -INFINITY ? -INFINITY : m_ref;
  if constexpr (G == 2) {
    // the second group hands its (max, sum, O) to the first through the tile stages
    // (every wavefront is past the last step's barrier: nobody reads tiles any more)
    float *xo = &Ks[0][0][0];  // [4 row chunks][16 * NT registers][64 lanes]
    float *xm = &Vs[0][0][0];  // [4][64] max, then [4][64] sum
    if (gidx == 1) {
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) xo[((wave * NT + t) * 16 + r) * 64 + lane] = o[t][r];
      xm[wave * 64 + lane] = m;
      xm[256 + wave * 64 + lane] = l;
    }
    __syncthreads();
    if (gidx == 1) return;
    const float m1 = xm[wave * 64 + lane], l1 = xm[256 + wave * 64 + lane];
    const float mnew = fmaxf(m, m1);
    // a side that saw no visible key has max -inf: its factor is 0 (and both may be, in a key chunk)
    const float a0 = m == -INFINITY ? 0.f : fast_exp2(m - mnew);
    const float a1 = m1 == -INFINITY ? 0.f : fast_exp2(m1 - mnew);
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[t][r] = o[t][r] * a0 + xo[((wave * NT + t) * 16 + r) * 64 + lane] * a1;
    l = l * a0 + l1 * a1;
    m = mnew;
  }
  if (SPLIT) {  // unnormalised partial of this key chunk: [128 virtual rows][HD], (max, sum) per row
    const long long pbase = (((long long)item * sh.KV + kvh) * ns + chunk) * 128 + wave * 32 + n;
    float *op = part_o + pbase * HD;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int d = NT * (8 * (r >> 2) + 4 * j + (r & 3));
      if constexpr (NT == 2) {
        *(float2 *)(op + d) = float2{o[0][r], o[1][r]};
      } else {
        *(f32x4 *)(op + d) = f32x4{o[0][r], o[1][r], o[2][r], o[3][r]};
      }
    }
    if (j == 0) *(float2 *)(part_ml + 2 * pbase) = float2{m, l};
  } else if (valid) {
    const float inv = 1.0f / l;
    float *op = out + qo_off;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int d = NT * (8 * (r >> 2) + 4 * j + (r & 3));
      if (PAD && d >= hd) continue;  // (hd is a multiple of 4 and d of NT = 2 or 4: a store lies inside or outside as a whole)
      if constexpr (NT == 2) {
        *(float2 *)(op + d) = float2{o[0][r] * inv, o[1][r] * inv};
      } else {
        *(f32x4 *)(op + d) = f32x4{o[0][r] * inv, o[1][r] * inv, o[2][r] * inv, o[3][r] * inv};
      }
    }
  }
}

template <int HD, bool SPLIT, int G, bool PAD>
__global__ __launch_bounds__(256 * G, G == 1 ? 2 : 1) void prefill_mfma_kernel(const float *__restrict__ q_rot,
                                                              const float *__restrict__ kc,
                                                              const float *__restrict__ vc,
                                                              float *__restrict__ out,
                                                              float *__restrict__ part_o,
                                                              float *__restrict__ part_ml, SeqTable st,
                                                              Shape sh, int ns, float c) {
  prefill_block<HD, SPLIT, G, PAD>(blockIdx.x, q_rot, kc, vc, out, part_o, part_ml, st, sh, ns, c);
}

// For launches of two or three row blocks per compute unit: a workgroup takes, in turn, block b
// of the launch (blocks are numbered by decreasing key range), block 2N - 1 - b and block
// 2N + b (N workgroups): long, short and shorter ones that add up to about the same work for
// every workgroup, instead of the dispatcher starting another workgroup where one has ended
// (3.5 us later, measured).
template <int HD, int G, bool PAD>
__global__ __launch_bounds__(256 * G, 1) void prefill_turns_kernel(const float *__restrict__ q_rot,
                                                                   const float *__restrict__ kc,
                                                                   const float *__restrict__ vc,
                                                                   float *__restrict__ out, SeqTable st, Shape sh,
                                                                   int n_blocks, float c) {
  const int N = gridDim.x, b = blockIdx.x;
  for (int turn = 0; turn < 3; ++turn) {
    const int bid = (turn & 1) ? (turn + 1) * N - 1 - b : turn * N + b;
    if (bid >= n_blocks) continue;
    if (turn) __syncthreads();  // the LDS stages are free: nobody is still merging the last block's halves
    prefill_block<HD, false, G, PAD>(bid, q_rot, kc, vc, out, nullptr, nullptr, st, sh, 1, c);
  }
}

// Merge the key chunks of one (row block, kv head): online-softmax combine per row.
// Four workgroups per block (32 of its 128 virtual rows each, blockIdx.y) and up to eight
// chunks' loads in flight per thread: the kernel is bound by load latency, not by bytes.
__global__ __launch_bounds__(256) void prefill_combine_kernel(const float *__restrict__ part_o,
                                                              const float *__restrict__ part_ml,
                                                              float *__restrict__ out, SeqTable st, Shape sh,
                                                              int ns, float c, int tile_hd) {
  // tile_hd: floats per row of a partial (the head dimension the tiles were laid out for)
  const int kvh = blockIdx.x % sh.KV, item = blockIdx.x / sh.KV;
  int s, vb;
  locate_block(st, item, s, vb);
  const int g = sh.g, hd = sh.hd, hd4 = hd >> 2;
  const int VR = st.n_new[s] * g;
  const long long base = ((long long)item * sh.KV + kvh) * ns * 128;
  for (int idx = threadIdx.x; idx < 32 * hd4; idx += 256) {
    const int vl = blockIdx.y * 32 + idx / hd4, d4 = idx % hd4;
    const int v = vb * 128 + vl;
    if (v >= VR) continue;
    const int row = v / g, hg = v - row * g;
    float mm = -INFINITY;
    for (int k0 = 0; k0 < ns; k0 += 8) {
      float mk[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) mk[u] = part_ml[2 * (base + (long long)min(k0 + u, ns - 1) * 128 + vl)];
#pragma unroll
      for (int u = 0; u < 8; ++u) mm = fmaxf(mm, mk[u]);
    }
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    float ls = 0.f;
    for (int k0 = 0; k0 < ns; k0 += 8) {
      f32x4 x[8];
      float mk[8], lk[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const long long pi = base + (long long)min(k0 + u, ns - 1) * 128 + vl;
        x[u] = *(const f32x4 *)(part_o + pi * tile_hd + 4 * d4);
        mk[u] = part_ml[2 * pi];
        lk[u] = part_ml[2 * pi + 1];
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        // 0 for a chunk that saw no visible key, and for the clamped repeats past the last chunk
        const float f = k0 + u < ns ? fast_exp2((mk[u] - mm) * c) : 0.f;
        acc += f * x[u];
        ls += f * lk[u];
      }
    }
    *(f32x4 *)(out + ((long long)(st.tok_off[s] + row) * sh.H + kvh * g + hg) * hd + 4 * d4) = acc * (1.0f / ls);
  }
}

// ---------------------------------------------------------------------------
// Any head_dim up to 256: one wavefront per (row, head), lane = key for the
// scores, lane = d for the output.
__global__ __launch_bounds__(64) void generic_attn_kernel(const float *__restrict__ q_rot,
                                                          const float *__restrict__ kc,
                                                          const float *__restrict__ vc,
                                                          float *__restrict__ out, SeqTable st, Shape sh,
                                                          float scale) {
  extern __shared__ float smem[];
  const int hd = sh.hd;
  float *q_s = smem, *p_s = smem + hd;
  const int token = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int s = find_seq(st, token, st.tok_off);
  const int visible = st.start_pos[s] + (token - st.tok_off[s]) + 1;
  const int kvh = h / sh.g;
  const long long head_base = (long long)st.slot[s] * sh.seq_stride + (long long)kvh * sh.cap * hd;
  const float *kbase = kc + head_base, *vbase = vc + head_base;
  const long long qo = ((long long)token * sh.H + h) * hd;
  for (int d = lane; d < hd; d += 64) q_s[d] = q_rot[qo + d];
  __syncthreads();
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  for (int j0 = 0; j0 < visible; j0 += 64) {
    const int jj = j0 + lane;
    float sv = -INFINITY;
    if (jj < visible) {
      const float *kr = kbase + (long long)jj * hd;
      float dot = 0.f;
      for (int d = 0; d < hd; ++d) dot += q_s[d] * kr[d];
      sv = dot * scale;
    }
    float mx = sv;
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    const float mnew = fmaxf(m, mx);
    const float alpha = expf(m - mnew);
    const float p = expf(sv - mnew);
    float ps = p;
    for (int o = 32; o > 0; o >>= 1) ps += __shfl_xor(ps, o);
    l = l * alpha + ps;
    m = mnew;
    p_s[lane] = p;
    __syncthreads();
    const int cnt = min(64, visible - j0);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int d = lane + 64 * u;
      if (d < hd) {
        float a = acc[u] * alpha;
        for (int t = 0; t < cnt; ++t) a += p_s[t] * vbase[(long long)(j0 + t) * hd + d];
        acc[u] = a;
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int d = lane + 64 * u;
    if (d < hd) out[qo + d] = acc[u] / l;
  }
}

constexpr float kLog2e = 1.4426950408889634f;

}  // namespace

bool decode_entries(const SeqTable &st, const Shape &sh, SeqTable &out) {
  if (sh.g < 1 || sh.g > 16) return false;
  const int per = 16 / sh.g;  // rows whose columns fill one tile
  memset(&out, 0, sizeof out);
  int n = 0;
  for (int s = 0; s < st.n_seqs; ++s) {
    const int groups = (st.n_new[s] + per - 1) / per;
    if (groups > 2 || n + groups > kMaxSeqs) return false;
    for (int k = 0; k < groups; ++k, ++n) {
      const int first = k * per, rows = st.n_new[s] - first < per ? st.n_new[s] - first : per;
      out.slot[n] = st.slot[s];
      out.start_pos[n] = st.start_pos[s] + first;  // the rows before them are in the cache already
      out.n_new[n] = rows;
      out.tok_off[n] = st.tok_off[s] + first;
    }
  }
  out.n_seqs = n;
  out.tok_off[n] = st.tok_off[st.n_seqs];
  return true;
}

int prefill_tile_head_dim(int hd) {
  if (hd < 4 || (hd & 3) || hd > 128) return 0;
  return hd <= 64 ? 64 : 128;
}

Path choose_path(const SeqTable &st, const Shape &sh) {
  // a few new rows per sequence: rows x heads of a group fit the 16 columns of the split-K
  // kernel's MFMA tiles, which then streams K and V once for all of them; up to twice as many
  // rows go to it as two entries (decode_entries), which still beats the key-chunked prefill.
  // Its tiles take any head dimension up to 256 that is a multiple of 4 (padded to 64, 128 or 256).
  SeqTable tmp;
  if (decode_tile_head_dim(sh.hd) && decode_entries(st, sh, tmp)) return Path::kDecodeSplitK;
  // the MFMA prefill kernel's tiles: head dimensions up to 128 (padded to 64 or 128)
  if (!prefill_tile_head_dim(sh.hd)) return Path::kGeneric;
  return Path::kPrefillMfma;
}

int plan_work(SeqTable &st, const Shape &sh, Path path) {
  st.work_off[0] = 0;
  for (int s = 0; s < st.n_seqs; ++s) {
    int items;
    if (path == Path::kPrefillMfma)
      items = (st.n_new[s] * sh.g + 127) / 128;
    else
      items = st.n_new[s];
    st.work_off[s + 1] = st.work_off[s] + items;
  }
  const int total = st.work_off[st.n_seqs];
  if (path == Path::kPrefillMfma) {
    // the prefill kernel wants per-sequence block counts and the sequences sorted by them
    for (int s = 0; s < st.n_seqs; ++s) st.work_off[s] = st.work_off[s + 1] - st.work_off[s];
    for (int s = 0; s < st.n_seqs; ++s) st.ord[s] = s;
    for (int a = 1; a < st.n_seqs; ++a)  // insertion sort, descending, stable
      for (int b = a; b > 0 && st.work_off[st.ord[b]] > st.work_off[st.ord[b - 1]]; --b) {
        const int t = st.ord[b];
        st.ord[b] = st.ord[b - 1];
        st.ord[b - 1] = t;
      }
  }
  return total;
}

static bool table_ok(const SeqTable &st, const Shape &sh) {
  if (st.n_seqs < 1 || st.n_seqs > kMaxSeqs || sh.g < 1 || sh.H != sh.KV * sh.g) return false;
  for (int s = 0; s < st.n_seqs; ++s)
    if (st.n_new[s] < 1 || st.start_pos[s] < 0 || st.start_pos[s] + st.n_new[s] > sh.cap || st.slot[s] < 0)
      return false;
  return true;
}

int prefill_key_splits(const SeqTable &st, const Shape &sh, int items) {
  const long long wgs = (long long)items * sh.KV;
  if (wgs >= 384) return 1;
  int longest = 0;  // key tiles of the longest row block
  for (int s = 0; s < st.n_seqs; ++s) {
    const int t = (st.start_pos[s] + st.n_new[s] + 31) / 32;
    longest = t > longest ? t : longest;
  }
  int ns = (int)((512 + wgs - 1) / wgs);
  // With long key ranges, about 1024 workgroups: four-wavefront workgroups that share the
  // compute units two or more at a time and drift apart then do better than 512 of eight
  // wavefronts, one per unit, whose two wavefronts per SIMD move in step (512 rows on 16384
  // cached, 128 row blocks: 1078 -> 1053 us); chunks under 32 tiles lose more to their set-up
  // (1024 rows into an empty cache: 109 -> 115 us).
  const int ns_1024 = (int)((1024 + wgs - 1) / wgs);
  if (longest / ns_1024 >= 32) ns = ns_1024;
  const int cap = longest / 8;  // at least eight key tiles per chunk
  if (ns > cap) ns = cap;
  if (ns > 16) ns = 16;
  return ns < 1 ? 1 : ns;
}

size_t prefill_partial_floats(const Shape &sh, int items, int ns) {
  return ns > 1 ? (size_t)items * sh.KV * ns * 128 * (prefill_tile_head_dim(sh.hd) + 2) : 0;
}

PrefillLaunch plan_prefill_launch(const Shape &sh, int items, int ns, int wgs_per_cu, int groups) {
  PrefillLaunch p;
  p.n_wgs = (long long)items * sh.KV * ns;
  // With fewer workgroups than three per compute unit everything is resident at
  // once: run one workgroup per compute unit (below) and give it eight wavefronts,
  // two per SIMD (G = 2).  Larger launches already have several workgroups per unit.
  p.groups = groups == 1 || groups == 2 ? groups : (p.n_wgs <= 768 ? 2 : 1);
  // static LDS of the kernel: two stages of `groups` padded K tiles and V tiles
  const int tile_hd = prefill_tile_head_dim(sh.hd);
  const size_t static_lds = (size_t)2 * p.groups * (32 * (tile_hd + 4) + 32 * tile_hd) * sizeof(float);
  p.pad = 0;
  // With fewer workgroups than three per compute unit everything is resident at
  // once and the dispatcher cannot balance the triangular work: one workgroup per
  // compute unit lets it hand the short row blocks to whichever unit finishes first.
  if (wgs_per_cu == 0 && p.n_wgs <= 768) wgs_per_cu = 1;
  p.wgs_per_cu = wgs_per_cu >= 1 && wgs_per_cu <= 3 ? wgs_per_cu : 0;
  if (p.wgs_per_cu) {
    const size_t want = (size_t)160 * 1024 / wgs_per_cu;  // one more workgroup would not fit
    const size_t floor_ = (size_t)160 * 1024 / (wgs_per_cu + 1) + 256;
    if (static_lds < floor_ && floor_ <= want) p.pad = floor_ - static_lds;
  }
  static const bool turns_off = getenv("SHAINET_HIP_PREFILL_NO_TURNS") != nullptr;
  // Turns only when the blocks fill them: otherwise compute units would stand idle where the
  // dispatcher's own hand-out keeps them busy (12 % slower at 640 blocks)
  const int turns = (int)((p.n_wgs + 255) / 256);
  p.turns = !turns_off && ns == 1 && p.groups == 2 && p.n_wgs > 256 && p.n_wgs <= 768 &&
                    p.n_wgs * 100 >= (long long)turns * 256 * 97
                ? turns
                : 0;
  return p;
}

hipError_t launch_prefill(const float *q_rot, const float *kc, const float *vc, float *out, float *partials,
                          const SeqTable &st, const Shape &sh, int items, int ns, float scale,
                          hipStream_t stream, int wgs_per_cu, int groups_wanted, hipEvent_t before, hipEvent_t after) {
  const int tile_hd = prefill_tile_head_dim(sh.hd);
  if (!table_ok(st, sh) || !tile_hd || items < 1 || ns < 1 || (ns > 1 && !partials)) return hipErrorInvalidValue;
  const bool pad = tile_hd != sh.hd;
  const PrefillLaunch plan = plan_prefill_launch(sh, items, ns, wgs_per_cu, groups_wanted);
  const long long n_wgs = plan.n_wgs;
  if (n_wgs > 0x7fffffffLL) return hipErrorInvalidValue;
  // the kernels address a row of a (sequence, kv head) by a 32-bit byte offset from its first row
  if ((long long)sh.cap * sh.hd * 4 > 0xffffffffLL) return hipErrorInvalidValue;
  const float c = scale * kLog2e;
  dim3 grid((unsigned)n_wgs);
  float *part_o = partials;
  float *part_ml = partials ? partials + (size_t)items * sh.KV * ns * 128 * tile_hd : nullptr;
  const int groups = plan.groups;
  const size_t lds_pad = plan.pad;
  if (plan.turns) {
    const int turns = plan.turns;
    dim3 fewer((unsigned)((n_wgs + turns - 1) / turns));
#define SHAINET_LAUNCH_TURNS(HD_, PAD_)                                                                          \
  SHAINET_LAUNCH_TIMED((prefill_turns_kernel<HD_, 2, PAD_>), fewer, dim3(512), 0, stream, before, after, q_rot, kc, \
                       vc, out, st, sh, (int)n_wgs, c)
    if (tile_hd == 64) {
      if (pad)
        SHAINET_LAUNCH_TURNS(64, true);
      else
        SHAINET_LAUNCH_TURNS(64, false);
    } else {
      if (pad)
        SHAINET_LAUNCH_TURNS(128, true);
      else
        SHAINET_LAUNCH_TURNS(128, false);
    }
#undef SHAINET_LAUNCH_TURNS
    return hipGetLastError();
  }
  hipEvent_t main_after = ns == 1 ? after : nullptr;  // with key chunks the combine kernel ends the timed stretch
#define SHAINET_LAUNCH_PREFILL(HD_, SPLIT_, PAD_)                                                              \
  do {                                                                                                          \
    if (groups == 2)                                                                                            \
      SHAINET_LAUNCH_TIMED((prefill_mfma_kernel<HD_, SPLIT_, 2, PAD_>), grid, dim3(512), lds_pad, stream, before, \
                           main_after, q_rot, kc, vc, out, part_o, part_ml, st, sh, ns, c);                     \
    else                                                                                                        \
      SHAINET_LAUNCH_TIMED((prefill_mfma_kernel<HD_, SPLIT_, 1, PAD_>), grid, dim3(256), lds_pad, stream, before, \
                           main_after, q_rot, kc, vc, out, part_o, part_ml, st, sh, ns, c);                     \
  } while (0)
#define SHAINET_LAUNCH_PREFILL_HD(HD_, PAD_) \
  do {                                        \
    if (ns > 1)                               \
      SHAINET_LAUNCH_PREFILL(HD_, true, PAD_);   \
    else                                      \
      SHAINET_LAUNCH_PREFILL(HD_, false, PAD_);  \
  } while (0)
  if (tile_hd == 64) {
    if (pad)
      SHAINET_LAUNCH_PREFILL_HD(64, true);
    else
      SHAINET_LAUNCH_PREFILL_HD(64, false);
  } else {
    if (pad)
      SHAINET_LAUNCH_PREFILL_HD(128, true);
    else
      SHAINET_LAUNCH_PREFILL_HD(128, false);
  }
#undef SHAINET_LAUNCH_PREFILL_HD
#undef SHAINET_LAUNCH_PREFILL
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || ns == 1) return e;
  hipEvent_t none = nullptr;
  SHAINET_LAUNCH_TIMED(prefill_combine_kernel, dim3((unsigned)(items * sh.KV), 4), dim3(256), 0, stream, none, after,
                       part_o, part_ml, out, st, sh, ns, 1.0f, tile_hd);  // the partials' maxima are already in log2 units
  return hipGetLastError();
}

hipError_t launch_generic(const float *q_rot, const float *kc, const float *vc, float *out,
                          const SeqTable &st, const Shape &sh, int total_tokens, float scale,
                          hipStream_t stream) {
  if (!table_ok(st, sh) || sh.hd < 1 || sh.hd > 256 || total_tokens < 1) return hipErrorInvalidValue;
  const size_t smem = (size_t)(sh.hd + 64) * sizeof(float);
  hipLaunchKernelGGL(generic_attn_kernel, dim3((unsigned)total_tokens, (unsigned)sh.H), dim3(64), smem, stream,
                     q_rot, kc, vc, out, st, sh, scale);
  return hipGetLastError();
}

}  // namespace shainet
