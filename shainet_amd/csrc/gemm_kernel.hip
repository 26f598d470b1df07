// Row-major fp32 product y[T,N] = x[T,K] W[K,N] (+ res) for gfx950, for more than 16 rows: the
// projections of a prefill (llama_block.cr:253-255, 298; swiglu_ff.cr:76-91), where the
// reference's GPU branch calls cuBLAS SGEMM (llama_block.cr:726-768, cuda.cr:237-247) and its CPU
// branch SimpleMatrix#* (simple_matrix.cr:61-74).
//
// A workgroup of four wavefronts owns a 128 x 128 tile of y; each wavefront owns 32 of its rows
// and all 128 columns (four blocks of v_mfma_f32_32x32x2_f32) and the workgroup walks K in steps
// of 32; two workgroups share a compute unit, so that each SIMD holds two wavefronts and one's
// barrier and memory waits hide behind the other's MFMAs (256 x 128 tiles, one workgroup per
// compute unit and twice the MFMAs per LDS read, were 7 % slower: 128 against 137 TFLOP/s).  Both operands go global memory -> registers -> LDS (two LDS stages, one barrier per
// step) and are read from LDS with ds_read_b128:
//   x tile [rows][32 k], row stride 36 floats: a lane reads four consecutive k of its row;
//   W tile [32 k][128 columns] as it lies in memory: lane n of a block owns columns 4 n + b of
//     the four blocks b, so one 16-byte read of a W row feeds the four blocks, and a lane's
//     results for one row of y are four neighbouring columns (16-byte stores).
// An MFMA may visit the contraction index in any order as long as both operands agree: MFMA i of
// a k step of 8 takes k = 8 s + 4 j + i from lane half j, on both sides.
// MFMA 32x32x2 layout (lane l): A[m = l % 32][k = l / 32], B[k = l / 32][n = l % 32],
// D[m = 8 (r / 4) + 4 (l / 32) + r % 4][n = l % 32] for accumulator register r.
// Tile loads take a scalar base that moves along K plus a per-thread 32-bit offset, so the loop
// holds next to no vector instructions besides the MFMAs (fp32 MFMAs run on the vector ALU's
// lanes: every other vector instruction is paid in matrix throughput).
//
// Work is counted in units of one K step of one tile.  When the tiles do not fill whole rounds of
// the chip (512 workgroups run at once), the units are dealt out evenly instead: a workgroup takes
// a contiguous run of units, which may end inside a tile (it leaves that piece as a partial product
// in its own slot of a scratch array and marks the slot's flag word) and may begin inside one (it
// then finishes that tile: waits for the flag words of the workgroups that hold the tile's earlier
// pieces, adds their partial products to its own in a fixed order and stores y).  Which
// workgroup holds which piece depends on the shape only, so results do not depend on scheduling.
// A workgroup waits only for workgroups with a lower index, which were started before it and wait
// for nobody in turn while they compute the piece it needs (every workgroup computes the piece it
// leaves unfinished first).  That serves shapes where a tile is shared by two or three workgroups.
// Few tiles with a long K (512 rows of the 8192 -> 2048 down projection: 64 tiles for 256 compute
// units) are cut into more pieces per tile; one workgroup adding them one after the other would take
// longer than the product, so there every workgroup leaves its piece in its slot and a second
// kernel, with the whole chip, adds the pieces in a fixed order (and the residual).
#include "gemm_kernel.hpp"

#include <stdint.h>
#include <stdlib.h>

namespace shainet {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int TN = 128, TK = 32;
constexpr int AS = TK + 4;  // padded row stride of the x tile: conflict-free 16-byte reads down a column of rows

#define ORDER_LDS_AND_MFMA() __builtin_amdgcn_sched_barrier(0x7)

// A partial product is read by a workgroup that may sit on another XCD, whose L2 is not kept
// coherent with this one's for ordinary accesses: the store is written through to memory.
// (The compiler does not see a store in this text: the registers of v must not be written again
// before the store has read them, so callers keep every value they store in registers of its own
// until they have waited for the stores.)
__device__ __forceinline__ void coherent_store4(float *p, f32x4 v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(p), "v"(v) : "memory");
}

struct GemmArgs {
  const float *x;
  long long xs;
  const float *w;
  float *y;
  const float *res;  // nullable: y = res + x W
  float *partials;   // [workgroups][128 * 128]: the piece a workgroup leaves unfinished
  unsigned *flags;   // [workgroups], zero between launches
  unsigned *flag_set;  // where a piece is marked complete: `flags`, or elsewhere in the test of the give-up path
  int spin_limit;    // polls before a wait for a flag word is given up
  int *error;        // set to 1 then
  int T, K, N, tiles_m;
  int steps;            // K steps of 32 per tile
  int group_bits;       // workgroup id -> group id & (groups - 1), place id >> group_bits
  int tiles_per_group;  // a group's workgroups share a contiguous run of tiles (row tiles fastest)
  int quota;            // units per workgroup
  int pieces;           // 0: a workgroup's run of units starts where the one before it ends; > 0: every tile
                        // is cut into this many pieces of `quota` steps, a workgroup each, all left in their slots
};

// GUARD: K need not be a multiple of 32 (pieces beyond its end are loaded as zeros); without it
// every load of the loop is unconditional.
template <bool GUARD>
__global__ __launch_bounds__(256, 2) void sgemm_mfma_kernel(const GemmArgs g) {
  constexpr int TM = 128;
  constexpr int NA = 4;  // float4 of the x tile per thread
  __shared__ __attribute__((aligned(16))) float As[2][TM * AS];
  __shared__ __attribute__((aligned(16))) float Bs[2][TK * TN];

  // Workgroups go to the eight XCDs round-robin by index: the workgroups of a group (index modulo
  // the group count, a power of two up to 8) stay on the same XCDs and share a run of tiles, whose
  // operands and partial products they find in those XCDs' L2.
  const int group = blockIdx.x & ((1 << g.group_bits) - 1), place = blockIdx.x >> g.group_bits;
  const int steps = g.steps;
  int u0 = place * g.quota, u1 = min(u0 + g.quota, g.tiles_per_group * steps);
  if (g.pieces) {
    const int t = place / g.pieces;
    u0 = t * steps + (place - t * g.pieces) * g.quota;
    u1 = t < g.tiles_per_group ? min(u0 + g.quota, (t + 1) * steps) : u0;
  }
  if (u0 >= u1) return;
  const int t_first = u0 / steps, t_last = (u1 - 1) / steps;
  const bool leaves_piece = u1 < (t_last + 1) * steps;  // the run ends inside tile t_last

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int ln = lane & 31, j = lane >> 5;
  const int T = g.T, K = g.K, N = g.N;

  // staging: x tile, NA float4 per thread: row = idx / 8, k piece = idx % 8 (rows past the last
  // one repeat it: their products are never stored); W tile, 4 float4 per thread: row = idx / 32,
  // columns 4 (idx % 32) .. + 3 (columns past the last one repeat the last four: never stored)
  int a_lds[NA], b_lds[4];
#pragma unroll
  for (int u = 0; u < NA; ++u) {
    const int idx = threadIdx.x + 256 * u;
    a_lds[u] = (idx >> 3) * AS + 4 * (idx & 7);
  }
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int idx = threadIdx.x + 256 * u;
    b_lds[u] = (idx >> 5) * TN + 4 * (idx & 31);
  }
  // operand fragments of one k step of 8: x rows (four k each), W rows per MFMA i (four columns =
  // the four blocks each)
  const int a_off = (wave * 32 + ln) * AS + 4 * j, b_off = 4 * j * TN + 4 * ln;
  const long long w_step = (long long)TK * N * 4;

  for (int visit = 0; visit <= t_last - t_first; ++visit) {
    // the tile this run leaves unfinished comes first: the workgroup that finishes it needs the piece
    const int t = leaves_piece ? (visit == 0 ? t_last : t_first + visit - 1) : t_first + visit;
    const int s_begin = t == t_first ? u0 - t_first * steps : 0;
    const int s_end = t == t_last ? u1 - t_last * steps : steps;
    const int tile = group * g.tiles_per_group + t;
    const int tm = tile % g.tiles_m, tn = tile / g.tiles_m;
    const int m0 = tm * TM, n0 = tn * TN;
    const int k_begin = s_begin * TK, k_end = min(K, s_end * TK);
    const int nk = s_end - s_begin;

    unsigned x_off[NA], w_off[4];
#pragma unroll
    for (int u = 0; u < NA; ++u) {
      const int idx = threadIdx.x + 256 * u;
      x_off[u] = (unsigned)(((long long)min(m0 + (idx >> 3), T - 1) * g.xs + 4 * (idx & 7)) * 4);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int idx = threadIdx.x + 256 * u;
      w_off[u] = (unsigned)(((long long)(idx >> 5) * N + min(n0 + 4 * (idx & 31), N - 4)) * 4);
    }
    const char *x_base = (const char *)(g.x + k_begin);
    const char *w_base = (const char *)(g.w + (long long)k_begin * N);

    // two register sets: the tiles of step t travel in set t & 1 and are requested two steps ahead
    // (one step, 1.7 us of MFMAs, is not always enough for a load to come back: 114 against 125 TFLOP/s)
    f32x4 sa[2][NA], sb[2][4];
    int k_next = k_begin;
    auto load_tiles = [&](f32x4 (&ra)[NA], f32x4 (&rb)[4]) {
#pragma unroll
      for (int u = 0; u < NA; ++u) {
        const int c4 = (threadIdx.x + 256 * u) & 7;
        if (GUARD)  // a piece beyond the end of K contributes nothing: zero on the x side is enough
          ra[u] = k_next + 4 * c4 < k_end ? *(const f32x4 *)(x_base + x_off[u]) : f32x4{0.f, 0.f, 0.f, 0.f};
        else
          ra[u] = *(const f32x4 *)(x_base + x_off[u]);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int row = (threadIdx.x + 256 * u) >> 5;
        if (GUARD)
          rb[u] = k_next + row < k_end ? *(const f32x4 *)(w_base + w_off[u]) : f32x4{0.f, 0.f, 0.f, 0.f};
        else
          rb[u] = *(const f32x4 *)(w_base + w_off[u]);
      }
      x_base += TK * 4;
      w_base += w_step;
      k_next += TK;
    };
    auto park_tiles = [&](const f32x4 (&ra)[NA], const f32x4 (&rb)[4], int buf) {
#pragma unroll
      for (int u = 0; u < NA; ++u) *(f32x4 *)&As[buf][a_lds[u]] = ra[u];
#pragma unroll
      for (int u = 0; u < 4; ++u) *(f32x4 *)&Bs[buf][b_lds[u]] = rb[u];
    };

    f32x16 acc[4];
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[b][r] = 0.f;

    f32x4 af[2], bf[2][4];  // [k step parity]
    auto fetch = [&](int par, int buf, int s) {
      af[par] = *(const f32x4 *)&As[buf][a_off + 8 * s];
#pragma unroll
      for (int i = 0; i < 4; ++i) bf[par][i] = *(const f32x4 *)&Bs[buf][b_off + (8 * s + i) * TN];
    };

    // (after the last barrier of the tile before this one nobody reads LDS any more)
    load_tiles(sa[0], sb[0]);
    if (nk > 1) load_tiles(sa[1], sb[1]);
    park_tiles(sa[0], sb[0], 0);
    if (nk > 2) load_tiles(sa[0], sb[0]);
    __syncthreads();
    fetch(0, 0, 0);

    // Per step of 32 along K: the MFMAs of the four k steps of 8 run with the fragments of each
    // fetched one k step ahead; before the last of them (its fragments are in registers by then)
    // the next step's tiles go from their registers to the other LDS stage, the one barrier of the
    // step follows, the tiles of a later step are requested into the registers just freed, and the
    // first fragments of the next step are fetched: neither the barrier nor an LDS round trip
    // stands between two steps' MFMAs.
    auto step = [&](const int kt, f32x4 (&ra)[NA], f32x4 (&rb)[4]) {  // ra, rb: the set that holds step kt + 1
      const int buf = kt & 1;
      const bool more = kt + 1 < nk;
#pragma unroll
      for (int s = 0; s < TK / 8; ++s) {
        const int cur = s & 1, nxt = cur ^ 1;
        if (s + 1 < TK / 8) {
          fetch(nxt, buf, s + 1);
        } else {
          if (more) park_tiles(ra, rb, buf ^ 1);
          __syncthreads();
          if (kt + 3 < nk) load_tiles(ra, rb);
          if (more) fetch(nxt, buf ^ 1, 0);
        }
        ORDER_LDS_AND_MFMA();
        // the accumulators take turns: no MFMA waits for the one before it
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int b = 0; b < 4; ++b)
            acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[cur][i], bf[cur][i][b], acc[b], 0, 0, 0);
        ORDER_LDS_AND_MFMA();
      }
    };
    for (int kt = 0; kt < nk; kt += 2) {
      step(kt, sa[1], sb[1]);
      if (kt + 1 < nk) step(kt + 1, sa[0], sb[0]);
    }

    // A piece travels as [register r][thread] float4: consecutive threads, consecutive 16 bytes.
    constexpr long long kSlot = (long long)TM * TN;
    f32x4 out[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) out[r] = f32x4{acc[0][r], acc[1][r], acc[2][r], acc[3][r]};
    // (the thread's offset is taken afresh per tile, or the compiler computes all sixteen addresses
    // before the loops and keeps them in scratch memory)
    int in_slot = 4 * threadIdx.x;
    asm volatile("" : "+v"(in_slot));
    if (g.pieces) {  // the second kernel adds the pieces
      float *slot = g.partials + blockIdx.x * kSlot + in_slot;
#pragma unroll
      for (int r = 0; r < 16; ++r) *(f32x4 *)(slot + r * 1024) = out[r];
      return;
    }
    if (s_end < steps) {
      float *slot = g.partials + blockIdx.x * kSlot + in_slot;
      __builtin_amdgcn_sched_barrier(0);  // all of out[] is in place before the first store is issued
#pragma unroll
      for (int r = 0; r < 16; ++r) coherent_store4(slot + r * 1024, out[r]);
      // the stores are acknowledged (s_waitcnt vmcnt(0): the barrier alone does not wait for them)
      // before the piece is marked complete
      __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();
      if (threadIdx.x == 0) __hip_atomic_store(g.flag_set + blockIdx.x, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      continue;
    }
    if (s_begin > 0) {
      // the tile's earlier pieces lie with the places before this one, from the one that holds the tile's first unit on
      const int p_first = t * steps / g.quota, n_before = place - p_first;
      if (wave == 0) {
        for (int spins = 0;; ++spins) {
          bool ok = true;
          for (int i = lane; i < n_before; i += 64)
            ok = ok && __hip_atomic_load(g.flags + (((p_first + i) << g.group_bits) | group), __ATOMIC_RELAXED,
                                         __HIP_MEMORY_SCOPE_AGENT) != 0u;
          if (__all(ok)) {
            for (int i = lane; i < n_before; i += 64)
              __hip_atomic_store(g.flags + (((p_first + i) << g.group_bits) | group), 0u, __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_AGENT);
            break;
          }
          if (spins >= g.spin_limit) {
            if (lane == 0) *g.error = 1;
            break;
          }
          __builtin_amdgcn_s_sleep(2);
        }
      }
      __syncthreads();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
      // ((own piece + piece 0) + piece 1) + ...
      const float *piece = g.partials + (long long)((p_first << g.group_bits) | group) * kSlot + in_slot;
      const long long piece_step = kSlot << g.group_bits;
      for (int i = 0; i < n_before; ++i) {
        f32x4 v[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) v[r] = *(const f32x4 *)(piece + i * piece_step + r * 1024);
        __builtin_amdgcn_sched_barrier(0);  // all sixteen loads in flight before the first sum waits
#pragma unroll
        for (int r = 0; r < 16; ++r) out[r] += v[r];
      }
    }
    const int col = n0 + 4 * ln;
    if (col < N) {  // N is a multiple of 4: a lane's four columns are inside together
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wave * 32 + 8 * (r >> 2) + 4 * j + (r & 3);
        if (row < T) {
          const long long o = (long long)row * N + col;
          f32x4 v = out[r];
          if (g.res) v = *(const f32x4 *)(g.res + o) + v;
          *(f32x4 *)(g.y + o) = v;
        }
      }
    }
  }
}

// y tile = (res +) piece 0 + piece 1 + ... of the tile, in that order.  A piece lies in its
// workgroup's slot as [register r][thread] float4, the layout of the product kernel's accumulators.
__global__ __launch_bounds__(256) void sgemm_reduce_kernel(const GemmArgs g, int tiles) {
  const int tile = blockIdx.x >> 4, r = blockIdx.x & 15;  // sixteen workgroups per tile, a register each
  if (tile >= tiles) return;
  const int group = tile / g.tiles_per_group, t = tile - group * g.tiles_per_group;
  constexpr long long kSlot = 128LL * TN;
  const float *piece = g.partials + (long long)(((t * g.pieces) << g.group_bits) | group) * kSlot + r * 1024 + 4 * threadIdx.x;
  const long long piece_step = kSlot << g.group_bits;
  const int n = min(g.pieces, (g.steps + g.quota - 1) / g.quota);  // pieces that hold any steps
  f32x4 acc = *(const f32x4 *)piece;
  for (int c = 1; c < n; ++c) acc += *(const f32x4 *)(piece + c * piece_step);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int row = (tile % g.tiles_m) * 128 + wave * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
  const int col = (tile / g.tiles_m) * TN + 4 * (lane & 31);
  if (row < g.T && col < g.N) {
    const long long o = (long long)row * g.N + col;
    if (g.res) acc = *(const f32x4 *)(g.res + o) + acc;
    *(f32x4 *)(g.y + o) = acc;
  }
}

// Any shape (K or N not a multiple of 4, unaligned rows): one thread per element of y, W read
// coalesced along n.  For the small odd shapes of tests; the MFMA kernel takes everything else.
__global__ __launch_bounds__(256) void sgemm_plain_kernel(const float *__restrict__ x, long long xs,
                                                          const float *__restrict__ w, float *__restrict__ y,
                                                          const float *__restrict__ res, int T, int K, int N) {
  const int n = blockIdx.x * 256 + threadIdx.x;
  if (n >= N) return;
  for (int t = blockIdx.y; t < T; t += gridDim.y) {  // the grid's second dimension ends at 65535
    const float *xr = x + (long long)t * xs;
    float acc = 0.f;
    for (int k = 0; k < K; ++k) acc += xr[k] * w[(long long)k * N + n];
    const long long o = (long long)t * N + n;
    y[o] = res ? res[o] + acc : acc;
  }
}

}  // namespace

GemmPlan plan_gemm(int T, int K, int N, long long x_stride) {
  GemmPlan p = {};
  // (the kernel addresses the rows of x by 32-bit byte offsets from a base that moves along K)
  p.mfma = T >= 1 && K >= 4 && N >= 4 && (K & 3) == 0 && (N & 3) == 0 && (x_stride & 3) == 0 &&
           (long long)T * x_stride * 4 < 0xffffffffLL && (long long)TK * N * 4 < 0xffffffffLL;
  p.tiles_m = (T + 127) / 128;
  p.tiles_n = (N + TN - 1) / TN;
  if (!p.mfma) return p;
  const int slots = 512;  // workgroups the chip runs at once: two per compute unit
  const int tiles = p.tiles_m * p.tiles_n;
  p.steps = (K + TK - 1) / TK;
  // groups of workgroups that stay on the same XCDs: as many (of 8, 4, 2, 1) as divide the tiles evenly
  p.group_bits = 3;
  while (tiles & ((1 << p.group_bits) - 1)) --p.group_bits;
  const int groups = 1 << p.group_bits;
  p.tiles_per_group = tiles / groups;
  if (tiles % slots == 0) {  // whole rounds of the chip: a workgroup per tile
    p.quota = p.steps;
    p.workgroups = tiles;
    return p;
  }
  // Otherwise one round of workgroups shares the K steps of all tiles evenly.
  const long long units = (long long)p.tiles_per_group * p.steps;
  int places = slots / groups;
  int quota = (int)((units + places - 1) / places);
  if (quota < 8) quota = p.steps < 8 ? p.steps : 8;  // a workgroup's start and end must not outweigh its loop
  if (2 * quota >= p.steps) {  // a tile is shared by two or three workgroups: the one that ends it adds the pieces
    p.quota = quota;
    p.workgroups = (int)((units + quota - 1) / quota) * groups;
    p.flag_words = (size_t)p.workgroups;
  } else {
    // more pieces per tile: as many as fill one round, of at least 8 steps each, all equal; the
    // second kernel adds them
    int pieces = slots / tiles;
    static const int pieces_knob = getenv("SHAINET_HIP_GEMM_PIECES") ? atoi(getenv("SHAINET_HIP_GEMM_PIECES")) : 0;
    if (pieces > 16) pieces = 16;  // (128 rows of 8192 -> 2048: 32 pieces 56 us, 16 pieces 48.5 us)
    if (pieces_knob > 0) pieces = pieces_knob;  // SHAINET_HIP_GEMM_PIECES: a tuning knob
    if (pieces > p.steps / 8) pieces = p.steps / 8;
    if (pieces < 1) pieces = 1;
    p.quota = (p.steps + pieces - 1) / pieces;
    p.pieces = pieces;
    p.workgroups = tiles * pieces;
    if (pieces == 1) return p;  // (short K: a workgroup per tile after all)
  }
  p.partial_floats = (size_t)p.workgroups * 128 * TN;
  return p;
}

hipError_t launch_gemm(const float *x, long long x_stride, const float *w, float *y, const float *res, float *partials,
                       unsigned *flags, int *error, int T, int K, int N, const GemmPlan &p, hipStream_t stream,
                       unsigned *flag_set, int spin_limit) {
  if (!x || !w || !y || T < 1 || K < 1 || N < 1 || x_stride < K) return hipErrorInvalidValue;
  const bool aligned = !(((uintptr_t)x | (uintptr_t)w | (uintptr_t)y | (uintptr_t)res) & 15);
  if (!p.mfma || !aligned) {
    hipLaunchKernelGGL(sgemm_plain_kernel, dim3((unsigned)((N + 255) / 256), (unsigned)(T < 65535 ? T : 65535)), dim3(256), 0, stream, x,
                       x_stride, w, y, res, T, K, N);
    return hipGetLastError();
  }
  if (p.partial_floats && !partials) return hipErrorInvalidValue;
  if (p.flag_words && (!flags || !error)) return hipErrorInvalidValue;
  GemmArgs g = {};
  g.x = x;
  g.xs = x_stride;
  g.w = w;
  g.y = y;
  g.res = res;
  g.partials = partials;
  g.flags = flags;
  g.flag_set = flag_set ? flag_set : flags;
  g.spin_limit = spin_limit > 0 ? spin_limit : 1 << 21;  // polls of about a microsecond each: seconds
  g.error = error;
  g.T = T;
  g.K = K;
  g.N = N;
  g.tiles_m = p.tiles_m;
  g.steps = p.steps;
  g.group_bits = p.group_bits;
  g.tiles_per_group = p.tiles_per_group;
  g.quota = p.quota;
  g.pieces = p.pieces > 1 ? p.pieces : 0;
  const dim3 grid((unsigned)p.workgroups);
  if (K % TK != 0)
    hipLaunchKernelGGL(sgemm_mfma_kernel<true>, grid, dim3(256), 0, stream, g);
  else
    hipLaunchKernelGGL(sgemm_mfma_kernel<false>, grid, dim3(256), 0, stream, g);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || !g.pieces) return e;
  const int tiles = p.tiles_m * p.tiles_n;
  hipLaunchKernelGGL(sgemm_reduce_kernel, dim3((unsigned)tiles * 16), dim3(256), 0, stream, g, tiles);
  return hipGetLastError();
}

}  // namespace shainet
