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
// Few rows with a long K (512 rows of the 8192 -> 2048 down projection: 64 tiles for 256 compute
// units) are cut along K into chunks that run as separate workgroups and leave partial
// products; a second kernel adds them in a fixed order (and the residual), so results do not depend
// on scheduling.
#include "gemm_kernel.hpp"

#include <stdint.h>

namespace shainet {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int TN = 128, TK = 32;
constexpr int AS = TK + 4;  // padded row stride of the x tile: conflict-free 16-byte reads down a column of rows

#define ORDER_LDS_AND_MFMA() __builtin_amdgcn_sched_barrier(0x7)

// XCD-aware numbering: workgroups go to the eight XCDs round-robin by index, so the workgroups
// of one XCD are given a contiguous run of tiles (row tiles fastest: they share W's column tile
// in that XCD's L2).
__device__ __forceinline__ int tile_of_workgroup(int id, int n_tiles) {
  const int per = (n_tiles + 7) >> 3;
  return (id & 7) * per + (id >> 3);  // >= n_tiles: nothing to do (the grid is rounded up to a multiple of 8)
}

// res != nullptr (and one K chunk only): y = res + x W.  With chunks, y is the partial-product
// array [chunks][T][N] and the workgroup writes its chunk's slice.
// GUARD: the contraction range of a workgroup need not be a multiple of 32 (pieces beyond its end
// are loaded as zeros); without it every load of the loop is unconditional.
template <bool GUARD>
__global__ __launch_bounds__(256, 2) void sgemm_mfma_kernel(const float *__restrict__ x, long long xs,
                                                                          const float *__restrict__ w,
                                                                          float *__restrict__ y,
                                                                          const float *__restrict__ res, int T, int K,
                                                                          int N, int tiles_m, int tiles_n, int k_chunk) {
  constexpr int MB = 1;       // blocks of 32 rows per wavefront
  constexpr int TM = 128 * MB;
  constexpr int NA = 4 * MB;  // float4 of the x tile per thread
  __shared__ __attribute__((aligned(16))) float As[2][TM * AS];
  __shared__ __attribute__((aligned(16))) float Bs[2][TK * TN];

  const int n_tiles = tiles_m * tiles_n;
  const int tile = tile_of_workgroup(blockIdx.x, n_tiles);
  if (tile >= n_tiles) return;
  const int tm = tile % tiles_m, tn = tile / tiles_m;
  const int m0 = tm * TM, n0 = tn * TN;
  const int k_begin = blockIdx.y * k_chunk, k_end = min(K, k_begin + k_chunk);
  const int nk = (k_end - k_begin + TK - 1) / TK;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int ln = lane & 31, j = lane >> 5;

  // staging: x tile, NA float4 per thread: row = idx / 8, k piece = idx % 8 (rows past the last
  // one repeat it: their products are never stored); W tile, 4 float4 per thread: row = idx / 32,
  // columns 4 (idx % 32) .. + 3 (columns past the last one repeat the last four: never stored)
  unsigned x_off[NA], w_off[4];
  int a_lds[NA], b_lds[4];
#pragma unroll
  for (int u = 0; u < NA; ++u) {
    const int idx = threadIdx.x + 256 * u;
    const int row = idx >> 3, c4 = idx & 7;
    x_off[u] = (unsigned)(((long long)min(m0 + row, T - 1) * xs + 4 * c4) * 4);
    a_lds[u] = row * AS + 4 * c4;
  }
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int idx = threadIdx.x + 256 * u;
    const int row = idx >> 5, c = idx & 31;
    w_off[u] = (unsigned)(((long long)row * N + min(n0 + 4 * c, N - 4)) * 4);
    b_lds[u] = row * TN + 4 * c;
  }
  const char *x_base = (const char *)(x + k_begin);
  const char *w_base = (const char *)(w + (long long)k_begin * N);
  const long long w_step = (long long)TK * N * 4;

  // two register sets: the tiles of step t travel in set t & 1 and are requested two steps ahead
  // (one step, 1.7 us of MFMAs, is not always enough for a load to come back: 114 against 125 TFLOP/s)
  constexpr int SETS = 2;
  f32x4 sa[SETS][NA], sb[SETS][4];
  int k_next = k_begin;
  auto load_tiles = [&](f32x4 (&ra)[NA], f32x4 (&rb)[4]) {
#pragma unroll
    for (int u = 0; u < NA; ++u) {
      const int c4 = (threadIdx.x + 256 * u) & 7;
      if (GUARD)  // a piece beyond this chunk's end contributes nothing: zero on the x side is enough
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

  f32x16 acc[MB][4];
#pragma unroll
  for (int a = 0; a < MB; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  // operand fragments of one k step of 8: x rows per block a (four k each), W rows per MFMA i
  // (four columns = the four blocks each)
  const int a_off = (wave * 32 * MB + ln) * AS + 4 * j, b_off = 4 * j * TN + 4 * ln;
  f32x4 af[2][MB], bf[2][4];  // [k step parity]
  auto fetch = [&](int par, int buf, int s) {
#pragma unroll
    for (int a = 0; a < MB; ++a) af[par][a] = *(const f32x4 *)&As[buf][a_off + a * 32 * AS + 8 * s];
#pragma unroll
    for (int i = 0; i < 4; ++i) bf[par][i] = *(const f32x4 *)&Bs[buf][b_off + (8 * s + i) * TN];
  };

  if (nk > 0) {
    load_tiles(sa[0], sb[0]);
    if (SETS == 2 && nk > 1) load_tiles(sa[SETS - 1], sb[SETS - 1]);
    park_tiles(sa[0], sb[0], 0);
    if (SETS == 2 ? nk > 2 : nk > 1) load_tiles(sa[0], sb[0]);
  }
  __syncthreads();
  if (nk > 0) fetch(0, 0, 0);

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
        if (kt + 1 + SETS < nk) load_tiles(ra, rb);
        if (more) fetch(nxt, buf ^ 1, 0);
      }
      ORDER_LDS_AND_MFMA();
      // the accumulators take turns: no MFMA waits for the one before it
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int a = 0; a < MB; ++a)
#pragma unroll
          for (int b = 0; b < 4; ++b)
            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[cur][a][i], bf[cur][i][b], acc[a][b], 0, 0, 0);
      ORDER_LDS_AND_MFMA();
    }
  };
  for (int kt = 0; kt < nk; kt += 2) {
    step(kt, sa[SETS - 1], sb[SETS - 1]);
    if (kt + 1 < nk) step(kt + 1, sa[0], sb[0]);
  }

  float *out = y + (long long)blockIdx.y * T * N;
  const int col = n0 + 4 * ln;
  if (col < N) {  // N is a multiple of 4: a lane's four columns are inside together
#pragma unroll
    for (int a = 0; a < MB; ++a)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wave * 32 * MB + a * 32 + 8 * (r >> 2) + 4 * j + (r & 3);
        if (row < T) {
          const long long o = (long long)row * N + col;
          f32x4 v = {acc[a][0][r], acc[a][1][r], acc[a][2][r], acc[a][3][r]};
          if (res) v = *(const f32x4 *)(res + o) + v;
          *(f32x4 *)(out + o) = v;
        }
      }
  }
}

// y = (res +) partials[0] + partials[1] + ... in that order; n4 = T * N / 4
__global__ __launch_bounds__(256) void sgemm_reduce_kernel(const float *__restrict__ partials,
                                                           const float *__restrict__ res, float *__restrict__ y,
                                                           long long n4, int chunks) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n4) return;
  f32x4 acc = ((const f32x4 *)partials)[i];
  for (int c = 1; c < chunks; ++c) acc += ((const f32x4 *)partials)[(long long)c * n4 + i];
  if (res) acc = ((const f32x4 *)res)[i] + acc;
  ((f32x4 *)y)[i] = acc;
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
  GemmPlan p;
  // (the kernel addresses the rows of x by 32-bit byte offsets from a base that moves along K)
  p.mfma = T >= 1 && K >= 4 && N >= 4 && (K & 3) == 0 && (N & 3) == 0 && (x_stride & 3) == 0 &&
           (long long)T * x_stride * 4 < 0xffffffffLL && (long long)TK * N * 4 < 0xffffffffLL;
  p.tiles_m = (T + 127) / 128;
  p.tiles_n = (N + TN - 1) / TN;
  p.chunks = 1;
  p.k_chunk = K;
  p.partial_floats = 0;
  if (!p.mfma) return p;
  // Fewer tiles than the chip runs at once (two workgroups share a compute unit) and a K that
  // is long enough: cut K so that one round fills the chip, keeping at least 8 steps of 32 per
  // chunk.  More chunks than fit that one round would leave a second round mostly empty.
  const int slots = 512;
  const int tiles = p.tiles_m * p.tiles_n;
  const int steps = (K + TK - 1) / TK;
  int chunks = 1;
  if (tiles <= slots / 2) {
    chunks = slots / tiles;
    if (chunks > steps / 8) chunks = steps / 8;
    if (chunks > 16) chunks = 16;
    if (chunks < 1) chunks = 1;
  }
  const int steps_per = (steps + chunks - 1) / chunks;
  p.k_chunk = steps_per * TK;
  p.chunks = (K + p.k_chunk - 1) / p.k_chunk;
  if (p.chunks > 1) p.partial_floats = (size_t)p.chunks * T * N;
  return p;
}

hipError_t launch_gemm(const float *x, long long x_stride, const float *w, float *y, const float *res, float *partials,
                       int T, int K, int N, const GemmPlan &p, hipStream_t stream) {
  if (!x || !w || !y || T < 1 || K < 1 || N < 1 || x_stride < K) return hipErrorInvalidValue;
  const bool aligned = !(((uintptr_t)x | (uintptr_t)w | (uintptr_t)y | (uintptr_t)res) & 15);
  if (!p.mfma || !aligned) {
    hipLaunchKernelGGL(sgemm_plain_kernel, dim3((unsigned)((N + 255) / 256), (unsigned)(T < 65535 ? T : 65535)), dim3(256), 0, stream, x,
                       x_stride, w, y, res, T, K, N);
    return hipGetLastError();
  }
  if (p.chunks > 1 && !partials) return hipErrorInvalidValue;
  const int tiles = p.tiles_m * p.tiles_n;
  const dim3 grid((unsigned)((tiles + 7) / 8 * 8), (unsigned)p.chunks);
  float *dst = p.chunks > 1 ? partials : y;
  const float *r = p.chunks > 1 ? nullptr : res;
  const bool guard = K % TK != 0;  // k_chunk is a multiple of 32 by construction
  if (guard)
    hipLaunchKernelGGL(sgemm_mfma_kernel<true>, grid, dim3(256), 0, stream, x, x_stride, w, dst, r, T, K, N, p.tiles_m,
                       p.tiles_n, p.k_chunk);
  else
    hipLaunchKernelGGL(sgemm_mfma_kernel<false>, grid, dim3(256), 0, stream, x, x_stride, w, dst, r, T, K, N, p.tiles_m,
                       p.tiles_n, p.k_chunk);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || p.chunks == 1) return e;
  const long long n4 = (long long)T * N / 4;
  hipLaunchKernelGGL(sgemm_reduce_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, stream, partials, res, y, n4,
                     p.chunks);
  return hipGetLastError();
}

}  // namespace shainet
