// y[T,N] = f(x)[T,K] * W[K,N] for a few rows (T <= 16), fp32: the projections of a
// decode step (llama_block.cr:253-255, 298; swiglu_ff.cr:76-91; the lm_head product
// of network_run.cr:1390-1404) with weights in the reference's [in, out] layout.
//
// The product is bound by reading W once from HBM, so the work is cut along K as
// well as along N to put enough workgroups in flight: a wavefront owns 256
// consecutive columns (one float4 per lane, 1 KiB per W row) and a run of rows of
// W; the four wavefronts of a workgroup take four runs and add up through LDS.
// With more than one workgroup along K, each leaves a partial sum and marks it
// complete in a flag word; the last workgroup along K of a column tile waits for
// the flags of the others, adds the partials in a fixed order, so results do not
// depend on scheduling, and applies the epilogue.  Everything a decode step does around a product rides along:
//   * prologue: RMSNorm of the x rows (rms_norm.cr:18-37, fp64 as there), so the
//     normalised activations never go to memory;
//   * epilogue: residual add (simple_matrix.cr:39-48), the SwiGLU gate
//     (swiglu_ff.cr:84-89) over a [K, 2*ff] matrix holding gate_proj | up_proj, or,
//     for the q | k | v product, bias -> QK-norm -> RoPE -> cache append
//     (llama_block.cr:256-286, 332-344) on each head row where it is summed up.
#include "attn_kernels.hpp"
#include "prep_math.hpp"

#include <math.h>
#include <stdint.h>
#include <stdlib.h>

namespace shainet {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

// Partial sums cross workgroups that may sit on different XCDs, whose L2 caches
// are not kept coherent with each other for ordinary accesses: the store is
// written through to memory (sc1 = device scope), 16 bytes at a time.
__device__ __forceinline__ void coherent_store4(float *p, f32x4 v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(p), "v"(v) : "memory");
}

__device__ __forceinline__ float swiglu1(float gate, float up) {
  const double g = (double)gate;
  return (float)((g / (1.0 + exp(-g))) * (double)up);
}

__device__ __forceinline__ f32x4 apply_epilogue(int epi, f32x4 a, f32x4 b, const float *res) {
  if (epi == kGemvSwiglu) return f32x4{swiglu1(a.x, b.x), swiglu1(a.y, b.y), swiglu1(a.z, b.z), swiglu1(a.w, b.w)};
  if (epi == kGemvResidual) {
    const f32x4 r = *(const f32x4 *)res;
    return f32x4{(float)((double)r.x + (double)a.x), (float)((double)r.y + (double)a.y),
                 (float)((double)r.z + (double)a.z), (float)((double)r.w + (double)a.w)};
  }
  return a;
}

// One row of the q | k | v product, complete in tile[CW] (columns tile0 ...): each
// wavefront takes whole heads of it through the arithmetic of prep_rows_kernel.
__device__ __forceinline__ void prep_tile_row(const GemvPrep &p, const float *tile, int tile0, int cw, int t,
                                              int wave, int lane) {
  const int hd = p.hd, half = hd >> 1;
  const bool active = lane < half;
  const int i = active ? lane : 0;
  const int pos = p.start_pos + t;
  for (int hh = wave; hh * hd < cw; hh += 4) {
    const int r = tile0 / hd + hh;  // head row of the token: H query, KV key, KV value heads
    if (r >= p.H + 2 * p.KV) break;
    float x0 = tile[hh * hd + i], x1 = tile[hh * hd + i + half];
    const float *bias, *w = nullptr;
    float *dst;
    bool rotate = true;
    if (r < p.H) {
      bias = p.b_q ? p.b_q + r * hd : nullptr;
      w = p.q_norm;
      dst = p.q_rot + (long long)t * p.H * hd + r * hd;
    } else {
      const bool is_v = r - p.H >= p.KV;
      const int c = is_v ? r - p.H - p.KV : r - p.H;
      const long long row = ((long long)c * p.cap + pos) * hd;
      bias = is_v ? (p.b_v ? p.b_v + c * hd : nullptr) : (p.b_k ? p.b_k + c * hd : nullptr);
      w = is_v ? nullptr : p.k_norm;
      dst = (is_v ? p.vc : p.kc) + row;
      rotate = !is_v;
    }
    if (bias) {
      x0 = x0 + bias[i];
      x1 = x1 + bias[i + half];
    }
    float y0 = x0, y1 = x1;
    if (rotate) {
      const float w0 = w ? w[i] : 1.0f, w1 = w ? w[i + half] : 1.0f;
      const float2 cs = p.rope_tab[(long long)pos * half + i];
      norm_rotate_pair(x0, x1, w != nullptr, w0, w1, p.eps, hd, half, cs, y0, y1);
    }
    if (active) {
      dst[i] = y0;
      dst[i + half] = y1;
    }
  }
}

// The same for one pair (x0 = element i, x1 = element i + hd / 2) of head row r of a single token,
// without QK-norm (which needs the whole head), in two steps: what does not depend on the sums (where
// the pair goes, its bias values, its cos and sin) is asked for while the weights are still on
// their way, so that no load stands between the finished sums and the stores.
struct PairTarget {
  float *dst;      // element i of the head row in q_rot or in the cache
  int half;
  float b0, b1;    // bias of the two elements (0 without one)
  bool has_bias, rotate;
  float2 cs;
};
__device__ __forceinline__ PairTarget prep_pair_begin(const GemvPrep &p, int r, int i) {
  PairTarget t;
  const int hd = p.hd, half = hd >> 1;
  const int pos = p.start_pos;
  const float *bias;
  t.rotate = true;
  if (r < p.H) {
    bias = p.b_q ? p.b_q + r * hd : nullptr;
    t.dst = p.q_rot + r * hd + i;
  } else {
    const bool is_v = r - p.H >= p.KV;
    const int c = is_v ? r - p.H - p.KV : r - p.H;
    bias = is_v ? (p.b_v ? p.b_v + c * hd : nullptr) : (p.b_k ? p.b_k + c * hd : nullptr);
    t.dst = (is_v ? p.vc : p.kc) + ((long long)c * p.cap + pos) * hd + i;
    t.rotate = !is_v;
  }
  t.half = half;
  t.has_bias = bias != nullptr;
  t.b0 = bias ? bias[i] : 0.f;
  t.b1 = bias ? bias[i + half] : 0.f;
  t.cs = p.rope_tab[(long long)pos * half + i];
  return t;
}
__device__ __forceinline__ void prep_pair_end(const GemvPrep &p, const PairTarget &t, float x0, float x1) {
  if (t.has_bias) {
    x0 = x0 + t.b0;
    x1 = x1 + t.b1;
  }
  float y0 = x0, y1 = x1;
  if (t.rotate) norm_rotate_pair(x0, x1, false, 1.0f, 1.0f, p.eps, p.hd, t.half, t.cs, y0, y1);
  t.dst[0] = y0;
  t.dst[t.half] = y1;
}

// NACC = 1, or 2 for the SwiGLU epilogue (gate and up accumulators).
// PREP: the kGemvQkvPrep epilogue (NACC = 1).
// RPI = rows of W per load instruction: 1 (a wavefront spans 256 columns) or 4
// (16 lanes per row, 64 columns, four consecutive rows at once).  Narrow tiles give
// a matrix with few columns enough column tiles that 16 workgroups along K
// suffice: the arrivals at a tile's counter serialise at roughly 0.1 us each.
template <int TT, int NACC, int RPI, bool PREP>
__global__ __launch_bounds__(256) void gemv_fused_kernel(GemvArgs a) {
  constexpr int LPR = 64 / RPI;  // lanes across a row
  constexpr int CW = LPR * 4;    // columns per tile
  extern __shared__ float smem[];  // xs[TT][4 * rows_per_wave]; reused for the cross-wavefront sums
  __shared__ double rms_s[TT];
  __shared__ double red_s[4];
  __shared__ __align__(16) float tile_s[PREP ? 256 : 4];  // PREP: one finished row of this column tile
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int cl = lane % LPR, sub = lane / LPR;
  const int T = a.T, K = a.K, N = a.N;
  const int rpw = a.rows_per_wave, span = 4 * rpw;  // rpw is a multiple of 8 * RPI
  const int col = blockIdx.x * CW + cl * 4;
  const int k_wg = blockIdx.y * span;
  const int ldw = NACC * N;  // row pitch of W
  const bool have_col = col < N;  // N is a multiple of 4

  // The first eight row loads of W do not depend on x: they are issued before the prologue
  // and land while the norm is computed and x is staged (a product of 128 rows per
  // workgroup with 4 rows per instruction is these eight loads and nothing more).
  const int kk0 = wave * rpw;  // this wavefront's rows, relative to k_wg
  f32x4 r_first[NACC][8];
  const bool have_first = have_col && k_wg + kk0 < K;
  if (have_first) {
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int row = min(k_wg + kk0 + u * RPI + sub, K - 1);
#pragma unroll
      for (int c = 0; c < NACC; ++c) r_first[c][u] = __builtin_nontemporal_load((const f32x4 *)(a.w + (long long)row * ldw + c * N + col));
    }
  }

  // ---- prologue: the x values of this workgroup's K range, normalised if asked;
  // zero beyond K and beyond T, so that clamped loads below contribute nothing
  if (a.norm) {
    for (int t = 0; t < T; ++t) {
      const float *xr = a.x + (long long)t * a.x_stride;
      double sq = 0.0;
      if (((K | a.x_stride) & 3) == 0) {
        for (int k = threadIdx.x * 4; k < K; k += 1024) {
          const f32x4 v = *(const f32x4 *)(xr + k);
          sq += (double)v.x * (double)v.x + (double)v.y * (double)v.y;
          sq += (double)v.z * (double)v.z + (double)v.w * (double)v.w;
        }
      } else {
        for (int k = threadIdx.x; k < K; k += 256) sq += (double)xr[k] * (double)xr[k];
      }
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) sq += __shfl_xor(sq, o);
      if (lane == 0) red_s[wave] = sq;
      __syncthreads();
      if (threadIdx.x == 0) rms_s[t] = sqrt(((red_s[0] + red_s[1]) + (red_s[2] + red_s[3])) / (double)K + a.eps);
      __syncthreads();
    }
  }
  for (int idx = threadIdx.x; idx < TT * span; idx += 256) {
    const int t = idx / span, kk = idx - t * span, k = k_wg + kk;
    float v = 0.f;
    if (t < T && k < K) {
      v = a.x[(long long)t * a.x_stride + k];
      if (a.norm) v = (float)(((double)v / rms_s[t]) * (double)(a.gamma ? a.gamma[k] : 1.f));
    }
    smem[idx] = v;
  }
  __syncthreads();

  // ---- main loop: eight load instructions (8 * RPI rows of W) in flight per wavefront
  f32x4 acc[NACC][TT];
#pragma unroll
  for (int c = 0; c < NACC; ++c)
#pragma unroll
    for (int t = 0; t < TT; ++t) acc[c][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  if (have_first) {
    for (int kb = 0; kb < rpw && k_wg + kk0 + kb < K; kb += 8 * RPI) {
      f32x4 r[NACC][8];
      if (kb == 0) {
#pragma unroll
        for (int u = 0; u < 8; ++u)
#pragma unroll
          for (int c = 0; c < NACC; ++c) r[c][u] = r_first[c][u];
      } else {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int row = min(k_wg + kk0 + kb + u * RPI + sub, K - 1);
#pragma unroll
          for (int c = 0; c < NACC; ++c) r[c][u] = __builtin_nontemporal_load((const f32x4 *)(a.w + (long long)row * ldw + c * N + col));
        }
      }
#pragma unroll
      for (int u = 0; u < 8; ++u)
#pragma unroll
        for (int t = 0; t < TT; ++t) {
          const float xv = smem[t * span + kk0 + kb + u * RPI + sub];  // one address per row: broadcasts
#pragma unroll
          for (int c = 0; c < NACC; ++c) acc[c][t] += xv * r[c][u];
        }
    }
  }
  if constexpr (RPI > 1) {  // add the RPI row groups of the wavefront: every lane ends up with the sum
#pragma unroll
    for (int c = 0; c < NACC; ++c)
#pragma unroll
      for (int t = 0; t < TT; ++t)
#pragma unroll
        for (int o = LPR; o < 64; o <<= 1) {
          acc[c][t].x += __shfl_xor(acc[c][t].x, o);
          acc[c][t].y += __shfl_xor(acc[c][t].y, o);
          acc[c][t].z += __shfl_xor(acc[c][t].z, o);
          acc[c][t].w += __shfl_xor(acc[c][t].w, o);
        }
  }

  // ---- the four wavefronts add up through LDS (the x staging area is free now),
  // one accumulator set at a time to keep the footprint at [3][TT][64] float4
  f32x4 *red = (f32x4 *)smem;
  const int splits = gridDim.y;
#pragma unroll
  for (int c = 0; c < NACC; ++c) {
    __syncthreads();
    if (wave > 0) {
#pragma unroll
      for (int t = 0; t < TT; ++t) red[((wave - 1) * TT + t) * 64 + lane] = acc[c][t];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int t = 0; t < TT; ++t)
        acc[c][t] = (acc[c][t] + red[(0 * TT + t) * 64 + lane]) + (red[(1 * TT + t) * 64 + lane] + red[(2 * TT + t) * 64 + lane]);
    }
  }
  const bool writer = wave == 0 && sub == 0 && have_col;
  if (splits == 1) {
#pragma unroll
    for (int t = 0; t < TT; ++t)
      if (t < T) {
        if constexpr (PREP) {
          if (writer) *(f32x4 *)(tile_s + cl * 4) = acc[0][t];
          __syncthreads();
          prep_tile_row(a.prep, tile_s, blockIdx.x * CW, CW, t, wave, lane);
          __syncthreads();
        } else if (writer) {
          const float *res = a.res ? a.res + (long long)t * N + col : nullptr;
          *(f32x4 *)(a.y + (long long)t * N + col) = apply_epilogue(a.epilogue, acc[0][t], acc[NACC - 1][t], res);
        }
      }
    return;
  }
  if (writer) {
#pragma unroll
    for (int t = 0; t < TT; ++t)
      if (t < T) {
#pragma unroll
        for (int c = 0; c < NACC; ++c)
          coherent_store4(a.partials + (((long long)blockIdx.y * T + t) * NACC + c) * N + col, acc[c][t]);
      }
  }

  // ---- the last workgroup along K of this column tile adds the partials in a fixed order.
  // The partial stores above are acknowledged (s_waitcnt vmcnt(0): the barrier alone does
  // not wait for them) before the partial is marked complete in its flag word; the merging
  // workgroup clears the words it waited for, so they are zero between launches.
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();
  unsigned *flags = a.flags + (long long)blockIdx.x * splits;
  if ((int)blockIdx.y != splits - 1) {
    if (threadIdx.x == 0)
      __hip_atomic_store((a.flag_set ? a.flag_set : a.flags) + (long long)blockIdx.x * splits + blockIdx.y, 1u,
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return;
  }
  // the others have lower indices, were started before this workgroup and wait for nobody
  if (wave == 0) {
    for (int spins = 0;; ++spins) {
      bool ok = true;
      for (int i = lane; i < splits - 1; i += 64)
        ok = ok && __hip_atomic_load(flags + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u;
      if (__all(ok)) {
        for (int i = lane; i < splits - 1; i += 64)
          __hip_atomic_store(flags + i, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
      if (spins >= (a.spin_limit > 0 ? a.spin_limit : 1 << 21)) {  // (by default: seconds)
        if (lane == 0) *a.error = 1;
        break;
      }
      __builtin_amdgcn_s_sleep(2);
    }
  }
  __syncthreads();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  for (int t = 0; t < T; ++t) {
    // row group g = wave * RPI + sub adds splits g, g + 4 * RPI, ... (FL loads in flight);
    // then the groups of a wavefront are added by shuffles and the wavefronts through LDS
    f32x4 part[NACC];
#pragma unroll
    for (int c = 0; c < NACC; ++c) part[c] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (have_col) {
      constexpr int FL = NACC == 1 ? 8 : 4;  // loads in flight per lane
      for (int s0 = wave * RPI + sub; s0 < splits; s0 += 4 * RPI * FL) {
        f32x4 v[NACC][FL];
#pragma unroll
        for (int u = 0; u < FL; ++u) {
          const int s = min(s0 + 4 * RPI * u, splits - 1);
#pragma unroll
          for (int c = 0; c < NACC; ++c)
            v[c][u] = *(const f32x4 *)(a.partials + (((long long)s * T + t) * NACC + c) * N + col);
        }
#pragma unroll
        for (int u = 0; u < FL; ++u)
          if (s0 + 4 * RPI * u < splits) {
#pragma unroll
            for (int c = 0; c < NACC; ++c) part[c] += v[c][u];
          }
      }
    }
    if constexpr (RPI > 1) {
#pragma unroll
      for (int c = 0; c < NACC; ++c)
#pragma unroll
        for (int o = LPR; o < 64; o <<= 1) {
          part[c].x += __shfl_xor(part[c].x, o);
          part[c].y += __shfl_xor(part[c].y, o);
          part[c].z += __shfl_xor(part[c].z, o);
          part[c].w += __shfl_xor(part[c].w, o);
        }
    }
    __syncthreads();
#pragma unroll
    for (int c = 0; c < NACC; ++c) red[(wave * NACC + c) * 64 + lane] = part[c];
    __syncthreads();
    if (writer) {
      f32x4 sum[NACC];
#pragma unroll
      for (int c = 0; c < NACC; ++c)
        sum[c] = (red[(0 * NACC + c) * 64 + lane] + red[(1 * NACC + c) * 64 + lane]) +
                 (red[(2 * NACC + c) * 64 + lane] + red[(3 * NACC + c) * 64 + lane]);
      if constexpr (PREP) {
        *(f32x4 *)(tile_s + cl * 4) = sum[0];
      } else {
        const float *res = a.res ? a.res + (long long)t * N + col : nullptr;
        *(f32x4 *)(a.y + (long long)t * N + col) = apply_epilogue(a.epilogue, sum[0], sum[NACC - 1], res);
      }
    }
    if constexpr (PREP) {
      __syncthreads();  // the row is complete in tile_s; the next round's first barrier protects it
      prep_tile_row(a.prep, tile_s, blockIdx.x * CW, CW, t, wave, lane);
    }
  }
}


// ---- one row of x against weights kept transposed: wt [N, K] (row n = column n of W) --------
// Every output element is one contiguous row of wt, so a wavefront owns whole outputs: it reads
// a row with KV4 16-byte loads per lane, all in flight at once, multiplies by the x values it
// holds and adds up across its lanes.  Nothing crosses workgroups: no partial sums in memory, no
// flag words, no wait, and a launch ends when its rows have streamed (a 2048 x 2048 product:
// 4.8 us back to back against 8.8 us for the split product above).  What it costs is the second
// copy of the matrix.  NACC = 2: the SwiGLU epilogue; the wavefront reads row n (gate) and row
// N + n (up).  SP = 2: two wavefronts share an output, half a row each, and add up through LDS
// (rows of 8192 values; NACC = 1, no norm).  K = 256 KV4 SP.  The RMSNorm prologue is done by every
// wavefront for itself: the mean of squares in fp64 as rms_norm.cr:18-37, and the factor 1 / rms
// applied to the finished sum, sum_k w[n][k] (x[k] gamma[k]), rather than to every x[k] (a division per
// element in every wavefront cost 5 of the 26 us of a 2048 -> 2 x 8192 product, and two fp64
// products per element, on the path between x and the first multiply-add, still 1.4 us), once for the
// a.rows_per_wave consecutive outputs it takes (more than one where N is large, so that the
// prologue does not outweigh the rows: 128 256 outputs with a wavefront each took 199 us, the
// split product 169 us).  The next row's loads are issued before the current row is added up.
// MULTI: a wavefront takes more than one output; only then are there registers for a second row.
// PREP (NACC = 1, a.N = the number of pairs): the kGemvQkvPrep epilogue of a q | k | v product without
// QK-norm.  Output n is the pair (i, i + hd / 2) of head row r, n = r * hd / 2 + i: rows r * hd + i and
// r * hd + i + hd / 2 of the matrix, whose two sums are all that bias, RoPE and the cache append of
// the pair need (llama_block.cr:256-286, 332-344), so the head rows never go through memory either.
// A workgroup takes two pairs: wavefronts 0 and 1 their lower rows, 2 and 3 their upper rows, and
// the sums meet in LDS (a wavefront per pair, two rows each, took 0.85 us longer for 3072 rows).
template <int KV4, int NACC, int SP, bool MULTI, bool PREP = false>
__global__ __launch_bounds__(256) void gemvt_kernel(GemvArgs a) {
  static_assert(!PREP || (NACC == 1 && SP == 1 && !MULTI), "the q | k | v epilogue: one row per wavefront");
  // x: up to 2048 values stay in registers.  Longer (half) rows: a wavefront with one output reads
  // them again from memory (the L2), eight 16-byte pieces at a time, where they are used; one with
  // several outputs keeps its own normed copy in LDS
  // One output per wavefront (XSH): the workgroup puts x into LDS once, asked for before the
  // weights, each thread a share of it; the share's squares give the norm's sum once per workgroup
  // (rows of 8192 first: read piece by piece from the L2 where it was used, x came back behind the
  // weight loads it was issued after, a round trip at the end of every wavefront, and the
  // registers for it left room for two wavefronts per SIMD).  Several outputs per wavefront:
  // x in registers (XREG) or a normed copy per wavefront in LDS (XLDS), as described above.
  constexpr bool XSH = !MULTI, XREG = !XSH && KV4 <= 8, XLDS = !XSH && !XREG;
  __shared__ __align__(16) float xs[XLDS ? 4 * 256 * KV4 : 4];
  __shared__ __align__(16) float xsh[XSH ? 256 * KV4 * SP : 4];
  __shared__ float half_s[4], sq_s[4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int rpw = a.rows_per_wave;
  const int N = a.N;
  const int n_own = PREP ? blockIdx.x * 2 + (wave & 1) : (blockIdx.x * (4 / SP) + wave / SP) * rpw;
  // (PREP: an odd number of pairs leaves two wavefronts of the last workgroup without one: they go
  // through the motions on the last pair, for the barrier's sake, and store nothing)
  const bool live = n_own < N;
  const int n0 = PREP ? min(n_own, N - 1) : n_own;  // this wavefront's first output
  const int seg = wave % SP;
  constexpr int KW = 256 * KV4;  // values per wavefront and row
  constexpr int K = KW * SP;
  // (with SP = 2 both wavefronts of a pair see the same n0: they are live or not together; XSH:
  // wavefronts without an output stay for the workgroup's x and leave after its barrier)
  if (!PREP && !XSH && !live) return;
  const int half_hd = PREP ? a.prep.hd >> 1 : 1;
  const int half_shift = PREP ? __builtin_ctz(half_hd) : 0;
  const int upper = PREP ? wave >> 1 : 0;
  auto load_row = [&](f32x4 (&w)[NACC][KV4], int n) {
#pragma unroll
    for (int c = 0; c < NACC; ++c) {
      const long long wrow = PREP ? (long long)n + (((n >> half_shift) + upper) << half_shift) : (long long)c * N + n;
      const float *row = a.w + wrow * K + seg * KW + 4 * lane;
#pragma unroll
      for (int i = 0; i < KV4; ++i) w[c][i] = __builtin_nontemporal_load((const f32x4 *)(row + 256 * i));
    }
  };
  f32x4 wa[NACC][KV4], wb[MULTI ? NACC : 1][MULTI ? KV4 : 1];
  float rms = 1.0f;  // 1 / the root mean square
  constexpr bool NORMS = SP == 1;  // (rows shared by two wavefronts come without the norm: gemvt_takes)
  f32x4 x_own[XSH ? K / 1024 : 1], g_own[XSH && NORMS ? K / 1024 : 1];  // this thread's share of x (and gamma) on its way to LDS
  if constexpr (XSH) {
#pragma unroll
    for (int i = 0; i < K / 1024; ++i) x_own[i] = *(const f32x4 *)(a.x + 4 * threadIdx.x + 1024 * i);
    if (NORMS && a.norm && a.gamma) {
#pragma unroll
      for (int i = 0; i < K / 1024; ++i) g_own[i] = *(const f32x4 *)(a.gamma + 4 * threadIdx.x + 1024 * i);
    }
  }
  if (live || PREP) load_row(wa, n0);
  if constexpr (XSH) {
    if (NORMS && a.norm) {
      // squares, their sums and the root in fp32 (a reciprocal square root and one Newton step):
      // within a few 1e-7 of the fp64 factor of rms_norm.cr:18-37
      f32x4 q = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < K / 1024; ++i) q += x_own[i] * x_own[i];
      float sq = (q.x + q.y) + (q.z + q.w);
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) sq += __shfl_xor(sq, o);
      if (lane == 0) sq_s[wave] = sq;
      if (a.gamma) {
#pragma unroll
        for (int i = 0; i < K / 1024; ++i) x_own[i] = x_own[i] * g_own[i];  // (1 / rms multiplies the finished sum)
      }
    }
#pragma unroll
    for (int i = 0; i < K / 1024; ++i) *(f32x4 *)(xsh + 4 * threadIdx.x + 1024 * i) = x_own[i];
    __syncthreads();
    if (!PREP && !live) return;
    if (NORMS && a.norm) {
      const float m = ((sq_s[0] + sq_s[1]) + (sq_s[2] + sq_s[3])) / (float)K + (float)a.eps;
      float r = rsqrtf(m);
      rms = r * (1.5f - 0.5f * m * r * r);
    }
  }
  // what the epilogue of the first output reads besides: asked for now, behind the weights
  const bool residual = !PREP && a.epilogue == kGemvResidual;
  float res_first = 0.f;
  if (residual) res_first = a.res[n0];
  PairTarget target = {};
  // (head_dim is a power of two here: gemvt_takes)
  if constexpr (PREP) target = prep_pair_begin(a.prep, n0 >> half_shift, n0 & (half_hd - 1));

  constexpr int XC = KV4 < 8 ? KV4 : 8;
  const float *xp = a.x + seg * KW + 4 * lane;
  float *my_xs = xs + (XLDS ? wave * KW : 0) + 4 * lane;
  f32x4 xv[XREG ? KV4 : 1];
  if constexpr (XREG) {  // x is loaded once, into the registers it stays in
#pragma unroll
    for (int i = 0; i < KV4; ++i) xv[i] = *(const f32x4 *)(xp + 256 * i);
  }
  if (!XSH && a.norm) {
    // every wavefront of the launch runs this, so it is kept short: squares, their sums and the
    // root in fp32 (a reciprocal square root and one Newton step; all of it in fp64 as
    // rms_norm.cr does cost 0.4 us of a 3072-row product for the sums and as much for the root);
    // the factor is within a few 1e-7 of the fp64 one
    f32x4 q = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c0 = 0; c0 < KV4; c0 += XC) {
      f32x4 t[XC];
#pragma unroll
      for (int i = 0; i < XC; ++i) t[i] = XREG ? xv[c0 + i] : *(const f32x4 *)(xp + 256 * (c0 + i));
#pragma unroll
      for (int i = 0; i < XC; ++i) q += t[i] * t[i];
    }
    float sq = (q.x + q.y) + (q.z + q.w);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) sq += __shfl_xor(sq, o);
    const float m = sq / (float)K + (float)a.eps;
    float r = rsqrtf(m);
    r = r * (1.5f - 0.5f * m * r * r);
    rms = r;
  }
  // pieces c0 .. c0 + XC - 1 of x times gamma (for the copy of XLDS)
  auto x_pieces = [&](f32x4 (&t)[XC], int c0) {
#pragma unroll
    for (int i = 0; i < XC; ++i) t[i] = *(const f32x4 *)(xp + 256 * (c0 + i));
    if (a.norm) {
#pragma unroll
      for (int i = 0; i < XC; ++i) {
        f32x4 g = {1.f, 1.f, 1.f, 1.f};
        if (a.gamma) g = *(const f32x4 *)(a.gamma + seg * KW + 4 * lane + 256 * (c0 + i));
        t[i] = t[i] * g;  // (1 / rms multiplies the finished sum instead of every element)
      }
    }
  };
  if constexpr (XREG) {
    if (a.norm && a.gamma) {
#pragma unroll
      for (int i = 0; i < KV4; ++i) xv[i] = xv[i] * *(const f32x4 *)(a.gamma + 4 * lane + 256 * i);
    }
  } else if constexpr (XLDS) {
#pragma unroll
    for (int c0 = 0; c0 < KV4; c0 += XC) {
      f32x4 t[XC];
      x_pieces(t, c0);
#pragma unroll
      for (int i = 0; i < XC; ++i) *(f32x4 *)(my_xs + 256 * (c0 + i)) = t[i];  // read back by this lane only: no barrier
    }
  }

  auto finish_row = [&](const f32x4 (&w)[NACC][KV4], int n, float res_v) {
    f32x4 acc[NACC];
#pragma unroll
    for (int c = 0; c < NACC; ++c) acc[c] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c0 = 0; c0 < KV4; c0 += XC) {
      f32x4 t[XC];
      if constexpr (XREG) {
#pragma unroll
        for (int i = 0; i < XC; ++i) t[i] = xv[c0 + i];
      } else if constexpr (XLDS) {
#pragma unroll
        for (int i = 0; i < XC; ++i) t[i] = *(const f32x4 *)(my_xs + 256 * (c0 + i));
      } else {  // XSH
#pragma unroll
        for (int i = 0; i < XC; ++i) t[i] = *(const f32x4 *)(xsh + seg * KW + 4 * lane + 256 * (c0 + i));
      }
#pragma unroll
      for (int c = 0; c < NACC; ++c)
#pragma unroll
        for (int i = 0; i < XC; ++i) acc[c] += w[c][c0 + i] * t[i];
    }
    float s[NACC];
#pragma unroll
    for (int c = 0; c < NACC; ++c) {
      s[c] = (acc[c].x + acc[c].y) + (acc[c].z + acc[c].w);
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) s[c] += __shfl_xor(s[c], o);
    }
    if constexpr (SP == 2) {
      __syncthreads();  // (the pair's sums of the row before have been read)
      if (lane == 0) half_s[wave] = s[0];
      __syncthreads();
      s[0] = half_s[wave & ~1] + half_s[wave | 1];
      if (seg) return;
    }
    if (a.norm) {
#pragma unroll
      for (int c = 0; c < NACC; ++c) s[c] = s[c] * rms;
    }
    if constexpr (PREP) {
      if (lane == 0) half_s[wave] = s[0];
      __syncthreads();
      if (wave < 2 && lane == 0 && live) prep_pair_end(a.prep, target, half_s[wave], half_s[wave + 2]);
    } else if (lane == 0) {
      float v = s[0];
      if (a.epilogue == kGemvSwiglu) v = swiglu1(s[0], s[NACC - 1]);
      if (residual) v = (float)((double)res_v + (double)s[0]);
      a.y[n] = v;
    }
  };
  // (with SP = 2 every wavefront of the workgroup makes the same number of turns: the rows of
  // all pairs end together, launch_gemvt sees to it, so the barriers above are met by all)
  if constexpr (MULTI) {
    const int n_end = min(n0 + rpw, N);
    float res_a = res_first, res_b = 0.f;  // the residual values travel with the rows' loads
    for (int n = n0; n < n_end; n += 2) {
      if (n + 1 < n_end) {
        load_row(wb, n + 1);
        if (residual) res_b = a.res[n + 1];
      }
      finish_row(wa, n, res_a);
      if (n + 1 < n_end) {
        if (n + 2 < n_end) {
          load_row(wa, n + 2);
          if (residual) res_a = a.res[n + 2];
        }
        finish_row(wb, n + 1, res_b);
      }
    }
  } else {
    finish_row(wa, n0, res_first);
  }
}

}  // namespace

GemvPlan plan_gemv(int T, int K, int N, int epilogue, int head_dim) {
  GemvPlan p;
  const int nacc = epilogue == kGemvSwiglu ? 2 : 1;
  static const int wg_env = getenv("SHAINET_HIP_GEMV_WGS") ? atoi(getenv("SHAINET_HIP_GEMV_WGS")) : 0;
  // about 1024 workgroups per product (512 when each reads two matrices' worth) but at
  // most 16 along K; a matrix too narrow for that with 256-column tiles gets 64-column ones
  const int target = (wg_env > 0 ? wg_env : 1024) / nacc;
  p.rows_per_instr = ((N + 255) / 256) * 16 < target ? 4 : 1;
  if (epilogue == kGemvQkvPrep && head_dim > 64) p.rows_per_instr = 1;  // a 64-column tile cannot hold a head
  const int cw = 256 / p.rows_per_instr;
  const int col_tiles = (N + cw - 1) / cw;
  int splits = (target + col_tiles - 1) / col_tiles;
  if (splits > 16) splits = 16;
  // rows of W per wavefront: a multiple of what eight load instructions cover, at
  // most 256 or, with more than 4 rows of x, 128 (the x staging area in LDS holds
  // rows of x * 4 * rows_per_wave floats)
  const int quantum = 8 * p.rows_per_instr;
  const int max_rows = T > 4 ? 128 : 256;
  int rows = (K + 4 * splits - 1) / (4 * splits);
  rows = rows / quantum * quantum;
  if (rows < quantum) rows = quantum;
  if (rows > max_rows) rows = max_rows;
  splits = (K + 4 * rows - 1) / (4 * rows);
  p.rows_per_wave = rows;
  p.splits = splits;
  p.col_tiles = col_tiles;
  p.partial_floats = splits > 1 ? (size_t)splits * T * nacc * N : 0;
  return p;
}

hipError_t launch_gemv(const GemvArgs &args, const GemvPlan &p, hipStream_t stream) {
  GemvArgs a = args;
  if (a.T < 1 || a.T > 16 || a.K < 1 || a.N < 4 || (a.N & 3) || !a.x || !a.w || a.x_stride < a.K)
    return hipErrorInvalidValue;
  if (!a.y && a.epilogue != kGemvQkvPrep) return hipErrorInvalidValue;
  if (p.rows_per_instr != 1 && p.rows_per_instr != 4) return hipErrorInvalidValue;
  if (p.rows_per_wave < 8 * p.rows_per_instr || p.rows_per_wave % (8 * p.rows_per_instr)) return hipErrorInvalidValue;
  if (p.splits > 1 && (!a.partials || !a.flags || !a.error)) return hipErrorInvalidValue;
  if (a.epilogue == kGemvResidual && !a.res) return hipErrorInvalidValue;
  if (a.epilogue != kGemvResidual) a.res = nullptr;
  const bool prep = a.epilogue == kGemvQkvPrep;
  if (prep) {
    const GemvPrep &q = a.prep;
    const int cw = 256 / p.rows_per_instr;
    if (q.hd < 2 || q.hd > 128 || (q.hd & (q.hd - 1)) || cw % q.hd || q.H < 1 || q.KV < 1 ||
        a.N != (q.H + 2 * q.KV) * q.hd || !q.rope_tab || !q.q_rot || !q.kc || !q.vc || q.start_pos < 0 ||
        q.start_pos + a.T > q.cap)
      return hipErrorInvalidValue;
  }
  a.rows_per_wave = p.rows_per_wave;
  dim3 grid((unsigned)p.col_tiles, (unsigned)p.splits);
  const int nacc = a.epilogue == kGemvSwiglu ? 2 : 1;
  const int tt = a.T == 1 ? 1 : (a.T <= 4 ? 4 : 16);
  const size_t stage = (size_t)tt * 4 * p.rows_per_wave * sizeof(float);
  const size_t red = (size_t)(3 * tt > 4 * nacc ? 3 * tt : 4 * nacc) * 64 * sizeof(f32x4);
  const size_t smem = stage > red ? stage : red;
#define SHAINET_LAUNCH_GEMV(TT_, NACC_, RPI_, PREP_) \
  hipLaunchKernelGGL((gemv_fused_kernel<TT_, NACC_, RPI_, PREP_>), grid, dim3(256), smem, stream, a)
#define SHAINET_LAUNCH_GEMV_T(NACC_, RPI_, PREP_)   \
  do {                                              \
    if (tt == 1)                                    \
      SHAINET_LAUNCH_GEMV(1, NACC_, RPI_, PREP_);   \
    else if (tt == 4)                               \
      SHAINET_LAUNCH_GEMV(4, NACC_, RPI_, PREP_);   \
    else                                            \
      SHAINET_LAUNCH_GEMV(16, NACC_, RPI_, PREP_);  \
  } while (0)
  if (prep && p.rows_per_instr == 1)
    SHAINET_LAUNCH_GEMV_T(1, 1, true);
  else if (prep)
    SHAINET_LAUNCH_GEMV_T(1, 4, true);
  else if (nacc == 1 && p.rows_per_instr == 1)
    SHAINET_LAUNCH_GEMV_T(1, 1, false);
  else if (nacc == 1)
    SHAINET_LAUNCH_GEMV_T(1, 4, false);
  else if (p.rows_per_instr == 1)
    SHAINET_LAUNCH_GEMV_T(2, 1, false);
  else
    SHAINET_LAUNCH_GEMV_T(2, 4, false);
#undef SHAINET_LAUNCH_GEMV_T
#undef SHAINET_LAUNCH_GEMV
  return hipGetLastError();
}

bool gemvt_takes(int T, int K, int N, int epilogue, bool norm, const GemvPrep *prep) {
  if (T != 1 || N < 1) return false;
  if (epilogue == kGemvQkvPrep) {
    if (!prep || prep->q_norm || prep->k_norm || prep->hd < 2 || (prep->hd & (prep->hd - 1))) return false;
    return (K == 1024 || K == 2048 || K == 4096) && N == (prep->H + 2 * prep->KV) * prep->hd;
  }
  // rows of 8192: two wavefronts per output, which leaves out the norm prologue and SwiGLU
  if (K == 8192) return !norm && !(N & 1) && (epilogue == kGemvPlain || epilogue == kGemvResidual);
  if (K != 1024 && K != 2048 && K != 4096) return false;
  return epilogue == kGemvPlain || epilogue == kGemvResidual || epilogue == kGemvSwiglu;
}

hipError_t launch_gemvt(const GemvArgs &args, hipStream_t stream) {
  GemvArgs a = args;
  const bool prep = a.epilogue == kGemvQkvPrep;
  if (!gemvt_takes(a.T, a.K, a.N, a.epilogue, a.norm != 0, &a.prep) || !a.x || !a.w || (!a.y && !prep)) return hipErrorInvalidValue;
  if (a.epilogue == kGemvResidual && !a.res) return hipErrorInvalidValue;
  if (((uintptr_t)a.x | (uintptr_t)a.w | (uintptr_t)a.gamma) & 15) return hipErrorInvalidValue;
  if (prep) {
    const GemvPrep &q = a.prep;
    if (q.H < 1 || q.KV < 1 || !q.rope_tab || !q.q_rot || !q.kc || !q.vc || q.start_pos < 0 || q.start_pos + 1 > q.cap)
      return hipErrorInvalidValue;
    a.N = a.N / 2;  // pairs, two per workgroup
    a.rows_per_wave = 1;
    const dim3 pgrid((unsigned)((a.N + 1) / 2));
    switch (a.K) {
      case 1024: hipLaunchKernelGGL((gemvt_kernel<4, 1, 1, false, true>), pgrid, dim3(256), 0, stream, a); break;
      case 2048: hipLaunchKernelGGL((gemvt_kernel<8, 1, 1, false, true>), pgrid, dim3(256), 0, stream, a); break;
      default: hipLaunchKernelGGL((gemvt_kernel<16, 1, 1, false, true>), pgrid, dim3(256), 0, stream, a); break;
    }
    return hipGetLastError();
  }
  const bool two = a.epilogue == kGemvSwiglu;
  const int sp = a.K == 8192 ? 2 : 1;
  // outputs per wavefront: one until the launch has some 32 000 wavefronts, then more (128 256
  // outputs: 4 per wavefront; 8 per wavefront were 5 us slower, 2 per wavefront 11 us)
  static const int wave_target = getenv("SHAINET_HIP_GEMVT_WAVES") ? atoi(getenv("SHAINET_HIP_GEMVT_WAVES")) : 32768;
  int rpw = (int)(((long long)a.N * (two ? 2 : 1) * sp + wave_target - 1) / wave_target);
  if (sp == 2) {
    // all pairs of a workgroup must take the same number of rows: rpw divides N / 2 pairs' worth evenly
    while ((a.N / 2) % rpw) --rpw;
  }
  a.rows_per_wave = rpw;
  const int per_wg = (4 / sp) * rpw;
  const dim3 grid((unsigned)((a.N + per_wg - 1) / per_wg));
#define SHAINET_LAUNCH_GEMVT(KV4_)                                                            \
  do {                                                                                        \
    if (two && rpw > 1)                                                                       \
      hipLaunchKernelGGL((gemvt_kernel<KV4_, 2, 1, true>), grid, dim3(256), 0, stream, a);    \
    else if (two)                                                                             \
      hipLaunchKernelGGL((gemvt_kernel<KV4_, 2, 1, false>), grid, dim3(256), 0, stream, a);   \
    else if (rpw > 1)                                                                         \
      hipLaunchKernelGGL((gemvt_kernel<KV4_, 1, 1, true>), grid, dim3(256), 0, stream, a);    \
    else                                                                                      \
      hipLaunchKernelGGL((gemvt_kernel<KV4_, 1, 1, false>), grid, dim3(256), 0, stream, a);   \
  } while (0)
  switch (a.K) {
    case 1024: SHAINET_LAUNCH_GEMVT(4); break;
    case 2048: SHAINET_LAUNCH_GEMVT(8); break;
    case 4096: SHAINET_LAUNCH_GEMVT(16); break;
    default:  // 8192: two wavefronts per output
      if (rpw > 1)
        hipLaunchKernelGGL((gemvt_kernel<16, 1, 2, true>), grid, dim3(256), 0, stream, a);
      else
        hipLaunchKernelGGL((gemvt_kernel<16, 1, 2, false>), grid, dim3(256), 0, stream, a);
      break;
  }
#undef SHAINET_LAUNCH_GEMVT
  return hipGetLastError();
}

}  // namespace shainet
