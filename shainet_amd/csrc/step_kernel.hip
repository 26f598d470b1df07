// One decode step of a stack of LlamaBlocks (LlamaBlock#forward_cached for one new row,
// llama_block.cr:189-196, 246-299; swiglu_ff.cr:76-91; as Network#run walks the layers,
// network_run.cr:199-204) in ONE launch of one workgroup per compute unit.
//
// A decode step is bound by reading every weight once, and no weight depends on an
// activation.  With one launch per product the memory system idles through every launch,
// prologue and cross-workgroup reduction.  Here the workgroups stay resident for the whole
// step; the five phases of a block
//     q|k|v product -> attention -> output product -> gate|up product -> down product
// are separated by barriers over all workgroups, and every thread has issued the first loads
// of the NEXT product's weights before it arrives at a barrier, so the barrier, the sums of
// the previous phase's partial results and the attention hide under weight streaming.
//
// Every product is cut into column tiles and splits along K, one (tile, split) per
// workgroup; a workgroup leaves the partial sum of its split in memory (write-through
// stores) and the workgroups of the next phase add the partials they need, in a fixed
// order, while they build their x slice in LDS: results do not depend on timing.  The
// residual stream (one row of d_model floats) is kept by every workgroup in its own LDS.
//
// Barrier: after its stores are acknowledged a workgroup arrives at a counter of its group of
// 16, the group's last arrival at a counter of the groups, and the last of those releases
// everybody through one word per group (bounded polls: a give-up sets the error word and the
// launch still ends).  Nothing is reset between launches: the numbers keep counting up.
#include "step_kernel.hpp"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>

#include "prep_math.hpp"

namespace shainet {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int NT = kStepThreads;
constexpr int NW = NT / 64;

__device__ __forceinline__ void coherent_store4(float *p, f32x4 v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void coherent_store(float *p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Partial results of other workgroups are read past the caches, which may hold a stale line of
// another XCD's data.  (Invalidating the caches once per phase and reading with ordinary loads
// was measured too: slower.)
__device__ __forceinline__ float part_load(const float *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ float swiglu1(float gate, float up) {  // swiglu_ff.cr:84-89
  const double g = (double)gate;
  return (float)((g / (1.0 + exp(-g))) * (double)up);
}

#define STEP_TRACE(slot)                                                                          \
  do {                                                                                            \
    if (TRACE && a.trace && threadIdx.x == 0)                                                     \
      a.trace[(long long)blockIdx.x * (1 + kStepTraceSlots * a.n_layers) + (slot)] = wall_clock64();           \
  } while (0)

// The numbers every phase works with.  The kernel makes a fresh copy at the start of each phase
// and hides where it came from (fresh_view): everything is the same in every block of the
// stack, and the compiler otherwise computes the addresses of all phases once, before the loop
// over the blocks, and runs out of registers keeping them.
struct View {
  int tid;
  int d, hd, KV, ff, pos, ck, chunks;
};
__device__ __forceinline__ View fresh_view(const StepArgs &a) {
  View v;
  v.tid = threadIdx.x;
  v.d = a.d;
  v.hd = a.hd;
  v.KV = a.KV;
  v.ff = a.ff;
  v.pos = a.pos;
  v.ck = a.attn_ck;
  v.chunks = a.attn_chunks;
  asm volatile("" : "+v"(v.tid));
  asm volatile("" : "+s"(v.d), "+s"(v.hd), "+s"(v.KV), "+s"(v.ff), "+s"(v.pos), "+s"(v.ck), "+s"(v.chunks));
  return v;
}

// ---- barrier over all workgroups --------------------------------------------------------
// Two levels of arrival counters (groups of kBarGroup workgroups, then the groups), each on a
// line of its own; the last arrival of all writes the barrier's number into one release word
// per group, which the group's workgroups poll.  Counters and release words keep counting up
// over barriers and launches (all comparisons are modulo 2^32), so nothing is ever reset.
// all_waves: every wavefront has stores to memory that the others must see; otherwise only
// wavefront 0 has (the others keep their weight loads in flight across the barrier).
// Layout of a.bar in 32-bit words: group g's counter at 64 g, its release word at 64 g + 32,
// the top counter at 64 * groups.
__device__ __forceinline__ void grid_barrier(const StepArgs &a, unsigned epoch, bool all_waves) {
  const int tid = threadIdx.x;
  if (all_waves) {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the stores are acknowledged
    __syncthreads();
  }
  if (tid < 64) {
    __builtin_amdgcn_s_waitcnt(0x0F70);
    if (tid == 0) {
      const unsigned n = gridDim.x, groups = (n + kStepBarGroup - 1) / kStepBarGroup, g = blockIdx.x / kStepBarGroup;
      const unsigned in_group = min((unsigned)kStepBarGroup, n - g * kStepBarGroup);
      const unsigned arrived = __hip_atomic_fetch_add(a.bar_set + 64 * g, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (arrived + 1 == epoch * in_group) {
        const unsigned top = __hip_atomic_fetch_add(a.bar_set + 64 * groups, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (top + 1 == epoch * groups)
          for (unsigned q = 0; q < groups; ++q)
            __hip_atomic_store(a.bar_set + 64 * q + 32, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      int spins = 0;
      while ((int)(__hip_atomic_load(a.bar + 64 * g + 32, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - epoch) < 0) {
        if (++spins > a.spin_limit) {
          *a.error = 1;
          break;
        }
        __builtin_amdgcn_s_sleep(1);
      }
    }
  }
  __syncthreads();
}

// ---- one product -------------------------------------------------------------------------
// What a thread does in one product: float4 column fc of the workgroup's tile, rows r0,
// r0 + RP, ... of the workgroup's split.
struct Geo {
  const float *w;     // the matrix (uniform over the workgroup)
  unsigned off0;      // bytes from w to the thread's first float4 (row k0 + r0, its column)
  unsigned off_max;   // bytes from w to its column in the split's last row: loads beyond are clamped to it
  unsigned step;      // bytes between two of its loads
  int n;              // loads per thread, the same for all threads of the workgroup; 0: no split for it
  int r0, RP, F;
  int k0, nrows;      // the workgroup's rows of W: [k0, k0 + nrows)
  int npad;           // entries of the x slice the threads read: [nrows, npad) must be zero
  int tile, split;
};

#define STEP_GLOBAL(T, p) ((const __attribute__((address_space(1))) T *)(p))

__device__ __forceinline__ int uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }

// Every thread of a workgroup makes the same number of loads (control flow stays uniform):
// threads without a column or beyond the split's rows, and workgroups without a split, load a
// valid address and multiply by the zeros behind the x slice.  (The matrices are smaller
// than 4 GiB: plan_step checks it.)
__device__ __forceinline__ Geo make_geo(const View &v, const StepProduct &pr, const float *w) {
  Geo g;
  const int tid = v.tid;
  g.w = w;
  const int wg = blockIdx.x;
  g.tile = uniform(pr.split_fast ? wg / pr.splits : wg % pr.col_tiles);
  g.split = uniform(pr.split_fast ? wg % pr.splits : wg / pr.col_tiles);
  g.F = pr.F;
  g.RP = uniform(NT / pr.F);
  const int fc = tid % pr.F;
  g.r0 = tid / pr.F;
  const int col = min((g.tile * pr.F + fc) * 4, pr.N - 4);
  const bool has_work = g.split < pr.splits && g.tile < pr.col_tiles;
  const int sp = has_work ? g.split : 0;
  g.nrows = uniform(has_work ? pr.bound[sp + 1] - pr.bound[sp] : 0);
  g.k0 = uniform(has_work ? pr.bound[sp] : 0);
  g.n = uniform((g.nrows + g.RP - 1) / g.RP);
  g.npad = (g.n + 24) * g.RP + (NT - 1) / pr.F + 1;  // the 16 rows ahead and groups of up to 8 rows may run past n
  g.off_max = ((unsigned)(g.k0 + max(g.nrows, 1) - 1) * (unsigned)pr.ldw + (unsigned)col) * 4u;
  g.off0 = min(((unsigned)(g.k0 + g.r0) * (unsigned)pr.ldw + (unsigned)col) * 4u, g.off_max);
  g.step = (unsigned)g.RP * (unsigned)pr.ldw * 4u;
  // The geometry is the same in every block of the stack; without this the compiler computes
  // every load offset of every product once, before the loop over the blocks.
  asm volatile("" : "+v"(g.off0), "+v"(g.off_max), "+v"(g.r0));
  return g;
}

__device__ __forceinline__ f32x4 load_w(const Geo &g, int i, int second_bytes) {
  const unsigned off = min(g.off0 + (unsigned)i * g.step, g.off_max) + (unsigned)second_bytes;
  return __builtin_nontemporal_load(STEP_GLOBAL(f32x4, (const char *)g.w + off));
}

// The first 16 / NACC rows of a thread's share of a product, requested long before they are
// used; in blocks of four rows, as far as the split has rows (a row beyond it would be a load
// of the split's last row again, and thousands of those to a few lines take tens of microseconds).
// second: floats from a gate column to its up column (NACC = 2).
template <int NACC>
__device__ __forceinline__ void issue_prefetch(const Geo &g, int second, f32x4 (&pre)[16]) {
  constexpr int PR = 16 / NACC;
#pragma unroll
  for (int b = 0; b < PR; b += 4)
    if (b < g.n) {
#pragma unroll
      for (int u = b; u < b + 4; ++u)
#pragma unroll
        for (int c = 0; c < NACC; ++c) pre[u * NACC + c] = load_w(g, u, c * second * 4);
    }
}

template <int NACC>
__device__ __forceinline__ void load_group(const Geo &g, int second, int i, f32x4 (&r)[8]) {
  constexpr int U = 8 / NACC;
#pragma unroll
  for (int u = 0; u < U; ++u)
#pragma unroll
    for (int c = 0; c < NACC; ++c) r[u * NACC + c] = load_w(g, i + u, c * second * 4);
}

template <int NACC>
__device__ __forceinline__ void consume_group(const Geo &g, const float *xs, int i, const f32x4 (&r)[8],
                                              f32x4 (&acc)[NACC]) {
  constexpr int U = 8 / NACC;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const float xv = xs[g.r0 + (i + u) * g.RP];
#pragma unroll
    for (int c = 0; c < NACC; ++c) acc[c] += xv * r[u * NACC + c];
  }
}

// acc = this thread's share of xs . W over the workgroup's split; `pre` holds the first rows
// (requested during the previous phase) and receives the first rows of the next product
// before the last rows of this one are used.  xs holds zeros from nrows up to g.npad.
template <int NACC, int NNEXT>
__device__ __forceinline__ void product(const Geo &g, int second, const float *xs, f32x4 (&pre)[16], const Geo &gn,
                                        int second_next, bool prefetch_next, f32x4 (&acc)[NACC]) {
  constexpr int PR = 16 / NACC, U = 8 / NACC;
#pragma unroll
  for (int c = 0; c < NACC; ++c) acc[c] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int n = g.n;
#pragma unroll
  for (int b = 0; b < PR; b += 4)
    if (b < n) {
#pragma unroll
      for (int u = b; u < b + 4; ++u) {
        const float xv = xs[g.r0 + u * g.RP];
#pragma unroll
        for (int c = 0; c < NACC; ++c) acc[c] += xv * pre[u * NACC + c];
      }
    }
  f32x4 ra[8];
  int i = PR;
  if (n > PR) {
    load_group<NACC>(g, second, i, ra);
    for (i += U; i < n; i += U) {
      f32x4 rb[8];
      load_group<NACC>(g, second, i, rb);
      consume_group<NACC>(g, xs, i - U, ra, acc);
#pragma unroll
      for (int u = 0; u < 8; ++u) ra[u] = rb[u];
    }
  }
  if (prefetch_next) issue_prefetch<NNEXT>(gn, second_next, pre);
  if (n > PR) consume_group<NACC>(g, xs, i - U, ra, acc);
}

// Adds the accumulators of the threads that share a column (a fixed tree through LDS) and
// leaves the workgroup's partial in memory: part[split][NACC][N].  Only wavefront 0 stores.
template <int NACC>
__device__ __forceinline__ void reduce_store(const View &v, const Geo &g, const StepProduct &pr,
                                             const f32x4 (&acc)[NACC], float *scr, float *part) {
  const int tid = v.tid, F = g.F, RP = g.RP;
  const int fc = tid % F, r0 = tid / F;
  f32x4 *red = (f32x4 *)scr;  // [NACC][RP][F]
  if (g.nrows > 0) {
    if (r0 < RP) {
#pragma unroll
      for (int c = 0; c < NACC; ++c) red[(c * RP + r0) * F + fc] = acc[c];
    }
    int n = RP, s = 1;
    while (s < RP) s <<= 1;
    for (s >>= 1; s > 0; s >>= 1) {
      __syncthreads();
      if (r0 < s && r0 + s < n) {
#pragma unroll
        for (int c = 0; c < NACC; ++c) red[(c * RP + r0) * F + fc] += red[(c * RP + r0 + s) * F + fc];
      }
      n = s;
    }
    __syncthreads();
    if (tid < NACC * F) {  // NACC * F <= 64
      const int c = tid / F, f = tid % F;
      const int col = (g.tile * F + f) * 4;
      if (col < pr.N) coherent_store4(part + ((long long)(g.split * NACC + c) * pr.N + col), red[(c * RP) * F + f]);
    }
  }
}

// ---- the residual stream and the x slices ---------------------------------------------------
// xfull[i] += sum over splits of part[s][i], for all i < d; every workgroup does all of it.
// Returns this thread's share of the sum of squares of the new xfull (for the norm that follows).
__device__ __forceinline__ double add_partials(const View &vw, float *xfull, const float *part, int splits) {
  const int d = vw.d;
  double sq = 0.0;
  for (int i0 = 0; i0 < d; i0 += 4 * NT) {
    float sum[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < splits; s0 += 8) {
      float v[4][8];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int i = i0 + e * NT + vw.tid;
#pragma unroll
        for (int u = 0; u < 8; ++u)
          v[e][u] = (i < d && s0 + u < splits) ? part_load(part + (long long)(s0 + u) * d + i) : 0.f;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int u = 0; u < 8; ++u) sum[e] += v[e][u];
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int i = i0 + e * NT + vw.tid;
      if (i < d) {
        const float x = (float)((double)xfull[i] + (double)sum[e]);  // simple_matrix.cr:39-48
        xfull[i] = x;
        sq += (double)x * (double)x;
      }
    }
  }
  return sq;
}

// This thread's share of the sum of squares of xfull, as add_partials returns it.
__device__ __forceinline__ double local_sumsq(const View &v, const float *xfull) {
  double sq = 0.0;
  for (int i = v.tid; i < v.d; i += NT) sq += (double)xfull[i] * (double)xfull[i];
  return sq;
}

// The zeros behind a workgroup's x slice (the caller's next barrier publishes them).
__device__ __forceinline__ void zero_tail(const View &v, const Geo &g, float *xs) {
  for (int t = g.nrows + v.tid; t < g.npad; t += NT) xs[t] = 0.f;
}

// xs[t] = RMSNorm(xfull)[k0 + t] for t < nrows (rms_norm.cr:18-37, fp64 as there); sq = this
// thread's share of the sum of squares (the barrier inside also publishes the caller's xfull).
__device__ __forceinline__ void norm_slice(const View &v, double sq, const float *xfull, const float *gamma, double eps,
                                           int k0, int nrows, float *xs, double *red_d) {
  const int tid = v.tid, d = v.d;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) sq += __shfl_xor(sq, o);
  if ((tid & 63) == 0) red_d[tid >> 6] = sq;
  __syncthreads();
  double total = 0.0;
#pragma unroll
  for (int w = 0; w < NW; ++w) total += red_d[w];
  const double rms = sqrt(total / (double)d + eps);
  for (int t = tid; t < nrows; t += NT) {
    const int k = k0 + t;
    xs[t] = (float)(((double)xfull[k] / rms) * (double)(gamma ? gamma[k] : 1.f));
  }
  __syncthreads();
}

// xs[t] = silu(gate[k0 + t]) * up[k0 + t], gate and up summed over the splits of the
// gate | up product: part[s][2][ff].
__device__ __forceinline__ void hidden_slice(const View &v, const float *part, int splits, int k0, int nrows,
                                             float *xs) {
  const int ff = v.ff;
  for (int t0 = 0; t0 < nrows; t0 += 4 * NT) {
    float gate[4] = {0.f, 0.f, 0.f, 0.f}, up[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < splits; s0 += 4) {
      float vg[4][4], vu[4][4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int t = t0 + e * NT + v.tid;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const bool on = t < nrows && s0 + u < splits;
          const float *q = part + (long long)(s0 + u) * 2 * ff + k0 + t;
          vg[e][u] = on ? part_load(q) : 0.f;
          vu[e][u] = on ? part_load(q + ff) : 0.f;
        }
      }
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          gate[e] += vg[e][u];
          up[e] += vu[e][u];
        }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int t = t0 + e * NT + v.tid;
      if (t < nrows) xs[t] = swiglu1(gate[e], up[e]);
    }
  }
  __syncthreads();
}

// ---- attention ------------------------------------------------------------------------------
// Attention of the new row's query heads of kv head c over keys [key0, key1) (key `pos` is the
// new row itself).  The group's q heads, k and v come from the q|k|v partials (bias, QK-norm
// and RoPE with the arithmetic of prep_rows_kernel: llama_block.cr:256-286, 332-344); with
// `append` the new k and v rows also go to the cache (283-286; read by later steps only).
// Every wavefront streams keys with an online softmax per head of the group; what it leaves
// in LDS, wm[wavefront][head][hd + 4] = (O unnormalised, max, sum), is merged by the caller.
template <int GQ, bool TRACE>
__device__ __forceinline__ void attention_group(const View &v, const StepArgs &a, const StepLayer &L, float *scr, int c,
                                                int key0, int key1, bool append) {
  const int tid = v.tid, lane = tid & 63, wave = uniform(tid >> 6);
  const int hd = v.hd, KV = v.KV, pos = v.pos, half = hd >> 1;
  float *raw = scr;                   // [(GQ + 2)][hd]: the group's q heads, k, v as the product left them
  float *qs = raw + (GQ + 2) * hd;    // [GQ][hd] rotated
  float *kn = qs + GQ * hd;           // [hd] rotated new key
  float *vn = kn + hd;                // [hd]
  float *wm = vn + hd;                // [NW][GQ][hd + 4]
  const int q_dim = a.H * hd, kv_dim = KV * hd, wide = q_dim + 2 * kv_dim;
  const int splits = a.qkv.splits;
  for (int t0 = 0; t0 < (GQ + 2) * hd; t0 += NT) {
    const int t = min(t0 + tid, (GQ + 2) * hd - 1);
    const int row = t / hd, e = t - row * hd;
    const int col = row < GQ ? (c * GQ + row) * hd + e : (row == GQ ? q_dim : q_dim + kv_dim) + c * hd + e;
    float sum = 0.f;
    for (int s0 = 0; s0 < splits; s0 += 8) {
      float pv[8];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        pv[u] = part_load(a.qkv_part + (long long)min(s0 + u, splits - 1) * wide + col);
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (s0 + u < splits) sum += pv[u];
    }
    if (t0 + tid < (GQ + 2) * hd) raw[t] = sum;
  }
  __syncthreads();
  for (int row = wave; row < GQ + 2; row += NW) {
    const bool act = lane < half;
    const int i = act ? lane : 0;
    float x0 = raw[row * hd + i], x1 = raw[row * hd + i + half];
    const float *bias = row < GQ ? (L.b_q ? L.b_q + (c * GQ + row) * hd : nullptr)
                                 : (row == GQ ? (L.b_k ? L.b_k + c * hd : nullptr) : (L.b_v ? L.b_v + c * hd : nullptr));
    if (bias) {
      x0 = x0 + bias[i];
      x1 = x1 + bias[i + half];
    }
    float y0 = x0, y1 = x1;
    if (row <= GQ) {
      const float *w = row < GQ ? L.q_norm : L.k_norm;
      const float w0 = w ? w[i] : 1.0f, w1 = w ? w[i + half] : 1.0f;
      const float2 cs = L.rope_tab[(long long)pos * half + i];
      norm_rotate_pair(x0, x1, w != nullptr, w0, w1, a.qk_eps, hd, half, cs, y0, y1);
    }
    float *dst = row < GQ ? qs + row * hd : (row == GQ ? kn : vn);
    if (act) {
      dst[i] = y0;
      dst[i + half] = y1;
      if (append && row >= GQ) {
        float *cache = (row == GQ ? L.kc : L.vc) + ((long long)c * L.cap + pos) * hd;
        cache[i] = y0;
        cache[i + half] = y1;
      }
    }
  }
  __syncthreads();

  const int LPK = hd >> 2, KPI = 64 / LPK;  // lanes per key, keys per load instruction
  const int ks = lane / LPK, f4 = lane - ks * LPK;
  const int stride = NW * KPI;
  f32x4 q4[GQ], o[GQ];
  float m[GQ], l[GQ];
#pragma unroll
  for (int h = 0; h < GQ; ++h) {
    q4[h] = ((const f32x4 *)qs)[h * LPK + f4];
    o[h] = f32x4{0.f, 0.f, 0.f, 0.f};
    m[h] = -INFINITY;
    l[h] = 0.f;
  }
  const float *kbase = L.kc + (long long)c * L.cap * hd + f4 * 4;
  const float *vbase = L.vc + (long long)c * L.cap * hd + f4 * 4;
  const f32x4 kn4 = ((const f32x4 *)kn)[f4], vn4 = ((const f32x4 *)vn)[f4];
  auto fetch = [&](int kb, f32x4 &k4, f32x4 &v4) {
    const int key = kb + ks;
    const long long row = (key < key1 && key < pos) ? key : 0;  // row 0 always exists; masked below
    k4 = __builtin_nontemporal_load(STEP_GLOBAL(f32x4, kbase + row * hd));
    v4 = __builtin_nontemporal_load(STEP_GLOBAL(f32x4, vbase + row * hd));
  };
  auto visit = [&](int kb, f32x4 k4, f32x4 v4) {
    const int key = kb + ks;
    const bool valid = key < key1;
    if (key == pos) {
      k4 = kn4;
      v4 = vn4;
    }
#pragma unroll
    for (int h = 0; h < GQ; ++h) {
      float s = (k4.x * q4[h].x + k4.y * q4[h].y) + (k4.z * q4[h].z + k4.w * q4[h].w);
      for (int off = LPK >> 1; off > 0; off >>= 1) s += __shfl_xor(s, off);
      s *= a.scale;
      if (valid) {
        const float mn = fmaxf(m[h], s);
        const float alpha = __expf(m[h] - mn), p = __expf(s - mn);  // m = -inf: alpha = 0
        l[h] = l[h] * alpha + p;
        o[h] = o[h] * alpha + p * v4;
        m[h] = mn;
      }
    }
  };
  // D key slots of loads in flight per wavefront (fewer when the group's heads fill the registers).
  // Slot i of a wavefront holds keys key0 + (wave + NW i) KPI ...
  constexpr int D = GQ <= 2 ? 4 : 2;
  const int first = key0 + wave * KPI;
  const int n_slots = first < key1 ? (key1 - first + stride - 1) / stride : 0;
  if (n_slots > 0) {
    int nxt = 0;  // next slot to fetch
    auto slot_key = [&](int sl) { return first + sl * stride; };
    f32x4 kq[D], vq[D];
    int kbq[D];
#pragma unroll
    for (int u = 0; u < D; ++u) {
      kbq[u] = u < n_slots ? slot_key(nxt) : key1;  // key1: nothing valid
      fetch(kbq[u], kq[u], vq[u]);
      nxt = nxt + 1 == n_slots ? 0 : nxt + 1;
    }
    for (int done = 0; done < n_slots; done += D) {
      f32x4 kx[D], vx[D];
      int kbx[D];
#pragma unroll
      for (int u = 0; u < D; ++u) {
        kbx[u] = done + D + u < n_slots ? slot_key(nxt) : key1;
        fetch(kbx[u], kx[u], vx[u]);
        nxt = nxt + 1 == n_slots ? 0 : nxt + 1;
      }
#pragma unroll
      for (int u = 0; u < D; ++u) visit(kbq[u], kq[u], vq[u]);
#pragma unroll
      for (int u = 0; u < D; ++u) {
        kq[u] = kx[u];
        vq[u] = vx[u];
        kbq[u] = kbx[u];
      }
    }
  }
  // the key slots of a wavefront
  for (int off = LPK; off < 64; off <<= 1) {
#pragma unroll
    for (int h = 0; h < GQ; ++h) {
      const float m2 = __shfl_xor(m[h], off), l2 = __shfl_xor(l[h], off);
      f32x4 o2;
      o2.x = __shfl_xor(o[h].x, off);
      o2.y = __shfl_xor(o[h].y, off);
      o2.z = __shfl_xor(o[h].z, off);
      o2.w = __shfl_xor(o[h].w, off);
      const float mn = fmaxf(m[h], m2);
      const float a1 = m[h] == -INFINITY ? 0.f : __expf(m[h] - mn), a2 = m2 == -INFINITY ? 0.f : __expf(m2 - mn);
      l[h] = l[h] * a1 + l2 * a2;
      o[h] = o[h] * a1 + o2 * a2;
      m[h] = mn;
    }
  }
  if (lane < LPK) {
#pragma unroll
    for (int h = 0; h < GQ; ++h) {
      float *w = wm + (wave * GQ + h) * (hd + 4);
      ((f32x4 *)w)[f4] = o[h];
      if (lane == 0) {
        w[hd] = m[h];
        w[hd + 1] = l[h];
      }
    }
  }
  __syncthreads();
}

// Element e of head h of the group as the wavefronts left it: (unnormalised O, max, sum) merged.
template <int GQ>
__device__ __forceinline__ void merge_waves(const float *wm, int hd, int h, int e, float &acc, float &mx, float &ls) {
  mx = -INFINITY;
#pragma unroll
  for (int w = 0; w < NW; ++w) mx = fmaxf(mx, wm[(w * GQ + h) * (hd + 4) + hd]);
  acc = 0.f;
  ls = 0.f;
#pragma unroll
  for (int w = 0; w < NW; ++w) {
    const float *p = wm + (w * GQ + h) * (hd + 4);
    const float f = p[hd] == -INFINITY ? 0.f : __expf(p[hd] - mx);
    acc += f * p[e];
    ls += f * p[hd + 1];
  }
}

// Long contexts: a phase of its own.  Workgroup w takes kv head c = w % KV and key chunk
// j = w / KV; the chunk's (max, sum, O) goes to memory, part[c][j][head of the group][hd + 2],
// for merge_attention in the next phase.  Chunk 0 appends the new k and v rows.
template <int GQ, bool TRACE>
__device__ __forceinline__ void attention_phase(const View &v, const StepArgs &a, const StepLayer &L, float *scr) {
  const int hd = v.hd;
  const int c = blockIdx.x % v.KV, j = blockIdx.x / v.KV;
  const int key0 = j * v.ck;
  const int key1 = min(v.pos + 1, key0 + v.ck);
  if (j >= v.chunks || key0 >= key1) return;  // uniform over the workgroup
  attention_group<GQ, TRACE>(v, a, L, scr, c, key0, key1, j == 0);
  const float *wm = scr + (GQ + 2) * hd + GQ * hd + 2 * hd;
  float *part = a.attn_part + ((long long)(c * v.chunks + j) * GQ) * (hd + 2);
  for (int t = v.tid; t < GQ * hd; t += NT) {
    const int h = t / hd, e = t - h * hd;
    float acc, mx, ls;
    merge_waves<GQ>(wm, hd, h, e, acc, mx, ls);
    coherent_store(part + h * (hd + 2) + e, acc);
    if (e == 0) {
      coherent_store(part + h * (hd + 2) + hd, mx);
      coherent_store(part + h * (hd + 2) + hd + 1, ls);
    }
  }
}

// xs[t] = attention output element k0 + t of the new row (t < nrows): the chunks' partials of
// its head merged in chunk order.
template <int GQ>
__device__ __forceinline__ void merge_attention(const View &v, const StepArgs &a, int k0, int nrows, float *xs) {
  const int hd = v.hd;
  const int chunks = (v.pos + v.ck) / v.ck;  // ceil((pos + 1) / ck)
  const long long cstride = (long long)GQ * (hd + 2);
  for (int t0 = 0; t0 < nrows; t0 += NT) {
    const int t = t0 + v.tid;
    const int eg = k0 + min(t, nrows - 1), head = eg / hd, e = eg - head * hd;
    const int c = head / GQ, h = head - c * GQ;
    const float *base = a.attn_part + ((long long)c * v.chunks * GQ + h) * (hd + 2);
    float mx = -INFINITY, acc = 0.f, ls = 0.f;
    for (int j0 = 0; j0 < chunks; j0 += 8) {
      float vm[8], vl[8], vo[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const float *p = base + (long long)min(j0 + u, chunks - 1) * cstride;
        vm[u] = part_load(p + hd);
        vl[u] = part_load(p + hd + 1);
        vo[u] = part_load(p + e);
      }
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (j0 + u < chunks) {
          const float mn = fmaxf(mx, vm[u]);
          const float a1 = mx == -INFINITY ? 0.f : __expf(mx - mn), a2 = __expf(vm[u] - mn);
          acc = acc * a1 + vo[u] * a2;
          ls = ls * a1 + vl[u] * a2;
          mx = mn;
        }
    }
    if (t < nrows) xs[t] = acc / ls;
  }
  __syncthreads();
}

template <int GQ, bool TRACE>
__global__ __launch_bounds__(NT) void llama_step_kernel(StepArgs a) {
  extern __shared__ __align__(16) float lds[];
  __shared__ double red_d[NW];
  float *xfull = lds;                    // the residual stream
  float *xs = xfull + ((a.d + 3) & ~3);  // this workgroup's slice of a product's x
  float *scr = xs + kStepMaxSlice + kStepSlicePad;  // reductions and the attention phase
  unsigned epoch = a.epoch0;
  // wavefront 0 makes the stores and the arrival of its workgroup: loads it had requested before would
  // hold both up (memory operations of a wavefront complete in order), so it requests its share after the barrier
  const bool wave0 = uniform(threadIdx.x >> 6) == 0;
  const bool ahead = !wave0, behind = wave0;
  f32x4 pre[16];
  f32x4 acc1[1], acc2[2];
  STEP_TRACE(0);
  Geo g_qkv;
  {
    const View v = fresh_view(a);
    g_qkv = make_geo(v, a.qkv, a.layers[0].w_qkv);
    issue_prefetch<1>(g_qkv, 0, pre);
    const int tok = *a.token;  // embedding_layer.cr:129-153
    for (int i = v.tid; i < v.d; i += NT) xfull[i] = a.embedding[(long long)tok * v.d + i];
    __syncthreads();
  }
  for (int li = 0; li < a.n_layers; ++li) {
    const StepLayer &L = a.layers[li];
    const int tb = 1 + kStepTraceSlots * li;
    Geo g_o, g_gu, g_dn;
    {  // 1: q | k | v = RMSNorm(x) W_qkv
      const View v = fresh_view(a);
      double sq;
      if (li > 0) {
        sq = add_partials(v, xfull, a.down_part, a.down.splits);
      } else {
        sq = local_sumsq(v, xfull);
      }
      zero_tail(v, g_qkv, xs);
      norm_slice(v, sq, xfull, L.norm1, a.eps, g_qkv.k0, g_qkv.nrows, xs, red_d);
      STEP_TRACE(tb + 0);
      g_o = make_geo(v, a.wo, L.w_o);
      product<1, 1>(g_qkv, 0, xs, pre, g_o, 0, ahead, acc1);
      STEP_TRACE(tb + 17);
      reduce_store<1>(v, g_qkv, a.qkv, acc1, scr, a.qkv_part);
      STEP_TRACE(tb + 1);
      grid_barrier(a, ++epoch, false);
      if (behind) issue_prefetch<1>(g_o, 0, pre);
    }
    {  // 2: attention over the cache and the new row
      const View v = fresh_view(a);
      STEP_TRACE(tb + 2);
      attention_phase<GQ, TRACE>(v, a, L, scr);
      STEP_TRACE(tb + 3);
      grid_barrier(a, ++epoch, true);
    }
    {  // 3: h = x + attention W_o
      const View v = fresh_view(a);
      STEP_TRACE(tb + 4);
      zero_tail(v, g_o, xs);
      merge_attention<GQ>(v, a, g_o.k0, g_o.nrows, xs);
      STEP_TRACE(tb + 13);
      g_gu = make_geo(v, a.gu, L.w_gu);
      product<1, 2>(g_o, 0, xs, pre, g_gu, v.ff, ahead, acc1);
      STEP_TRACE(tb + 14);
      reduce_store<1>(v, g_o, a.wo, acc1, scr, a.o_part);
      STEP_TRACE(tb + 5);
      grid_barrier(a, ++epoch, false);
      if (behind) issue_prefetch<2>(g_gu, a.ff, pre);
    }
    {  // 4: hidden = silu(RMSNorm(h) W_gate) * (RMSNorm(h) W_up)
      const View v = fresh_view(a);
      STEP_TRACE(tb + 6);
      const double sq = add_partials(v, xfull, a.o_part, a.wo.splits);
      STEP_TRACE(tb + 10);
      zero_tail(v, g_gu, xs);
      norm_slice(v, sq, xfull, L.norm2, a.eps, g_gu.k0, g_gu.nrows, xs, red_d);
      STEP_TRACE(tb + 11);
      g_dn = make_geo(v, a.down, L.w_down);
      product<2, 1>(g_gu, v.ff, xs, pre, g_dn, 0, ahead, acc2);
      STEP_TRACE(tb + 12);
      reduce_store<2>(v, g_gu, a.gu, acc2, scr, a.gu_part);
      STEP_TRACE(tb + 7);
      grid_barrier(a, ++epoch, false);
      if (behind) issue_prefetch<1>(g_dn, 0, pre);
    }
    {  // 5: x = h + hidden W_down
      const View v = fresh_view(a);
      STEP_TRACE(tb + 8);
      zero_tail(v, g_dn, xs);
      hidden_slice(v, a.gu_part, a.gu.splits, g_dn.k0, g_dn.nrows, xs);
      STEP_TRACE(tb + 15);
      const bool last = li + 1 == a.n_layers;
      g_qkv = make_geo(v, a.qkv, a.layers[last ? li : li + 1].w_qkv);
      product<1, 1>(g_dn, 0, xs, pre, g_qkv, 0, !last && ahead, acc1);  // nothing follows the last block: no loads ahead
      STEP_TRACE(tb + 16);
      reduce_store<1>(v, g_dn, a.down, acc1, scr, a.down_part);
      STEP_TRACE(tb + 9);
      grid_barrier(a, ++epoch, false);
      if (behind && !last) issue_prefetch<1>(g_qkv, 0, pre);
    }
  }
  if (blockIdx.x == 0) {
    const View v = fresh_view(a);
    add_partials(v, xfull, a.down_part, a.down.splits);
    __syncthreads();
    for (int i = v.tid; i < v.d; i += NT) a.x_out[i] = xfull[i];
  }
}

// Relative streaming speed of the eight XCDs (thousandths), for the row shares of the splits: a
// tuning knob.  With a split kept on fixed XCDs equal shares measured best.
const int *xcd_speeds() {
  static int speed[8] = {1000, 1000, 1000, 1000, 1000, 1000, 1000, 1000};
  static const bool init = [] {
    if (const char *env = getenv("SHAINET_HIP_STEP_XCD_SPEEDS")) {
      int v[8];
      if (sscanf(env, "%d,%d,%d,%d,%d,%d,%d,%d", v, v + 1, v + 2, v + 3, v + 4, v + 5, v + 6, v + 7) == 8) {
        bool ok = true;
        for (int i = 0; i < 8; ++i) ok = ok && v[i] >= 100 && v[i] <= 10000;
        if (ok)
          for (int i = 0; i < 8; ++i) speed[i] = v[i];
      }
    }
    return true;
  }();
  (void)init;
  return speed;
}

// One product's cut for n_wgs workgroups.  All workgroups stream at once, so a product takes as
// long as its busiest thread has loads: the cut with the fewest loads per thread wins; among
// equals one whose splits stay on fixed XCDs (their row shares then follow the XCDs' speed),
// then the one with the fewest splits (fewer partials to add up).  forced_cw: 0, or the tile width.
bool plan_product(StepProduct &p, int K, int N, int ldw, int nacc, int n_wgs, int forced_cw) {
  static const int widths[] = {256, 192, 128, 96, 64, 32, 16};
  double best = -1.0;
  for (int cw : widths) {
    if (forced_cw > 0 && cw != forced_cw) continue;
    const int F = cw / 4;
    if (nacc * F > 64) continue;
    const int col_tiles = (N + cw - 1) / cw;
    if (col_tiles > n_wgs) continue;
    const int RP = NT / F;
    int splits = n_wgs / col_tiles;
    const int max_splits = K / RP > 1 ? K / RP : 1;  // a split of less than one pass of rows is no use
    if (splits > max_splits) splits = max_splits;
    if (splits > kStepMaxSplits) splits = kStepMaxSplits;
    int rps = (K + splits - 1) / splits;
    if (rps > kStepMaxSlice) continue;
    splits = (K + rps - 1) / rps;
    const int loads = (rps + RP - 1) / RP;
    // splits of 2, 4, 8 or 16 with the split as the fast index keep a split on XCDs of one parity
    const bool aligned = n_wgs % 8 == 0 && (splits == 2 || splits == 4 || splits == 8 || splits == 16);
    const double score = (cw >= 32 ? 1.0 : 0.8) / (double)loads + (aligned ? 2e-5 : 0.0) - 1e-6 * splits;
    if (score > best) {
      best = score;
      p.K = K;
      p.N = N;
      p.ldw = ldw;
      p.F = F;
      p.col_tiles = col_tiles;
      p.splits = splits;
      p.split_fast = aligned ? 1 : 0;
      const int *speed = xcd_speeds();
      double total = 0.0, share[kStepMaxSplits];
      for (int s = 0; s < splits; ++s) {
        share[s] = 1.0;
        if (aligned) {  // split s runs on the XCDs x with x % splits == s % 8 ... (workgroup index = tile * splits + s)
          share[s] = 0.0;
          int cnt = 0;
          for (int x = 0; x < 8; ++x)
            if (x % (splits < 8 ? splits : 8) == s % 8 % (splits < 8 ? splits : 8)) {
              share[s] += speed[x];
              ++cnt;
            }
          share[s] /= cnt;
        }
        total += share[s];
      }
      double acc = 0.0;
      p.bound[0] = 0;
      for (int s = 0; s < splits; ++s) {
        acc += share[s];
        int b = (int)((double)K * acc / total + 0.5);
        if (b < p.bound[s]) b = p.bound[s];
        if (b > K || s == splits - 1) b = K;
        p.bound[s + 1] = b;
      }
      for (int s = splits + 1; s <= kStepMaxSplits; ++s) p.bound[s] = K;
    }
  }
  if (best <= 0.0) return false;
  for (int s = 0; s < p.splits; ++s)
    if (p.bound[s + 1] - p.bound[s] > kStepMaxSlice) return false;
  return true;
}

}  // namespace

StepPlan plan_step(int d, int H, int KV, int hd, int ff, int n_wgs) {
  StepPlan p = {};
  p.ok = false;
  if (d < 4 || (d & 3) || ff < 4 || (ff & 3) || hd < 4 || hd > 128 || (hd & (hd - 1)) || KV < 1 || H < KV ||
      H % KV || n_wgs < KV || n_wgs < 1 || n_wgs > 1024 || d > 16384)
    return p;
  const int g = H / KV;
  if (g != 1 && g != 2 && g != 4 && g != 8) return p;
  const int q_dim = H * hd, kv_dim = KV * hd, wide = q_dim + 2 * kv_dim;
  // tuning knob: the column-tile widths (floats) of the four products, e.g. "96,64,32,64"; 0 = planner's choice
  static int forced[4] = {0, 0, 0, 0};
  static const bool have_env = [] {
    if (const char *env = getenv("SHAINET_HIP_STEP_TILE_WIDTHS")) sscanf(env, "%d,%d,%d,%d", forced, forced + 1, forced + 2, forced + 3);
    return true;
  }();
  (void)have_env;
  if (!plan_product(p.qkv, d, wide, wide, 1, n_wgs, forced[0]) || !plan_product(p.wo, q_dim, d, d, 1, n_wgs, forced[1]) ||
      !plan_product(p.gu, d, ff, 2 * ff, 2, n_wgs, forced[2]) || !plan_product(p.down, ff, d, d, 1, n_wgs, forced[3]))
    return p;
  p.attn_chunks = n_wgs / KV;
  const size_t attn_scr = (size_t)(g + 2) * hd + (size_t)g * hd + 2 * hd + (size_t)NW * g * (hd + 4);
  size_t scr = (size_t)NT * 2 * 4;
  if (attn_scr > scr) scr = attn_scr;
  size_t lds = ((size_t)((d + 3) & ~3) + kStepMaxSlice + kStepSlicePad + scr) * sizeof(float);
  const size_t one_per_unit = (size_t)160 * 1024 / 2 + 256;  // a second workgroup would not fit the compute unit
  if (lds < one_per_unit) lds = one_per_unit;
  if (lds > (size_t)150 * 1024) return p;
  p.lds_bytes = lds;
  p.qkv_floats = (size_t)p.qkv.splits * wide;
  p.attn_floats = (size_t)KV * p.attn_chunks * g * (hd + 2);
  p.o_floats = (size_t)p.wo.splits * d;
  p.gu_floats = (size_t)p.gu.splits * 2 * ff;
  p.down_floats = (size_t)p.down.splits * d;
  p.ok = true;
  return p;
}

int step_keys_per_chunk(const StepPlan &p, int pos) {
  const int n_keys = pos + 1;
  int ck = (n_keys + p.attn_chunks - 1) / p.attn_chunks;
  if (ck < 32) ck = 32;  // a chunk keeps every wavefront of its workgroup busy for at least one load
  return ck;
}

hipError_t launch_step(const StepArgs &a, int n_wgs, size_t lds_bytes, hipStream_t stream) {
  if (!a.layers || a.n_layers < 1 || !a.embedding || !a.token || !a.x_out || !a.qkv_part || !a.attn_part ||
      !a.o_part || !a.gu_part || !a.down_part || !a.bar || !a.bar_set || !a.error || a.pos < 0 || a.attn_ck < 1 ||
      a.attn_chunks < 1 || (long long)a.attn_chunks * a.KV > n_wgs ||
      (a.pos + a.attn_ck) / a.attn_ck > a.attn_chunks)
    return hipErrorInvalidValue;
  const int g = a.H / a.KV;
  dim3 grid((unsigned)n_wgs), block(NT);
#define SHAINET_LAUNCH_STEP(GQ_)                                                                   \
  do {                                                                                             \
    if (a.trace)                                                                                   \
      hipLaunchKernelGGL((llama_step_kernel<GQ_, true>), grid, block, lds_bytes, stream, a);       \
    else                                                                                           \
      hipLaunchKernelGGL((llama_step_kernel<GQ_, false>), grid, block, lds_bytes, stream, a);      \
  } while (0)
  switch (g) {
    case 1: SHAINET_LAUNCH_STEP(1); break;
    case 2: SHAINET_LAUNCH_STEP(2); break;
    case 4: SHAINET_LAUNCH_STEP(4); break;
    case 8: SHAINET_LAUNCH_STEP(8); break;
    default: return hipErrorInvalidValue;
  }
#undef SHAINET_LAUNCH_STEP
  return hipGetLastError();
}

}  // namespace shainet
