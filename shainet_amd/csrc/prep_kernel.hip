// bias -> per-head QK-RMSNorm -> half-split RoPE -> KV-cache append, on the device.
//
// Restates llama_block.cr:256-286 (K) and 332-344 (Q) with the reference's
// number types and evaluation order, so that the rotated Q rows and the cache
// contents are bit-identical to the reference's CPU path:
//   * bias is one fp32 add (llama_block.cr:596);
//   * the sum of squares is fp32, sequential over the head dimension
//     (626-632); the factor is (float)(1.0 / sqrt((double)(ss / hd) + eps)) (633);
//   * v * inv * w[d] are two fp32 products, left to right (636);
//   * cos/sin come from a table built on the host as cosf/sinf((float)pos * freq)
//     (275-277), and x0*c - x1*s, x1*c + x0*s are separately rounded (280-281).
// This file is compiled with -ffp-contract=off: no product may fuse into an add.
#include "attn_kernels.hpp"
#include "prep_math.hpp"

#include <stdint.h>

#pragma clang fp contract(off)

namespace shainet {

namespace {

struct RowRef {
  const float *src, *bias, *w;
  float *dst;
  int pos;
  bool rotate, valid;
};

// Row r of a token: the H query heads, then the KV key heads, then the KV value heads.
__device__ __forceinline__ RowRef locate_row(const PrepArgs &a, const SeqTable &st, const Shape &sh, int token,
                                             int r, int total_tokens) {
  RowRef rr;
  rr.valid = r < sh.H + 2 * sh.KV;
  if (!rr.valid) r = 0;
  int s = token;
  if (total_tokens != st.n_seqs) {  // not one row per sequence: search the prefix sums
    s = 0;
    while (s + 1 < st.n_seqs && token >= st.tok_off[s + 1]) ++s;
  }
  rr.pos = st.start_pos[s] + (token - st.tok_off[s]);
  const int hd = sh.hd, q_dim = sh.H * hd;
  rr.rotate = true;
  if (r < sh.H) {
    rr.src = a.q + (long long)token * a.q_stride + r * hd;
    rr.bias = a.b_q ? a.b_q + r * hd : nullptr;
    rr.w = a.q_norm;
    rr.dst = a.q_rot + (long long)token * q_dim + r * hd;
  } else {
    const bool is_v = (r - sh.H) >= sh.KV;
    const int c = is_v ? r - sh.H - sh.KV : r - sh.H;
    const long long row = (long long)st.slot[s] * sh.seq_stride + ((long long)c * sh.cap + rr.pos) * hd;
    if (is_v) {
      rr.src = a.v + (long long)token * a.v_stride + c * hd;
      rr.bias = a.b_v ? a.b_v + c * hd : nullptr;
      rr.w = nullptr;
      rr.dst = a.vc + row;
      rr.rotate = false;
    } else {
      rr.src = a.k + (long long)token * a.k_stride + c * hd;
      rr.bias = a.b_k ? a.b_k + c * hd : nullptr;
      rr.w = a.k_norm;
      rr.dst = a.kc + row;
    }
  }
  return rr;
}

// Even head_dim up to 128: R head rows per wavefront, lane i < hd/2 owns the pair
// (i, i + hd/2).  All loads of the R rows are issued before any arithmetic.
// DEV: the sequence table is read from *dev (written by the step's plan kernel earlier on the
// stream); a step that the plan kernel marked as skipped writes nothing.
template <int R, bool DEV>
__global__ __launch_bounds__(256) void prep_rows_kernel(PrepArgs a, SeqTable st_arg, Shape sh, int total_tokens,
                                                        const DecodeDevicePlan *__restrict__ dev) {
  if (DEV && dev->skip) return;
  const SeqTable &st = DEV ? dev->st : st_arg;
  const int lane = threadIdx.x & 63;
  const int hd = sh.hd, half = hd >> 1;
  const int token = blockIdx.y;
  const int r0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * R;
  const bool active = lane < half;
  const int i = active ? lane : 0;
  RowRef rr[R];
  float x0[R], x1[R], w0[R], w1[R];
  float2 cs[R];
#pragma unroll
  for (int u = 0; u < R; ++u) {
    rr[u] = locate_row(a, st, sh, token, r0 + u, total_tokens);
    x0[u] = rr[u].src[i];
    x1[u] = rr[u].src[i + half];
    if (rr[u].bias) {
      x0[u] = x0[u] + rr[u].bias[i];
      x1[u] = x1[u] + rr[u].bias[i + half];
    }
    w0[u] = rr[u].w ? rr[u].w[i] : 1.0f;
    w1[u] = rr[u].w ? rr[u].w[i + half] : 1.0f;
    cs[u] = rr[u].rotate ? a.rope_tab[(long long)rr[u].pos * half + i] : float2{1.0f, 0.0f};
  }
#pragma unroll
  for (int u = 0; u < R; ++u) {
    if (!rr[u].valid) continue;  // uniform over the wavefront
    float *dst = rr[u].dst;
    if (!rr[u].rotate) {  // V rows are stored as they are (llama_block.cr:284)
      if (active) {
        dst[i] = x0[u];
        dst[i + half] = x1[u];
      }
      continue;
    }
    float y0, y1;
    norm_rotate_pair(x0[u], x1[u], rr[u].w != nullptr, w0[u], w1[u], a.eps, hd, half, cs[u], y0, y1);
    if (active) {
      dst[i] = y0;
      dst[i + half] = y1;
    }
  }
}

// Many rows without QK-norm (prefill of the Llama shapes): nothing crosses lanes, so a
// lane takes four neighbouring pairs of one head row with 16-byte accesses.  head_dim is
// a multiple of 8 and every row start is 16-byte aligned.  Same products and sums as
// norm_rotate_pair without weights.
__global__ __launch_bounds__(256) void prep_rows_vec_kernel(PrepArgs a, SeqTable st, Shape sh, int total_tokens,
                                                            long long n_items) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= n_items) return;
  const int half = sh.hd >> 1, tpr = half >> 2, rows = sh.H + 2 * sh.KV;
  const int j = (int)(idx % tpr);
  const long long row_g = idx / tpr;
  const int token = (int)(row_g / rows), r = (int)(row_g - (long long)token * rows);
  const RowRef rr = locate_row(a, st, sh, token, r, total_tokens);
  const int i0 = 4 * j;
  float4 x0 = *(const float4 *)(rr.src + i0), x1 = *(const float4 *)(rr.src + half + i0);
  if (rr.bias) {
    const float4 b0 = *(const float4 *)(rr.bias + i0), b1 = *(const float4 *)(rr.bias + half + i0);
    x0 = float4{x0.x + b0.x, x0.y + b0.y, x0.z + b0.z, x0.w + b0.w};
    x1 = float4{x1.x + b1.x, x1.y + b1.y, x1.z + b1.z, x1.w + b1.w};
  }
  if (rr.rotate) {
    const float4 *cs = (const float4 *)(a.rope_tab + (long long)rr.pos * half + i0);
    const float4 cs01 = cs[0], cs23 = cs[1];  // (cos, sin) of pairs i0, i0 + 1 and i0 + 2, i0 + 3
    float4 y0, y1;
#define SHAINET_ROTATE(f, c, s)            \
  {                                        \
    const float p0 = x0.f * c, p1 = x1.f * s, p2 = x1.f * c, p3 = x0.f * s; \
    y0.f = p0 - p1;                        \
    y1.f = p2 + p3;                        \
  }
    SHAINET_ROTATE(x, cs01.x, cs01.y)
    SHAINET_ROTATE(y, cs01.z, cs01.w)
    SHAINET_ROTATE(z, cs23.x, cs23.y)
    SHAINET_ROTATE(w, cs23.z, cs23.w)
#undef SHAINET_ROTATE
    x0 = y0;
    x1 = y1;
  }
  *(float4 *)(rr.dst + i0) = x0;
  *(float4 *)(rr.dst + half + i0) = x1;
}

// Many rows with QK-norm (prefill of the Qwen3 shapes).  The sum of squares of a head row
// must be added up in the reference's order, one fp32 add per element, which leaves a
// wavefront per row waiting on a chain of hd dependent adds (25 us for 20 480 rows of 128).
// Here a workgroup takes ROWS head rows through LDS: all threads load them (bias added),
// then one lane per row walks its row (row stride hd + 1 floats: no bank conflicts), then
// all threads normalise, rotate and store pair by pair with coalesced accesses.  The same
// products and sums as norm_rotate_pair, the same bits.
template <int ROWS>
__global__ __launch_bounds__(256) void prep_rows_norm_kernel(PrepArgs a, SeqTable st, Shape sh, int total_tokens,
                                                             long long n_rows) {
  extern __shared__ float xs[];  // [ROWS][hd + 1]
  __shared__ const float *src_s[ROWS], *bias_s[ROWS], *w_s[ROWS];
  __shared__ float *dst_s[ROWS];
  __shared__ int pos_s[ROWS];
  __shared__ bool rot_s[ROWS];
  __shared__ float inv_s[ROWS];
  const int hd = sh.hd, half = hd >> 1, stride = hd + 1, per_token = sh.H + 2 * sh.KV;
  const long long row0 = (long long)blockIdx.x * ROWS;
  const int t = threadIdx.x;
  if (t < ROWS) {
    const long long row_g = row0 + t;
    RowRef rr;
    rr.src = nullptr;
    if (row_g < n_rows) {
      const int token = (int)(row_g / per_token);
      rr = locate_row(a, st, sh, token, (int)(row_g - (long long)token * per_token), total_tokens);
    }
    src_s[t] = rr.src;
    if (rr.src) {
      bias_s[t] = rr.bias;
      w_s[t] = rr.w;
      dst_s[t] = rr.dst;
      pos_s[t] = rr.pos;
      rot_s[t] = rr.rotate;
    }
  }
  __syncthreads();
  for (int idx = t; idx < ROWS * hd; idx += 256) {
    const int r = idx / hd, d = idx - r * hd;
    const float *src = src_s[r];
    float x = 0.0f;
    if (src) {
      x = src[d];
      const float *bias = bias_s[r];
      if (bias) x = x + bias[d];
    }
    xs[r * stride + d] = x;
  }
  __syncthreads();
  if (t < ROWS && src_s[t] && w_s[t]) {  // llama_block.cr:626-633
    const float *row = xs + t * stride;
    float ss = 0.0f;
#pragma unroll 8
    for (int d = 0; d < hd; ++d) {
      const float v = row[d];
      const float sq = v * v;
      ss = ss + sq;
    }
    const float mean = ss / (float)hd;
    inv_s[t] = (float)(1.0 / sqrt((double)mean + a.eps));
  }
  __syncthreads();
  for (int idx = t; idx < ROWS * half; idx += 256) {
    const int r = idx / half, i = idx - r * half;
    if (!src_s[r]) continue;
    float x0 = xs[r * stride + i], x1 = xs[r * stride + i + half];
    float *dst = dst_s[r];
    if (rot_s[r]) {
      const float *w = w_s[r];
      if (w) {  // 636
        const float inv = inv_s[r];
        x0 = x0 * inv;
        x0 = x0 * w[i];
        x1 = x1 * inv;
        x1 = x1 * w[i + half];
      }
      const float2 cs = a.rope_tab[(long long)pos_s[r] * half + i];
      const float p0 = x0 * cs.x, p1 = x1 * cs.y, p2 = x1 * cs.x, p3 = x0 * cs.y;
      x0 = p0 - p1;
      x1 = p2 + p3;
    }
    dst[i] = x0;
    dst[i + half] = x1;
  }
}

// Any head_dim (odd ones included): one wavefront per head row.
__global__ __launch_bounds__(256) void prep_rows_generic_kernel(PrepArgs a, SeqTable st, Shape sh, int total_tokens) {
  const int lane = threadIdx.x & 63;
  const RowRef rr = locate_row(a, st, sh, blockIdx.y, blockIdx.x * 4 + (threadIdx.x >> 6), total_tokens);
  if (!rr.valid) return;
  const int hd = sh.hd, half = hd >> 1;
  const float *src = rr.src, *bias = rr.bias, *w = rr.w;
  float *dst = rr.dst;
  const int pos = rr.pos;

  if (!rr.rotate) {  // V rows are stored as they are (llama_block.cr:284)
    for (int d = lane; d < hd; d += 64) dst[d] = bias ? src[d] + bias[d] : src[d];
    return;
  }

  float inv = 1.0f;
  if (w) {
    // The sum of squares must run in the reference's order (d ascending, one fp32
    // add per element).  The row is fetched 64 elements per load, and every lane
    // then walks it through lane broadcasts, so all lanes hold the same sum.
    float ss = 0.0f;
    for (int d0 = 0; d0 < hd; d0 += 64) {
      const int d = d0 + lane;
      float x = 0.0f;
      if (d < hd) x = bias ? src[d] + bias[d] : src[d];
      const int n = min(64, hd - d0);
      for (int t = 0; t < n; ++t) {
        const float v = lane_value(x, t);
        const float sq = v * v;
        ss = ss + sq;
      }
    }
    float mean = ss / (float)hd;
    inv = (float)(1.0 / sqrt((double)mean + a.eps));
  }
  for (int i = lane; i < half; i += 64) {
    float x0 = bias ? src[i] + bias[i] : src[i];
    float x1 = bias ? src[i + half] + bias[i + half] : src[i + half];
    if (w) {
      x0 = x0 * inv;
      x0 = x0 * w[i];
      x1 = x1 * inv;
      x1 = x1 * w[i + half];
    }
    const float2 cs = a.rope_tab[(long long)pos * half + i];
    const float p0 = x0 * cs.x, p1 = x1 * cs.y, p2 = x1 * cs.x, p3 = x0 * cs.y;
    dst[i] = p0 - p1;
    dst[i + half] = p2 + p3;
  }
  if ((hd & 1) && lane == 0) dst[hd - 1] = 0.0f;  // Array.new(head_dim, 0.0): an odd last slot stays 0
}

__global__ void legacy_append_kernel(const float *__restrict__ staging, float *__restrict__ kc,
                                     float *__restrict__ vc, int new_tokens, int start_pos, int num_kv_heads,
                                     int head_dim, int capacity) {
  const long long chunk = (long long)new_tokens * head_dim;  // floats per kv head per tensor
  const long long total = chunk * num_kv_heads;
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= 2 * total) return;
  const bool is_v = idx >= total;
  const long long r = is_v ? idx - total : idx;
  const long long kv_h = r / chunk;
  const long long dst = (kv_h * capacity + start_pos) * head_dim + (r - kv_h * chunk);
  (is_v ? vc : kc)[dst] = staging[idx];
}

}  // namespace

hipError_t launch_prep(const PrepArgs &a, const SeqTable &st, const Shape &sh, int total_tokens,
                       hipStream_t stream, const DecodeDevicePlan *dev) {
  if (total_tokens <= 0) return hipSuccess;
  const int rows = sh.H + 2 * sh.KV;
  const bool fast = sh.hd <= 128 && (sh.hd & 1) == 0;
  if (dev) {  // one row per sequence, positions known to the device only
    if (!fast || total_tokens != st.n_seqs || total_tokens > kMaxSeqs) return hipErrorInvalidValue;
    dim3 grid((unsigned)((rows + 3) / 4), (unsigned)total_tokens);
    hipLaunchKernelGGL((prep_rows_kernel<1, true>), grid, dim3(256), 0, stream, a, st, sh, total_tokens, dev);
    return hipGetLastError();
  }
  // few rows (decode): one row per wavefront keeps the latency short; many rows
  // (prefill): four rows per wavefront amortise the load latency
  const int rows_per_wave = fast && (long long)total_tokens * rows >= 8192 ? 4 : 1;
  const int per_wg = 4 * rows_per_wave;
  const auto aligned16 = [](const void *p) { return ((uintptr_t)p & 15) == 0; };
  const bool vec = !a.q_norm && !a.k_norm && (sh.hd & 7) == 0 && (long long)total_tokens * rows >= 8192 &&
                   ((a.q_stride | a.k_stride | a.v_stride) & 3) == 0 && aligned16(a.q) && aligned16(a.k) &&
                   aligned16(a.v) && aligned16(a.q_rot) && aligned16(a.kc) && aligned16(a.vc) && aligned16(a.b_q) &&
                   aligned16(a.b_k) && aligned16(a.b_v) && aligned16(a.rope_tab);
  // (for a decode step's few hundred rows the one-wavefront-per-row kernel is the shorter one: 5.8 against 10 us)
  if (fast && (a.q_norm || a.k_norm) && (long long)total_tokens * rows >= 8192) {
    constexpr int kRows = 16;  // small groups: many workgroups per compute unit hide each other's latencies
    const long long n_rows = (long long)total_tokens * rows;
    const long long blocks = (n_rows + kRows - 1) / kRows;
    if (blocks <= 0x7fffffffLL) {
      const size_t lds = (size_t)kRows * (sh.hd + 1) * sizeof(float);
      hipLaunchKernelGGL(prep_rows_norm_kernel<kRows>, dim3((unsigned)blocks), dim3(256), lds, stream, a, st, sh,
                         total_tokens, n_rows);
      return hipGetLastError();
    }
  }
  if (vec) {
    const long long n_items = (long long)total_tokens * rows * (sh.hd >> 3);
    const long long blocks = (n_items + 255) / 256;
    if (blocks <= 0x7fffffffLL) {
      hipLaunchKernelGGL(prep_rows_vec_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, a, st, sh,
                         total_tokens, n_items);
      return hipGetLastError();
    }
  }
  // blockIdx.y is the token; a launch takes at most 65535 of them
  for (int t0 = 0; t0 < total_tokens; t0 += 65535) {
    const int nt = total_tokens - t0 < 65535 ? total_tokens - t0 : 65535;
    PrepArgs b = a;
    b.q += (long long)t0 * a.q_stride;
    b.k += (long long)t0 * a.k_stride;
    b.v += (long long)t0 * a.v_stride;
    b.q_rot += (long long)t0 * sh.H * sh.hd;
    SeqTable sub = st;
    if (t0) {  // the kernel indexes tokens from 0: shift the prefix sums
      for (int s = 0; s <= st.n_seqs; ++s) sub.tok_off[s] = st.tok_off[s] - t0;
    }
    dim3 grid((unsigned)((rows + per_wg - 1) / per_wg), (unsigned)nt);
    // n_seqs == tokens means one row per sequence (decode) only for the whole call
    const int tt = t0 == 0 && nt == total_tokens ? total_tokens : -1;
    if (!fast)
      hipLaunchKernelGGL(prep_rows_generic_kernel, grid, dim3(256), 0, stream, b, sub, sh, tt);
    else if (rows_per_wave == 4)
      hipLaunchKernelGGL((prep_rows_kernel<4, false>), grid, dim3(256), 0, stream, b, sub, sh, tt, nullptr);
    else
      hipLaunchKernelGGL((prep_rows_kernel<1, false>), grid, dim3(256), 0, stream, b, sub, sh, tt, nullptr);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

hipError_t launch_legacy_append(const float *staging, float *kc, float *vc, int new_tokens, int start_pos,
                                int num_kv_heads, int head_dim, int capacity, hipStream_t stream) {
  const long long total = 2LL * num_kv_heads * new_tokens * head_dim;
  if (total <= 0) return hipSuccess;
  if (start_pos < 0 || start_pos + new_tokens > capacity) return hipErrorInvalidValue;
  const long long blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  hipLaunchKernelGGL(legacy_append_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, staging, kc, vc,
                     new_tokens, start_pos, num_kv_heads, head_dim, capacity);
  return hipGetLastError();
}

}  // namespace shainet
