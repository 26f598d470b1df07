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

#pragma clang fp contract(off)

namespace shainet {

namespace {

// One wavefront per (token, head row): H query rows, KV key rows, KV value rows.
__global__ __launch_bounds__(256) void prep_rows_kernel(PrepArgs a, SeqTable st, Shape sh, int total_tokens) {
  const int lane = threadIdx.x & 63;
  const int rows_per_token = sh.H + 2 * sh.KV;
  const long long item = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= (long long)total_tokens * rows_per_token) return;
  const int token = (int)(item / rows_per_token);
  const int r = (int)(item - (long long)token * rows_per_token);
  int s = 0;
  while (s + 1 < st.n_seqs && token >= st.tok_off[s + 1]) ++s;
  const int pos = st.start_pos[s] + (token - st.tok_off[s]);
  const int hd = sh.hd, half = hd >> 1;
  const int q_dim = sh.H * hd, kv_dim = sh.KV * hd;

  const float *src, *bias, *w;
  float *dst;
  bool rotate = true;
  if (r < sh.H) {
    src = a.q + (long long)token * q_dim + r * hd;
    bias = a.b_q ? a.b_q + r * hd : nullptr;
    w = a.q_norm;
    dst = a.q_rot + (long long)token * q_dim + r * hd;
  } else {
    const int c = (r - sh.H) % sh.KV;
    const bool is_v = (r - sh.H) >= sh.KV;
    const long long row = (long long)st.slot[s] * sh.seq_stride + ((long long)c * sh.cap + pos) * hd;
    if (is_v) {
      src = a.v + (long long)token * kv_dim + c * hd;
      bias = a.b_v ? a.b_v + c * hd : nullptr;
      w = nullptr;
      dst = a.vc + row;
      rotate = false;
    } else {
      src = a.k + (long long)token * kv_dim + c * hd;
      bias = a.b_k ? a.b_k + c * hd : nullptr;
      w = a.k_norm;
      dst = a.kc + row;
    }
  }

  if (!rotate) {  // V rows are stored as they are (llama_block.cr:284)
    for (int d = lane; d < hd; d += 64) dst[d] = bias ? src[d] + bias[d] : src[d];
    return;
  }

  float inv = 1.0f;
  if (w) {
    // The sum of squares must run in the reference's order (d ascending, one fp32
    // add per element).  The row is fetched once, 64 elements per load, and every
    // lane then walks it through lane broadcasts, so all lanes hold the same sum.
    float ss = 0.0f;
    for (int d0 = 0; d0 < hd; d0 += 64) {
      const int d = d0 + lane;
      float x = 0.0f;
      if (d < hd) x = bias ? src[d] + bias[d] : src[d];
      const int n = min(64, hd - d0);
      for (int t = 0; t < n; ++t) {
        const float v = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), t));
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
                       hipStream_t stream) {
  if (total_tokens <= 0) return hipSuccess;
  const long long items = (long long)total_tokens * (sh.H + 2 * sh.KV);
  const long long blocks = (items + 3) / 4;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  hipLaunchKernelGGL(prep_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, a, st, sh, total_tokens);
  return hipGetLastError();
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
