// The kernels of a LlamaBlock around attention, and of the steps after the last
// block, for gfx950.  They restate the reference's host loops with its number
// types, so that results agree with its CPU path to the last bit or two:
//   RMSNorm#forward        rms_norm.cr:18-37   sum of squares, the root and the
//                                              scaling in fp64, one rounding to fp32
//   SimpleMatrix#+         simple_matrix.cr:39-48   fp64 add, rounded to fp32
//   SwiGLUFF#forward       swiglu_ff.cr:76-91  g / (1 + exp(-g)) * up in fp64
//   EmbeddingLayer#embed_cpu   embedding_layer.cr:129-153   row gather
//   Sampler                text/sampler.cr:38-120   greedy, repetition penalty, top-k
// All of them are bound by HBM (or by latency at decode sizes); fp64 arithmetic is
// free at these intensities on this part.
#include "block_kernels.hpp"

#include <math.h>
#include <stdint.h>

namespace shainet {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

// One workgroup per row.
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float *__restrict__ x, long long x_stride,
                                                      const float *__restrict__ gamma, float *__restrict__ out,
                                                      int cols, double eps) {
  __shared__ double red[4];
  const float *xr = x + (long long)blockIdx.x * x_stride;
  float *orow = out + (long long)blockIdx.x * cols;
  const bool vec = (cols & 3) == 0 && (x_stride & 3) == 0;
  double sq = 0.0;
  if (vec) {
    for (int j = threadIdx.x * 4; j < cols; j += 1024) {
      const f32x4 v = *(const f32x4 *)(xr + j);
      sq += (double)v.x * (double)v.x + (double)v.y * (double)v.y;
      sq += (double)v.z * (double)v.z + (double)v.w * (double)v.w;
    }
  } else {
    for (int j = threadIdx.x; j < cols; j += 256) sq += (double)xr[j] * (double)xr[j];
  }
  sq = wave_sum(sq);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = sq;
  __syncthreads();
  const double total = (red[0] + red[1]) + (red[2] + red[3]);
  const double rms = sqrt(total / (double)cols + eps);
  if (vec) {
    for (int j = threadIdx.x * 4; j < cols; j += 1024) {
      const f32x4 v = *(const f32x4 *)(xr + j);
      f32x4 gm = {1.f, 1.f, 1.f, 1.f};
      if (gamma) gm = *(const f32x4 *)(gamma + j);
      f32x4 y;
      y.x = (float)(((double)v.x / rms) * (double)gm.x);
      y.y = (float)(((double)v.y / rms) * (double)gm.y);
      y.z = (float)(((double)v.z / rms) * (double)gm.z);
      y.w = (float)(((double)v.w / rms) * (double)gm.w);
      *(f32x4 *)(orow + j) = y;
    }
  } else {
    for (int j = threadIdx.x; j < cols; j += 256)
      orow[j] = (float)(((double)xr[j] / rms) * (double)(gamma ? gamma[j] : 1.f));
  }
}

__global__ __launch_bounds__(256) void add_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                                  float *__restrict__ out, long long n) {
  const long long i = ((long long)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i + 3 < n) {
    const f32x4 x = *(const f32x4 *)(a + i), y = *(const f32x4 *)(b + i);
    f32x4 r;
    r.x = (float)((double)x.x + (double)y.x);
    r.y = (float)((double)x.y + (double)y.y);
    r.z = (float)((double)x.z + (double)y.z);
    r.w = (float)((double)x.w + (double)y.w);
    *(f32x4 *)(out + i) = r;
  } else {
    for (long long j = i; j < n; ++j) out[j] = (float)((double)a[j] + (double)b[j]);
  }
}

__device__ __forceinline__ float swiglu(float gate, float up) {
  const double g = (double)gate;
  return (float)((g / (1.0 + exp(-g))) * (double)up);
}

__global__ __launch_bounds__(256) void swiglu_act_kernel(const float *__restrict__ gate_up, float *__restrict__ hidden,
                                                         int ff) {
  const int r = blockIdx.y;
  const float *gr = gate_up + (long long)r * 2 * ff;
  float *hr = hidden + (long long)r * ff;
  const int j = (blockIdx.x * 256 + threadIdx.x) * 4;
  if (j + 3 < ff && (ff & 3) == 0) {
    const f32x4 g = *(const f32x4 *)(gr + j), u = *(const f32x4 *)(gr + ff + j);
    *(f32x4 *)(hr + j) = f32x4{swiglu(g.x, u.x), swiglu(g.y, u.y), swiglu(g.z, u.z), swiglu(g.w, u.w)};
  } else {
    for (int k = j; k < ff && k < j + 4; ++k) hr[k] = swiglu(gr[k], gr[ff + k]);
  }
}

__global__ __launch_bounds__(256) void embed_kernel(const float *__restrict__ table, const int *__restrict__ tokens,
                                                    float *__restrict__ out, int d_model) {
  const float *src = table + (long long)tokens[blockIdx.x] * d_model;
  float *dst = out + (long long)blockIdx.x * d_model;
  for (int j = threadIdx.x; j < d_model; j += 256) dst[j] = src[j];
}

__global__ __launch_bounds__(256) void add_bias_row_kernel(float *__restrict__ logits, const float *__restrict__ bias,
                                                           int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  // matrix[i, j] += b[0, j] on SimpleMatrix: fp64 add, rounded (network_run.cr:221-225)
  if (i < n) logits[i] = (float)((double)logits[i] + (double)bias[i]);
}

// The reference walks the ids in order and rewrites the logit once per occurrence,
// so an id that repeats is penalised repeatedly; one thread keeps that order.
__global__ void repetition_penalty_kernel(float *logits, int vocab, const int *ids, int n, double p) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  for (int i = 0; i < n; ++i) {
    const int id = ids[i];
    if (id >= 0 && id < vocab) {
      const float v = logits[id];
      logits[id] = (float)(v > 0.f ? (double)v / p : (double)v * p);
    }
  }
}

// ---- top-k ------------------------------------------------------------------
// A candidate is a 64-bit key: the float's bits mapped to an unsigned integer of
// the same order in the high word, ~index in the low word, so that the largest
// key is the largest value and, among equal values, the smallest index.  Key 0
// means "no candidate".
__device__ __forceinline__ unsigned long long make_key(float v, int idx, bool finite_only) {
  if (v != v) return 0ull;
  if (finite_only && (v == INFINITY || v == -INFINITY)) return 0ull;
  unsigned u = __float_as_uint(v);
  u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
  // -0.0 and +0.0 compare equal in the reference (v > x is false both ways)
  if (v == 0.f) u = 0x80000000u;
  return ((unsigned long long)u << 32) | (unsigned)(~(unsigned)idx);
}
__device__ __forceinline__ float key_value(unsigned long long key, const float *logits) {
  return logits[~(unsigned)(key & 0xffffffffu)];
}

__device__ __forceinline__ unsigned long long wave_max(unsigned long long v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const unsigned long long other = __shfl_xor(v, o);
    v = other > v ? other : v;
  }
  return v;
}

constexpr int kTopkChunk = 2048;  // logits per workgroup in the first pass; 8 keys per thread

// k rounds of "take the largest key and retire it" over keys held in registers.
// n_mine keys per thread; writes the k winners (descending) to `dst`.
template <int PER_THREAD>
__device__ __forceinline__ void select_k(unsigned long long (&keys)[PER_THREAD], int k, unsigned long long *dst) {
  __shared__ unsigned long long red[4];
  for (int round = 0; round < k; ++round) {
    unsigned long long best = 0ull;
#pragma unroll
    for (int u = 0; u < PER_THREAD; ++u) best = keys[u] > best ? keys[u] : best;
    best = wave_max(best);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = best;
    __syncthreads();
    unsigned long long w = red[0];
#pragma unroll
    for (int i = 1; i < 4; ++i) w = red[i] > w ? red[i] : w;
    __syncthreads();
    if (threadIdx.x == 0) dst[round] = w;
    if (w == 0ull) {  // nothing left: the remaining rounds are empty too
      for (int r = round + 1 + (int)threadIdx.x; r < k; r += 256) dst[r] = 0ull;
      return;
    }
#pragma unroll
    for (int u = 0; u < PER_THREAD; ++u)
      if (keys[u] == w) keys[u] = 0ull;  // keys are unique (the index is part of them)
  }
}

__global__ __launch_bounds__(256) void topk_chunk_kernel(const float *__restrict__ logits, int vocab, int k,
                                                         int finite_only, unsigned long long *__restrict__ cand) {
  unsigned long long keys[8];
  const int base = blockIdx.x * kTopkChunk;
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const int idx = base + u * 256 + threadIdx.x;
    keys[u] = idx < vocab ? make_key(logits[idx], idx, finite_only != 0) : 0ull;
  }
  select_k<8>(keys, k, cand + (long long)blockIdx.x * k);
}

// One workgroup merges the chunks' candidates (n_cand keys), 2048 at a time, keeping
// the running top-k among them.
__global__ __launch_bounds__(256) void topk_merge_kernel(const float *__restrict__ logits,
                                                         unsigned long long *__restrict__ cand, int n_cand, int k,
                                                         unsigned long long *__restrict__ winners,
                                                         int *__restrict__ out_ids, float *__restrict__ out_vals,
                                                         int *__restrict__ out_count, int fallback_id) {
  // winners[0..k) holds the best so far; each pass selects among them and the next 2048 - 256 candidates
  for (int r = threadIdx.x; r < k; r += 256) winners[r] = 0ull;
  __syncthreads();
  constexpr int kStep = 7 * 256;
  for (int c0 = 0; c0 < n_cand || c0 == 0; c0 += kStep) {
    unsigned long long keys[8];
    keys[0] = (int)threadIdx.x < k ? winners[threadIdx.x] : 0ull;  // k <= 256
#pragma unroll
    for (int u = 1; u < 8; ++u) {
      const int i = c0 + (u - 1) * 256 + threadIdx.x;
      keys[u] = i < n_cand ? cand[i] : 0ull;
    }
    __syncthreads();
    select_k<8>(keys, k, winners);
    __syncthreads();
  }
  int count = 0;
  for (int r = threadIdx.x; r < k; r += 256) {
    const unsigned long long key = winners[r];
    if (key != 0ull) {
      out_ids[r] = (int)(~(unsigned)(key & 0xffffffffu));
      if (out_vals) out_vals[r] = key_value(key, logits);
    } else {
      out_ids[r] = fallback_id;
      if (out_vals) out_vals[r] = 0.f;
    }
  }
  if (threadIdx.x == 0 && out_count) {
    while (count < k && winners[count] != 0ull) ++count;
    *out_count = count;
  }
}

// Sampler#sample after its top-k selection (text/sampler.cr:118-150): the temperature softmax over
// the survivors and the inverse-CDF pick for the uniform draw r, one lane, in the reference's order
// and number types (fp64 throughout).  ids / vals: the selection, descending; *count entries.
__global__ void sample_pick_kernel(const int *__restrict__ ids, const float *__restrict__ vals,
                                   const int *__restrict__ count, double temperature, double r, int *__restrict__ out) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  const int n = *count;
  if (n <= 0) {  // all-NaN row: nothing to sample (sampler.cr:121)
    *out = 0;
    return;
  }
  const double max_val = (double)vals[0] / temperature;  // descending order: element 0 is the maximum
  double sum = 0.0;
  for (int i = 0; i < n; ++i) sum += exp((double)vals[i] / temperature - max_val);
  const double inv_sum = 1.0 / sum;
  double cumulative = 0.0;
  int best = ids[n - 1];
  for (int i = 0; i < n; ++i) {
    cumulative += exp((double)vals[i] / temperature - max_val) * inv_sum;
    if (r <= cumulative) {
      best = ids[i];
      break;
    }
  }
  *out = best;
}

// RoPE.apply (rope.cr:7-33): one lane per (row, pair).  Everything in fp64 as the reference has
// it (Float32 operands widened, `theta ** (2.0 * i / head_dim)`, the angle, Math.cos / Math.sin,
// both products and their difference or sum), rounded once when the result is stored.
__global__ __launch_bounds__(256) void rope_apply_kernel(const float *__restrict__ x, float *__restrict__ out,
                                                         int seq_len, int head_dim, int start_pos, double theta) {
  const int half = head_dim / 2;
  const long long per_row = half + (head_dim & 1);  // the odd trailing column rides along as one more item
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long long)seq_len * per_row) return;
  const int pos = (int)(idx / per_row), i = (int)(idx - (long long)pos * per_row);
  const float *xr = x + (long long)pos * head_dim;
  float *orow = out + (long long)pos * head_dim;
  if (i == half) {
    orow[head_dim - 1] = xr[head_dim - 1];
    return;
  }
  const double freq = 1.0 / pow(theta, 2.0 * (double)i / (double)head_dim);
  const double angle = (double)(pos + start_pos) * freq;
  const double c = cos(angle), s = sin(angle);
  const double x0 = (double)xr[i], x1 = (double)xr[i + half];
  orow[i] = (float)(x0 * c - x1 * s);
  orow[i + half] = (float)(x1 * c + x0 * s);
}

// 32 x 32 tiles through LDS: coalesced on both sides
// (row_scale, nullable: row r of src is multiplied by row_scale[r] on its way)
__global__ __launch_bounds__(256) void transpose_kernel(const float *__restrict__ src, float *__restrict__ dst, int rows,
                                                        int cols, const float *__restrict__ row_scale) {
  __shared__ float tile[32][33];
  const int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  for (int i = ty; i < 32; i += 8)
    if (r0 + i < rows && c0 + tx < cols)
      tile[i][tx] = src[(long long)(r0 + i) * cols + c0 + tx] * (row_scale ? row_scale[r0 + i] : 1.0f);
  __syncthreads();
  for (int i = ty; i < 32; i += 8)
    if (c0 + i < cols && r0 + tx < rows) dst[(long long)(c0 + i) * rows + r0 + tx] = tile[tx][i];
}

__global__ __launch_bounds__(256) void transposed_differ_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                                                int rows, int cols, int *__restrict__ differ) {
  __shared__ unsigned tile[32][33];
  const int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  for (int i = ty; i < 32; i += 8)
    if (r0 + i < rows && c0 + tx < cols) tile[i][tx] = __float_as_uint(a[(long long)(r0 + i) * cols + c0 + tx]);
  __syncthreads();
  bool bad = false;
  for (int i = ty; i < 32; i += 8)
    if (c0 + i < cols && r0 + tx < rows) bad = bad || __float_as_uint(b[(long long)(c0 + i) * rows + r0 + tx]) != tile[tx][i];
  if (bad) *differ = 1;
}

}  // namespace

hipError_t launch_transposed_differ(const float *a, const float *b, int rows, int cols, int *differ, hipStream_t stream) {
  if (!a || !b || !differ || rows < 1 || cols < 1 || (rows + 31) / 32 > 65535) return hipErrorInvalidValue;
  hipLaunchKernelGGL(transposed_differ_kernel, dim3((unsigned)((cols + 31) / 32), (unsigned)((rows + 31) / 32)), dim3(256),
                     0, stream, a, b, rows, cols, differ);
  return hipGetLastError();
}

hipError_t launch_transpose(const float *src, float *dst, int rows, int cols, hipStream_t stream, const float *row_scale) {
  if (!src || !dst || rows < 1 || cols < 1 || (rows + 31) / 32 > 65535) return hipErrorInvalidValue;
  hipLaunchKernelGGL(transpose_kernel, dim3((unsigned)((cols + 31) / 32), (unsigned)((rows + 31) / 32)), dim3(256), 0,
                     stream, src, dst, rows, cols, row_scale);
  return hipGetLastError();
}

hipError_t launch_rmsnorm(const float *x, long long x_stride, const float *gamma, float *out, int rows, int cols,
                          double eps, hipStream_t stream) {
  if (rows < 1 || cols < 1 || x_stride < cols) return hipErrorInvalidValue;
  hipLaunchKernelGGL(rmsnorm_kernel, dim3((unsigned)rows), dim3(256), 0, stream, x, x_stride, gamma, out, cols, eps);
  return hipGetLastError();
}

hipError_t launch_add(const float *a, const float *b, float *out, long long n, hipStream_t stream) {
  if (n < 1) return hipErrorInvalidValue;
  const long long blocks = (n + 1023) / 1024;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  hipLaunchKernelGGL(add_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, a, b, out, n);
  return hipGetLastError();
}

hipError_t launch_swiglu_act(const float *gate_up, float *hidden, int rows, int ff, hipStream_t stream) {
  if (rows < 1 || rows > 65535 || ff < 1) return hipErrorInvalidValue;
  hipLaunchKernelGGL(swiglu_act_kernel, dim3((unsigned)((ff + 1023) / 1024), (unsigned)rows), dim3(256), 0, stream,
                     gate_up, hidden, ff);
  return hipGetLastError();
}

hipError_t launch_embed(const float *table, const int *tokens, float *out, int n_tokens, int d_model,
                        hipStream_t stream) {
  if (n_tokens < 1 || d_model < 1) return hipErrorInvalidValue;
  hipLaunchKernelGGL(embed_kernel, dim3((unsigned)n_tokens), dim3(256), 0, stream, table, tokens, out, d_model);
  return hipGetLastError();
}

hipError_t launch_add_bias_row(float *logits, const float *bias, int n, hipStream_t stream) {
  if (n < 1) return hipErrorInvalidValue;
  hipLaunchKernelGGL(add_bias_row_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, logits, bias, n);
  return hipGetLastError();
}

hipError_t launch_repetition_penalty(float *logits, int vocab, const int *ids, int n, double penalty,
                                     hipStream_t stream) {
  if (n < 1) return hipSuccess;
  hipLaunchKernelGGL(repetition_penalty_kernel, dim3(1), dim3(64), 0, stream, logits, vocab, ids, n, penalty);
  return hipGetLastError();
}

hipError_t launch_rope_apply(const float *x, float *out, int seq_len, int head_dim, int start_pos, double theta,
                             hipStream_t stream) {
  if (!x || !out || seq_len < 0 || head_dim < 1) return hipErrorInvalidValue;
  const long long items = (long long)seq_len * (head_dim / 2 + (head_dim & 1));
  if (items == 0) return hipSuccess;
  if ((items + 255) / 256 > 0x7fffffffLL) return hipErrorInvalidValue;
  hipLaunchKernelGGL(rope_apply_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, stream, x, out, seq_len,
                     head_dim, start_pos, theta);
  return hipGetLastError();
}

hipError_t launch_sample_pick(const int *ids, const float *vals, const int *count, double temperature, double r,
                              int *out, hipStream_t stream) {
  if (!ids || !vals || !count || !out || !(temperature > 0.0)) return hipErrorInvalidValue;
  hipLaunchKernelGGL(sample_pick_kernel, dim3(1), dim3(64), 0, stream, ids, vals, count, temperature, r, out);
  return hipGetLastError();
}

size_t topk_scratch_bytes(int vocab, int k) {
  const size_t chunks = (size_t)(vocab + kTopkChunk - 1) / kTopkChunk;
  return (chunks * k + k) * sizeof(unsigned long long);
}

hipError_t launch_topk(const float *logits, int vocab, int k, bool finite_only, void *scratch, int *out_ids,
                       float *out_vals, int *out_count, hipStream_t stream, int fallback_id) {
  if (vocab < 1 || k < 1 || k > kMaxTopK || !scratch) return hipErrorInvalidValue;
  const int chunks = (vocab + kTopkChunk - 1) / kTopkChunk;
  unsigned long long *cand = (unsigned long long *)scratch;
  unsigned long long *winners = cand + (size_t)chunks * k;
  hipLaunchKernelGGL(topk_chunk_kernel, dim3((unsigned)chunks), dim3(256), 0, stream, logits, vocab, k,
                     finite_only ? 1 : 0, cand);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(topk_merge_kernel, dim3(1), dim3(256), 0, stream, logits, cand, chunks * k, k, winners, out_ids,
                     out_vals, out_count, fallback_id);
  return hipGetLastError();
}

}  // namespace shainet
