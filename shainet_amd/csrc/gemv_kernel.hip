// y[T,N] = x[T,K] * W[K,N] for a few rows (T <= 16), fp32: the Q/K/V/O projections
// of a decode step (llama_block.cr:253-255, 298 with weights in the reference's
// [in, out] layout).  The product is bound by reading W once from HBM, so the
// work is cut along K as well as along N to put enough workgroups in flight: a
// wavefront owns 256 consecutive columns (one float4 per lane, 1 KiB per W row)
// and a run of rows of W; the four wavefronts of a workgroup take four runs and
// add up through LDS; a second kernel adds the workgroups' partial sums in a
// fixed order (no atomics: results do not depend on scheduling).
#include "attn_kernels.hpp"

namespace shainet {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int TT>
__global__ __launch_bounds__(256) void gemv_partial_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                           float *__restrict__ part, int T, int K, int N,
                                                           int rows_per_wave) {
  __shared__ f32x4 red[4][TT][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = blockIdx.x * 256 + lane * 4;
  const int k0 = (blockIdx.y * 4 + wave) * rows_per_wave;
  const int k1 = min(K, k0 + rows_per_wave);
  f32x4 acc[TT];
#pragma unroll
  for (int t = 0; t < TT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  if (col < N) {  // N is a multiple of 4
    const float *wp = w + (long long)k0 * N + col;
    int k = k0;
    for (; k + 4 <= k1; k += 4) {  // four rows of W in flight
      f32x4 r[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) r[u] = *(const f32x4 *)(wp + (long long)u * N);
      wp += 4LL * N;
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int t = 0; t < TT; ++t) {
          const float xv = t < T ? x[(long long)t * K + k + u] : 0.f;  // uniform over the wavefront
          acc[t] += xv * r[u];
        }
    }
    for (; k < k1; ++k) {
      const f32x4 r = *(const f32x4 *)wp;
      wp += N;
#pragma unroll
      for (int t = 0; t < TT; ++t) {
        const float xv = t < T ? x[(long long)t * K + k] : 0.f;
        acc[t] += xv * r;
      }
    }
  }
#pragma unroll
  for (int t = 0; t < TT; ++t) red[wave][t][lane] = acc[t];
  __syncthreads();
  if (wave == 0 && col < N) {
#pragma unroll
    for (int t = 0; t < TT; ++t)
      if (t < T) {
        const f32x4 sum = (red[0][t][lane] + red[1][t][lane]) + (red[2][t][lane] + red[3][t][lane]);
        *(f32x4 *)(part + ((long long)blockIdx.y * T + t) * N + col) = sum;
      }
  }
}

__global__ __launch_bounds__(256) void gemv_reduce_kernel(const float *__restrict__ part, float *__restrict__ y,
                                                          int total, int splits) {
  const int i = blockIdx.x * 256 + threadIdx.x;  // over T*N/4 float4
  if (i >= total) return;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < splits; ++s) acc += ((const f32x4 *)part)[(long long)s * total + i];
  ((f32x4 *)y)[i] = acc;
}

}  // namespace

GemvPlan plan_gemv(int T, int K, int N) {
  GemvPlan p;
  const int col_tiles = (N + 255) / 256;
  // about 1024 workgroups per product, at least 8 rows of W per wavefront
  int splits = (1024 + col_tiles - 1) / col_tiles;
  int rows = (K + 4 * splits - 1) / (4 * splits);
  if (rows < 8) rows = 8;
  splits = (K + 4 * rows - 1) / (4 * rows);
  p.rows_per_wave = rows;
  p.splits = splits;
  p.partial_floats = (size_t)splits * T * N;
  return p;
}

hipError_t launch_gemv(const float *x, const float *w, float *y, float *partials, int T, int K, int N,
                       const GemvPlan &p, hipStream_t stream) {
  if (T < 1 || T > 16 || K < 1 || N < 4 || (N & 3) || !partials) return hipErrorInvalidValue;
  dim3 grid((unsigned)((N + 255) / 256), (unsigned)p.splits);
#define SHAINET_LAUNCH_GEMV(TT_) \
  hipLaunchKernelGGL(gemv_partial_kernel<TT_>, grid, dim3(256), 0, stream, x, w, partials, T, K, N, p.rows_per_wave)
  if (T == 1)
    SHAINET_LAUNCH_GEMV(1);
  else if (T <= 4)
    SHAINET_LAUNCH_GEMV(4);
  else
    SHAINET_LAUNCH_GEMV(16);
#undef SHAINET_LAUNCH_GEMV
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  const int total = T * N / 4;
  hipLaunchKernelGGL(gemv_reduce_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, partials, y,
                     total, p.splits);
  return hipGetLastError();
}

}  // namespace shainet
