// Plain streaming kernels of known size.  They calibrate what the HBM counters of
// rocprofv3 (FETCH_SIZE, WRITE_SIZE) read per byte moved and what bandwidth a
// perfectly coalesced stream reaches on the device, the yardsticks the attention
// kernels' traffic and bandwidth figures are compared with.  A loop of nothing but
// fp32 MFMAs does the same for the matrix cores: the rate they sustain at the clock
// the device holds under that load, which the prefill kernels are compared with.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <algorithm>
#include <vector>

#include "../../include/shainet_hip_attn.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void copy_f32x4_kernel(const f32x4 *__restrict__ src, f32x4 *__restrict__ dst,
                                                         long long n4) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) dst[i] = src[i];
}

// Reads everything (non-temporal loads, as the kernels that stream once through their data do:
// 10 % faster than plain loads on buffers far larger than the caches), writes one float per workgroup.
__global__ __launch_bounds__(256) void read_f32x4_kernel(const f32x4 *__restrict__ src, float *__restrict__ sink,
                                                         long long n4) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  for (; i + 3 * stride < n4; i += 4 * stride) {
    const f32x4 a = __builtin_nontemporal_load(src + i), b = __builtin_nontemporal_load(src + i + stride),
                c = __builtin_nontemporal_load(src + i + 2 * stride), d = __builtin_nontemporal_load(src + i + 3 * stride);
    acc += (a + b) + (c + d);
  }
  for (; i < n4; i += stride) acc += __builtin_nontemporal_load(src + i);
  float s = (acc.x + acc.y) + (acc.z + acc.w);
  for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
  if ((threadIdx.x & 63) == 0) atomicAdd(&sink[blockIdx.x], s);
}

typedef float f32x16 __attribute__((ext_vector_type(16)));

// Every wavefront issues `iters` rounds of four independent v_mfma_f32_32x32x2_f32 (four
// accumulators, so no instruction waits for the one before it) and folds the accumulators
// into one float per lane so that the work cannot be dropped.
__global__ __launch_bounds__(512, 1) void mfma_f32_loop_kernel(float *__restrict__ sink, int iters, float a0, float b0) {
  f32x16 acc[4];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;
  const float a = a0 + 1e-6f * threadIdx.x, b = b0;
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int t = 0; t < 4; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[t], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[t][r];
  sink[(long long)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// One workgroup of `lanes` lanes that does nothing: what a launch costs with no work in it.
__global__ void empty_kernel(int *never) {
  if (never && threadIdx.x == 12345) *never = 1;
}

}  // namespace

extern "C" {

int shainet_hip_stream_copy_f32(const float *src, float *dst, long long n, int workgroups, void *stream) {
  if (!src || !dst || n < 0 || (n & 3) || workgroups < 1) return SHAINET_HIP_ERR_ARGUMENT;
  hipLaunchKernelGGL(copy_f32x4_kernel, dim3((unsigned)workgroups), dim3(256), 0, (hipStream_t)stream,
                     (const f32x4 *)src, (f32x4 *)dst, n / 4);
  return hipGetLastError() == hipSuccess ? SHAINET_HIP_OK : SHAINET_HIP_ERR_RUNTIME;
}

int shainet_hip_stream_read_f32(const float *src, float *sink, long long n, int workgroups, void *stream) {
  if (!src || !sink || n < 0 || (n & 3) || workgroups < 1) return SHAINET_HIP_ERR_ARGUMENT;
  hipLaunchKernelGGL(read_f32x4_kernel, dim3((unsigned)workgroups), dim3(256), 0, (hipStream_t)stream,
                     (const f32x4 *)src, sink, n / 4);
  return hipGetLastError() == hipSuccess ? SHAINET_HIP_OK : SHAINET_HIP_ERR_RUNTIME;
}

int shainet_hip_mfma_f32_loop(float *sink, int iters, int workgroups, long long *flops, void *stream) {
  if (!sink || iters < 1 || workgroups < 1) return SHAINET_HIP_ERR_ARGUMENT;
  hipLaunchKernelGGL(mfma_f32_loop_kernel, dim3((unsigned)workgroups), dim3(512), 0, (hipStream_t)stream, sink, iters,
                     0.5f, 0.25f);
  // 16 MFMAs per round and wavefront, 2 * 32 * 32 * 2 flops each, 8 wavefronts per workgroup
  if (flops) *flops = (long long)workgroups * 8 * iters * 16 * 4096;
  return hipGetLastError() == hipSuccess ? SHAINET_HIP_OK : SHAINET_HIP_ERR_RUNTIME;
}

int shainet_hip_launch_latency(int chain, int reps, int workgroups, float *us_out, void *stream_) {
  if (chain < 1 || chain > 64 || reps < 1 || reps > 10000 || workgroups < 1 || !us_out) return SHAINET_HIP_ERR_ARGUMENT;
  hipStream_t stream = (hipStream_t)stream_;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return SHAINET_HIP_ERR_RUNTIME;
  std::vector<float> us;
  int rc = SHAINET_HIP_OK;
  for (int r = 0; r < reps + 3 && rc == SHAINET_HIP_OK; ++r) {
    // the first kernel hands its own first clock reading to e0, the last its last one to e1
    for (int i = 0; i < chain; ++i)
      hipExtLaunchKernelGGL(empty_kernel, dim3((unsigned)workgroups), dim3(256), 0, stream, i == 0 ? e0 : nullptr,
                            i == chain - 1 ? e1 : nullptr, 0, (int *)nullptr);
    float ms = 0.f;
    if (hipGetLastError() != hipSuccess || hipStreamSynchronize(stream) != hipSuccess ||
        hipEventElapsedTime(&ms, e0, e1) != hipSuccess)
      rc = SHAINET_HIP_ERR_RUNTIME;
    else if (r >= 3)
      us.push_back(ms * 1e3f);
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (rc == SHAINET_HIP_OK) {
    std::sort(us.begin(), us.end());
    *us_out = us[us.size() / 2];
  }
  return rc;
}

}  // extern "C"
