// Launcher of the fp32 MFMA product y[T,N] = x[T,K] W[K,N] (+ res) for more than 16 rows.
#pragma once
#include <hip/hip_runtime.h>

namespace shainet {

struct GemmPlan {
  bool mfma;              // false: K, N or the row stride of x is not a multiple of 4 -> the plain kernel
  int tiles_m, tiles_n;   // 128 x 128 tiles of y
  int chunks;             // pieces K is cut into; > 1 adds the kernel that sums the partial products
  int k_chunk;            // contraction length per piece, a multiple of 32
  size_t partial_floats;  // scratch the launch needs (chunks * T * N when chunks > 1)
};
GemmPlan plan_gemm(int T, int K, int N, long long x_stride);
// Device pointers, 16-byte aligned for the MFMA kernel; rows of x are x_stride floats apart, y and
// res are dense [T, N]; res nullable (y = res + x W; res == y is allowed).  partials:
// p.partial_floats floats.
hipError_t launch_gemm(const float *x, long long x_stride, const float *w, float *y, const float *res, float *partials,
                       int T, int K, int N, const GemmPlan &p, hipStream_t stream);

}  // namespace shainet
