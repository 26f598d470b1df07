// Shared by the host mirrors of LlamaBlock and of the model around it: grow-only
// device buffers and the row-major projection y = x W.
#pragma once
#include <hip/hip_runtime.h>

#include <string>

namespace shainet {

struct DevF {
  float *p = nullptr;
  size_t cap = 0;
  bool reserve(size_t n);
  void release();
};

// y[T,N] = x[T,K] * W[K,N], all row-major on the device: a hand-written split
// GEMV for up to 16 rows (decode), rocBLAS SGEMM (the counterpart of the
// reference's cuBLAS SGEMM, cuda.cr:237-247) for more.
struct Projector {
  void *blas = nullptr;
  DevF scratch;
  // returns a SHAINET_HIP_* status; the message is left for shainet_hip_last_error
  int project(const float *x, const float *w, float *y, int T, int K, int N, hipStream_t stream);
  void release();
};

// Replace *dst (device, hipMalloc'ed or null) by a copy of n host floats.
int upload_floats(float **dst, const float *src, size_t n);
// Two host matrices [rows, n_a] and [rows, n_b] side by side into one device matrix [rows, n_a + n_b].
int upload_side_by_side(float **dst, const float *a, int n_a, const float *b, int n_b, int rows);

int llama_fail(int code, const std::string &msg);

}  // namespace shainet
