// Launcher of the fp32 MFMA product y[T,N] = x[T,K] W[K,N] (+ res) for more than 16 rows.
#pragma once
#include <hip/hip_runtime.h>

namespace shainet {

struct GemmPlan {
  bool mfma;              // false: K, N or the row stride of x is not a multiple of 4 -> the plain kernel
  int tiles_m, tiles_n;   // 128 x 128 tiles of y
  int steps;              // K steps of 32 per tile; a unit of work is one step of one tile
  int group_bits;         // 2^group_bits groups of workgroups, each with an equal run of the tiles
  int tiles_per_group;
  int quota;              // consecutive units per workgroup (= steps: a workgroup per tile, nothing shared)
  int pieces;             // > 1: every tile is cut into this many pieces of `quota` steps and a second kernel adds them
  int workgroups;
  size_t partial_floats;  // scratch for the pieces of tiles that two or more workgroups share (0: none)
  size_t flag_words;      // words, zero before the first launch (the kernel leaves them zero), that mark pieces complete
};
GemmPlan plan_gemm(int T, int K, int N, long long x_stride);
// Device pointers, 16-byte aligned for the MFMA kernel; rows of x are x_stride floats apart, y and
// res are dense [T, N]; res nullable (y = res + x W; res == y is allowed).  partials, flags:
// p.partial_floats floats and p.flag_words words (unused when those are 0); error: a word the
// kernel sets to 1 when it gives up a wait for another workgroup's piece (y is invalid then).
// flag_set, spin_limit: for the test of the give-up path only (marks go to flag_set, p.flag_words
// words of their own, instead of flags, and a wait ends after spin_limit polls); null / 0 otherwise.
hipError_t launch_gemm(const float *x, long long x_stride, const float *w, float *y, const float *res, float *partials,
                       unsigned *flags, int *error, int T, int K, int N, const GemmPlan &p, hipStream_t stream,
                       unsigned *flag_set = nullptr, int spin_limit = 0);

}  // namespace shainet
