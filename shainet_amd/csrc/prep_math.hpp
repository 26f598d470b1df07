// The arithmetic of bias -> per-head QK-RMSNorm -> half-split RoPE for one head
// row held by one wavefront, with the reference's number types and evaluation
// order (llama_block.cr:596, 626-636, 274-281 and 332-344), so that results are
// bit-identical to its CPU path.  No product may fuse into an add here, whatever
// the including file is compiled with.
#pragma once
#include <hip/hip_runtime.h>

namespace shainet {

__device__ __forceinline__ float lane_value(float x, int t) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), t));
}

// Lane i < half holds x0 = row[i], x1 = row[i + half] (bias already added; lanes
// >= half hold anything).  has_w: apply the norm with weights w0 = w[i], w1 = w[i + half].
// cs = (cos, sin) of this row's position for rotation index i.  Wavefront-uniform
// control flow only (lane broadcasts inside).
__device__ __forceinline__ void norm_rotate_pair(float x0, float x1, bool has_w, float w0, float w1, double eps,
                                                 int hd, int half, float2 cs, float &r0, float &r1) {
#pragma clang fp contract(off)
  if (has_w) {
    // sum of squares in the reference's order: d ascending, one fp32 add per
    // element; first the lower halves of the pairs, then the upper halves
    float ss = 0.0f;
    for (int t0 = 0; t0 < half; t0 += 16) {
#pragma unroll
      for (int k = 0; k < 16; ++k)
        if (t0 + k < half) {
          const float v = lane_value(x0, t0 + k);
          const float sq = v * v;
          ss = ss + sq;
        }
    }
    for (int t0 = 0; t0 < half; t0 += 16) {
#pragma unroll
      for (int k = 0; k < 16; ++k)
        if (t0 + k < half) {
          const float v = lane_value(x1, t0 + k);
          const float sq = v * v;
          ss = ss + sq;
        }
    }
    const float mean = ss / (float)hd;
    const float inv = (float)(1.0 / sqrt((double)mean + eps));
    x0 = x0 * inv;
    x0 = x0 * w0;
    x1 = x1 * inv;
    x1 = x1 * w1;
  }
  const float p0 = x0 * cs.x, p1 = x1 * cs.y, p2 = x1 * cs.x, p3 = x0 * cs.y;
  r0 = p0 - p1;
  r1 = p2 + p3;
}

}  // namespace shainet
