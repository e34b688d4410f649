// Arithmetic shared by the kernels that turn attention scores into int8 probabilities: one fixed
// sequence of IEEE fp32 operations, so every kernel (and a CPU restatement of the same sequence)
// produces the same bits.
#pragma once
#include "ti_common.h"

namespace ti {

// e^x for x <= 0: Cody-Waite reduction x = n ln2 + r, |r| <= ln2/2, degree-6
// polynomial in Horner form with fma, scaling by 2^n through the exponent
// field.  x below -87 gives 0.  About 1 ulp.
// Straight-line on purpose: the out-of-range case is a select at the end (on an argument clamped to -87, so
// that every intermediate is an ordinary number), not a branch around the polynomial.  A branch per value costs
// three scalar instructions and a fetch bubble, and keeps the four values of a lane from overlapping.
__device__ __forceinline__ float exp_nonpos(float x) {
  const float xc = __builtin_fmaxf(x, -87.0f);  // NaN -> -87
  const float n = __builtin_rintf(xc * 1.44269504088896341f);
  float r = __builtin_fmaf(n, -0.693145751953125f, xc);       // ln2 high part (exact product for |n| < 2^11)
  r = __builtin_fmaf(n, -1.42860682030941723e-6f, r);         // ln2 low part
  float p = 1.0f / 720.0f;
  p = __builtin_fmaf(p, r, 1.0f / 120.0f);
  p = __builtin_fmaf(p, r, 1.0f / 24.0f);
  p = __builtin_fmaf(p, r, 1.0f / 6.0f);
  p = __builtin_fmaf(p, r, 0.5f);
  p = __builtin_fmaf(p, r, 1.0f);
  p = __builtin_fmaf(p, r, 1.0f);
  const int e = (int)n + 127;  // in [1, 127]
  const float v = p * __int_as_float(e << 23);
  return x > -87.0f ? v : 0.0f;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float o = __shfl_xor(v, off, 64);
    v = v > o ? v : o;
  }
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = v + __shfl_xor(v, off, 64);
  return v;
}

}  // namespace ti
