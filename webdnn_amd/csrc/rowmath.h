// Cross-lane reductions and the exponential shared by the row kernels (Softmax,
// LayerNormalization) and the fused attention kernel, so that the fused and the
// unfused softmax round alike.
#pragma once
#include <hip/hip_runtime.h>
#include <math.h>

namespace wdh {
namespace rowmath {

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
// e^x through the hardware's 2^r: x*log2(e) is split into the nearest integer n and a
// remainder r (|r| <= 1/2) that keeps the bits the single-precision product would drop,
// so the result is within two ulp for every x, large negative ones included.
__device__ __forceinline__ float exp_f32(float x) {
  x = x < -150.0f ? -150.0f : x;  // e^-150 is already 0 in single precision; NaN stays NaN
  const float log2e_hi = 1.44269502162933349609375f, log2e_lo = 1.925963033500011e-8f;
  const float n = __builtin_rintf(x * log2e_hi);
  float r = __builtin_fmaf(x, log2e_hi, -n);
  r = __builtin_fmaf(x, log2e_lo, r);
  return __builtin_ldexpf(__builtin_amdgcn_exp2f(r), (int)n);
}

}  // namespace rowmath
}  // namespace wdh
