// Cross-lane reductions and the exponential shared by the row kernels (Softmax,
// LayerNormalization) and the fused attention kernel, so that the fused and the
// unfused softmax round alike.
#pragma once
#include <hip/hip_runtime.h>
#include <math.h>

namespace wdh {
namespace rowmath {

// Reductions over the 64 lanes through DPP operands (the exchange rides on the arithmetic
// instruction: no LDS crossbar, no lane-index arithmetic): within quads, across the quads of a
// row of 16 (half mirror, mirror), then lane 15 of rows 0 and 2 into rows 1 and 3, lane 31 into
// rows 2 and 3; lane 63 holds the result, which leaves through a scalar register.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_take(float idle, float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, idle), __builtin_bit_cast(int, v),
                                                              CTRL, ROW_MASK, 0xf, false));
}
constexpr int DPP_XOR1 = 0xB1, DPP_XOR2 = 0x4E, DPP_HALF_MIRROR = 0x141, DPP_MIRROR = 0x140;
constexpr int DPP_BCAST15 = 0x142, DPP_BCAST31 = 0x143;

__device__ __forceinline__ float wave_max(float v) {
  const float idle = -INFINITY;
  v = fmaxf(v, dpp_take<DPP_XOR1, 0xf>(idle, v));
  v = fmaxf(v, dpp_take<DPP_XOR2, 0xf>(idle, v));
  v = fmaxf(v, dpp_take<DPP_HALF_MIRROR, 0xf>(idle, v));
  v = fmaxf(v, dpp_take<DPP_MIRROR, 0xf>(idle, v));
  v = fmaxf(v, dpp_take<DPP_BCAST15, 0xa>(idle, v));
  v = fmaxf(v, dpp_take<DPP_BCAST31, 0xc>(idle, v));
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_take<DPP_XOR1, 0xf>(0.0f, v);
  v += dpp_take<DPP_XOR2, 0xf>(0.0f, v);
  v += dpp_take<DPP_HALF_MIRROR, 0xf>(0.0f, v);
  v += dpp_take<DPP_MIRROR, 0xf>(0.0f, v);
  v += dpp_take<DPP_BCAST15, 0xa>(0.0f, v);
  v += dpp_take<DPP_BCAST31, 0xc>(0.0f, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
// e^x through the hardware's 2^r: x*log2(e) is split into the nearest integer n and a
// remainder r (|r| <= 1/2) that keeps the bits the single-precision product would drop,
// so the result is within two ulp for every x, large negative ones included.
__device__ __forceinline__ float exp_f32(float x) {
  const float log2e_hi = 1.44269502162933349609375f, log2e_lo = 1.925963033500011e-8f;
  // n is held at -200 or above: 2^-200 is already 0 in single precision, and for x = -inf the
  // remainder then comes out as -inf (2^-inf = 0) instead of inf - inf.  A NaN x passes through n
  // (fmaxf returns -200) into r and out of 2^r.
  const float n = fmaxf(__builtin_rintf(x * log2e_hi), -200.0f);
  float r = __builtin_fmaf(x, log2e_hi, -n);
  r = __builtin_fmaf(x, log2e_lo, r);
  return __builtin_ldexpf(__builtin_amdgcn_exp2f(r), (int)n);
}

}  // namespace rowmath
}  // namespace wdh
