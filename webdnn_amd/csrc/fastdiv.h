// Exact division by a launch-time constant, shared by the contraction and the copy kernels.
#pragma once
#include <hip/hip_runtime.h>

namespace wdh {

// Division of a non-negative 32-bit integer by a divisor fixed for the launch: the
// host turns the divisor into a multiplier and a shift, the kernel pays one
// multiply-high and one shift instead of the ~40 instructions of a hardware-less
// integer division.  Exact for 0 <= n < 2^31.
struct FastDiv {
  unsigned mul;    // 0: the divisor is 1
  unsigned shift;
  int d;
};
inline FastDiv make_fastdiv(long long divisor) {
  FastDiv f = {0u, 0u, (int)divisor};
  if (divisor <= 1) return f;
  unsigned lg = 0;
  while ((1ll << lg) < divisor) lg++;
  const unsigned pw = 31 + lg;
  f.mul = (unsigned)((((unsigned long long)1 << pw) + (unsigned long long)divisor - 1) /
                     (unsigned long long)divisor);
  f.shift = pw - 32;
  return f;
}
__device__ __forceinline__ int fdiv(int n, const FastDiv &f) {
  return f.mul ? (int)(__umulhi((unsigned)n, f.mul) >> f.shift) : n;
}

}  // namespace wdh
