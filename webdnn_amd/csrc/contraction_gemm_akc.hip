// One family of contraction kernels of libwebdnn_hip.so, in a translation unit of its own so that
// the families compile side by side (contraction.h holds the kernels and says what they compute).
#include "contraction.h"

namespace wdhc {
// Gemm / MatMul with A contiguous along K
int launch_gemm_a_kc(bool b_kc, Params &p, int nz, bool vec) {
  return b_kc ? launch<true, B_KC>(p, nz, vec) : launch<true, B_MC>(p, nz, vec);
}
}  // namespace wdhc
