// One family of contraction kernels of libwebdnn_hip.so, in a translation unit of its own so that
// the families compile side by side (contraction.h holds the kernels and says what they compute).
#include "contraction.h"

namespace wdhc {
// Gemm / MatMul with A contiguous along M (transA)
int launch_gemm_a_mc(bool b_kc, Params &p, int nz, bool vec) {
  return b_kc ? launch<false, B_KC>(p, nz, vec) : launch<false, B_MC>(p, nz, vec);
}
}  // namespace wdhc
