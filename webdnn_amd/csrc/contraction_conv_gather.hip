// One family of contraction kernels of libwebdnn_hip.so, in a translation unit of its own so that
// the families compile side by side (contraction.h holds the kernels and says what they compute).
#include "contraction.h"

namespace wdhc {
// Conv with taps gathered through a tap table
int launch_conv_gather(int mode, Params &p, int nz, bool vec) {
  if (mode == B_IM2COL32) return launch<true, B_IM2COL32>(p, nz, vec);
  if (mode == B_IM2COL64) return launch<true, B_IM2COL64>(p, nz, vec);
  return launch<true, B_IM2COL_BIG>(p, nz, vec);
}
}  // namespace wdhc
