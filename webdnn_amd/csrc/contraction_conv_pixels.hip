// One family of contraction kernels of libwebdnn_hip.so, in a translation unit of its own so that
// the families compile side by side (contraction.h holds the kernels and says what they compute).
#include "contraction.h"

namespace wdhc {
// 1x1 stride-1 Conv reading X in place
int launch_conv_pixels(Params &p, int nz, bool vec) { return launch<true, B_PIXELS>(p, nz, vec); }
}  // namespace wdhc
