// One family of contraction kernels of libwebdnn_hip.so, in a translation unit of its own so that
// the families compile side by side (contraction.h holds the kernels and says what they compute).
#include "contraction.h"

namespace wdhc {
// 1x1 unpadded Conv reading X in place: every pixel (stride 1), or every other pixel of a row
int launch_conv_pixels(Params &p, int nz, bool vec, bool stride2) {
  return stride2 ? launch<true, B_PIXELS_S2>(p, nz, vec) : launch<true, B_PIXELS>(p, nz, vec);
}
}  // namespace wdhc
