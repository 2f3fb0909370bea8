// One family of contraction kernels of libwebdnn_hip.so, in a translation unit of its own so that
// the families compile side by side (contraction.h holds the kernels and says what they compute).
#include "contraction.h"

namespace wdhc {
// 3x3 stride-1 Conv with the input rows of a tile staged in LDS
int launch_conv3x3(int tile, Params &p, int nz, int vecw) {
  switch (tile) {
    case T128x128: return launch_halo_tile<128, 128, 2, 2>(p, nz, vecw);
    case T64x256: return launch_halo_tile<64, 256, 1, 4>(p, nz, vecw);
    case T64x128: return launch_halo_tile<64, 128, 1, 4>(p, nz, vecw);
    case T128x64: return launch_halo_tile<128, 64, 2, 2>(p, nz, vecw);
    default: return launch_halo_tile<64, 64, 2, 2>(p, nz, vecw);
  }
}
}  // namespace wdhc
