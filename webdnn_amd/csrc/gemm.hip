// fp32 MFMA contraction kernels for gfx950: Gemm / batched MatMul and Conv as
// implicit GEMM, sharing one LDS-tiled main loop.
//
// Semantics follow the reference CPU operators
//   Gemm   : src/descriptor_runner/operators/cpu/operators/standard/gemm.ts:21-61
//   MatMul : src/descriptor_runner/operators/cpu/operators/standard/matmul.ts:58-111
//   Conv   : src/descriptor_runner/operators/cpu/operators/standard/conv.ts:134-333
// (those accumulate in double; here the accumulation is fp32 on the matrix
// cores, and the rounding points after the sum are kept: alpha*sum is rounded
// to fp32 before the C/bias term is added).
//
// Tiling: one 256-thread workgroup (4 wavefronts of 64) owns a BM x BN tile of
// the result, split over a WM x WN grid of wavefronts; each wavefront owns
// MT x NT v_mfma_f32_32x32x2_f32 tiles (16 accumulator registers per lane
// each).  K advances 16 at a time through two LDS buffers; the next K slab is
// fetched from global memory into registers while the current one feeds the
// matrix cores, so there is one barrier per slab.  Tile shapes: 128x128 for
// large problems, 64x256 / 64x128 when there are at most 64 result rows worth
// filling (ResNet stage-1 convs have 64 output channels), 64x64 when a larger
// tile would leave most of the 256 CUs idle.
//
// Operand layouts in LDS depend on which index is contiguous in global memory:
//   "KC" (k contiguous, e.g. A of a non-transposed Gemm, conv weights):
//        tile[row][k], row stride 20 floats; a lane reads 4 consecutive k with
//        one ds_read_b128.  The 16 k of a slab are consumed in the order
//        k = 8*(s/4) + 4*half + s%4 for MFMA step s and lane half (lane/32);
//        both operands use the same order, so the sum is over the same set.
//   "MC" (row/column index contiguous, e.g. B of a non-transposed Gemm, the
//        im2col view of a conv input): tile[k][col], row stride extent+8
//        floats; a lane reads one float per step, lanes 0..31 hit consecutive
//        banks and the two lane halves land 32 banks apart.
//
// Conv is Y[co][pixel] = W[co][k] * im2col[k][pixel] with k = (ci, ky, kx) and
// pixel = (image, oy, ox): M = output channels, N = batch*oh*ow.  The im2col
// matrix is never materialised: each thread owns one output pixel of the tile
// and gathers its taps straight from X (NCHW), consecutive lanes reading
// consecutive addresses; the epilogue scatters rows back to NCHW and fuses
// bias, residual and Relu.
//
// Global loads go through buffer descriptors wherever an operand spans less
// than 2 GiB: every per-thread address term is folded into one byte offset
// before the K loop, K advances through the instruction's scalar offset, and a
// conv tap that falls in the padding is given an offset outside the
// descriptor's window so that the hardware returns 0 for it.  The main loop
// then holds no vector-ALU address arithmetic at all (vector-ALU instructions
// issue in the same slot as the matrix-core ones and were measured to cost
// about 2.5 cycles of matrix-core time each).  Ragged K ends, edge tiles of
// an operand contiguous along M/N and operands of 2 GiB or more take a slower
// flat-load path in a separate general loop.
//
// Work decomposition (plan_work): whole tiles fill complete rounds over the
// CUs; the tiles left over, or every tile when there are too few to occupy
// the chip, are cut along K into chunks whose partial sums a second kernel
// adds in a fixed order.
#include <string.h>

#include <map>
#include <vector>

#include "contraction.h"

// The library's own workspace for partial sums, held in its image instead of pool memory.
// Two users:
//  * launches scheduled as streams of K slabs (see stream_next): the partial tile a
//    workgroup hands to its neighbour and one flag per workgroup, in the first
//    SK_PARTIAL_FLOATS + SK_FLAG_WORDS words.  Flags are 0 between launches: the
//    workgroup that consumes a partial tile clears its flag;
//  * wdh_gemm_static, for the chunk sums of plans that cut tiles across workgroups, so
//    that the call allocates nothing: the whole array.
// Every GPU the library runs on holds one copy until the process ends.
using namespace wdhc;
static __device__ __align__(256) float scratch[WDH_STATIC_SCRATCH_FLOATS];
static_assert(sizeof(float) * WDH_STATIC_SCRATCH_FLOATS == WDH_STATIC_SCRATCH_BYTES,
              "the header states the workspace size");
// In host code `scratch` is only a stand-in for the symbol: the array's device address is
// looked up once per device (wdh_init, with that device current) and kept here.
constexpr int kMaxDevices = 64;
static float *g_scratch_ptr[kMaxDevices] = {};

namespace wdh {
int init_static_scratch(int device) {
  if (device < 0 || device >= kMaxDevices)
    return fail(WDH_ENODEV, "wdh_init: device %d beyond the %d this library keeps a workspace for",
                device, kMaxDevices);
  if (g_scratch_ptr[device]) return WDH_OK;
  float *ptr = nullptr;
  hipError_t e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !ptr) {
    (void)hipGetLastError();
    return fail(WDH_EHIP, "wdh_init: address of the static workspace on device %d: %s", device,
                e == hipSuccess ? "null" : hipGetErrorString(e));
  }
  g_scratch_ptr[device] = ptr;
  return WDH_OK;
}
}  // namespace wdh
namespace wdhc {

float *static_scratch() { return g_scratch_ptr[wdh::device()]; }
// Side lanes: a workspace of the same layout from the driver (contraction_lane_init), so that what is
// recorded on a side lane takes the same kernels and adds in the same order as on lane 0.
static float *g_lane_workspace[WDH_LANES] = {};
float *stream_workspace() { return wdh::lane() == 0 ? static_scratch() : g_lane_workspace[wdh::lane()]; }


// Tile choice for Gemm / MatMul, from sweeps of all tile shapes over 30 problem sizes:
// 128x128 tiles (four accumulator tiles per wavefront, a quarter of the LDS reads per
// MFMA) win by 3-11 % once there are at least two of them per CU; below that the 64x64
// tile's finer granularity wins by up to 40 % (2048x2048x576: 46 us against 62), and the
// two rectangular shapes are never ahead of both by more than 2 %.  They and 64x256 stay
// reachable through wdh_set_option.
TileId pick_tile(int m, int n, int nz) {
  const long long tiles128 = (long long)((m + 127) / 128) * ((n + 127) / 128) * nz;
  // a 128-row tile over 64 rows (or 128 columns over 64) would compute mostly padding
  const double filled = (double)m * n * nz / ((double)tiles128 * 128.0 * 128.0);
  return tiles128 >= 2LL * wdh::compute_units() && filled >= 0.8 ? T128x128 : T64x64;
}
int g_forced_tile = -1;   // >= 0: overrides pick_tile (tuning hook)
int g_tile_hint = -1;     // >= 0: the caller inside the library knows the tile for its next product
int g_forced_split = -1;  // >= 1: overrides the split-K heuristic
int g_descriptors = 1;    // 0: every operand is treated as if it spanned 2 GiB or more
// what launch_planned decided for the most recent launch (wdh_last_plan)
LastPlan g_last_plan = {};
int g_last_form = 0;
bool g_static_scratch = false;  // set for the duration of a wdh_gemm_static call
int g_wavesplit = 1;      // 0: small products take the ordinary tiles too
int g_halo = 1;           // 0: 3x3 stride-1 convs use the gathered form too
// wdh_linear_group: while set, products that qualify for gemm_wavesplit_kernel are queued here
// instead of being launched, and leave together in one launch per kernel variant
struct GroupQueue {
  bool collecting = false;
  int count = 0;
  Params p[16];
  long long blocks[16];
  int variant[16];  // 2 * B_IS_KC + VEC
} g_group;
int g_stem = 1;           // 0: the 7x7 stride-2 stem conv gathers its taps like any other geometry
int g_pixels_s2 = 1;      // 0: 1x1 convs with a column stride of 2 gather their taps like any other geometry
int g_winograd4_channels = 0;  // when not 0: "conv3x3_winograd" 1 takes F(4x4, 3x3) from this many input and output channels on
int g_winograd = 1;       // 3x3 stride-1 convs by minimal filtering: 0 never, 1 = F(2x2, 3x3) where it wins, 2 / 3 = F(2x2, 3x3) / F(4x4, 3x3) wherever legal
int g_wide_stores = 1;    // 0: whole tiles store one element per lane and instruction
int g_stream = 1;         // launches scheduled as streams of K slabs: 0 never, 1 where the plan below gains, 2 wherever legal
int g_stream_wgs = 4;     // workgroups per CU of a stream launch (at most what the kernel's resources allow)
int g_stream_spin = 1 << 22;  // polls of a partial tile's flag before a workgroup gives up
unsigned *g_stream_error = nullptr;       // pinned host word the kernels set when a wait gave up
unsigned *g_stream_error_dev = nullptr;   // its device address
// Whether whole tiles may leave in 16-byte stores: Y (and the residual, which has Y's
// layout) must be 16-byte aligned with rows and z steps that keep the alignment, and the
// C term must be a value per row or contiguous along the columns.
static void set_wide(Params &p, bool conv) {
  auto aligned = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  bool ok = g_wide_stores && p.y_bytes > 0 && aligned(p.Y) && (!p.R || aligned(p.R));
  if (conv) {
    ok = ok && (p.cv.oh * p.cv.ow) % 4 == 0;
  } else {
    ok = ok && p.sY0 % 4 == 0 && p.sYb % 4 == 0;
    if (p.C) ok = ok && (p.sC1 == 0 || (p.sC1 == 1 && p.sC0 % 4 == 0 && aligned(p.C)));
  }
  p.wide = ok ? 1 : 0;
}
// A launch keeps every CU busy for ceil(tiles / CUs) tile times, so a tile count
// just above a multiple of the CU count wastes most of a round, and a CU that
// holds only one or two workgroups cannot hide their latencies.  Candidate
// plans -- nothing split, only the tiles beyond the last full round split, or
// every tile split -- are compared with a small model in microseconds: a CU
// works through its workgroups' K slabs at slab_us each, but never finishes
// sooner than `solo` times the longest single workgroup (the slow-down of a
// workgroup that runs alone on a CU); every workgroup adds a start-up/epilogue
// cost and a split adds the reduce pass over the partial sums.
WorkPlan plan_work(long long tiles, int k, int bm, int bn, bool gather, int kgran) {
  // kgran: the K loop advances in units of this many elements (a chunk is a whole number of them);
  // the model's constants are per 16 elements
  const long long cus = wdh::compute_units();
  const int slabs = (k + kgran - 1) / kgran;
  const double per16 = kgran / 16.0;
  WorkPlan w = {tiles, 0, 1, 0};
  auto with_split = [&](long long tail, int s) {
    WorkPlan r;
    r.kchunk = ((slabs + s - 1) / s) * kgran;
    r.split = (k + r.kchunk - 1) / r.kchunk;
    if (r.split < 1) r.split = 1;
    r.tail = r.split > 1 ? tail : 0;
    r.full = tiles - r.tail;
    return r;
  };
  if (g_forced_split >= 1) {
    // tuning / test hook: every tile is split this many ways
    const int s = g_forced_split < slabs ? g_forced_split : (slabs > 0 ? slabs : 1);
    return s > 1 ? with_split(tiles, s) : w;
  }
  if (slabs * per16 < 8) return w;
  const double area = (double)bm * bn / (64.0 * 64.0);
  const double slab_us = 0.30 * area * per16;
  const double start_us = 0.9 * (area > 1.0 ? 2.0 : 1.0);
  const double tile_bytes = (double)bm * bn * 4.0;
  // A launch cannot finish sooner than its longest workgroup, and with the CU mostly to
  // itself a workgroup is bound by the latency of its loads, slab after slab: about 2.5
  // times its nominal time (measured inside whole graphs, where operands arrive cold).
  auto floor_us = [](double longest) { return 2.5 * longest; };
  auto cost = [&](long long tail, int s) {
    const long long full_rounds = (tiles - tail) / cus;  // tiles - tail is a multiple of cus or 0
    const long long tail_rounds = (tail * s + cus - 1) / cus;
    const double chunk_us = (double)slabs / s * slab_us + start_us;
    const double whole_us = slabs * slab_us + start_us;
    const double work = full_rounds * whole_us + tail_rounds * chunk_us;
    const double longest = full_rounds > 0 ? whole_us : chunk_us;
    double t = work > floor_us(longest) ? work : floor_us(longest);
    // reduce pass: a launch, a serial walk over the s partial sums of each element (what
    // the deep splits of small Gemms feel; convs split at most ~8 ways), and the partial
    // sums written and read back (mostly through the last-level cache, ~8 TB/s)
    if (s > 1) t += (gather ? 6.0 : 4.0 + 0.26 * s) + 2.0 * tail * s * tile_bytes / 8.0e6;
    return t;
  };
  const long long rem = tiles % cus;
  // at least 64 elements of K per chunk
  const int min_units = per16 >= 4.0 ? 1 : (int)(4.0 / per16 + 0.999);
  const int max_s = slabs / min_units < 32 ? slabs / min_units : 32;
  double best;
  // unsplit: the remainder tiles make one more (partial) round of whole tiles
  {
    const long long rounds = (tiles + cus - 1) / cus;
    const double whole_us = slabs * slab_us + start_us;
    const double work = rounds * whole_us;
    best = work > floor_us(whole_us) ? work : floor_us(whole_us);
  }
  long long best_tail = 0;
  int best_s = 1;
  for (int s = 2; s <= max_s; s++) {
    if (rem) {
      const double c = cost(rem, s);
      if (c < best) { best = c; best_tail = rem; best_s = s; }
    }
    const double c = cost(tiles, s);
    if (c < best) { best = c; best_tail = tiles; best_s = s; }
  }
  return best_s > 1 ? with_split(best_tail, best_s) : w;
}
// Whether (and how wide) a launch runs as a stream of K slabs: workgroups per XCD, 0 = not.
// `w` is what the tile-per-workgroup plan would do.
int stream_width(long long tiles, int slabs, int kgran, const WorkPlan &w, int tile_floats, int max_wgs_per_cu) {
  if (!g_stream || g_forced_split >= 1 || !stream_workspace() || !g_stream_error_dev || tiles <= 0 || slabs <= 0) return 0;
  // while a side branch is open two launches of one recording may run at the same time, and the lane has
  // one set of slots and flags: neither side takes the stream form then
  if (wdh::branch_open()) return 0;
  const long long cus = wdh::compute_units();
  if (g_stream == 1) {
    // Measured on the ResNet-50 and DETR layer shapes: resident workgroups that walk segments
    // lose to one short-lived workgroup per tile wherever the plain plan needs no cut (more
    // wavefronts in flight hide the start and the end of a tile better than a longer-lived
    // workgroup does), and they win for 1x1 convs that read X in place where the plain plan
    // would cut every tile of a launch that has at least a tile per CU (392 tiles of K 1024:
    // 45 -> 40 us; 850 tiles of K 256 on a 50x68 plane: 31 -> 27 us): there the stream saves
    // the reduce pass and evens out the 1.5 tiles per CU.  With fewer tiles than CUs each tile
    // is shared by many workgroups and the chunk plan's parallel reduce wins; 3x3 convs gain 2 %
    // on ResNet-50's 14x14 planes and lose 8-10 % on DETR's 100x136 and 25x34 planes.
    if (!(w.tail == tiles && tiles >= cus && (g_last_form == B_PIXELS || g_last_form == B_PIXELS_S2))) return 0;
  }
  int per_cu = g_stream_wgs < max_wgs_per_cu ? g_stream_wgs : max_wgs_per_cu;
  if (per_cu < 1) per_cu = 1;
  long long wgs = cus * per_cu / XCDS;  // per XCD
  // every workgroup of an XCD that has tiles gets at least 64 elements of K
  const long long base = tiles / XCDS > 0 ? tiles / XCDS : 1;
  const int min_units = kgran >= 64 ? 1 : (64 + kgran - 1) / kgran;
  if (wgs > base * slabs / min_units) wgs = base * slabs / min_units;
  if (wgs < 1) wgs = 1;
  while (wgs * XCDS > SK_MAX_WGS || wgs * XCDS * tile_floats > (long long)SK_PARTIAL_FLOATS) wgs--;
  if (wgs < 1) return 0;
  const long long units = (tiles / XCDS + 1) * slabs;
  if (wgs * units >= 0x7fffffffLL) return 0;
  return (int)wgs;
}
// Fills in the LDS layout of the input tile for BN-pixel tiles; false if the geometry
// does not fit the kernel's LDS budget (the gathered form serves it then).
bool halo_fits(ConvGeom &cv, int bn, int nimg, int vecw, int pr) {
  const int up = [](int v, int to) { return (v + to - 1) / to * to; }(cv.pl, vecw);
  cv.col0 = up;
  cv.pitch = up + cv.w + (pr + vecw - 1) / vecw * vecw;
  int rows = 2 + (bn - 2) / cv.ow;
  int imgs = 2 + (bn - 2) / (cv.oh * cv.ow);
  if (imgs > nimg) imgs = nimg;
  if (rows > nimg * cv.oh) rows = nimg * cv.oh;
  cv.slots = rows + 2 * imgs;
  cv.fd_oh2 = make_fastdiv(cv.oh + 2);
  cv.fd_pg = make_fastdiv(cv.pitch / vecw);
  cv.fd_upc = make_fastdiv((long long)cv.slots * (cv.pitch / vecw));
  const long long pieces = (long long)HALO_CB * cv.slots * (cv.pitch / vecw);
  cv.units = (int)((pieces + NTHREADS - 1) / NTHREADS);
  return (long long)cv.slots * cv.pitch <= halo_plane(bn) && cv.units <= halo_units(vecw, bn);
}
bool aligned16(const void *ptr) { return ((uintptr_t)ptr & 15) == 0; }

// Largest element offset the strided view touches, for bounds checking.
long long span(long long nb, long long sb, long long n0, long long s0,
               long long n1, long long s1) {
  return (nb - 1) * sb + (n0 - 1) * s0 + (n1 - 1) * s1 + 1;
}
}  // namespace wdhc

using wdh::fail;

// Whether a product is one for gemm_wavesplit_kernel: few result blocks and a K worth cutting.
static bool wavesplit_suits(int batch, int m, int n, int k) {
  if (!g_wavesplit || g_forced_tile >= 0 || g_forced_split >= 0 || k < 128) return false;
  const long long blocks32 = (long long)((m + 31) / 32) * ((n + 31) / 32) * batch;
  const long long tiles64 = (long long)((m + 63) / 64) * ((n + 63) / 64) * batch;
  // (few blocks each streaming a long K would leave the weights to a handful of CUs: the 32 x 1000 x 2048
  // classifier head takes 17.2 us this way, 13.3 us as 64x64 tiles cut 16 ways along K plus their reduce pass)
  return blocks32 <= 4LL * wdh::compute_units() && tiles64 < 2LL * wdh::compute_units() &&
         (blocks32 * 2 >= wdh::compute_units() || k <= 512);
}

extern "C" int wdh_set_option(const char *name, int value) {
  if (!name) return fail(WDH_EINVAL, "wdh_set_option: name is NULL");
  if (strcmp(name, "contraction_tile") == 0) {
    if (value < -1 || value > T128x64)
      return fail(WDH_EINVAL, "wdh_set_option: contraction_tile %d outside -1..%d", value,
                  (int)T128x64);
    g_forced_tile = value;
    return WDH_OK;
  }
  if (strcmp(name, "split_k") == 0) {
    if (value < -1 || value == 0 || value > 64)
      return fail(WDH_EINVAL, "wdh_set_option: split_k %d (use -1 or 1..64)", value);
    g_forced_split = value;
    return WDH_OK;
  }
  if (strcmp(name, "descriptor_loads") == 0) {
    if (value != 0 && value != 1)
      return fail(WDH_EINVAL, "wdh_set_option: descriptor_loads %d (use 0 or 1)", value);
    g_descriptors = value;
    return WDH_OK;
  }
  if (strcmp(name, "gemm_wavesplit") == 0) {
    if (value != 0 && value != 1)
      return fail(WDH_EINVAL, "wdh_set_option: gemm_wavesplit %d (use 0 or 1)", value);
    g_wavesplit = value;
    return WDH_OK;
  }
  if (strcmp(name, "wide_stores") == 0) {
    if (value != 0 && value != 1)
      return fail(WDH_EINVAL, "wdh_set_option: wide_stores %d (use 0 or 1)", value);
    g_wide_stores = value;
    return WDH_OK;
  }
  if (strcmp(name, "conv_stem") == 0) {
    if (value != 0 && value != 1)
      return fail(WDH_EINVAL, "wdh_set_option: conv_stem %d (use 0 or 1)", value);
    g_stem = value;
    return WDH_OK;
  }
  if (strcmp(name, "conv3x3_winograd") == 0) {
    if (value < 0 || value > 3) return fail(WDH_EINVAL, "wdh_set_option: conv3x3_winograd %d (use 0..3)", value);
    g_winograd = value;
    return WDH_OK;
  }
  if (strcmp(name, "conv3x3_f4x4_channels") == 0) {
    if (value < 0) return fail(WDH_EINVAL, "wdh_set_option: conv3x3_f4x4_channels %d (use 0 or more)", value);
    g_winograd4_channels = value;
    return WDH_OK;
  }
  if (strcmp(name, "conv1x1_stride2_in_place") == 0) {
    if (value != 0 && value != 1)
      return fail(WDH_EINVAL, "wdh_set_option: conv1x1_stride2_in_place %d (use 0 or 1)", value);
    g_pixels_s2 = value;
    return WDH_OK;
  }
  if (strcmp(name, "stream_k") == 0) {
    if (value < 0 || value > 2) return fail(WDH_EINVAL, "wdh_set_option: stream_k %d (use 0, 1 or 2)", value);
    g_stream = value;
    return WDH_OK;
  }
  if (strcmp(name, "stream_wgs") == 0) {
    if (value < 1 || value > 8) return fail(WDH_EINVAL, "wdh_set_option: stream_wgs %d (use 1..8)", value);
    g_stream_wgs = value;
    return WDH_OK;
  }
  if (strcmp(name, "stream_spin") == 0) {
    if (value < 0) return fail(WDH_EINVAL, "wdh_set_option: stream_spin %d (use >= 0)", value);
    g_stream_spin = value;
    return WDH_OK;
  }
  if (strcmp(name, "conv3x3_halo") == 0) {
    if (value != 0 && value != 1)
      return fail(WDH_EINVAL, "wdh_set_option: conv3x3_halo %d (use 0 or 1)", value);
    g_halo = value;
    return WDH_OK;
  }
  if (strcmp(name, "memory_limit_mib") == 0) {
    if (value < 0) return fail(WDH_EINVAL, "wdh_set_option: memory_limit_mib %d (use 0 for none, or a size)", value);
    wdh::set_memory_limit((uint64_t)value << 20);
    return WDH_OK;
  }
  return fail(WDH_EINVAL, "wdh_set_option: unknown option \"%s\"", name);
}

extern "C" int wdh_last_plan(int *tile_m, int *tile_n, int64_t *whole_tiles, int64_t *split_tiles,
                             int *split, int *form) {
  if (tile_m) *tile_m = g_last_plan.bm;
  if (tile_n) *tile_n = g_last_plan.bn;
  if (whole_tiles) *whole_tiles = g_last_plan.full;
  if (split_tiles) *split_tiles = g_last_plan.tail;
  if (split) *split = g_last_plan.split;
  if (form) *form = g_last_plan.form;
  return WDH_OK;
}

extern "C" int wdh_gemm_static(wdh_buf hA, wdh_buf hB, wdh_buf hC, wdh_buf hY,
                               int batch, int m, int n, int k, int64_t sAb,
                               int64_t sA0, int64_t sA1, int64_t sBb, int64_t sB0,
                               int64_t sB1, int64_t sC0, int64_t sC1, float alpha,
                               float beta, int epilogue, wdh_buf hR) {
  WDH_REQUIRE_INIT();
  WDH_REQUIRE_COMPUTE_LANE();
  if (wdh::lane() != 0)
    return fail(WDH_ESTATE, "wdh_gemm_static: the static workspace belongs to lane 0 (a run recorded on lane %d "
                            "could be replayed next to one that uses it)", wdh::lane());
  g_static_scratch = true;
  const int rc = wdh_gemm(hA, hB, hC, hY, batch, m, n, k, sAb, sA0, sA1, sBb, sB0, sB1, sC0, sC1,
                          alpha, beta, epilogue, hR);
  g_static_scratch = false;
  return rc;
}

extern "C" int wdh_gemm(wdh_buf hA, wdh_buf hB, wdh_buf hC, wdh_buf hY,
                        int batch, int m, int n, int k, int64_t sAb,
                        int64_t sA0, int64_t sA1, int64_t sBb, int64_t sB0,
                        int64_t sB1, int64_t sC0, int64_t sC1, float alpha,
                        float beta, int epilogue, wdh_buf hR) {
  return wdh_gemm_ex(hA, hB, hC, hY, batch, m, n, k, sAb, sA0, sA1, sBb, sB0, sB1, sC0, sC1, alpha, beta,
                     epilogue, hR, (int64_t)m * n, n);
}

extern "C" int wdh_gemm_ex(wdh_buf hA, wdh_buf hB, wdh_buf hC, wdh_buf hY,
                           int batch, int m, int n, int k, int64_t sAb,
                           int64_t sA0, int64_t sA1, int64_t sBb, int64_t sB0,
                           int64_t sB1, int64_t sC0, int64_t sC1, float alpha,
                           float beta, int epilogue, wdh_buf hR, int64_t sYb, int64_t sY0) {
  WDH_REQUIRE_INIT();
  WDH_REQUIRE_COMPUTE_LANE();
  if (batch < 0 || m < 0 || n < 0 || k < 0)
    return fail(WDH_EINVAL, "wdh_gemm: negative extent (batch=%d m=%d n=%d k=%d)",
                batch, m, n, k);
  if (batch > 65535)
    return fail(WDH_EINVAL, "wdh_gemm: batch %d exceeds 65535", batch);
  if (sAb < 0 || sA0 < 0 || sA1 < 0 || sBb < 0 || sB0 < 0 || sB1 < 0 ||
      sC0 < 0 || sC1 < 0)
    return fail(WDH_EINVAL, "wdh_gemm: negative stride");
  if (epilogue != WDH_EPI_NONE && epilogue != WDH_EPI_RELU)
    return fail(WDH_EINVAL, "wdh_gemm: unknown epilogue %d", epilogue);
  const long long out_elems = (long long)batch * m * n;
  if (out_elems == 0) return WDH_OK;
  // Y (and R) rows are contiguous; rows and batch entries may be spaced out, either batch
  // entries apart (sYb >= m*sY0) or interleaved row by row (sY0 >= batch*sYb)
  if (sY0 < n || sYb < 0 ||
      (batch > 1 && !(sYb >= (int64_t)m * sY0 || (sYb >= n && sY0 >= (int64_t)batch * sYb))))
    return fail(WDH_EINVAL, "wdh_gemm: result strides (%lld, %lld) make rows overlap", (long long)sYb,
                (long long)sY0);
  const long long y_span = span(batch, sYb, m, sY0, n, 1);

  Params p = {};
  void *ptr;
  size_t need_a = k ? (size_t)span(batch, sAb, m, sA0, k, sA1) * 4 : 0;
  size_t need_b = k ? (size_t)span(batch, sBb, k, sB0, n, sB1) * 4 : 0;
  if (!wdh::operand(hA, need_a, "wdh_gemm: A", &ptr)) return WDH_EINVAL;
  p.A = (const float *)ptr;
  if (!wdh::operand(hB, need_b, "wdh_gemm: B", &ptr)) return WDH_EINVAL;
  p.B = (const float *)ptr;
  if (hC) {
    size_t need_c = (size_t)span(1, 0, m, sC0, n, sC1) * 4;
    if (!wdh::operand(hC, need_c, "wdh_gemm: C", &ptr)) return WDH_EINVAL;
    p.C = (const float *)ptr;
  }
  if (hR) {
    if (!wdh::operand(hR, (size_t)y_span * 4, "wdh_gemm: R", &ptr)) return WDH_EINVAL;
    p.R = (const float *)ptr;
  }
  if (!wdh::operand(hY, (size_t)y_span * 4, "wdh_gemm: Y", &ptr)) return WDH_EINVAL;
  p.Y = (float *)ptr;
  p.sYb = sYb; p.sY0 = sY0;
  p.m = m; p.n = n; p.k = k;
  p.sAb = sAb; p.sA0 = sA0; p.sA1 = sA1;
  p.sBb = sBb; p.sB0 = sB0; p.sB1 = sB1;
  p.sC0 = sC0; p.sC1 = sC1;
  p.alpha = alpha; p.beta = beta; p.epilogue = epilogue;

  // Which index of each operand is contiguous?  An extent of 1 makes the
  // stride along it irrelevant.
  const bool a_kc = (sA1 == 1 || k == 1), a_mc = (sA0 == 1 || m == 1);
  const bool b_kc = (sB0 == 1 || k == 1), b_mc = (sB1 == 1 || n == 1);
  if (!(a_kc || a_mc) || !(b_kc || b_mc) ||
      ((long long)(m + 63) / 64) * ((n + 63) / 64) > 0x7fffffffLL) {
    const long long sblocks = ((long long)m * n + 255) / 256;
    if (sblocks > 0x7fffffffLL)
      return fail(WDH_EINVAL, "wdh_gemm: %lld x %lld results exceed the grid limit of the strided form",
                  (long long)m, (long long)n);
    dim3 grid((unsigned)sblocks, (unsigned)batch);
    hipLaunchKernelGGL(contraction_strided_kernel, grid, dim3(256), 0,
                       wdh::stream(), p);
    WDH_LAUNCH_CHECK();
    return WDH_OK;
  }
  // Prefer the layout that allows 16-byte loads.
  auto vec_ok = [&](const float *base, long long ld, long long sb) {
    return aligned16(base) && ld % 4 == 0 && sb % 4 == 0;
  };
  bool useA_kc, useB_kc;
  if (a_kc && a_mc) useA_kc = vec_ok(p.A, sA0, sAb) || !vec_ok(p.A, sA1, sAb);
  else useA_kc = a_kc;
  if (b_kc && b_mc) useB_kc = vec_ok(p.B, sB1, sBb) || !vec_ok(p.B, sB0, sBb);
  else useB_kc = b_kc;
  // When k == 1 (or m/n == 1) the "contiguous" stride may not literally be 1;
  // the loaders index with the leading stride only, so normalise.
  if (useA_kc) p.sA1 = 1; else p.sA0 = 1;
  if (useB_kc) p.sB0 = 1; else p.sB1 = 1;
  const bool vec = vec_ok(p.A, useA_kc ? p.sA0 : p.sA1, sAb) &&
                   vec_ok(p.B, useB_kc ? p.sB1 : p.sB0, sBb);
  // Descriptor loads address one batch entry with 32-bit byte offsets (a
  // clamped edge row plus a 16-byte piece may reach 12 bytes past the span).
  const long long a_bytes = k ? span(1, 0, m, p.sA0, k, p.sA1) * 4 : 0;
  const long long b_bytes = k ? span(1, 0, k, p.sB0, n, p.sB1) * 4 : 0;
  // (the margin covers the columns an edge tile reads past the matrix)
  p.fast = g_descriptors && a_bytes < 0x7fffffffLL - 4096 && b_bytes < 0x7fffffffLL - 4096;
  p.a_bytes = p.fast ? (int)a_bytes : 0;
  p.b_bytes = p.fast ? (int)b_bytes : 0;
  {
    const long long y_bytes = y_span * 4;
    const long long c_bytes = p.C ? span(1, 0, m, p.sC0, n, p.sC1) * 4 : 0;
    const bool ok = g_descriptors && y_bytes < 0x7fffffffLL && c_bytes < 0x7fffffffLL;
    p.y_bytes = ok ? (int)y_bytes : 0;
    p.c_bytes = ok ? (int)c_bytes : 0;
    set_wide(p, false);
  }
  // Few result tiles and a K worth cutting: one launch with K cut across the wavefronts of a
  // workgroup (gemm_wavesplit_kernel) instead of chunks in a workspace and a reduce pass
  if (useA_kc && p.fast && wavesplit_suits(batch, m, n, k)) {
    const long long blocks32 = (long long)((m + 31) / 32) * ((n + 31) / 32) * batch;
    if (useB_kc || (long long)(k - 1) * p.sB0 * 4 < 0x7fffffffLL) {
      p.tiles_m = (m + 31) / 32;
      p.tiles_n = (n + 31) / 32;
      p.nz = batch;
      p.fd_tiles_per_z = make_fastdiv((long long)p.tiles_m * p.tiles_n);
      p.fd_group = make_fastdiv(p.tiles_n);
      p.kchunk = ((k + BK - 1) / BK + WS_WAVES - 1) / WS_WAVES * BK;  // slabs per wavefront, in elements
      g_last_plan = {32, 32, WS_WAVES, useB_kc ? WDH_FORM_GEMM_KC : WDH_FORM_GEMM_MC, blocks32, 0};
      if (g_group.collecting && g_group.count < 16) {
        g_group.p[g_group.count] = p;
        g_group.blocks[g_group.count] = blocks32;
        g_group.variant[g_group.count] = 2 * (useB_kc ? 1 : 0) + (vec ? 1 : 0);
        g_group.count++;
        return WDH_OK;
      }
      const dim3 grid((unsigned)blocks32), block(64 * WS_WAVES);
      if (useB_kc && vec)
        hipLaunchKernelGGL((gemm_wavesplit_kernel<true, true>), grid, block, 0, wdh::stream(), p);
      else if (useB_kc)
        hipLaunchKernelGGL((gemm_wavesplit_kernel<true, false>), grid, block, 0, wdh::stream(), p);
      else if (vec)
        hipLaunchKernelGGL((gemm_wavesplit_kernel<false, true>), grid, block, 0, wdh::stream(), p);
      else
        hipLaunchKernelGGL((gemm_wavesplit_kernel<false, false>), grid, block, 0, wdh::stream(), p);
      WDH_LAUNCH_CHECK();
      return WDH_OK;
    }
  }
  return useA_kc ? launch_gemm_a_kc(useB_kc, p, batch, vec) : launch_gemm_a_mc(useB_kc, p, batch, vec);
}

namespace {
// Launches what wdh_linear_group queued: one launch per kernel variant and GROUP_MAX problems.
int flush_group() {
  for (int variant = 0; variant < 4; variant++) {
    GroupParams g;
    g.count = 0;
    long long blocks = 0;
    auto launch_now = [&]() -> int {
      if (g.count == 0) return WDH_OK;
      g.first[g.count] = (int)blocks;
      const dim3 grid((unsigned)blocks), block(64 * WS_WAVES);
      switch (variant) {
        case 3: hipLaunchKernelGGL((gemm_wavesplit_group_kernel<true, true>), grid, block, 0, wdh::stream(), g); break;
        case 2: hipLaunchKernelGGL((gemm_wavesplit_group_kernel<true, false>), grid, block, 0, wdh::stream(), g); break;
        case 1: hipLaunchKernelGGL((gemm_wavesplit_group_kernel<false, true>), grid, block, 0, wdh::stream(), g); break;
        default: hipLaunchKernelGGL((gemm_wavesplit_group_kernel<false, false>), grid, block, 0, wdh::stream(), g); break;
      }
      WDH_LAUNCH_CHECK();
      g.count = 0;
      blocks = 0;
      return WDH_OK;
    };
    for (int i = 0; i < g_group.count; i++) {
      if (g_group.variant[i] != variant) continue;
      if (g.count == GROUP_MAX || blocks + g_group.blocks[i] > 0x3fffffffLL)
        if (int rc = launch_now()) return rc;
      g.first[g.count] = (int)blocks;
      g.p[g.count] = g_group.p[i];
      blocks += g_group.blocks[i];
      g.count++;
    }
    if (int rc = launch_now()) return rc;
  }
  return WDH_OK;
}
}  // namespace

extern "C" int wdh_linear_group(int count, const wdh_buf *hA, const wdh_buf *hW, const wdh_buf *hBias,
                                const wdh_buf *hY, const int *m, const int *n, const int *k, int epilogue) {
  WDH_REQUIRE_INIT();
  WDH_REQUIRE_COMPUTE_LANE();
  if (count < 0 || count > 16) return fail(WDH_EINVAL, "wdh_linear_group: %d problems (0..16)", count);
  if (count > 0 && (!hA || !hW || !hY || !m || !n || !k)) return fail(WDH_EINVAL, "wdh_linear_group: NULL array");
  // the results must be distinct buffers, none of them an input: the products run in no particular order
  for (int i = 0; i < count; i++)
    for (int j = 0; j < count; j++)
      if ((j != i && hY[i] == hY[j]) || hY[i] == hA[j] || hY[i] == hW[j] || (hBias && hBias[j] && hY[i] == hBias[j]))
        return fail(WDH_EINVAL, "wdh_linear_group: result %d is also an operand or another result", i);
  g_group.collecting = true;
  g_group.count = 0;
  int rc = WDH_OK;
  for (int i = 0; i < count && rc == WDH_OK; i++)
    rc = wdh_gemm_ex(hA[i], hW[i], hBias ? hBias[i] : 0, hY[i], 1, m[i], n[i], k[i], 0, k[i], 1, 0, n[i], 1, 0, 1,
                     1.0f, 1.0f, epilogue, 0, (int64_t)m[i] * n[i], n[i]);
  g_group.collecting = false;
  // (what was queued before a failure still runs: every queued problem passed its checks)
  const int rc2 = flush_group();
  g_group.count = 0;
  return rc != WDH_OK ? rc : rc2;
}

// ---- conv ----------------------------------------------------------------

namespace {

// Tap tables per conv geometry, built on the host once and kept on the device
// for the life of the library.
struct KtabKey {
  int c_in_g, kh, kw, dh, dw, h, w, mode;
  bool operator<(const KtabKey &o) const {
    return memcmp(this, &o, sizeof(*this)) < 0;
  }
};
struct KtabVal {
  int2 *ktab;
};

std::map<KtabKey, KtabVal> g_ktabs;

// Transformed filters (U of the F(2x2, 3x3) form) of weight buffers whose owner promised not to
// write to them (WDH_CONV_CONSTANT_WEIGHTS): weight handle -> a pool block that holds U.
struct FilterEntry {
  wdh_buf u;
  int cout, c, r;  // r: 2 or 4, the form the filters were transformed for
};
std::map<wdh_buf, FilterEntry> g_filters;

}  // namespace

namespace wdh {
void release_conv_tables() {
  for (auto &kv : g_ktabs) {
    (void)hipFree(kv.second.ktab);
  }
  g_ktabs.clear();
}
// The word a stream launch sets when one of its workgroups gave up waiting for a partial tile
// lives in pinned host memory the device writes to directly, so the host can look at it after
// any synchronisation without a copy.
// The buffer behind `h` is about to be freed or written to: data derived from it is stale.
void conv_forget_weights(wdh_buf h) {
  if (g_filters.empty()) return;
  auto it = g_filters.find(h);
  if (it == g_filters.end()) return;
  const wdh_buf u = it->second.u;
  g_filters.erase(it);  // first: wdh_free comes back here for `u`
  (void)wdh_free(u);
}

int init_contraction(int device) {
  if (g_stream_error) return WDH_OK;
  void *host = nullptr, *dev = nullptr;
  if (hipHostMalloc(&host, 64, hipHostMallocMapped) != hipSuccess ||
      hipHostGetDevicePointer(&dev, host, 0) != hipSuccess) {
    (void)hipGetLastError();
    if (host) (void)hipHostFree(host);
    return fail(WDH_ENOMEM, "wdh_init: pinned status word of the contraction kernels");
  }
  memset(host, 0, 64);
  g_stream_error = static_cast<unsigned *>(host);
  g_stream_error_dev = static_cast<unsigned *>(dev);
  // the flags of the static workspace start at zero and are left at zero by every launch; a
  // launch that was cut short (a failed run before a new wdh_init) may have left some raised
  float *base = device >= 0 && device < kMaxDevices ? g_scratch_ptr[device] : nullptr;
  if (base && hipMemset(base + SK_PARTIAL_FLOATS, 0, (size_t)SK_FLAG_WORDS * 4) != hipSuccess) {
    (void)hipGetLastError();
    return fail(WDH_EHIP, "wdh_init: clearing the workspace flags");
  }
  return WDH_OK;
}
// A side lane's own slots and flags for launches scheduled as streams of K slabs (they may run next to
// lane 0's, so they cannot share its static workspace).  Called once, when the lane is created.
int contraction_lane_init(int lane) {
  if (lane <= 0 || lane >= WDH_LANES || wdhc::g_lane_workspace[lane]) return WDH_OK;
  void *ptr = nullptr;
  if (hipMalloc(&ptr, WDH_STATIC_SCRATCH_BYTES) != hipSuccess) {
    (void)hipGetLastError();
    return fail(WDH_ENOMEM, "wdh_set_lane: %u bytes of workspace for lane %d", (unsigned)WDH_STATIC_SCRATCH_BYTES, lane);
  }
  if (hipMemset((float *)ptr + SK_PARTIAL_FLOATS, 0, (size_t)SK_FLAG_WORDS * 4) != hipSuccess) {
    (void)hipGetLastError();
    (void)hipFree(ptr);
    return fail(WDH_EHIP, "wdh_set_lane: clearing the workspace flags of lane %d", lane);
  }
  wdhc::g_lane_workspace[lane] = (float *)ptr;
  return WDH_OK;
}
void release_contraction() {
  for (float *&ws : wdhc::g_lane_workspace) {
    if (ws) (void)hipFree(ws);
    ws = nullptr;
  }
  g_filters.clear();  // (the blocks go with the pool)
  if (g_stream_error) (void)hipHostFree(g_stream_error);
  g_stream_error = g_stream_error_dev = nullptr;
}
// After the stream has drained: did a stream launch report a wait that gave up?
int contraction_check() {
  if (!g_stream_error || *reinterpret_cast<volatile unsigned *>(g_stream_error) == 0) return WDH_OK;
  *reinterpret_cast<volatile unsigned *>(g_stream_error) = 0;
  float *base = g_scratch_ptr[device()];
  if (base) (void)hipMemset(base + SK_PARTIAL_FLOATS, 0, (size_t)SK_FLAG_WORDS * 4);
  for (float *ws : wdhc::g_lane_workspace)
    if (ws) (void)hipMemset(ws + SK_PARTIAL_FLOATS, 0, (size_t)SK_FLAG_WORDS * 4);
  return fail(WDH_EHIP, "a contraction kernel gave up waiting for a partial tile of a neighbouring workgroup; "
                        "results since the last synchronisation are not valid");
}
}  // namespace wdh

extern "C" int wdh_conv2d(wdh_buf hX, wdh_buf hW, wdh_buf hBias, wdh_buf hY,
                          int n, int c, int h, int w, int cout, int kh, int kw,
                          int pt, int pl, int pb, int pr, int sh, int sw,
                          int dh, int dw, int group, int epilogue, wdh_buf hR) {
  return wdh_conv2d_ex(hX, hW, hBias, hY, n, c, h, w, cout, kh, kw, pt, pl, pb, pr, sh, sw, dh, dw, group, epilogue,
                       hR, 0);
}

extern "C" int wdh_conv2d_ex(wdh_buf hX, wdh_buf hW, wdh_buf hBias, wdh_buf hY,
                             int n, int c, int h, int w, int cout, int kh, int kw,
                             int pt, int pl, int pb, int pr, int sh, int sw,
                             int dh, int dw, int group, int epilogue, wdh_buf hR, int flags) {
  WDH_REQUIRE_INIT();
  WDH_REQUIRE_COMPUTE_LANE();
  if (flags & ~WDH_CONV_CONSTANT_WEIGHTS) return fail(WDH_EINVAL, "wdh_conv2d_ex: unknown flags %d", flags);
  if (n < 0 || c <= 0 || h <= 0 || w <= 0 || cout <= 0 || kh <= 0 || kw <= 0 ||
      sh <= 0 || sw <= 0 || dh <= 0 || dw <= 0 || group <= 0 || pt < 0 ||
      pl < 0 || pb < 0 || pr < 0)
    return fail(WDH_EINVAL, "wdh_conv2d: bad geometry");
  if (c % group || cout % group)
    return fail(WDH_EINVAL, "wdh_conv2d: channels (%d in, %d out) not divisible by group %d",
                c, cout, group);
  if (epilogue != WDH_EPI_NONE && epilogue != WDH_EPI_RELU)
    return fail(WDH_EINVAL, "wdh_conv2d: unknown epilogue %d", epilogue);
  if (group > 65535) return fail(WDH_EINVAL, "wdh_conv2d: group %d exceeds 65535", group);
  // floor division, as Math.floor in base/conv.ts:43-59
  auto out_dim = [](int in, int p0, int p1, int d, int k, int s) {
    int num = in + p0 + p1 - d * (k - 1) - 1;
    int q = num >= 0 ? num / s : -((-num + s - 1) / s);
    return q + 1;
  };
  const int oh = out_dim(h, pt, pb, dh, kh, sh), ow = out_dim(w, pl, pr, dw, kw, sw);
  if (oh <= 0 || ow <= 0)
    return fail(WDH_EINVAL, "wdh_conv2d: empty output (%d x %d)", oh, ow);
  if ((kh - 1) * dh > 0x7fff || (kw - 1) * dw > 0x7fff)
    return fail(WDH_EINVAL, "wdh_conv2d: kernel extent too large");
  const int c_in_g = c / group, cout_g = cout / group;
  const long long kdim = (long long)c_in_g * kh * kw;
  const long long npix = (long long)n * oh * ow;
  if (kdim > 0x7fffffffLL || npix > 0x7fffffffLL ||
      (long long)c * h * w > 0x7fffffffLL)
    return fail(WDH_EINVAL, "wdh_conv2d: extent exceeds 2^31");
  if (npix == 0) return WDH_OK;

  Params p = {};
  void *ptr;
  if (!wdh::operand(hX, (size_t)n * c * h * w * 4, "wdh_conv2d: X", &ptr)) return WDH_EINVAL;
  p.B = (const float *)ptr;
  if (!wdh::operand(hW, (size_t)cout * kdim * 4, "wdh_conv2d: W", &ptr)) return WDH_EINVAL;
  p.A = (const float *)ptr;
  if (hBias) {
    if (!wdh::operand(hBias, (size_t)cout * 4, "wdh_conv2d: Bias", &ptr)) return WDH_EINVAL;
    p.C = (const float *)ptr;
  }
  const size_t out_bytes = (size_t)npix * cout * 4;
  if (hR) {
    if (!wdh::operand(hR, out_bytes, "wdh_conv2d: R", &ptr)) return WDH_EINVAL;
    p.R = (const float *)ptr;
  }
  if (!wdh::operand(hY, out_bytes, "wdh_conv2d: Y", &ptr)) return WDH_EINVAL;
  p.Y = (float *)ptr;

  p.cv.fd_ow = make_fastdiv(ow);
  p.cv.fd_oh = make_fastdiv(oh);
  p.cv.fd_ohw = make_fastdiv((long long)oh * ow);
  p.cv.fd_plane = make_fastdiv((long long)h * w);

  if (g_stem && g_descriptors && wdh::conv_patch_applies(c, cout, kh, kw, sh, sw, dh, dw, group, h, w, pt, pl, oh, ow)) {
    const long long tiles = (long long)n * ((oh + 7) / 8) * ((ow + 15) / 16);
    g_last_plan = {64, 128, 1, WDH_FORM_CONV_STEM, tiles, 0};
    return wdh::conv_patch_launch(p.B, p.A, p.C, p.R, p.Y, n, h, w, oh, ow, pt, pl, epilogue == WDH_EPI_RELU);
  }

  const int ntaps = kh * kw;
  // Descriptor loads need every byte offset formed in the kernel (X, shifted up
  // by the top-left padding, and one group's weights) to stay below 2^31.
  const long long x_bytes = ((long long)n * c * h * w + (long long)pt * w + pl) * 4;
  const long long w_bytes = (long long)cout_g * kdim * 4;
  const bool small = g_descriptors && x_bytes < 0x7fffffffLL && w_bytes < 0x7fffffffLL;
  const bool vec = aligned16(p.A) && kdim % 4 == 0 && ((long long)cout_g * kdim) % 4 == 0;
  // 1x1, stride 1, no padding: X is the B matrix as it lies (B_PIXELS), provided every K slab
  // is whole and four consecutive pixels never straddle two images.  The last tile may hang
  // over the end of the pixels: its surplus columns read the next k row or, past the last
  // image, the zeros the descriptor returns, and are never stored.
  const long long plane = (long long)h * w;
  // The same with a column stride of 2 (the stride-2 1x1 convs that open a ResNet stage), when output
  // rows hold an even number of pixels: two neighbouring output pixels are elements 0 and 2 of four
  // consecutive input floats (B_PIXELS_S2).
  const bool unpadded_1x1 = small && vec && ntaps == 1 && pt == 0 && pl == 0 && pb == 0 && pr == 0 &&
                            plane % 4 == 0 && kdim % BK == 0 && aligned16(p.B);
  const bool in_place = unpadded_1x1 && sh == 1 && sw == 1;
  const bool in_place_s2 = unpadded_1x1 && g_pixels_s2 && sw == 2 && ow % 2 == 0 && ((long long)sh * w) % 4 == 0 && w % 4 == 0;
  if (in_place || in_place_s2) {
    p.m = cout_g; p.n = (int)npix; p.k = (int)kdim;
    p.sAb = (long long)cout_g * kdim; p.sA0 = kdim; p.sA1 = 1;
    p.sBb = (long long)c_in_g * plane; p.sB0 = plane; p.sB1 = 1;
    p.alpha = 1.0f; p.beta = 1.0f; p.epilogue = epilogue;
    p.cv.c_in_g = c_in_g; p.cv.h = h; p.cv.w = w; p.cv.oh = oh; p.cv.ow = ow;
    p.cv.sh = sh; p.cv.sw = sw;
    p.cv.kh = p.cv.kw = p.cv.dh = p.cv.dw = 1;
    p.cv.c_total = c; p.cv.cout_total = cout; p.cv.cout_g = cout_g;
    p.cv.ntaps = 1; p.cv.npix = npix;
    p.fast = 1;
    p.a_bytes = (int)w_bytes;
    p.b_bytes = (int)x_bytes;  // window of group 0; the kernel shortens it per group
    p.y_bytes = g_descriptors && out_bytes < 0x7fffffffULL ? (int)out_bytes : 0;
    p.c_bytes = cout * 4;
    set_wide(p, true);
    return launch_conv_pixels(p, group, true, in_place_s2);
  }
  // 3x3, stride 1, no dilation, one group, many channels: minimal filtering -- filters and input patches
  // are transformed, the positions of the transform domain (16 for F(2x2, 3x3), 36 for F(4x4, 3x3)) are
  // one batched product M[xi] = U[xi] [cout, c] x V[xi] [c, tiles] with 4/9 or 1/4 of the direct form's
  // multiplications, and the products are transformed back under the epilogue (winograd.hip).
  // g_winograd: 0 never; 1 = F(2x2, 3x3) from 128 channels on (F(4x4, 3x3) from g_winograd4_channels on, when
  // that is set: faster from 64 channels on, but its rounding errors are about ten times the direct form's,
  // which a 50-layer network's logits show); 2 / 3 = F(2x2, 3x3) / F(4x4, 3x3) wherever legal.
  const int wino_min = c < cout ? c : cout;
  int wino_r = 0;
  if (g_winograd == 2) wino_r = 2;
  else if (g_winograd == 3) wino_r = 4;
  else if (g_winograd == 1) wino_r = g_winograd4_channels && wino_min >= g_winograd4_channels ? 4 : wino_min >= 128 ? 2 : 0;
  if (wino_r && kh == 3 && kw == 3 && sh == 1 && sw == 1 && dh == 1 && dw == 1 && group == 1 && c % BK == 0 &&
      g_forced_tile < 0 && g_forced_split < 0) {
    const int r = wino_r, positions = (r + 2) * (r + 2);
    const long long tiles = wdh::wino_pitch(wdh::wino_tiles(r, n, oh, ow));  // (row length of V and M)
    const size_t u_bytes = (size_t)positions * cout * c * 4, v_bytes = (size_t)positions * c * tiles * 4,
                 m_bytes = (size_t)positions * cout * tiles * 4;
    if (tiles < 0x7fffffffLL && v_bytes < ((size_t)1 << 33) && m_bytes < ((size_t)1 << 33)) {
      // the transformed filters: kept from call to call when the caller vouches for the weights
      // (a block allocated while a graph is being recorded belongs to that graph, so nothing is kept then)
      wdh_buf hU = 0;
      bool u_kept = false, u_ready = false;
      if (flags & WDH_CONV_CONSTANT_WEIGHTS) {
        auto it = g_filters.find(hW);
        if (it != g_filters.end() && it->second.cout == cout && it->second.c == c && it->second.r == r) {
          hU = it->second.u;
          u_kept = u_ready = true;
        } else if (!wdh::capturing()) {
          wdh::conv_forget_weights(hW);
          hU = wdh_alloc(u_bytes);
          if (hU) {
            g_filters[hW] = FilterEntry{hU, cout, c, r};
            u_kept = true;
          }
        }
      }
      if (!hU) hU = wdh_alloc(u_bytes);
      const wdh_buf hV = wdh_alloc(v_bytes), hM = wdh_alloc(m_bytes);
      int rc = WDH_OK;
      if (!(hU && hV && hM)) {
        // no room for the transform-domain tensors: the direct forms below need none
        if (hU && !u_kept) (void)wdh_free(hU);
        if (u_kept && !u_ready) wdh::conv_forget_weights(hW);  // (registered above, never filled)
        if (hV) (void)wdh_free(hV);
        if (hM) (void)wdh_free(hM);
        wdh::clear_error();
        goto direct_forms;
      }
      {
        float *U = (float *)wdh::resolve(hU, nullptr), *V = (float *)wdh::resolve(hV, nullptr);
        if (!u_ready) rc = wdh::wino_filter_launch(r, p.A, U, cout, c);
        if (rc == WDH_OK) rc = wdh::wino_input_launch(r, p.B, V, n, c, h, w, oh, ow, pt, pl);
      }
      if (rc == WDH_OK) {
        // (64x64 tiles: the 16 products have K = c, short against their extent; measured best on
        // every 3x3 layer shape of ResNet-50 and DETR, 35 against 44 us where the general choice
        // takes 128x128)
        g_tile_hint = T64x64;
        rc = wdh_gemm(hU, hV, 0, hM, positions, cout, (int)tiles, c, (int64_t)cout * c, c, 1, (int64_t)c * tiles, tiles, 1,
                      0, 0, 1.0f, 1.0f, WDH_EPI_NONE, 0);
        g_tile_hint = -1;
      }
      if (rc == WDH_OK) {
        g_last_plan.form = r == 2 ? WDH_FORM_CONV3X3_WINOGRAD : WDH_FORM_CONV3X3_WINOGRAD4;
        rc = wdh::wino_output_launch(r, (const float *)wdh::resolve(hM, nullptr), p.C, p.R, p.Y, n, cout, oh, ow,
                                     epilogue == WDH_EPI_RELU);
      }
      // (the blocks go back to the pool at once: whoever gets them next is ordered behind these kernels)
      if (rc != WDH_OK && u_kept && !u_ready) wdh::conv_forget_weights(hW);  // (may not have been filled)
      if (hU && !u_kept) (void)wdh_free(hU);
      if (hV) (void)wdh_free(hV);
      if (hM) (void)wdh_free(hM);
      return rc;
    }
  }
direct_forms:
  // 3x3, stride 1, no dilation, input channels in blocks of 8: taps read from an input
  // tile staged in LDS (conv3x3_halo_kernel)
  if (g_halo && small && kh == 3 && kw == 3 && sh == 1 && sw == 1 && dh == 1 && dw == 1 &&
      c_in_g % HALO_CB == 0 && aligned16(p.A)) {
    const int vecw = (w % 4 == 0 && aligned16(p.B)) ? 4 : ((w % 2 == 0 && ((uintptr_t)p.B & 7) == 0) ? 2 : 1);
    p.cv.h = h; p.cv.w = w; p.cv.oh = oh; p.cv.ow = ow; p.cv.pt = pt; p.cv.pl = pl;
    // tile: 64x128 (each wavefront 64 rows x 32 pixels: one LDS read of the input feeds two
    // matrix-core steps) where the pixel count fills the chip with such tiles, 64x64 below
    TileId tile = g_forced_tile >= 0 ? (TileId)g_forced_tile : T64x64;
    if (g_forced_tile < 0 && (npix + 127) / 128 * ((cout_g + 63) / 64) * group >= 2LL * wdh::compute_units())
      tile = T64x128;
    const int bn = kTileN[tile];
    if (halo_fits(p.cv, bn, n, vecw, pr)) {
      p.m = cout_g; p.n = (int)npix; p.k = (int)kdim;
      p.sAb = (long long)cout_g * kdim; p.sA0 = kdim; p.sA1 = 1;
      p.alpha = 1.0f; p.beta = 1.0f; p.epilogue = epilogue;
      p.cv.c_in_g = c_in_g; p.cv.sh = p.cv.sw = p.cv.dh = p.cv.dw = 1; p.cv.kh = p.cv.kw = 3;
      p.cv.c_total = c; p.cv.cout_total = cout; p.cv.cout_g = cout_g;
      p.cv.ntaps = 9; p.cv.npix = npix;
      p.fast = 1;
      p.a_bytes = (int)w_bytes;
      p.b_bytes = (int)((long long)n * c * h * w * 4);
      p.y_bytes = g_descriptors && out_bytes < 0x7fffffffULL ? (int)out_bytes : 0;
      p.c_bytes = cout * 4;
      set_wide(p, true);
      return launch_conv3x3(tile, p, group, vecw);
    }
  }
  const int mode = !small || ntaps > 63 ? B_IM2COL_BIG : (ntaps > 31 ? B_IM2COL64 : B_IM2COL32);
  KtabKey key;
  memset(&key, 0, sizeof(key));
  key.c_in_g = c_in_g; key.kh = kh; key.kw = kw; key.dh = dh; key.dw = dw;
  key.h = h; key.w = w; key.mode = mode;
  auto it = g_ktabs.find(key);
  if (it == g_ktabs.end()) {
    if (wdh::capturing()) {
      // building the table takes a synchronous copy
      wdh::poison_capture();
      return fail(WDH_ESTATE, "wdh_conv2d: first use of this geometry; run it once before capturing a graph");
    }
    const int pad_tap = mode == B_IM2COL32 ? 31 : 63;
    std::vector<int2> tab((size_t)((kdim + BK - 1) / BK * BK),
                          mode == B_IM2COL_BIG ? int2{0, 0} : int2{0, pad_tap});
    size_t idx = 0;
    for (int ci = 0; ci < c_in_g; ci++)
      for (int ky = 0; ky < kh; ky++)
        for (int kx = 0; kx < kw; kx++) {
          const int packed = ((ky * dh) << 16) | (kx * dw);
          const int off = ci * h * w + ky * dh * w + kx * dw;
          if (mode == B_IM2COL_BIG) {
            tab[idx].x = off;
            tab[idx].y = packed;
          } else {
            tab[idx].x = off * 4;
            tab[idx].y = ky * kw + kx;
          }
          idx++;
        }
    KtabVal val = {nullptr};
    if (hipMalloc(&val.ktab, tab.size() * sizeof(int2)) != hipSuccess) {
      (void)hipGetLastError();
      return fail(WDH_ENOMEM, "wdh_conv2d: tap table allocation failed");
    }
    // synchronous copy: the host vector dies at the end of this scope
    WDH_HIP_CHECK(hipMemcpy(val.ktab, tab.data(), tab.size() * sizeof(int2),
                            hipMemcpyHostToDevice));
    it = g_ktabs.emplace(key, val).first;
  }

  p.m = cout_g; p.n = (int)npix; p.k = (int)kdim;
  p.sAb = (long long)cout_g * kdim; p.sA0 = kdim; p.sA1 = 1;
  p.sBb = 0; p.sB0 = 0; p.sB1 = 0;
  p.alpha = 1.0f; p.beta = 1.0f; p.epilogue = epilogue;
  p.cv.c_in_g = c_in_g; p.cv.h = h; p.cv.w = w; p.cv.oh = oh; p.cv.ow = ow;
  p.cv.pt = pt; p.cv.pl = pl; p.cv.sh = sh; p.cv.sw = sw;
  p.cv.c_total = c; p.cv.cout_total = cout; p.cv.cout_g = cout_g;
  p.cv.ntaps = ntaps;
  p.cv.npix = npix; p.cv.ktab = it->second.ktab;
  p.cv.kh = kh; p.cv.kw = kw; p.cv.dh = dh; p.cv.dw = dw;
  p.fast = small ? 1 : 0;
  p.a_bytes = small ? (int)w_bytes : 0;
  // a group's window runs from its first byte (shifted down by the padding) to the end of X
  p.b_bytes = small ? (int)x_bytes : 0;  // window of group 0; the kernel shortens it per group
  p.y_bytes = g_descriptors && out_bytes < 0x7fffffffULL ? (int)out_bytes : 0;
  p.c_bytes = cout * 4;
  set_wide(p, true);
  return launch_conv_gather(mode, p, group, vec);
}
