// The 7x7, stride-2 stem convolution of an image network (3 input channels, 64 output
// channels): reference semantics src/descriptor_runner/operators/cpu/operators/standard/conv.ts:223-333
// (im2col + matmul + bias), computed here as one contraction per output tile with both
// operands in LDS.
//
// Why it has a kernel of its own: K = 3*7*7 = 147 is short and every k is a different tap,
// so the gathered form spends one 4-byte global load per (pixel, k) and pads K to 160.
// Here a workgroup
//   * copies all 64x147 weights into LDS once (42 KB) and then walks output tiles,
//   * stages the 21x37x3 input patch of a tile of 8 rows x 16 columns of output pixels in
//     LDS (10 KB, double-buffered: the next tile's patch travels while this one is
//     multiplied), even and odd input columns in separate half-rows, so that the 16 pixels
//     of an output row read 16 consecutive floats for any tap and the two pixel rows of a
//     wavefront's block land 16 banks apart: no bank conflicts,
//   * reads every B element for the matrix cores from LDS at a compile-time offset from one
//     of three per-lane base addresses.
//
// K order.  v_mfma_f32_32x32x2_f32 takes k and k+1 of a step from the two halves of the
// wavefront, so the two k of a step must lie a fixed distance apart in the patch:
//   9 steps per kx : (c, ky = 2r) with (c, ky = 2r + 1), one input row apart,
//   1 step  per kx : (c = 0, ky = 6) with (c = 1, ky = 6), one channel plane apart,
//   1 step  per kx : (c = 2, ky = 6) alone (the other half multiplies zeros),
// 77 steps = 154 k for 147 taps.  The weights are permuted into this order as they are
// copied to LDS.  Sums therefore associate differently from the gathered form (as between
// any two tile shapes); both are within the contraction tolerance of the oracle.
#include "common.h"
#include "fastdiv.h"

namespace {

using wdh::FastDiv;
using wdh::fdiv;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int KH = 7, KW = 7, STRIDE = 2, CIN = 3, COUT = 64;
constexpr int TH = 8, TW = 16;                       // output pixels per tile: 8 rows of 16
constexpr int PH = (TH - 1) * STRIDE + KH;           // 21 input rows
constexpr int PW = (TW - 1) * STRIDE + KW;           // 37 input columns
constexpr int HALF_W = 20;                           // floats per half-row (19 even / 18 odd columns used)
constexpr int ROWP = 2 * HALF_W;                     // 40: an input row = even columns, then odd columns
constexpr int PLANE = PH * ROWP;                     // 840 floats per channel
constexpr int PATCH = CIN * PLANE;                   // 2520 floats
constexpr int PATCH_ELEMS = CIN * PH * PW;           // 2331 input elements per tile
constexpr int NTHREADS = 256;
constexpr int NFETCH = (PATCH_ELEMS + NTHREADS - 1) / NTHREADS;  // 10 per thread
constexpr int STEPS_PER_KX = 11, STEPS = KW * STEPS_PER_KX;      // 77
constexpr int STEP_GROUPS = (STEPS + 3) / 4;                     // 20 groups of four steps
constexpr int LDW = 8 * STEP_GROUPS + 4;             // 164 floats per weight row (164/4 odd: 16-byte reads spread over all banks)
static_assert(STRIDE * ROWP % 32 == 16, "the two pixel rows of a block must land 16 banks apart");
static_assert((LDW / 4) % 2 == 1, "weight rows must not line up on the banks");

// Y and the residual are written and read through buffer descriptors that span one image's
// 64 planes: the lane's part of the address is one byte offset per tile, the channel's part a
// scalar offset, and a lane whose pixel lies outside the image carries an offset outside
// every window, which the hardware drops: no address arithmetic and no branch per element.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
constexpr int BUF_WORD3 = 0x00020000;
constexpr int BUF_OUTSIDE = (int)0x80000000u;
__device__ __forceinline__ rsrc_t make_rsrc(const void *base, int bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, bytes, BUF_WORD3);
}

struct PatchParams {
  const float *X, *W, *Bias, *R;
  float *Y;
  int n, h, w, oh, ow, pt, pl;
  int tiles_x, tiles_y, ntiles;
  FastDiv fd_per_image, fd_tiles_x;
  int relu;
};

// Step t, half h -> index of the weight in a row of W (c*49 + ky*7 + kx), or -1 for none.
__host__ __device__ constexpr int weight_index(int t, int h) {
  const int kx = t / STEPS_PER_KX, u = t % STEPS_PER_KX;
  if (t >= STEPS) return -1;
  if (u < 9) return (u / 3) * (KH * KW) + (2 * (u % 3) + h) * KW + kx;
  if (u == 9) return h * (KH * KW) + 6 * KW + kx;
  return h == 0 ? 2 * (KH * KW) + 6 * KW + kx : -1;
}
// Step t -> offset (floats) of its half-0 element from the lane's pixel corner.
__host__ __device__ constexpr int step_offset(int t) {
  const int kx = t / STEPS_PER_KX, u = t % STEPS_PER_KX;
  const int col = (kx & 1) * HALF_W + (kx >> 1);
  if (u < 9) return (u / 3) * PLANE + 2 * (u % 3) * ROWP + col;
  if (u == 9) return 6 * ROWP + col;
  return 2 * PLANE + 6 * ROWP + col;
}

__device__ __forceinline__ float relu_js(float v) {
  // Math.max(v, 0): NaN stays NaN (the comparison is false for it), -0 becomes +0.
  return v <= 0.0f ? 0.0f : v;
}

__global__ __launch_bounds__(NTHREADS, 2) void conv7x7s2_patch_kernel(PatchParams p) {
  __shared__ __attribute__((aligned(16))) float wl[COUT * LDW];
  __shared__ __attribute__((aligned(16))) float patch[2][PATCH];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int li = lane & 31, half = lane >> 5;

  // ---- weights -> LDS, in step order: row m, position 8*(t/4) + 4*half + t%4 --------------
  // (all of a thread's 40 loads are issued before the first is stored: one memory round
  // trip per workgroup, not forty)
  {
    constexpr int ROW = 8 * STEP_GROUPS, PER_THREAD = COUT * ROW / NTHREADS;
    static_assert(COUT * ROW % NTHREADS == 0, "whole passes");
    float wv[PER_THREAD];
#pragma unroll
    for (int i = 0; i < PER_THREAD; i++) {
      const int e = tid + NTHREADS * i;
      const int m = e / ROW, pos = e - m * ROW;
      const int k = weight_index(4 * (pos >> 3) + (pos & 3), (pos >> 2) & 1);
      const float v = p.W[m * (CIN * KH * KW) + (k >= 0 ? k : 0)];
      wv[i] = k >= 0 ? v : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < PER_THREAD; i++) {
      const int e = tid + NTHREADS * i;
      const int m = e / ROW, pos = e - m * ROW;
      wl[m * LDW + pos] = wv[i];
    }
  }

  // ---- what this thread copies of every patch: element e = tid + 256 i -> (c, iy, ix) -------
  // (tile-independent: where the element lies relative to the patch's corner in X, its
  // row and column for the bounds test, and where it goes in LDS)
  int rel[NFETCH], src_y[NFETCH], src_x[NFETCH], dst[NFETCH];
#pragma unroll
  for (int i = 0; i < NFETCH; i++) {
    const int e = tid + NTHREADS * i;
    const int c = e / (PH * PW), r = e - c * (PH * PW);
    const int iy = r / PW, ix = r - iy * PW;
    src_y[i] = e < PATCH_ELEMS ? iy : -0x40000000;  // surplus threads fail every bounds test
    src_x[i] = ix;
    rel[i] = (c * p.h + iy) * p.w + ix;
    dst[i] = e < PATCH_ELEMS ? c * PLANE + iy * ROWP + (ix & 1) * HALF_W + (ix >> 1) : -1;
  }
  const int per_image = p.tiles_x * p.tiles_y;
  struct Origin { int img, oy0, ox0; };
  auto tile_origin = [&](int tile) {
    Origin o;
    o.img = fdiv(tile, p.fd_per_image);
    const int r = tile - o.img * per_image;
    const int ty = fdiv(r, p.fd_tiles_x);
    o.oy0 = ty * TH;
    o.ox0 = (r - ty * p.tiles_x) * TW;
    return o;
  };
  float staged[NFETCH];
  auto fetch = [&](const Origin &o) {
    const int iy0 = o.oy0 * STRIDE - p.pt, ix0 = o.ox0 * STRIDE - p.pl;
    // the patch's corner in X (it may lie in the padding, before the image's first element)
    const float *corner_x = p.X + ((long long)o.img * CIN * p.h * p.w + (long long)iy0 * p.w + ix0);
#pragma unroll
    for (int i = 0; i < NFETCH; i++) {
      const bool in = (unsigned)(iy0 + src_y[i]) < (unsigned)p.h && (unsigned)(ix0 + src_x[i]) < (unsigned)p.w;
      staged[i] = in ? corner_x[rel[i]] : 0.0f;  // outside the image: the zero padding
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int i = 0; i < NFETCH; i++)
      if (dst[i] >= 0) patch[buf][dst[i]] = staged[i];
  };

  // bias of the 32 channels whose sums this lane holds: register r of block mt is channel
  // 32 mt + 8 (r/4) + 4 half + r%4
  float bias[2][16];
#pragma unroll
  for (int mt = 0; mt < 2; mt++)
#pragma unroll
    for (int r = 0; r < 16; r++)
      bias[mt][r] = (p.Bias ? p.Bias : p.W)[32 * mt + 8 * (r >> 2) + 4 * half + (r & 3)];  // (unused without a bias)

  // the lane's pixel within the tile: row 2*wave + li/16, column li%16
  const int py = 2 * wave + (li >> 4), px = li & 15;
  const int corner = py * (STRIDE * ROWP) + px;

  // ---- the epilogue of a tile, one element at a time ---------------------------------------
  // It runs while the NEXT tile is multiplied: a few elements after each group of matrix-core
  // instructions, whose 64 cycles apiece hide the additions and the stores.  (Run after the
  // tile's own last product instead, it left the matrix cores idle a third of the time: the
  // two workgroups of a CU fall into step, and then both are in their epilogue at once.)
  const int plane = p.oh * p.ow;  // 64 planes of it stay below 2^29 elements (checked by the host)
  struct Pending {
    f32x16 sums[2];
    rsrc_t y, r;
    int lane_off;   // bytes from the image's first result to channel 4*half of the lane's pixel
  };
  auto open_pending = [&](Pending &d, const Origin &o, bool valid) {
    const long long image = (long long)o.img * COUT * plane;
    d.y = make_rsrc(p.Y + image, COUT * plane * 4);
    d.r = make_rsrc((p.R ? p.R : p.Y) + image, COUT * plane * 4);
    const int oy = o.oy0 + py, ox = o.ox0 + px;
    d.lane_off = valid && oy < p.oh && ox < p.ow ? (4 * half * plane + oy * p.ow + ox) * 4 : BUF_OUTSIDE;
  };
  auto finish_element = [&](const Pending &d, int e) {  // e: compile-time 0..31
    const int mt = e >> 4, r = e & 15;
    const int soff = (32 * mt + 8 * (r >> 2) + (r & 3)) * plane * 4;
    float v = d.sums[mt][r];
    if (p.Bias) v = v + bias[mt][r];
    if (p.R) v = v + __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(d.r, d.lane_off, soff, 0));
    if (p.relu) v = relu_js(v);
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), d.y, d.lane_off, soff, 0);
  };

  int tile = blockIdx.x;  // the host launches at most ntiles workgroups
  Origin here = tile_origin(tile);
  fetch(here);
  stash(0);
  __syncthreads();
  int buf = 0;
  Pending done;
  open_pending(done, here, false);  // nothing to finish during the first tile
  for (;;) {
    const int next = tile + (int)gridDim.x;
    Origin there = here;
    if (next < p.ntiles) {
      there = tile_origin(next);
      fetch(there);
    }
    __builtin_amdgcn_sched_barrier(0);

    f32x16 acc[2];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[a][r] = 0.0f;
    const float *b0 = &patch[buf][corner];
    const float *b1 = b0 + half * ROWP;    // steps pairing two input rows
    const float *b2 = b0 + half * PLANE;   // steps pairing two channels
    const float *a0 = &wl[li * LDW + 4 * half];
    // Four steps at a time: the weights and patch elements of group g + 1 are requested
    // before the eight matrix-core instructions of group g are issued, so an LDS round trip
    // hides behind them (two wavefronts per SIMD are too few to hide it otherwise).
    struct Frag { f32x4 a0, a1; float b[4]; };
    auto read_group = [&](int g, Frag &f) {
      f.a0 = *reinterpret_cast<const f32x4 *>(a0 + 8 * g);
      f.a1 = *reinterpret_cast<const f32x4 *>(a0 + 32 * LDW + 8 * g);
#pragma unroll
      for (int s = 0; s < 4; s++) {
        const int t = 4 * g + s;
        const int u = t % STEPS_PER_KX;
        if (t >= STEPS) f.b[s] = 0.0f;
        else if (u < 9) f.b[s] = b1[step_offset(t)];
        else if (u == 9) f.b[s] = b2[step_offset(t)];
        else f.b[s] = half ? 0.0f : b0[step_offset(t)];  // no partner tap: a true zero, whatever lies there
      }
    };
    Frag cur, nxt;
    read_group(0, cur);
#pragma unroll
    for (int g = 0; g < STEP_GROUPS; g++) {
      if (g + 1 < STEP_GROUPS) read_group(g + 1, nxt);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < 4; s++) {
        if (4 * g + s >= STEPS) continue;
        acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(cur.a0[s], cur.b[s], acc[0], 0, 0, 0);
        acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(cur.a1[s], cur.b[s], acc[1], 0, 0, 0);
      }
      // two elements of the previous tile per group: 32 elements over the first 16 groups
      if (g < 16) {
        finish_element(done, 2 * g);
        finish_element(done, 2 * g + 1);
      }
      __builtin_amdgcn_sched_barrier(0);
      cur = nxt;
    }
    done.sums[0] = acc[0];
    done.sums[1] = acc[1];
    open_pending(done, here, true);
    if (next >= p.ntiles) break;
    stash(buf ^ 1);   // nobody reads that buffer: its tile was finished before the last barrier
    __syncthreads();
    buf ^= 1;
    tile = next;
    here = there;
  }
  // the last tile has no successor to hide behind
#pragma unroll
  for (int e = 0; e < 32; e++) finish_element(done, e);
}

}  // namespace

namespace wdh {

bool conv_patch_applies(int c, int cout, int kh, int kw, int sh, int sw, int dh, int dw, int group, int h, int w,
                        int pt, int pl, int oh, int ow) {
  // One image's results must fit a buffer descriptor's window (below 2 GiB), and the kernel
  // indexes an image's input with 32-bit element offsets ((c * h + iy) * w + ix, shifted up by
  // the padding): larger images are left to the gathered form and its 64-bit path.
  return group == 1 && c == CIN && cout == COUT && kh == KH && kw == KW && sh == STRIDE && sw == STRIDE &&
         dh == 1 && dw == 1 && (long long)COUT * oh * ow * 4 < 0x7fffffffLL &&
         (long long)CIN * h * w + (long long)pt * w + pl < 0x7fffffffLL / 4;
}

int conv_patch_launch(const float *X, const float *W, const float *Bias, const float *R, float *Y, int n,
                      int h, int w, int oh, int ow, int pt, int pl, int relu) {
  PatchParams p = {};
  p.X = X; p.W = W; p.Bias = Bias; p.R = R; p.Y = Y;
  p.n = n; p.h = h; p.w = w; p.oh = oh; p.ow = ow; p.pt = pt; p.pl = pl;
  p.tiles_x = (ow + TW - 1) / TW;
  p.tiles_y = (oh + TH - 1) / TH;
  const long long ntiles = (long long)n * p.tiles_x * p.tiles_y;
  if (ntiles > 0x7fffffffLL) return fail(WDH_EINVAL, "wdh_conv2d: %lld output tiles exceed the grid limit", ntiles);
  p.fd_per_image = wdh::make_fastdiv((long long)p.tiles_x * p.tiles_y);
  p.fd_tiles_x = wdh::make_fastdiv(p.tiles_x);
  p.ntiles = (int)ntiles;
  p.relu = relu;
  const long long cap = 2LL * compute_units();  // two workgroups fit a CU (62 KB of LDS each)
  const unsigned grid = (unsigned)(ntiles < cap ? ntiles : cap);
  hipLaunchKernelGGL(conv7x7s2_patch_kernel, dim3(grid), dim3(NTHREADS), 0, stream(), p);
  WDH_LAUNCH_CHECK();
  return WDH_OK;
}

}  // namespace wdh
