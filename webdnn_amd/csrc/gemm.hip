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

#include "common.h"
#include "fastdiv.h"

// Workspace of wdh_gemm_static: the partial sums of tiles cut along K, held in the
// library's own image instead of pool memory so that the call allocates nothing.
// Every GPU the library runs on holds one copy until the process ends.
#define WDH_STATIC_SCRATCH_FLOATS (4u << 20) /* 16 MiB */
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

namespace {

using wdh::FastDiv;
using wdh::make_fastdiv;
using wdh::fdiv;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef __amdgpu_buffer_rsrc_t rsrc_t;

// Buffer descriptors: untyped 32-bit data, a window of `bytes` (< 2^31) above
// the base that covers exactly the operand.  A byte offset outside the window
// makes the hardware return 0 without touching memory; an offset with bit 31
// set is outside every window, which is how padding taps of a convolution are
// read.
constexpr int BUF_WORD3 = 0x00020000;
constexpr int BUF_OOB = (int)0x80000000u;

__device__ __forceinline__ rsrc_t make_rsrc(const void *base, int bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, bytes, BUF_WORD3);
}
__device__ __forceinline__ float buf_load(rsrc_t r, int voff, int soff) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
}
__device__ __forceinline__ f32x4 buf_load4(rsrc_t r, int voff, int soff) {
  return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0));
}
__device__ __forceinline__ void buf_store(rsrc_t r, float v, int voff, int soff) {
  __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), r, voff, soff, 0);
}
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
// No scalar-offset parameter on purpose: a buffer_store_dwordx4 whose scalar offset is a
// register gets no wait states from the compiler before its data registers are written again,
// and the chip then now and then stores the new values (seen in about one quad in a thousand).
// Every term of the address goes into `voff`.  test_sixteen_byte_stores_hold_the_bits_of_four_byte_stores (tests/test_gpu_parity.py)
// compares these stores with the 4-byte ones on every tile and must pass after a toolchain change.
__device__ __forceinline__ void buf_store4(rsrc_t r, f32x4 v, int voff) {
  __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), r, voff, 0, 0);
}

constexpr int BK = 16;
constexpr int NTHREADS = 256;
constexpr int LDK = BK + 4;  // KC tile row stride (floats)
constexpr int MC_PAD = 8;    // MC tile row stride = extent + 8 (floats)

// B_IM2COL32 / B_IM2COL64: at most 31 / 63 taps and X below 2 GiB, read through
// a buffer descriptor; B_IM2COL_BIG: anything else, read with flat loads.
// B_PIXELS: a 1x1, stride-1, unpadded conv.  Its B matrix is X itself, k rows of
// h*w contiguous pixels per image, so it is fetched like B_MC (16-byte pieces)
// with the image jump folded into each thread's column offset; the host picks it
// only when every tile and K slab is whole (n % BN == 0, k % BK == 0, h*w % 4 == 0).
enum BMode { B_KC = 0, B_MC = 1, B_IM2COL32 = 2, B_IM2COL64 = 3, B_IM2COL_BIG = 4, B_PIXELS = 5 };

struct ConvGeom {
  int c_in_g;        // input channels per group
  int h, w;          // input spatial size
  int oh, ow;        // output spatial size
  int pt, pl;        // top / left padding
  int sh, sw;        // strides
  int kh, kw;        // kernel size
  int dh, dw;        // dilations
  int c_total;       // input channels (all groups)
  int cout_total;    // output channels (all groups)
  int cout_g;        // output channels per group
  int ntaps;         // kh*kw
  long long npix;    // batch * oh * ow
  // per k = (ci, ky, kx), padded to a multiple of 16 entries.
  // Descriptor modes: x = 4*(ci*h*w + ky*dh*w + kx*dw), the byte offset from
  // the receptive field's corner, y = tap index ky*kw+kx; padding entries
  // carry tap 31 (B_IM2COL32) or 63 (B_IM2COL64), which no pixel has.
  // B_IM2COL_BIG: x = the same offset in elements, y = (ky*dh)<<16 | kx*dw.
  const int2 *ktab;
  // conv3x3_halo_kernel only: the input rows a tile needs are staged in LDS as
  // rows of `pitch` floats, `slots` of them per channel, the first input column in
  // LDS column col0; pb/pr = bottom / right padding
  int pitch, slots, col0, units;
  FastDiv fd_ow, fd_oh, fd_ohw;      // output width, height, plane
  FastDiv fd_plane;                  // h*w
  FastDiv fd_oh2, fd_upc, fd_pg;     // oh+2, pieces per channel, pieces per row (halo kernel)
};

struct Params {
  const float *A;
  const float *B;
  const float *C;   // bias-like term, broadcast by (sC0, sC1); may be null
  const float *R;   // residual shaped like Y; may be null
  float *Y;
  int m, n, k;
  long long sAb, sA0, sA1;   // A[b, i, x] = A[b*sAb + i*sA0 + x*sA1]
  long long sBb, sB0, sB1;   // B[b, x, j] = B[b*sBb + x*sB0 + j*sB1]
  long long sC0, sC1;
  long long sYb, sY0;        // Gemm/MatMul: Y[b, i, j] = Y[b*sYb + i*sY0 + j] (and R alike)
  float alpha, beta;
  int epilogue;
  int tiles_m, tiles_n;
  FastDiv fd_tiles_per_z, fd_tail_tiles, fd_group, fd_last_rows;  // see decode_work / tile_coords
  // Work decomposition.  Tiles are numbered tile + z * tiles_m * tiles_n (z =
  // batch entry or conv group).  The first full_tiles of them are computed by
  // one workgroup each; every remaining ("tail") tile is cut along K into
  // tail_split chunks of kchunk elements, one workgroup per chunk, whose raw
  // sums go to `partial` and are added up by splitk_reduce_kernel.
  int nz;
  int full_tiles;
  int tail_tiles;
  int tail_split;   // 1: no tile is split
  int kchunk;       // a multiple of 16
  float *partial;   // [tail tile][chunk][BM][BN]
  int fast;         // every operand spans less than 2 GiB: descriptor loads allowed
  int a_bytes;      // fast: bytes of one z of A / of B (conv: of X from the first byte
  int b_bytes;      //       of a group to the end of the tensor, plus the padding shift)
  int y_bytes;      // > 0: bytes of the span of Y over all z, below 2 GiB, and C spans
  int c_bytes;      //      c_bytes (< 2 GiB): whole tiles may use the descriptor epilogue
  int wide;         // whole tiles may store four columns per lane (see finish_tile)
  ConvGeom cv;
};

__device__ __forceinline__ float relu_js(float v) {
  // Math.max(v, 0): NaN stays NaN (the comparison is false for it), -0 becomes +0.
  return v <= 0.0f ? 0.0f : v;
}

// Whole-tile workgroups: ids are dealt round-robin over the 8 XCDs by the
// hardware; this gives each XCD a contiguous range of tile numbers, so that
// tiles sharing A and B panels meet in one L2.
__device__ __forceinline__ int xcd_contiguous(int pid, int total) {
  constexpr int XCDS = 8;
  const int xcd = pid % XCDS, local = pid / XCDS;
  const int base = total / XCDS, rem = total % XCDS;
  return xcd * base + (xcd < rem ? xcd : rem) + local;
}

// Tile number within one z -> tile coordinates, visiting tiles in groups of 8
// tile-rows so that the panels a group touches stay resident in L2.
constexpr int TILE_GROUP = 8;
__device__ __forceinline__ void tile_coords(const Params &p, int id, int *tm, int *tn) {
  const int per_group = TILE_GROUP * p.tiles_n;
  const int group = fdiv(id, p.fd_group);
  const int first_m = group * TILE_GROUP;
  const int in_group = id - group * per_group;
  if (p.tiles_m - first_m >= TILE_GROUP) {
    *tn = in_group / TILE_GROUP;
    *tm = first_m + in_group % TILE_GROUP;
  } else {
    // the last, shorter group
    *tn = fdiv(in_group, p.fd_last_rows);
    *tm = first_m + in_group - *tn * p.fd_last_rows.d;
  }
}

// Which tile a workgroup computes and, for a chunk workgroup, which part of K.
struct TileWork {
  bool whole;
  int lin, chunk, bz, tm, tn;
};
__device__ __forceinline__ TileWork decode_work(const Params &p) {
  TileWork t;
  const int pid = blockIdx.x;
  t.whole = pid < p.full_tiles;
  t.chunk = 0;
  if (t.whole) {
    t.lin = xcd_contiguous(pid, p.full_tiles);
  } else {
    // chunk workgroups: an XCD takes a contiguous run of (chunk, tile) pairs with the
    // tile varying fastest, so that tiles which share a slice of B meet in one L2
    const int v = xcd_contiguous(pid - p.full_tiles, p.tail_tiles * p.tail_split);
    t.chunk = fdiv(v, p.fd_tail_tiles);
    t.lin = p.full_tiles + (v - t.chunk * p.tail_tiles);
  }
  const int tiles_per_z = p.tiles_m * p.tiles_n;
  t.bz = fdiv(t.lin, p.fd_tiles_per_z);  // batch entry (gemm) or group (conv)
  tile_coords(p, t.lin - t.bz * tiles_per_z, &t.tm, &t.tn);
  return t;
}

// ---- global -> register fetch of one K slab ------------------------------
// KC operand, EXT rows: thread t fetches rows (t>>2) + 64*i, k offsets 4*(t&3)..+3.
template <int EXT, bool VEC>
__device__ __forceinline__ void fetch_kc(const float *__restrict__ base,
                                         long long ld_row, int row0, int nrows,
                                         int k0, int kdim, int tid,
                                         f32x4 (&reg)[EXT / 64]) {
  const int k = k0 + (tid & 3) * 4;
#pragma unroll
  for (int i = 0; i < EXT / 64; i++) {
    int r = row0 + (tid >> 2) + i * 64;
    r = r < nrows ? r : nrows - 1;  // rows past the edge are never stored
    const float *p = base + (long long)r * ld_row + k;
    if (k + 3 < kdim) {
      // interior: plain loads, nothing between them and the LDS store
      if (VEC) reg[i] = *reinterpret_cast<const f32x4 *>(p);
      else reg[i] = f32x4{p[0], p[1], p[2], p[3]};
    } else {
      f32x4 v;
      v.x = (k + 0 < kdim) ? p[0] : 0.0f;
      v.y = (k + 1 < kdim) ? p[1] : 0.0f;
      v.z = (k + 2 < kdim) ? p[2] : 0.0f;
      v.w = (k + 3 < kdim) ? p[3] : 0.0f;
      reg[i] = v;
    }
  }
}

// MC operand, EXT columns: EXT/4 threads cover one k row with 16-byte loads.
template <int EXT, bool VEC>
__device__ __forceinline__ void fetch_mc(const float *__restrict__ base,
                                         long long ld_k, int col0, int ncols,
                                         int k0, int kdim, int tid,
                                         f32x4 (&reg)[EXT / 64]) {
  constexpr int TPR = EXT / 4;          // threads per k row
  constexpr int RPP = NTHREADS / TPR;   // k rows per pass
  const int c = col0 + (tid % TPR) * 4;
#pragma unroll
  for (int i = 0; i < EXT / 64; i++) {
    int k = k0 + tid / TPR + i * RPP;
    if (k < kdim) {
      const float *p = base + (long long)k * ld_k;
      if (VEC && c + 3 < ncols) {
        reg[i] = *reinterpret_cast<const f32x4 *>(p + c);
      } else {
        const int last = ncols - 1;
        f32x4 v;
        v.x = p[c + 0 < last ? c + 0 : last];
        v.y = p[c + 1 < last ? c + 1 : last];
        v.z = p[c + 2 < last ? c + 2 : last];
        v.w = p[c + 3 < last ? c + 3 : last];
        reg[i] = v;
      }
    } else {
      reg[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
  }
}

// im2col view of X, EXT pixels: thread t owns pixel (t % EXT) of the tile and
// the 16*EXT/256 consecutive k rows starting at (t / EXT) * 16*EXT/256.  The k
// rows are uniform across a wavefront, so their tap-table entries arrive with
// one scalar load.
struct PixelCtx {
  const float *xbase;       // X + (image*c_total + group*c_in_g)*h*w (image 0 past the edge)
  int pbase;                // iy0*w + ix0
  int iy0, ix0;             // corner of the receptive field (may be negative)
  unsigned long long mask;  // 1 for a pixel of the output, 0 past the edge
};

template <int EXT>
__device__ __forceinline__ unsigned fetch_im2col(const ConvGeom &cv,
                                                 const PixelCtx &px, int k0,
                                                 int kdim, int tid,
                                                 f32x4 (&reg)[EXT / 64]) {
  constexpr int G = NTHREADS / EXT;  // wavefront groups, each owning L consecutive k rows
  constexpr int L = BK / G;          // loads per thread
  const int kfirst = k0 + __builtin_amdgcn_readfirstlane(tid / EXT) * L;
  // the table is padded to a multiple of 16 entries; rows past kdim are
  // masked by the k < kdim test
  int2 e[L];
#pragma unroll
  for (int i = 0; i < L; i++) e[i] = cv.ktab[kfirst + i];
  unsigned okbits = 0;
#pragma unroll
  for (int i = 0; i < L; i++) {
    const int iy = px.iy0 + (e[i].y >> 16), ix = px.ix0 + (e[i].y & 0xffff);
    const bool ok = px.mask && (unsigned)iy < (unsigned)cv.h &&
                    (unsigned)ix < (unsigned)cv.w && kfirst + i < kdim;
    // Unconditional load from a safe address; the value is zeroed when it is
    // stored to LDS (stash_im2col), so nothing here waits for the load.
    reg[i >> 2][i & 3] = px.xbase[ok ? px.pbase + e[i].x : 0];
    okbits |= (ok ? 1u : 0u) << i;
  }
  return okbits;
}

// ---- the same fetches through a buffer descriptor --------------------------
// Everything a thread needs to know about its rows is folded into one byte
// offset per 16-byte piece before the K loop starts; advancing along K is a
// scalar offset, so a slab costs no vector ALU work beyond the loads.
template <int EXT, bool VEC>
__device__ __forceinline__ void fetch_rows_fast(rsrc_t r, const int (&voff)[EXT / 64],
                                                int soff, f32x4 (&reg)[EXT / 64]) {
#pragma unroll
  for (int i = 0; i < EXT / 64; i++) {
    if (VEC)
      reg[i] = buf_load4(r, voff[i], soff);
    else
      reg[i] = f32x4{buf_load(r, voff[i], soff), buf_load(r, voff[i] + 4, soff),
                     buf_load(r, voff[i] + 8, soff), buf_load(r, voff[i] + 12, soff)};
  }
}

// Per-thread constants of the descriptor im2col fetch.
struct PixelFast {
  int valid;            // byte offset of the receptive field's corner, biased to be >= 0
  unsigned pad_lo;      // bit t set: tap t of this pixel falls in the padding (taps 0..31)
  unsigned pad_hi;      // taps 32..63
};

template <int EXT, bool TAPS64>
__device__ __forceinline__ void fetch_im2col_fast(rsrc_t r, const int2 *__restrict__ ktab,
                                                  const PixelFast &px, int kfirst,
                                                  f32x4 (&reg)[EXT / 64]) {
  constexpr int G = NTHREADS / EXT, L = BK / G;
  int2 e[L];
#pragma unroll
  for (int i = 0; i < L; i++) e[i] = ktab[kfirst + i];
#pragma unroll
  for (int i = 0; i < L; i++) {
    const unsigned word = (TAPS64 && (e[i].y & 32)) ? px.pad_hi : px.pad_lo;
    // -1 when the tap is padding, 0 otherwise
    const int pad = __builtin_amdgcn_sbfe((int)word, (unsigned)e[i].y & 31u, 1u);
    reg[i >> 2][i & 3] = buf_load(r, (pad & BUF_OOB) | px.valid, e[i].x);
  }
}

// ---- register -> LDS -------------------------------------------------------
template <int EXT>
__device__ __forceinline__ void stash_kc(float *tile, int tid,
                                         const f32x4 (&reg)[EXT / 64]) {
#pragma unroll
  for (int i = 0; i < EXT / 64; i++)
    *reinterpret_cast<f32x4 *>(tile + ((tid >> 2) + i * 64) * LDK + (tid & 3) * 4) = reg[i];
}
template <int EXT>
__device__ __forceinline__ void stash_mc(float *tile, int tid,
                                         const f32x4 (&reg)[EXT / 64]) {
  constexpr int TPR = EXT / 4, RPP = NTHREADS / TPR, LD = EXT + MC_PAD;
#pragma unroll
  for (int i = 0; i < EXT / 64; i++)
    *reinterpret_cast<f32x4 *>(tile + (tid / TPR + i * RPP) * LD + (tid % TPR) * 4) = reg[i];
}
template <int EXT>
__device__ __forceinline__ void stash_im2col(float *tile, int tid,
                                             const f32x4 (&reg)[EXT / 64],
                                             unsigned okbits) {
  constexpr int G = NTHREADS / EXT, L = BK / G, LD = EXT + MC_PAD;
  const int kgroup = tid / EXT, pix = tid % EXT;
#pragma unroll
  for (int i = 0; i < L; i++)
    tile[(kgroup * L + i) * LD + pix] = ((okbits >> i) & 1u) ? reg[i >> 2][i & 3] : 0.0f;
}

// The descriptor gather leaves a thread with L consecutive k of one pixel: they go
// to LDS as they are, tile[pixel][k] (the KC layout), L/4 16-byte stores.
template <int EXT>
__device__ __forceinline__ void stash_im2col_fast(float *tile, int tid,
                                                  const f32x4 (&reg)[EXT / 64]) {
  constexpr int G = NTHREADS / EXT, L = BK / G;
  const int kgroup = tid / EXT, pix = tid % EXT;
#pragma unroll
  for (int i = 0; i < L / 4; i++)
    *reinterpret_cast<f32x4 *>(tile + pix * LDK + kgroup * L + 4 * i) = reg[i];
}

constexpr int tile_floats(bool kc, int ext) { return kc ? ext * LDK : BK * (ext + MC_PAD); }

// ---- adding up the chunks of a tail tile ---------------------------------------
// Four consecutive columns (tile-local element e .. e+3) of tail tile j: the
// chunks' partial sums are added in index order, then alpha, bias, residual
// and Relu are applied as in the whole-tile epilogue.
template <bool CONV>
__device__ __forceinline__ void reduce_quad(const Params &p, int bm, int bn, int j, int bz,
                                            int tm, int tn, int e) {
  const int lr = e / bn, lc = e - lr * bn;
  const int row = tm * bm + lr;
  if (row >= p.m) return;
  const float *part = p.partial + (long long)j * p.tail_split * (bm * bn) + e;
  f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int c = 0; c < p.tail_split; c++)
    acc += *reinterpret_cast<const f32x4 *>(part + (long long)c * (bm * bn));
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int col = tn * bn + lc + i;
    if (col >= p.n) break;
    float y = CONV ? acc[i] : p.alpha * acc[i];  // (a conv has alpha = beta = 1: the same bits, fewer instructions)
    long long off;
    if (CONV) {
      const int ohw = p.cv.oh * p.cv.ow;
      const int img = fdiv(col, p.cv.fd_ohw), q = col - img * ohw;
      off = ((long long)img * p.cv.cout_total + (long long)bz * p.cv.cout_g + row) * ohw + q;
      if (p.C) y = y + p.C[bz * p.cv.cout_g + row];
    } else {
      off = (long long)bz * p.sYb + (long long)row * p.sY0 + col;
      if (p.C) y = __builtin_fmaf(p.C[(long long)row * p.sC0 + (long long)col * p.sC1], p.beta, y);
    }
    if (p.R) y = y + p.R[off];
    if (p.epilogue == WDH_EPI_RELU) y = relu_js(y);
    p.Y[off] = y;
  }
}

// ---- epilogue shared by the contraction kernels ----------------------------------
// LDS a wavefront turns one 32x32 block through: rows of 36 floats (16-byte aligned, and
// the two halves of a wavefront land on different banks)
constexpr int STAGE_LD = 36;
constexpr int STAGE_FLOATS = 32 * STAGE_LD;

// A lane holds column (li) of each 32x32 block of its wavefront's part of the tile,
// rows 8*(r/4) + 4*half + r%4 for accumulator register r.  Chunk workgroups store raw
// sums for splitk_reduce_kernel; whole tiles apply alpha, the C/bias term, the
// residual and Relu and store to Y (NCHW for CONV).
template <int BM, int BN, int WM, int WN, bool CONV>
__device__ __forceinline__ void finish_tile(const Params &p,
                                            f32x16 (&acc)[BM / (WM * 32)][BN / (WN * 32)],
                                            bool whole, int lin, int chunk, int bz, int row0,
                                            int col0, float *stage) {
  constexpr int MT = BM / (WM * 32), NT = BN / (WN * 32);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int li = lane & 31, half = lane >> 5;
  const int wrow = wm * (MT * 32), wcol = wn * (NT * 32);
  if (!whole) {
    // raw sums of the whole tile (edge rows and columns included), tile-local
    float *part = p.partial +
                  ((long long)(lin - p.full_tiles) * p.tail_split + chunk) * (BM * BN);
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
#pragma unroll
      for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int lr = wrow + mt * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
          part[lr * BN + wcol + nt * 32 + li] = acc[mt][nt][r];
        }
    return;  // splitk_reduce_kernel adds the chunks up
  }
  // Whole tiles whose rows can be written 16 bytes at a time: each 32x32 block is
  // turned through the wavefront's own corner of the LDS the main loop has finished
  // with, so that a lane holds four neighbouring columns of a row and the block
  // leaves in four 16-byte stores (and its residual arrives in four loads) where
  // the accumulator layout would need sixteen of four bytes.  The epilogue is
  // bound by the number of memory instructions, not by the bytes.
  if (p.wide && row0 + BM <= p.m && col0 + BN <= p.n) {
    __syncthreads();  // no wavefront still reads the main loop's tiles
    float *st = stage;  // this wavefront's 32 rows of STAGE_LD
    const long long zoff = CONV ? 0 : (long long)bz * p.sYb;
    const int y_window = p.y_bytes - (int)(zoff * 4);
    const rsrc_t rsrc_y = make_rsrc(p.Y + zoff, y_window);
    const rsrc_t rsrc_r = make_rsrc(p.R ? p.R + zoff : p.Y + zoff, y_window);
    const rsrc_t rsrc_c = make_rsrc(p.C ? p.C : p.Y, p.C ? p.c_bytes : 0);
    const int lr = lane >> 3, lc = (lane & 7) * 4;  // row (of every eight) and first column
    const bool c_per_row = CONV || p.sC1 == 0;
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      const int col = col0 + wcol + nt * 32 + lc;
      int ybase, ystride, voff_c, cstride;  // in elements; byte offsets stay below 2^31
      if (CONV) {
        const unsigned ohw = (unsigned)(p.cv.oh * p.cv.ow);
        const unsigned img = (unsigned)fdiv(col, p.cv.fd_ohw);
        ybase = (int)((img * (unsigned)p.cv.cout_total + (unsigned)(bz * p.cv.cout_g)) * ohw +
                      ((unsigned)col - img * ohw));
        ystride = (int)ohw;
        voff_c = (bz * p.cv.cout_g + lr) * 4;
        cstride = 1;
      } else {
        ybase = col;
        ystride = (int)p.sY0;
        voff_c = (int)((lr * p.sC0 + col * p.sC1) * 4);
        cstride = (int)p.sC0;
      }
      const int voff_y = (ybase + lr * ystride) * 4;
#pragma unroll
      for (int mt = 0; mt < MT; mt++) {
        const int rbase = __builtin_amdgcn_readfirstlane(row0 + wrow + mt * 32);
        // Tiles with one or two blocks per wavefront have registers to spare and request the
        // bias / residual values of all four row groups before the first is used; the
        // 64-accumulator tiles request them row group by row group (anything else spills).
        constexpr bool AHEAD = MT * NT <= 2;
        f32x4 cv[AHEAD ? 4 : 1], rv[AHEAD ? 4 : 1];
        auto request = [&](int i, int slot) {
          if (p.C) {
            const int soff = (rbase + 8 * i) * cstride * 4;
            if (c_per_row) {
              const float c = buf_load(rsrc_c, voff_c, soff);
              cv[slot] = f32x4{c, c, c, c};
            } else {
              cv[slot] = buf_load4(rsrc_c, voff_c, soff);
            }
          }
          if (p.R) rv[slot] = buf_load4(rsrc_r, voff_y, (rbase + 8 * i) * ystride * 4);
        };
        if constexpr (AHEAD) {
#pragma unroll
          for (int i = 0; i < 4; i++) request(i, i);
        }
        __builtin_amdgcn_wave_barrier();  // the previous block's reads come first
#pragma unroll
        for (int r = 0; r < 16; r++)
          st[(8 * (r >> 2) + 4 * half + (r & 3)) * STAGE_LD + li] = acc[mt][nt][r];
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const int slot = AHEAD ? i : 0;
          if constexpr (!AHEAD) request(i, 0);
          const f32x4 v = *reinterpret_cast<const f32x4 *>(&st[(lr + 8 * i) * STAGE_LD + lc]);
          f32x4 y;
#pragma unroll
          for (int e = 0; e < 4; e++) {
            float t;
            if constexpr (CONV) {  // alpha = beta = 1: the same bits, two instructions fewer per element
              t = v[e];
              if (p.C) t = t + cv[slot][e];
            } else {
              t = p.alpha * v[e];
              if (p.C) t = __builtin_fmaf(cv[slot][e], p.beta, t);
            }
            if (p.R) t = t + rv[slot][e];
            if (p.epilogue == WDH_EPI_RELU) t = relu_js(t);
            y[e] = t;
          }
          // (row offset in the vector register: a 16-byte store whose scalar offset is a
          // register gets no wait states from the compiler before its data registers are
          // written again, and this chip then now and then stores the new value)
          buf_store4(rsrc_y, y, voff_y + (rbase + 8 * i) * ystride * 4);
        }
      }
    }
    return;
  }
  // Whole tiles of results below 2 GiB: every address is one per-lane byte
  // offset (column, plus the four rows by which the two halves of a wavefront
  // differ) and one scalar offset per accumulator row, so a stored element costs
  // no address arithmetic, no bounds test and no change of the execution mask.
  if (p.y_bytes > 0 && row0 + BM <= p.m && col0 + BN <= p.n) {
    // (Gemm: the window runs from this z's first element to the end of the span all z cover)
    const long long zoff = CONV ? 0 : (long long)bz * p.sYb;
    const int y_window = p.y_bytes - (int)(zoff * 4);
    const rsrc_t rsrc_y = make_rsrc(p.Y + zoff, y_window);
    const rsrc_t rsrc_r = make_rsrc(p.R ? p.R + zoff : p.Y + zoff, y_window);
    const rsrc_t rsrc_c = make_rsrc(p.C ? p.C : p.Y, p.C ? p.c_bytes : 0);
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      const int col = col0 + wcol + nt * 32 + li;
      int ybase, ystride, voff_c, cstride;  // in elements; byte offsets stay below 2^31
      if (CONV) {
        const unsigned ohw = (unsigned)(p.cv.oh * p.cv.ow);
        const unsigned img = (unsigned)fdiv(col, p.cv.fd_ohw);
        ybase = (int)((img * (unsigned)p.cv.cout_total + (unsigned)(bz * p.cv.cout_g)) * ohw +
                      ((unsigned)col - img * ohw));
        ystride = (int)ohw;
        voff_c = (bz * p.cv.cout_g + 4 * half) * 4;
        cstride = 1;
      } else {
        ybase = col;
        ystride = (int)p.sY0;
        voff_c = (int)((4 * half * p.sC0 + col * p.sC1) * 4);
        cstride = (int)p.sC0;
      }
      const int voff_y = (ybase + 4 * half * ystride) * 4;
#pragma unroll
      for (int mt = 0; mt < MT; mt++) {
        const int rbase = __builtin_amdgcn_readfirstlane(row0 + wrow + mt * 32);
#pragma unroll
        for (int hb = 0; hb < 2; hb++) {
          float cv[8], rv[8];
          if (p.C) {
#pragma unroll
            for (int j = 0; j < 8; j++)
              cv[j] = buf_load(rsrc_c, voff_c, (rbase + 16 * hb + 8 * (j >> 2) + (j & 3)) * cstride * 4);
          }
          if (p.R) {
#pragma unroll
            for (int j = 0; j < 8; j++)
              rv[j] = buf_load(rsrc_r, voff_y, (rbase + 16 * hb + 8 * (j >> 2) + (j & 3)) * ystride * 4);
          }
#pragma unroll
          for (int j = 0; j < 8; j++) {
            float y;
            if constexpr (CONV) {
              y = acc[mt][nt][8 * hb + j];
              if (p.C) y = y + cv[j];
            } else {
              y = p.alpha * acc[mt][nt][8 * hb + j];
              if (p.C) y = __builtin_fmaf(cv[j], p.beta, y);
            }
            if (p.R) y = y + rv[j];
            if (p.epilogue == WDH_EPI_RELU) y = relu_js(y);
            buf_store(rsrc_y, y, voff_y, (rbase + 16 * hb + 8 * (j >> 2) + (j & 3)) * ystride * 4);
          }
        }
      }
    }
    return;
  }
  // Edge tiles and larger results.  Bias and residual values of a 32x32 block
  // are all requested before the first is used, so the block pays one memory
  // round trip, not thirty-two.  Loads use clamped indices (always inside the
  // tensors); only the store is conditional.
#pragma unroll
  for (int nt = 0; nt < NT; nt++) {
    const int col = col0 + wcol + nt * 32 + li;
    const bool col_ok = col < p.n;
    const int colc = col_ok ? col : p.n - 1;
    long long ybase;     // offset of (row 0, this column) in Y
    long long ystride;   // distance between consecutive rows in Y
    if (CONV) {
      const unsigned ohw = (unsigned)(p.cv.oh * p.cv.ow);
      const unsigned img = (unsigned)fdiv(colc, p.cv.fd_ohw);
      const unsigned q = (unsigned)colc - img * ohw;
      ybase = ((long long)img * p.cv.cout_total + (long long)bz * p.cv.cout_g) * ohw + q;
      ystride = ohw;
    } else {
      ybase = (long long)bz * p.sYb + colc;
      ystride = p.sY0;
    }
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
      const int rfirst = row0 + wrow + mt * 32 + 4 * half;
      // eight rows at a time keeps the 64-register tiles from spilling
#pragma unroll
      for (int hb = 0; hb < 2; hb++) {
        float cv[8], rv[8];
        if (p.C) {
#pragma unroll
          for (int j = 0; j < 8; j++) {
            int row = rfirst + 16 * hb + 8 * (j >> 2) + (j & 3);
            row = row < p.m ? row : p.m - 1;
            cv[j] = CONV ? p.C[bz * p.cv.cout_g + row]
                           : p.C[(long long)row * p.sC0 + (long long)colc * p.sC1];
          }
        }
        if (p.R) {
#pragma unroll
          for (int j = 0; j < 8; j++) {
            int row = rfirst + 16 * hb + 8 * (j >> 2) + (j & 3);
            row = row < p.m ? row : p.m - 1;
            rv[j] = p.R[ybase + (long long)row * ystride];
          }
        }
#pragma unroll
        for (int j = 0; j < 8; j++) {
          const int row = rfirst + 16 * hb + 8 * (j >> 2) + (j & 3);
          float y = p.alpha * acc[mt][nt][8 * hb + j];
          if (p.C) y = __builtin_fmaf(cv[j], p.beta, y);
          if (p.R) y = y + rv[j];
          if (p.epilogue == WDH_EPI_RELU) y = relu_js(y);
          if (col_ok && row < p.m) p.Y[ybase + (long long)row * ystride] = y;
        }
      }
    }
  }
}

// ---- the kernel -------------------------------------------------------------
// Workgroups per CU the register budget must allow: the 64-accumulator tiles
// are held to 128 registers so that four of them share a CU, the
// 16-accumulator tiles to 64 registers so that eight do.
constexpr int min_blocks(int bm, int bn) {
  return (bm == 128 && bn == 128) ? 4 : (bm * bn <= 64 * 64 ? 8 : 1);
}

template <int BM, int BN, int WM, int WN, bool A_KC, int BMODE_, bool VEC>
__global__ __launch_bounds__(NTHREADS, min_blocks(BM, BN)) void contraction_kernel(Params p) {
  constexpr bool IM2COL_FAST = BMODE_ == B_IM2COL32 || BMODE_ == B_IM2COL64;
  constexpr bool IM2COL = IM2COL_FAST || BMODE_ == B_IM2COL_BIG;
  constexpr bool PIXELS = BMODE_ == B_PIXELS;
  constexpr bool CONV = IM2COL || PIXELS;  // Y is NCHW, the bias is per row
  constexpr bool B_IS_KC = BMODE_ == B_KC;
  // layout of the B tile in LDS: tile[column][k] for a k-contiguous B and for the
  // descriptor gather (whose threads hold consecutive k of one pixel)
  constexpr bool B_LDS_KC = B_IS_KC || IM2COL_FAST;
  static_assert(WM * WN == NTHREADS / 64, "four wavefronts");
  constexpr int MT = BM / (WM * 32), NT = BN / (WN * 32);
  static_assert(MT >= 1 && NT >= 1, "tile too small for the wavefront grid");
  constexpr int A_FLOATS = tile_floats(A_KC, BM);
  constexpr int B_FLOATS = tile_floats(B_LDS_KC, BN);
  constexpr int LDA = BM + MC_PAD, LDB = BN + MC_PAD;
  __shared__ __attribute__((aligned(16))) float lds_a[2][A_FLOATS];
  __shared__ __attribute__((aligned(16))) float lds_b[2][B_FLOATS];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int li = lane & 31, half = lane >> 5;
  const int wrow = wm * (MT * 32), wcol = wn * (NT * 32);

  // which tile, and which part of K
  const TileWork tw = decode_work(p);
  const bool whole = tw.whole;
  const int lin = tw.lin, chunk = tw.chunk, bz = tw.bz;
  const int row0 = tw.tm * BM, col0 = tw.tn * BN;

  const float *A = p.A + (long long)bz * p.sAb;
  const float *B = p.B + (long long)bz * p.sBb;
  const long long lda = A_KC ? p.sA0 : p.sA1;
  const long long ldb = B_IS_KC ? p.sB1 : p.sB0;

  // this workgroup's share of K
  const int kbeg = whole ? 0 : chunk * p.kchunk;
  const int kend = whole ? p.k : (kbeg + p.kchunk < p.k ? kbeg + p.kchunk : p.k);

  // ---- descriptor fetch plans: one byte offset per 16-byte piece -------------
  // Every operand below 2 GiB takes this path, edge tiles included.  Rows of a
  // row-major-in-K operand past the edge are clamped; an operand that is
  // contiguous along M or N simply reads on past its last row or column, into
  // the next k row (or, past the end of the matrix, zeros from the descriptor's
  // bounds check).  Either way the surplus rows and columns only feed products
  // that are never stored.
  const bool a_fast = p.fast;
  const bool b_fast = p.fast && BMODE_ != B_IM2COL_BIG;
  int voff_a[BM / 64], voff_b[BN / 64];
  if (A_KC) {
#pragma unroll
    for (int i = 0; i < BM / 64; i++) {
      int r = row0 + (tid >> 2) + i * 64;
      r = r < p.m ? r : p.m - 1;
      voff_a[i] = (int)(((long long)r * lda + (tid & 3) * 4) * 4);
    }
  } else {
    constexpr int TPR = BM / 4, RPP = NTHREADS / TPR;
#pragma unroll
    for (int i = 0; i < BM / 64; i++)
      voff_a[i] = (int)(((long long)(tid / TPR + i * RPP) * lda + row0 + (tid % TPR) * 4) * 4);
  }
  if (B_IS_KC) {
#pragma unroll
    for (int i = 0; i < BN / 64; i++) {
      int c = col0 + (tid >> 2) + i * 64;
      c = c < p.n ? c : p.n - 1;
      voff_b[i] = (int)(((long long)c * ldb + (tid & 3) * 4) * 4);
    }
  } else if (!IM2COL) {
    constexpr int TPR = BN / 4, RPP = NTHREADS / TPR;
    // B_PIXELS: column = pixel index over the batch; its four pixels share an image
    long long colpos = col0 + (tid % TPR) * 4;
    if (PIXELS) {
      const unsigned plane = (unsigned)(p.cv.h * p.cv.w);
      const unsigned img = (unsigned)fdiv((int)colpos, p.cv.fd_plane);
      colpos = (long long)img * p.cv.c_total * plane + ((unsigned)colpos - img * plane);
    }
#pragma unroll
    for (int i = 0; i < BN / 64; i++)
      voff_b[i] = (int)(((long long)(tid / TPR + i * RPP) * ldb + colpos) * 4);
  }
  const rsrc_t rsrc_a = make_rsrc(A, p.a_bytes);

  // ---- im2col: what this thread's pixel looks like ----------------------------
  PixelCtx px = {p.B, 0, 0, 0, 0ull};
  PixelFast pf = {0, 0xffffffffu, 0xffffffffu};
  const float *bbase = B;  // base of the B descriptor
  if (IM2COL) {
    const unsigned P = (unsigned)col0 + (unsigned)(tid % BN);  // npix < 2^31
    const long long plane = (long long)p.cv.h * p.cv.w;
    const int bias = p.cv.pt * p.cv.w + p.cv.pl;  // makes every corner offset >= 0
    px.xbase = p.B + (long long)bz * p.cv.c_in_g * plane;
    bbase = px.xbase - bias;
    if (P < (unsigned)p.cv.npix) {
      const unsigned ohw = (unsigned)(p.cv.oh * p.cv.ow);
      const unsigned img = (unsigned)fdiv((int)P, p.cv.fd_ohw);
      const unsigned q = P - img * ohw;
      const int oy = fdiv((int)q, p.cv.fd_ow), ox = (int)q - oy * p.cv.ow;
      const long long img_off = (long long)img * p.cv.c_total * plane;
      px.iy0 = oy * p.cv.sh - p.cv.pt;
      px.ix0 = ox * p.cv.sw - p.cv.pl;
      px.pbase = px.iy0 * p.cv.w + px.ix0;
      if (IM2COL_FAST) {
        pf.valid = (int)((img_off + px.pbase + bias) * 4);
        // which taps of this pixel fall inside the input: rows first, then columns
        unsigned long long inside = 0;
        int t = 0;
        for (int ky = 0; ky < p.cv.kh; ky++) {
          const bool row_in = (unsigned)(px.iy0 + ky * p.cv.dh) < (unsigned)p.cv.h;
          for (int kx = 0; kx < p.cv.kw; kx++, t++)
            if (row_in && (unsigned)(px.ix0 + kx * p.cv.dw) < (unsigned)p.cv.w)
              inside |= 1ull << t;
        }
        pf.pad_lo = ~(unsigned)inside;
        pf.pad_hi = ~(unsigned)(inside >> 32);
      } else {
        px.xbase += img_off;
        px.mask = 1ull;
      }
    }
  }
  // conv: p.b_bytes is group 0's window, later groups start further into X
  const int b_window =
      CONV ? p.b_bytes - (int)((long long)bz * p.cv.c_in_g * p.cv.h * p.cv.w * 4) : p.b_bytes;
  const rsrc_t rsrc_b = make_rsrc(bbase, b_window);
  // first of the L consecutive k rows this wavefront gathers in each slab
  const int kgroup0 = IM2COL ? __builtin_amdgcn_readfirstlane(tid / BN) * (BK / (NTHREADS / BN)) : 0;

  f32x16 acc[MT][NT];
#pragma unroll
  for (int a = 0; a < MT; a++)
#pragma unroll
    for (int b = 0; b < NT; b++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[a][b][r] = 0.0f;

  // Registers that carry one fetched K slab from global memory to LDS.
  struct Staged {
    f32x4 a[BM / 64], b[BN / 64];
    unsigned ok;  // flat im2col only: which fetched taps lie inside the input
  };
  // Descriptor-only fetch: legal for a slab that lies fully inside K when
  // both operands qualify (all_fast).
  auto fetch_fast = [&](int k0, Staged &st) {
    fetch_rows_fast<BM, VEC>(rsrc_a, voff_a, A_KC ? k0 * 4 : (int)(k0 * lda * 4), st.a);
    if (IM2COL_FAST)
      fetch_im2col_fast<BN, BMODE_ == B_IM2COL64>(rsrc_b, p.cv.ktab, pf, k0 + kgroup0, st.b);
    else if (!IM2COL)
      fetch_rows_fast<BN, VEC>(rsrc_b, voff_b, B_IS_KC ? k0 * 4 : (int)(k0 * ldb * 4), st.b);
  };
  // Fetch that copes with everything: ragged last slab, edge tiles, huge operands.
  auto fetch_any = [&](int k0, Staged &st) {
    const bool full = k0 + BK <= kend;
    if (a_fast && full) {
      fetch_rows_fast<BM, VEC>(rsrc_a, voff_a, A_KC ? k0 * 4 : (int)(k0 * lda * 4), st.a);
    } else if (A_KC) {
      fetch_kc<BM, VEC>(A, lda, row0, p.m, k0, kend, tid, st.a);
    } else {
      fetch_mc<BM, VEC>(A, lda, row0, p.m, k0, kend, tid, st.a);
    }
    if (IM2COL_FAST) {
      // padding entries of the tap table read as 0, so a ragged K needs no care
      fetch_im2col_fast<BN, BMODE_ == B_IM2COL64>(rsrc_b, p.cv.ktab, pf, k0 + kgroup0, st.b);
    } else if (IM2COL) {
      st.ok = fetch_im2col<BN>(p.cv, px, k0, kend, tid, st.b);
    } else if ((b_fast && full) || PIXELS) {
      fetch_rows_fast<BN, VEC>(rsrc_b, voff_b, B_IS_KC ? k0 * 4 : (int)(k0 * ldb * 4), st.b);
    } else if (B_IS_KC) {
      fetch_kc<BN, VEC>(B, ldb, col0, p.n, k0, kend, tid, st.b);
    } else {
      fetch_mc<BN, VEC>(B, ldb, col0, p.n, k0, kend, tid, st.b);
    }
  };
  auto stash = [&](int buf, const Staged &st) {
    if (A_KC)
      stash_kc<BM>(lds_a[buf], tid, st.a);
    else
      stash_mc<BM>(lds_a[buf], tid, st.a);
    if (B_IS_KC)
      stash_kc<BN>(lds_b[buf], tid, st.b);
    else if (IM2COL_FAST)
      stash_im2col_fast<BN>(lds_b[buf], tid, st.b);
    else if (IM2COL)
      stash_im2col<BN>(lds_b[buf], tid, st.b, st.ok);
    else
      stash_mc<BN>(lds_b[buf], tid, st.b);
  };
  // One K slab from LDS buffer `cur` through the matrix cores.
  auto compute = [&](int cur) {
    const float *ta = lds_a[cur];
    const float *tb = lds_b[cur];
    f32x4 av[MT][2], bv[NT][2];
    if (A_KC) {
#pragma unroll
      for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int j = 0; j < 2; j++)
          av[mt][j] = *reinterpret_cast<const f32x4 *>(
              ta + (wrow + mt * 32 + li) * LDK + 8 * j + 4 * half);
    }
    if (B_LDS_KC) {
#pragma unroll
      for (int nt = 0; nt < NT; nt++)
#pragma unroll
        for (int j = 0; j < 2; j++)
          bv[nt][j] = *reinterpret_cast<const f32x4 *>(
              tb + (wcol + nt * 32 + li) * LDK + 8 * j + 4 * half);
    }
#pragma unroll
    for (int st = 0; st < 8; st++) {
      const int kk = 8 * (st >> 2) + 4 * half + (st & 3);
      float a_el[MT], b_el[NT];
#pragma unroll
      for (int mt = 0; mt < MT; mt++)
        a_el[mt] = A_KC ? av[mt][st >> 2][st & 3] : ta[kk * LDA + wrow + mt * 32 + li];
#pragma unroll
      for (int nt = 0; nt < NT; nt++)
        b_el[nt] = B_LDS_KC ? bv[nt][st >> 2][st & 3] : tb[kk * LDB + wcol + nt * 32 + li];
#pragma unroll
      for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int nt = 0; nt < NT; nt++)
          acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(a_el[mt], b_el[nt],
                                                             acc[mt][nt], 0, 0, 0);
    }
  };

  // Slab s+1 travels global -> registers while slab s runs through the matrix
  // cores, then goes to the other LDS buffer.  (A second slab in flight was
  // measured and bought nothing.)  The main loop takes two slabs per trip, so
  // that LDS buffer indices are compile-time constants, and contains
  // descriptor fetches only; the few slabs it leaves over (and every slab of a
  // workgroup that cannot use descriptors) run in the general loop below it.
  const int nslabs = (kend - kbeg + BK - 1) / BK;
  const int nfull = (kend - kbeg) / BK;
  const bool all_fast = a_fast && b_fast && !(IM2COL && !IM2COL_FAST);
  const int nfast = all_fast ? nfull - 1 : 0;  // steps whose next slab is a full one
  Staged st0;
  fetch_any(kbeg, st0);
  stash(0, st0);
  __syncthreads();
  int s = 0;
  // The scheduling fences keep the compiler from sinking the loads below the
  // matrix-core work they are meant to overlap.
  for (; s + 2 <= nfast; s += 2) {
    fetch_fast(kbeg + (s + 1) * BK, st0);
    __builtin_amdgcn_sched_barrier(0);
    compute(0);
    stash(1, st0);
    __syncthreads();
    fetch_fast(kbeg + (s + 2) * BK, st0);
    __builtin_amdgcn_sched_barrier(0);
    compute(1);
    stash(0, st0);
    __syncthreads();
  }
  for (; s < nslabs; s++) {
    const int cur = s & 1;
    if (s + 1 < nslabs) fetch_any(kbeg + (s + 1) * BK, st0);
    compute(cur);
    if (s + 1 < nslabs) stash(cur ^ 1, st0);
    __syncthreads();
  }

  static_assert(2 * A_FLOATS >= 2 * STAGE_FLOATS && 2 * B_FLOATS >= 2 * STAGE_FLOATS, "epilogue staging");
  finish_tile<BM, BN, WM, WN, CONV>(p, acc, whole, lin, chunk, bz, row0, col0,
                                    (wave < 2 ? &lds_a[0][0] : &lds_b[0][0]) + (wave & 1) * STAGE_FLOATS);
}

// ---- 3x3, stride 1, dilation 1: taps read from an input tile staged in LDS -------
// Same contraction as the gathered form (M = output channels, N = pixels in
// (image, oy, ox) order, K = (channel, ky, kx)), same tiles, same work plan and
// epilogue.  What differs is how B reaches the matrix cores.  K advances in blocks of
// 8 input channels (72 k).  For a block, the workgroup copies the input rows its BN
// pixels touch -- whole rows, as they lie in X, with 16-, 8- or 4-byte loads -- into
// LDS: xs[channel][slot][column], where consecutive output rows of an image share
// slots (output row R of the tile, tap row ky -> slot (R - R0) + ky + 2 * (images
// after the tile's first)), columns left and right of the row and rows above and
// below the image are zero (requested through offsets outside the descriptor, so they
// cost no memory traffic).  A lane then reads tap (ky, kx) of channel c of its pixel at
// a fixed distance from its pixel's corner: one LDS address per tap and lane, computed
// once per tile, plus an immediate per channel.  No tap table, no padding masks, no
// address arithmetic in the loop; each input element is fetched once per tile and
// block instead of once per tap, and a block (36 MFMA steps) costs two barriers.
// The weights of a block, a[row][72 k] in the order they lie in W, are read with
// 16-byte LDS loads: the lower half of a wavefront multiplies channels 0-3 of the
// block (k 0..35), the upper half channels 4-7 (k 36..71), so the two k of one MFMA
// step are (c, tap) and (c + 4, tap).
constexpr int HALO_CB = 8;                 // channels per K block
constexpr int HALO_KB = HALO_CB * 9;       // k per block
constexpr int HALO_ROWA = HALO_KB + 4;     // weight tile row stride (floats)
constexpr int HALO_AROWS = 14;             // weight rows per pass: 256 threads = 14 rows x 18 pieces
// floats per channel of the input tile; 32 mod 64 so that the two halves of a
// wavefront (channels c and c + 4) fall on different LDS banks
constexpr int halo_plane(int bn) { return bn <= 64 ? 480 : (bn <= 128 ? 544 : 672); }
// most 16/8/4-byte pieces of the input tile a thread fetches per block (the launch says
// how many of them a geometry needs)
constexpr int halo_units(int vecw, int bn) {
  return vecw == 4 ? (bn <= 64 ? 4 : (bn <= 128 ? 5 : 6))
                   : (vecw == 2 ? (bn <= 64 ? 4 : (bn <= 128 ? 6 : 8)) : (bn <= 64 ? 5 : (bn <= 128 ? 8 : 12)));
}

typedef float f32x2 __attribute__((ext_vector_type(2)));
template <int VECW> struct HaloPiece;
template <> struct HaloPiece<4> {
  typedef f32x4 type;
  static __device__ __forceinline__ type load(rsrc_t r, int voff, int soff) {
    return buf_load4(r, voff, soff);
  }
};
template <> struct HaloPiece<2> {
  typedef f32x2 type;
  static __device__ __forceinline__ type load(rsrc_t r, int voff, int soff) {
    return __builtin_bit_cast(f32x2, __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, 0));
  }
};
template <> struct HaloPiece<1> {
  typedef float type;
  static __device__ __forceinline__ type load(rsrc_t r, int voff, int soff) {
    return buf_load(r, voff, soff);
  }
};

template <int BM, int BN, int WM, int WN, int VECW>
__global__ __launch_bounds__(NTHREADS, BM == 64 ? (BN == 64 ? 4 : (BN == 128 ? 3 : 2)) : 2) void conv3x3_halo_kernel(Params p) {
  static_assert(WM * WN == NTHREADS / 64, "four wavefronts");
  constexpr int MT = BM / (WM * 32), NT = BN / (WN * 32);
  constexpr int PLANE = halo_plane(BN);
  constexpr int AU = (BM + HALO_AROWS - 1) / HALO_AROWS;  // weight pieces per thread and block
  constexpr int XU = halo_units(VECW, BN);
  typedef typename HaloPiece<VECW>::type xpiece;
  __shared__ __attribute__((aligned(16))) float as[AU * HALO_AROWS * HALO_ROWA];
  __shared__ __attribute__((aligned(16))) float xs[HALO_CB * PLANE + 4];  // + a dump cell for idle pieces

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int li = lane & 31, half = lane >> 5;
  const int wrow = wm * (MT * 32), wcol = wn * (NT * 32);

  const TileWork t = decode_work(p);
  const int row0 = t.tm * BM, col0 = t.tn * BN;
  const int kbeg = t.whole ? 0 : t.chunk * p.kchunk;
  const int kend = t.whole ? p.k : (kbeg + p.kchunk < p.k ? kbeg + p.kchunk : p.k);

  const ConvGeom &cv = p.cv;
  const int plane_in = cv.h * cv.w;
  // first output row of the tile (rows numbered through the batch) and its image
  const int R0 = fdiv(col0, cv.fd_ow);
  const int img0 = fdiv(R0, cv.fd_oh);

  // ---- weights: piece (row r0 + 14 i, k 4q .. 4q+3) of the block -----------------
  // (threads 252..255 repeat pieces of row 13: same values to the same cells)
  const int q = tid % 18, r0 = tid / 18 < HALO_AROWS ? tid / 18 : HALO_AROWS - 1;
  int voff_a[AU];
#pragma unroll
  for (int i = 0; i < AU; i++) {
    int r = row0 + r0 + HALO_AROWS * i;
    r = r < p.m ? r : p.m - 1;  // rows past the edge are never stored
    voff_a[i] = (r * p.k + 4 * q) * 4;
  }
  const int lds_a_w = (r0 * HALO_ROWA + 4 * q) * 4;
  const rsrc_t rsrc_a = make_rsrc(p.A + (long long)t.bz * p.sAb, p.a_bytes);

  // ---- input rows: piece u = tid + 256 i -> (channel, slot, column group) ---------
  const int pg = cv.pitch / VECW;       // pieces per row
  const int upc = cv.slots * pg;        // pieces per channel
  const int first_rows = (img0 + 1) * cv.oh - R0;  // output rows from R0 to the end of its image
  const int xu = cv.units;  // pieces per thread this geometry needs (<= XU)
  int voff_x[XU], lds_x_w[XU];
#pragma unroll
  for (int i = 0; i < XU; i++) {
    const int u = tid + NTHREADS * i;
    const int c = fdiv(u, cv.fd_upc), rem = u - c * upc;
    const int slot = fdiv(rem, cv.fd_pg), cg = rem - slot * pg;
    // which input row the slot holds
    int d, iy;
    if (slot < first_rows + 2) {
      d = 0;
      iy = (R0 - img0 * cv.oh) - cv.pt + slot;
    } else {
      const int s2 = slot - first_rows - 2;
      const int dd = fdiv(s2, cv.fd_oh2);
      d = 1 + dd;
      iy = s2 - dd * (cv.oh + 2) - cv.pt;
    }
    const int img = img0 + d;
    const int ix = cg * VECW - cv.col0;
    const bool live = c < HALO_CB;
    const bool data = live && (long long)img * cv.oh * cv.ow < cv.npix && iy >= 0 && iy < cv.h &&
                      ix >= 0 && ix + VECW <= cv.w;
    voff_x[i] = data ? (((img * cv.c_total + c) * cv.h + iy) * cv.w + ix) * 4 : BUF_OOB;
    lds_x_w[i] = live ? (c * PLANE + slot * cv.pitch + cg * VECW) * 4 : HALO_CB * PLANE * 4;
  }
  const long long group_off = (long long)t.bz * cv.c_in_g * plane_in;
  const rsrc_t rsrc_x = make_rsrc(p.B + group_off, p.b_bytes - (int)(group_off * 4));

  // ---- where a lane finds its operands in LDS -------------------------------------
  int lds_a_r[MT];
#pragma unroll
  for (int mt = 0; mt < MT; mt++)
    lds_a_r[mt] = ((wrow + mt * 32 + li) * HALO_ROWA + 36 * half) * 4;
  int lds_b_r[NT][9];
#pragma unroll
  for (int nt = 0; nt < NT; nt++) {
    int P = col0 + wcol + nt * 32 + li;
    P = P < (int)cv.npix ? P : (int)cv.npix - 1;  // lanes past the edge are never stored
    const int R = fdiv(P, cv.fd_ow), ox = P - R * cv.ow;
    const int slot0 = (R - R0) + 2 * (fdiv(R, cv.fd_oh) - img0);
    const int corner = (4 * half * PLANE + slot0 * cv.pitch + cv.col0 - cv.pl + ox) * 4;
#pragma unroll
    for (int tap = 0; tap < 9; tap++)
      lds_b_r[nt][tap] = corner + ((tap / 3) * cv.pitch + tap % 3) * 4;
  }

  f32x16 acc[MT][NT];
#pragma unroll
  for (int a = 0; a < MT; a++)
#pragma unroll
    for (int b = 0; b < NT; b++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[a][b][r] = 0.0f;

  f32x4 ra[AU];
  xpiece rx[XU];
  auto fetch = [&](int k0) {
    const int soff_a = k0 * 4;
    const int soff_x = (k0 / 9) * plane_in * 4;
#pragma unroll
    for (int i = 0; i < AU; i++) ra[i] = buf_load4(rsrc_a, voff_a[i], soff_a);
#pragma unroll
    for (int i = 0; i < XU; i++)
      if (i < xu) rx[i] = HaloPiece<VECW>::load(rsrc_x, voff_x[i], soff_x);
  };
  auto stash = [&]() {
    char *const as_b = reinterpret_cast<char *>(as);
    char *const xs_b = reinterpret_cast<char *>(xs);
#pragma unroll
    for (int i = 0; i < AU; i++)
      *reinterpret_cast<f32x4 *>(as_b + lds_a_w + i * (HALO_AROWS * HALO_ROWA * 4)) = ra[i];
#pragma unroll
    for (int i = 0; i < XU; i++)
      if (i < xu) *reinterpret_cast<xpiece *>(xs_b + lds_x_w[i]) = rx[i];
  };
  auto compute = [&]() {
    const char *const as_b = reinterpret_cast<const char *>(as);
    const char *const xs_b = reinterpret_cast<const char *>(xs);
#pragma unroll
    for (int j = 0; j < 9; j++) {
      f32x4 av[MT];
#pragma unroll
      for (int mt = 0; mt < MT; mt++)
        av[mt] = *reinterpret_cast<const f32x4 *>(as_b + lds_a_r[mt] + 16 * j);
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const int kk = 4 * j + e, c = kk / 9, tap = kk % 9;
        float b_el[NT];
#pragma unroll
        for (int nt = 0; nt < NT; nt++)
          b_el[nt] = *reinterpret_cast<const float *>(xs_b + lds_b_r[nt][tap] + c * (PLANE * 4));
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
          for (int nt = 0; nt < NT; nt++)
            acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[mt][e], b_el[nt], acc[mt][nt], 0, 0, 0);
      }
    }
  };

  // One LDS buffer: block b+1 travels global -> registers while block b runs through
  // the matrix cores, and is written to LDS once every wavefront has finished reading.
  fetch(kbeg);
  for (int k0 = kbeg; k0 < kend; k0 += HALO_KB) {
    if (k0 != kbeg) __syncthreads();
    stash();
    __syncthreads();
    if (k0 + HALO_KB < kend) fetch(k0 + HALO_KB);
    __builtin_amdgcn_sched_barrier(0);
    compute();
  }
  static_assert(AU * HALO_AROWS * HALO_ROWA >= 4 * STAGE_FLOATS, "epilogue staging");
  finish_tile<BM, BN, WM, WN, true>(p, acc, t.whole, t.lin, t.chunk, t.bz, row0, col0,
                                    as + (threadIdx.x >> 6) * STAGE_FLOATS);
}

// ---- small products: K cut across the wavefronts of one workgroup -------------------
// A product with few result tiles (a transformer's 850x256 linear layers, attention x V,
// a classifier head) cannot fill the chip with 64x64 tiles, and cutting K across
// workgroups costs a second launch to add the pieces up.  Here a workgroup of 16
// wavefronts owns one 32x32 block of the result and every wavefront multiplies a 1/16
// share of K for the whole block: operand fragments go from global memory straight into
// the lanes the matrix core reads them from (A rows and k-contiguous B columns as 16-byte
// pieces, an n-contiguous B as one element per k), the 16 partial blocks meet in LDS and
// thread t adds up element t in wavefront order -- a fixed order, so results do not
// depend on scheduling -- before the usual epilogue.  One launch, no workspace.
constexpr int WS_WAVES = 16;
template <bool B_IS_KC, bool VEC>
__device__ __forceinline__ void wavesplit_block(const Params &p, int block) {
  __shared__ float part[WS_WAVES][16][64];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int li = lane & 31, half = lane >> 5;
  const int tiles_per_z = p.tiles_m * p.tiles_n;
  const int bz = fdiv(block, p.fd_tiles_per_z);
  const int tile = block - bz * tiles_per_z;
  const int tm = fdiv(tile, p.fd_group), tn = tile - tm * p.tiles_n;  // fd_group: division by tiles_n
  const int row0 = tm * 32, col0 = tn * 32;

  const rsrc_t rsrc_a = make_rsrc(p.A + (long long)bz * p.sAb, p.a_bytes);
  const rsrc_t rsrc_b = make_rsrc(p.B + (long long)bz * p.sBb, p.b_bytes);
  int ra = row0 + li;
  ra = ra < p.m ? ra : p.m - 1;  // rows and columns past the edge are never stored
  int cb = col0 + li;
  cb = cb < p.n ? cb : p.n - 1;
  const int lda = (int)p.sA0, ldb = B_IS_KC ? (int)p.sB1 : (int)p.sB0;
  const int voff_a = (ra * lda + 4 * half) * 4;
  const int voff_b = B_IS_KC ? (cb * ldb + 4 * half) * 4 : (4 * half * ldb + cb) * 4;

  // this wavefront's share of K, in slabs of 16 (made scalar explicitly: K offsets of loads are scalar operands)
  const int kbeg = __builtin_amdgcn_readfirstlane(wave) * p.kchunk;
  const int kend = kbeg + p.kchunk < p.k ? kbeg + p.kchunk : p.k;

  f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.0f;

  struct Frag {
    f32x4 a[2], b[2];
  };
  // the 16 k of a slab are consumed in the order k = 8*(s/4) + 4*half + s%4, s = 0..7
  auto fetch = [&](int k0, Frag &f) {
#pragma unroll
    for (int j = 0; j < 2; j++) {
      // (rows whose length is no multiple of four floats are not 16-byte aligned)
      if (VEC) {
        f.a[j] = buf_load4(rsrc_a, voff_a, (k0 + 8 * j) * 4);
      } else {
#pragma unroll
        for (int e = 0; e < 4; e++) f.a[j][e] = buf_load(rsrc_a, voff_a + 4 * e, (k0 + 8 * j) * 4);
      }
      if (B_IS_KC && VEC) {
        f.b[j] = buf_load4(rsrc_b, voff_b, (k0 + 8 * j) * 4);
      } else if (B_IS_KC) {
#pragma unroll
        for (int e = 0; e < 4; e++) f.b[j][e] = buf_load(rsrc_b, voff_b + 4 * e, (k0 + 8 * j) * 4);
      } else {
#pragma unroll
        for (int e = 0; e < 4; e++) f.b[j][e] = buf_load(rsrc_b, voff_b, (k0 + 8 * j + e) * ldb * 4);
      }
    }
  };
  // (a slab is touched only here, when it is used: the requests above stay requests)
  auto multiply = [&](Frag &f, int k0) {
    if (k0 + BK > p.k) {
      // ragged end of K: what lies past it belongs to the next row (or to nobody)
#pragma unroll
      for (int j = 0; j < 2; j++)
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (k0 + 8 * j + 4 * half + e >= p.k) {
            f.a[j][e] = 0.0f;
            f.b[j][e] = 0.0f;
          }
    }
#pragma unroll
    for (int s = 0; s < 8; s++)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(f.a[s >> 2][s & 3], f.b[s >> 2][s & 3], acc, 0, 0, 0);
  };
  // (four slabs in flight per wavefront instead of two, in whole branch-free trips, did not
  // help: 850x256x2048 21.4 us against 20.5, 850x256x1024 12.4 against 11.1)
  if (kbeg < kend) {
    Frag cur, nxt;
    fetch(kbeg, cur);
    for (int k0 = kbeg; k0 < kend; k0 += BK) {
      if (k0 + BK < kend) fetch(k0 + BK, nxt);
      multiply(cur, k0);
      cur = nxt;
    }
  }
#pragma unroll
  for (int r = 0; r < 16; r++) part[wave][r][lane] = acc[r];
  __syncthreads();

  // thread t owns element t of the block: accumulator register r = t / 64 of lane t % 64
  const int r = tid >> 6;
  float sum = 0.0f;
#pragma unroll
  for (int w = 0; w < WS_WAVES; w++) sum += part[w][r][lane];
  const int row = row0 + 8 * (r >> 2) + 4 * half + (r & 3), col = col0 + li;
  if (row >= p.m || col >= p.n) return;
  float y = p.alpha * sum;
  if (p.C) y = __builtin_fmaf(p.C[(long long)row * p.sC0 + (long long)col * p.sC1], p.beta, y);
  const long long off = (long long)bz * p.sYb + (long long)row * p.sY0 + col;
  if (p.R) y = y + p.R[off];
  if (p.epilogue == WDH_EPI_RELU) y = relu_js(y);
  p.Y[off] = y;
}

template <bool B_IS_KC, bool VEC>
__global__ __launch_bounds__(64 * WS_WAVES, 1) void gemm_wavesplit_kernel(Params p) {
  wavesplit_block<B_IS_KC, VEC>(p, (int)blockIdx.x);
}

// Several independent small products in one launch (the query, key and value projections
// of an attention block): the blocks of problem i follow those of problem i - 1 in the grid.
constexpr int GROUP_MAX = 6;
struct GroupParams {
  int count;
  int first[GROUP_MAX + 1];  // first block of each problem; first[count] = grid size
  Params p[GROUP_MAX];
};
template <bool B_IS_KC, bool VEC>
__global__ __launch_bounds__(64 * WS_WAVES, 1) void gemm_wavesplit_group_kernel(GroupParams g) {
  int i = 0;
#pragma unroll
  for (int j = 1; j < GROUP_MAX; j++)
    if (j < g.count && (int)blockIdx.x >= g.first[j]) i = j;
  wavesplit_block<B_IS_KC, VEC>(g.p[i], (int)blockIdx.x - g.first[i]);
}

// Reference-order scalar kernel for operands that are dense in neither index
// (never produced by the runner's dense tensors, kept so the entry point is total).
__global__ void contraction_strided_kernel(Params p) {
  long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  long long total = (long long)p.m * p.n;
  if (idx >= total) return;
  int bz = blockIdx.y;
  int i = (int)(idx / p.n), j = (int)(idx % p.n);
  const float *A = p.A + (long long)bz * p.sAb + (long long)i * p.sA0;
  const float *B = p.B + (long long)bz * p.sBb + (long long)j * p.sB1;
  float acc = 0.0f;
  for (int x = 0; x < p.k; x++)
    acc = __builtin_fmaf(A[(long long)x * p.sA1], B[(long long)x * p.sB0], acc);
  float y = p.alpha * acc;
  if (p.C) y = __builtin_fmaf(p.C[(long long)i * p.sC0 + (long long)j * p.sC1], p.beta, y);
  long long off = (long long)bz * p.sYb + (long long)i * p.sY0 + j;
  if (p.R) y = y + p.R[off];
  if (p.epilogue == WDH_EPI_RELU) y = relu_js(y);
  p.Y[off] = y;
}

// Second pass for the tail tiles: adds the chunks of each tile in index order
// (so the result does not depend on scheduling) and applies the epilogue.
// grid = (tail tiles, bm*bn/1024), 256 threads, 4 consecutive columns each.
template <bool CONV>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(Params p, int bm, int bn) {
  const int j = blockIdx.x;
  const int lin = p.full_tiles + j;
  const int tiles_per_z = p.tiles_m * p.tiles_n;
  const int bz = fdiv(lin, p.fd_tiles_per_z);
  int tm, tn;
  tile_coords(p, lin - bz * tiles_per_z, &tm, &tn);
  reduce_quad<CONV>(p, bm, bn, j, bz, tm, tn, ((int)blockIdx.y * 256 + (int)threadIdx.x) * 4);
}

// ---- host-side dispatch -------------------------------------------------------
enum TileId { T128x128 = 0, T64x256 = 1, T64x128 = 2, T64x64 = 3, T128x64 = 4 };
const int kTileM[] = {128, 64, 64, 64, 128};
const int kTileN[] = {128, 256, 128, 64, 64};

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
int g_forced_split = -1;  // >= 1: overrides the split-K heuristic
int g_descriptors = 1;    // 0: every operand is treated as if it spanned 2 GiB or more
// what launch_planned decided for the most recent launch (wdh_last_plan)
struct LastPlan { int bm, bn, split, form; long long full, tail; } g_last_plan = {};
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
int g_wide_stores = 1;    // 0: whole tiles store one element per lane and instruction

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

// How the tiles of one launch are spread over the chip.
struct WorkPlan {
  long long full;   // tiles computed by one workgroup each
  long long tail;   // tiles cut along K
  int split;        // chunks per tail tile
  int kchunk;       // K elements per chunk (a multiple of 16)
};

// A launch keeps every CU busy for ceil(tiles / CUs) tile times, so a tile count
// just above a multiple of the CU count wastes most of a round, and a CU that
// holds only one or two workgroups cannot hide their latencies.  Candidate
// plans -- nothing split, only the tiles beyond the last full round split, or
// every tile split -- are compared with a small model in microseconds: a CU
// works through its workgroups' K slabs at slab_us each, but never finishes
// sooner than `solo` times the longest single workgroup (the slow-down of a
// workgroup that runs alone on a CU); every workgroup adds a start-up/epilogue
// cost and a split adds the reduce pass over the partial sums.
WorkPlan plan_work(long long tiles, int k, int bm, int bn, bool gather, int kgran = BK) {
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

// Plans the work of one launch, provides the partial-sum workspace, starts the main
// kernel through `start(grid)` and, if tiles were cut along K, the reduce pass.
template <int BM, int BN, typename Start>
int launch_planned(Params &p, int nz, bool conv, int kgran, Start start) {
  p.tiles_m = (p.m + BM - 1) / BM;
  p.tiles_n = (p.n + BN - 1) / BN;
  const long long tiles = (long long)p.tiles_m * p.tiles_n * nz;
  const WorkPlan w = plan_work(tiles, p.k, BM, BN, conv, kgran);
  const long long blocks = w.full + w.tail * w.split;
  if (blocks > 0x7fffffffLL)
    return wdh::fail(WDH_EINVAL, "contraction: %lld workgroups exceed the grid limit", blocks);
  p.nz = nz;
  p.full_tiles = (int)w.full;
  p.tail_tiles = (int)w.tail;
  p.tail_split = w.split;
  p.kchunk = w.kchunk;
  g_last_plan = {BM, BN, w.split, g_last_form, w.full, w.tail};
  p.fd_tiles_per_z = make_fastdiv((long long)p.tiles_m * p.tiles_n);
  p.fd_tail_tiles = make_fastdiv(w.tail > 0 ? w.tail : 1);
  p.fd_group = make_fastdiv((long long)TILE_GROUP * p.tiles_n);
  p.fd_last_rows = make_fastdiv(p.tiles_m % TILE_GROUP ? p.tiles_m % TILE_GROUP : 1);
  wdh_buf pooled = 0;
  if (w.tail > 0) {
    const size_t need = (size_t)w.tail * w.split * BM * BN * sizeof(float);
    if (g_static_scratch) {
      // the caller cannot allocate: the chunks' sums go to the library's static workspace,
      // through its device address (every element a reduce pass reads is written first by
      // the launch before it, so nothing has to be cleared between calls)
      if (need > WDH_STATIC_SCRATCH_BYTES)
        return wdh::fail(WDH_EINVAL,
                         "wdh_gemm_static: this problem is cut into %lld x %d partial tiles of %d x %d, "
                         "%zu bytes; the static workspace holds %zu (set split_k to 1 to run it unsplit)",
                         w.tail, w.split, BM, BN, need, (size_t)WDH_STATIC_SCRATCH_BYTES);
      p.partial = g_scratch_ptr[wdh::device()];
      if (!p.partial) return wdh::fail(WDH_ESTATE, "wdh_gemm_static: no static workspace on device %d", wdh::device());
    } else {
      pooled = wdh_alloc(need);
      if (!pooled) return WDH_ENOMEM;
      p.partial = (float *)wdh::resolve(pooled, nullptr);
    }
  }
  start(dim3((unsigned)blocks));
  hipError_t e = hipGetLastError();
  if (e == hipSuccess && w.tail > 0) {
    dim3 rgrid((unsigned)w.tail, (unsigned)(BM * BN / 1024));
    if (conv)
      hipLaunchKernelGGL(splitk_reduce_kernel<true>, rgrid, dim3(256), 0, wdh::stream(), p,
                         BM, BN);
    else
      hipLaunchKernelGGL(splitk_reduce_kernel<false>, rgrid, dim3(256), 0, wdh::stream(), p,
                         BM, BN);
    e = hipGetLastError();
  }
  // The scratch block goes back to the pool right away: whoever gets it next
  // touches it through the same stream, behind the two kernels above.
  if (pooled) (void)wdh_free(pooled);
  if (e != hipSuccess)
    return wdh::fail(WDH_EHIP, "contraction launch failed: %s", hipGetErrorString(e));
  return WDH_OK;
}

template <int BM, int BN, int WM, int WN, bool A_KC, int BMODE>
int launch_tile(Params &p, int nz, bool vec) {
  g_last_form = BMODE;
  return launch_planned<BM, BN>(p, nz, BMODE >= B_IM2COL32, BK, [&](dim3 grid) {
    if (vec)
      hipLaunchKernelGGL((contraction_kernel<BM, BN, WM, WN, A_KC, BMODE, true>), grid,
                         dim3(NTHREADS), 0, wdh::stream(), p);
    else
      hipLaunchKernelGGL((contraction_kernel<BM, BN, WM, WN, A_KC, BMODE, false>), grid,
                         dim3(NTHREADS), 0, wdh::stream(), p);
  });
}

template <int BM, int BN, int WM, int WN>
int launch_halo_tile(Params &p, int nz, int vecw) {
  g_last_form = WDH_FORM_CONV3X3_LDS;
  return launch_planned<BM, BN>(p, nz, true, HALO_KB, [&](dim3 grid) {
    if (vecw == 4)
      hipLaunchKernelGGL((conv3x3_halo_kernel<BM, BN, WM, WN, 4>), grid, dim3(NTHREADS), 0,
                         wdh::stream(), p);
    else if (vecw == 2)
      hipLaunchKernelGGL((conv3x3_halo_kernel<BM, BN, WM, WN, 2>), grid, dim3(NTHREADS), 0,
                         wdh::stream(), p);
    else
      hipLaunchKernelGGL((conv3x3_halo_kernel<BM, BN, WM, WN, 1>), grid, dim3(NTHREADS), 0,
                         wdh::stream(), p);
  });
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

template <bool A_KC, int BMODE>
int launch(Params &p, int nz, bool vec) {
  // Convs measured best on 64x64 tiles at nearly every ResNet-50 layer shape;
  // Gemm/MatMul use the cost model.
  const bool conv = BMODE >= B_IM2COL32;
  // deep convs with many output channels (ResNet stage 3/4 3x3) gain ~5 % from two
  // accumulator tiles per wavefront
  const TileId conv_tile = (p.m >= 256 && p.k >= 2048) ? T128x64 : T64x64;
  TileId t = g_forced_tile >= 0 ? (TileId)g_forced_tile
                                : (conv ? conv_tile : pick_tile(p.m, p.n, nz));
  switch (t) {
    case T128x128: return launch_tile<128, 128, 2, 2, A_KC, BMODE>(p, nz, vec);
    case T64x256: return launch_tile<64, 256, 1, 4, A_KC, BMODE>(p, nz, vec);
    case T64x128: return launch_tile<64, 128, 1, 4, A_KC, BMODE>(p, nz, vec);
    case T128x64: return launch_tile<128, 64, 2, 2, A_KC, BMODE>(p, nz, vec);
    default: return launch_tile<64, 64, 2, 2, A_KC, BMODE>(p, nz, vec);
  }
}

bool aligned16(const void *ptr) { return ((uintptr_t)ptr & 15) == 0; }

// Largest element offset the strided view touches, for bounds checking.
long long span(long long nb, long long sb, long long n0, long long s0,
               long long n1, long long s1) {
  return (nb - 1) * sb + (n0 - 1) * s0 + (n1 - 1) * s1 + 1;
}

}  // namespace

using wdh::fail;

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
  if (strcmp(name, "conv3x3_halo") == 0) {
    if (value != 0 && value != 1)
      return fail(WDH_EINVAL, "wdh_set_option: conv3x3_halo %d (use 0 or 1)", value);
    g_halo = value;
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
  if (g_wavesplit && g_forced_tile < 0 && g_forced_split < 0 && useA_kc && p.fast && k >= 128) {
    const long long blocks32 = (long long)((m + 31) / 32) * ((n + 31) / 32) * batch;
    const long long tiles64 = (long long)((m + 63) / 64) * ((n + 63) / 64) * batch;
    // (few blocks each streaming a long K would leave the weights to a handful of CUs)
    if (blocks32 <= 4LL * wdh::compute_units() && tiles64 < 2LL * wdh::compute_units() &&
        (blocks32 * 2 >= wdh::compute_units() || k <= 512) &&
        (useB_kc || (long long)(k - 1) * p.sB0 * 4 < 0x7fffffffLL)) {
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
  if (useA_kc && useB_kc) return launch<true, B_KC>(p, batch, vec);
  if (useA_kc && !useB_kc) return launch<true, B_MC>(p, batch, vec);
  if (!useA_kc && useB_kc) return launch<false, B_KC>(p, batch, vec);
  return launch<false, B_MC>(p, batch, vec);
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

}  // namespace

namespace wdh {
void release_conv_tables() {
  for (auto &kv : g_ktabs) {
    (void)hipFree(kv.second.ktab);
  }
  g_ktabs.clear();
}
int init_contraction() { return WDH_OK; }
void release_contraction() {}
}  // namespace wdh

extern "C" int wdh_conv2d(wdh_buf hX, wdh_buf hW, wdh_buf hBias, wdh_buf hY,
                          int n, int c, int h, int w, int cout, int kh, int kw,
                          int pt, int pl, int pb, int pr, int sh, int sw,
                          int dh, int dw, int group, int epilogue, wdh_buf hR) {
  WDH_REQUIRE_INIT();
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
  if (small && vec && ntaps == 1 && sh == 1 && sw == 1 && pt == 0 && pl == 0 && pb == 0 && pr == 0 &&
      plane % 4 == 0 && kdim % BK == 0 && aligned16(p.B)) {
    p.m = cout_g; p.n = (int)npix; p.k = (int)kdim;
    p.sAb = (long long)cout_g * kdim; p.sA0 = kdim; p.sA1 = 1;
    p.sBb = (long long)c_in_g * plane; p.sB0 = plane; p.sB1 = 1;
    p.alpha = 1.0f; p.beta = 1.0f; p.epilogue = epilogue;
    p.cv.c_in_g = c_in_g; p.cv.h = h; p.cv.w = w; p.cv.oh = oh; p.cv.ow = ow;
    p.cv.sh = p.cv.sw = p.cv.kh = p.cv.kw = p.cv.dh = p.cv.dw = 1;
    p.cv.c_total = c; p.cv.cout_total = cout; p.cv.cout_g = cout_g;
    p.cv.ntaps = 1; p.cv.npix = npix;
    p.fast = 1;
    p.a_bytes = (int)w_bytes;
    p.b_bytes = (int)x_bytes;  // window of group 0; the kernel shortens it per group
    p.y_bytes = g_descriptors && out_bytes < 0x7fffffffULL ? (int)out_bytes : 0;
    p.c_bytes = cout * 4;
    set_wide(p, true);
    return launch<true, B_PIXELS>(p, group, true);
  }
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
      switch (tile) {
        case T128x128: return launch_halo_tile<128, 128, 2, 2>(p, group, vecw);
        case T64x256: return launch_halo_tile<64, 256, 1, 4>(p, group, vecw);
        case T64x128: return launch_halo_tile<64, 128, 1, 4>(p, group, vecw);
        case T128x64: return launch_halo_tile<128, 64, 2, 2>(p, group, vecw);
        default: return launch_halo_tile<64, 64, 2, 2>(p, group, vecw);
      }
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
  if (mode == B_IM2COL32) return launch<true, B_IM2COL32>(p, group, vec);
  if (mode == B_IM2COL64) return launch<true, B_IM2COL64>(p, group, vec);
  return launch<true, B_IM2COL_BIG>(p, group, vec);
}
