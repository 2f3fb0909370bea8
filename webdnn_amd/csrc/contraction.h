// The contraction kernels of libwebdnn_hip.so (fp32 MFMA Gemm / MatMul / Conv) and the launch
// planning they share.  Included by gemm.hip (entry points, planning, small-product kernels) and
// by the contraction_*.hip files, each of which instantiates the kernels of one family so that
// the families compile side by side.
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
#pragma once
#include <string.h>


#include "common.h"
#include "fastdiv.h"

namespace wdhc {

// Layout of the library's static workspace (the array itself lives in gemm.hip): partial tiles
// first, then one flag per workgroup of a stream launch, each in a 64-byte line of its own.
#define WDH_STATIC_SCRATCH_FLOATS (WDH_STATIC_SCRATCH_BYTES / 4)
constexpr unsigned SK_MAX_WGS = 2048;                 // workgroups of one stream launch
constexpr unsigned SK_FLAG_STRIDE = 16;               // one flag per 64-byte line
constexpr unsigned SK_FLAG_WORDS = SK_MAX_WGS * SK_FLAG_STRIDE + 64;
constexpr unsigned SK_PARTIAL_FLOATS = WDH_STATIC_SCRATCH_FLOATS - SK_FLAG_WORDS;


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
// B_PIXELS_S2: a 1x1 unpadded conv with column stride 2 (any row stride) whose output rows hold an
// even number of pixels: two neighbouring output pixels are elements 0 and 2 of four consecutive
// input floats, so a thread's four pixels arrive as two 16-byte pieces (each with its own offset:
// the two pairs may lie in different rows) of which every other element is kept.
enum BMode { B_KC = 0, B_MC = 1, B_IM2COL32 = 2, B_IM2COL64 = 3, B_IM2COL_BIG = 4, B_PIXELS = 5, B_PIXELS_S2 = 8 };

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
  // Stream schedule (stream != 0; see stream_next).  The launch has 8 * sk_wgs workgroups;
  // the tiles are dealt to the 8 XCDs in contiguous runs, and within an XCD the K slabs of
  // its tiles, numbered tile by tile, are cut into sk_wgs equal contiguous ranges.
  int stream;
  int sk_wgs;            // workgroups per XCD
  int sk_slabs;          // K slabs per tile (slab = BK elements, or HALO_KB for the LDS-tile conv)
  int sk_tiles;          // tiles of the launch (all z)
  FastDiv fd_sk_slabs, fd_sk_wgs;
  float *sk_partial;     // [workgroup][BM * BN]: the partial tile a workgroup hands on
  unsigned *sk_flags;    // [workgroup * SK_FLAG_STRIDE]: 1 once that partial tile is complete
  unsigned *sk_error;    // set when a wait for a flag gave up
  int sk_spin_limit;     // polls of a flag before giving up
  ConvGeom cv;
};

__device__ __forceinline__ float relu_js(float v) {
  // Math.max(v, 0): NaN stays NaN (the comparison is false for it), -0 becomes +0.
  return v <= 0.0f ? 0.0f : v;
}

constexpr int XCDS = 8;
// Whole-tile workgroups: ids are dealt round-robin over the 8 XCDs by the
// hardware; this gives each XCD a contiguous range of tile numbers, so that
// tiles sharing A and B panels meet in one L2.
__device__ __forceinline__ int xcd_contiguous(int pid, int total) {
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

// ---- stream schedule ---------------------------------------------------------------
// A launch keeps every CU busy for ceil(tiles / CUs) tile times, and a tile count that is no
// multiple of what the chip holds wastes the difference.  A stream launch instead has a fixed
// grid of 8 * sk_wgs workgroups that stay for the whole launch.  The tiles are dealt to the 8
// XCDs in contiguous runs (workgroup id % 8 is the XCD it runs on); within an XCD the K slabs
// of its tiles are numbered tile by tile and cut into sk_wgs equal contiguous ranges, one per
// workgroup, whatever the tile boundaries: every workgroup multiplies the same number of
// slabs.  A workgroup walks its range from the end to the start, one segment (the part of
// one tile inside the range) at a time:
//   * a segment that covers its tile's whole K is finished like any whole tile;
//   * a segment that stops short of K (only the first one walked can: the range's end lies
//     inside the tile) leaves its sums in the workgroup's slot of sk_partial and raises
//     the workgroup's flag;
//   * a segment that reaches K but starts after 0 (only the last one walked can) belongs to
//     the workgroup that finishes the tile: it adds the slots of the workgroups before it
//     that hold the tile's earlier K ranges, in order of K, then its own sums -- a fixed
//     order, so results do not depend on timing -- and applies the epilogue.
// The finishing workgroup only ever waits for workgroups with lower ids (dispatched before
// it) and for the first thing they compute, which it needs as the last thing it does, so
// the wait is short and cannot deadlock even if the grid is not resident all at once.
// Partial tiles cross CUs inside one launch: they are written and read with system-scope
// (sc0 sc1) accesses that bypass the non-coherent cache levels, the flag is raised after the
// stores have been acknowledged, and nothing needs a fence that writes back a whole L2.
constexpr int AUX_COHERENT = 17;  // sc0 | sc1 of a buffer instruction

struct StreamPos {
  int xcd, local;   // this workgroup: its XCD and its number within the XCD
  int tile0;        // launch-wide number of the XCD's first tile
  int units;        // slabs of the XCD: its tiles * sk_slabs
  int u0;           // first slab of this workgroup's range (numbered within the XCD)
  int cur_end;      // end of the part of the range not yet computed
};
struct Segment {
  int lin;          // tile (launch-wide number)
  int tile_begin;   // XCD-local slab number of the tile's first slab
  int sbeg, send;   // slabs of the tile this segment covers: [sbeg, send)
  bool first, last; // starts at slab 0 / ends with the tile's last slab
};
__device__ __forceinline__ StreamPos stream_begin(const Params &p) {
  StreamPos s;
  s.xcd = (int)blockIdx.x % XCDS;
  s.local = (int)blockIdx.x / XCDS;
  const int base = p.sk_tiles / XCDS, rem = p.sk_tiles % XCDS;
  s.tile0 = s.xcd * base + (s.xcd < rem ? s.xcd : rem);
  s.units = (base + (s.xcd < rem ? 1 : 0)) * p.sk_slabs;
  s.u0 = fdiv(s.local * s.units, p.fd_sk_wgs);            // (the host keeps sk_wgs * units below 2^31)
  s.cur_end = fdiv((s.local + 1) * s.units, p.fd_sk_wgs);
  return s;
}
// The segment that ends at pos.cur_end; moves cur_end to its start.
__device__ __forceinline__ Segment stream_next(const Params &p, StreamPos &pos) {
  Segment g;
  const int t = fdiv(pos.cur_end - 1, p.fd_sk_slabs);
  g.tile_begin = t * p.sk_slabs;
  const int seg_begin = pos.u0 > g.tile_begin ? pos.u0 : g.tile_begin;
  g.lin = pos.tile0 + t;
  g.sbeg = seg_begin - g.tile_begin;
  g.send = pos.cur_end - g.tile_begin;
  g.first = g.sbeg == 0;
  g.last = g.send == p.sk_slabs;
  pos.cur_end = seg_begin;
  return g;
}

// This workgroup's sums of a segment that stops short of K: to its slot, then the flag.
// Slot layout: [accumulator block][quad of registers][thread][4], so every lane reads back
// what the same lane of the finishing workgroup's same wavefront position wrote.
template <int MT, int NT>
__device__ __forceinline__ void stream_hand_on(const Params &p, f32x16 (&acc)[MT][NT]) {
  constexpr int TILE_FLOATS = MT * NT * 16 * NTHREADS;
  const rsrc_t slot = make_rsrc(p.sk_partial + (size_t)blockIdx.x * TILE_FLOATS, TILE_FLOATS * 4);
  const int voff = (int)threadIdx.x * 16;
#pragma unroll
  for (int mt = 0; mt < MT; mt++)
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const f32x4 v = {acc[mt][nt][4 * q], acc[mt][nt][4 * q + 1], acc[mt][nt][4 * q + 2], acc[mt][nt][4 * q + 3]};
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), slot,
                                               voff + ((mt * NT + nt) * 4 + q) * (NTHREADS * 16), 0, AUX_COHERENT);
      }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): every store above has been acknowledged
  __syncthreads();
  if (threadIdx.x == 0)
    __hip_atomic_store(p.sk_flags + (size_t)blockIdx.x * SK_FLAG_STRIDE, 1u, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_SYSTEM);
}

// The finishing workgroup: acc = (slot[a] + slot[a+1] + ... + slot[local-1]) + acc, where
// a .. local-1 are the workgroups of this XCD whose ranges hold the tile's earlier slabs.
template <int MT, int NT>
__device__ __forceinline__ void stream_collect(const Params &p, const StreamPos &pos, const Segment &g,
                                               f32x16 (&acc)[MT][NT]) {
  constexpr int TILE_FLOATS = MT * NT * 16 * NTHREADS;
  int a = pos.local - 1;
  while (a > 0 && fdiv(a * pos.units, p.fd_sk_wgs) > g.tile_begin) a--;
  if (threadIdx.x == 0) {
    for (int j = a; j < pos.local; j++) {
      const unsigned *flag = p.sk_flags + (size_t)(j * XCDS + pos.xcd) * SK_FLAG_STRIDE;
      int polls = 0;
      while (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) == 0u) {
        if (++polls > p.sk_spin_limit) {  // never hang: give up, say so, and go on with what is there
          __hip_atomic_store(p.sk_error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
          break;
        }
        __builtin_amdgcn_s_sleep(8);
      }
    }
  }
  __syncthreads();
  const int voff = (int)threadIdx.x * 16;
#pragma unroll
  for (int mt = 0; mt < MT; mt++)
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      f32x4 sum[4];
      for (int j = a; j < pos.local; j++) {
        const rsrc_t slot = make_rsrc(p.sk_partial + (size_t)(j * XCDS + pos.xcd) * TILE_FLOATS, TILE_FLOATS * 4);
#pragma unroll
        for (int q = 0; q < 4; q++) {
          const f32x4 v = __builtin_bit_cast(
              f32x4, __builtin_amdgcn_raw_buffer_load_b128(slot, voff + ((mt * NT + nt) * 4 + q) * (NTHREADS * 16), 0,
                                                           AUX_COHERENT));
          if (j == a) sum[q] = v;
          else sum[q] += v;
        }
      }
#pragma unroll
      for (int r = 0; r < 16; r++) acc[mt][nt][r] = sum[r >> 2][r & 3] + acc[mt][nt][r];
    }
  // the flags go back to 0 for the next launch (nobody raises them again in this one)
  if (threadIdx.x == 0)
    for (int j = a; j < pos.local; j++)
      __hip_atomic_store(p.sk_flags + (size_t)(j * XCDS + pos.xcd) * SK_FLAG_STRIDE, 0u, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_SYSTEM);
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
// resident workgroups per CU of a stream launch (at most; the host may ask for fewer)
constexpr int stream_blocks(int bm, int bn) {
  return bm * bn <= 64 * 64 ? 4 : (bm * bn <= 64 * 128 ? 3 : 2);
}

// STREAM: the launch is a stream of K slabs (stream_next): the body below runs once per segment
// of the workgroup's range.  Such a launch has a fixed number of resident workgroups per CU
// (stream_blocks), fewer than a tile-per-workgroup launch may have, so its kernels may use
// more registers.
template <int BM, int BN, int WM, int WN, bool A_KC, int BMODE_, bool VEC, bool STREAM>
__global__ __launch_bounds__(NTHREADS, STREAM ? stream_blocks(BM, BN) : min_blocks(BM, BN)) void contraction_kernel(Params p) {
  constexpr bool IM2COL_FAST = BMODE_ == B_IM2COL32 || BMODE_ == B_IM2COL64;
  constexpr bool IM2COL = IM2COL_FAST || BMODE_ == B_IM2COL_BIG;
  constexpr bool PIX_S2 = BMODE_ == B_PIXELS_S2;
  constexpr bool PIXELS = BMODE_ == B_PIXELS || PIX_S2;
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

  // Everything the loops need to know about one segment of work: the tile, the part of K, and
  // this thread's fetch plan (one byte offset per 16-byte piece, every address term folded in
  // before the K loop starts).
  struct Ctx {
    bool whole, first, last;
    int lin, chunk, bz, row0, col0, kbeg, kend;
    const float *A, *B;
    long long lda, ldb;
    int voff_a[BM / 64], voff_b[BN / 64];
    int voff_b2[BMODE_ == B_PIXELS_S2 ? BN / 64 : 1];  // B_PIXELS_S2: the piece of the second pixel pair
    rsrc_t rsrc_a, rsrc_b;
    PixelCtx px;
    PixelFast pf;
    int kgroup0;   // first of the L consecutive k rows this wavefront gathers in each slab
    int tile_begin;
  };
  const bool a_fast = p.fast;
  const bool b_fast = p.fast && BMODE_ != B_IM2COL_BIG;

  // ---- descriptor fetch plans --------------------------------------------------------
  // Every operand below 2 GiB takes this path, edge tiles included.  Rows of a
  // row-major-in-K operand past the edge are clamped; an operand that is
  // contiguous along M or N simply reads on past its last row or column, into
  // the next k row (or, past the end of the matrix, zeros from the descriptor's
  // bounds check).  Either way the surplus rows and columns only feed products
  // that are never stored.
  auto setup = [&](Ctx &c, int tm, int tn) {
    const int bz = c.bz;
    const int row0 = c.row0 = tm * BM, col0 = c.col0 = tn * BN;
    c.A = p.A + (long long)bz * p.sAb;
    c.B = p.B + (long long)bz * p.sBb;
    const long long lda = c.lda = A_KC ? p.sA0 : p.sA1;
    const long long ldb = c.ldb = B_IS_KC ? p.sB1 : p.sB0;
    if (A_KC) {
#pragma unroll
      for (int i = 0; i < BM / 64; i++) {
        int r = row0 + (tid >> 2) + i * 64;
        r = r < p.m ? r : p.m - 1;
        c.voff_a[i] = (int)(((long long)r * lda + (tid & 3) * 4) * 4);
      }
    } else {
      constexpr int TPR = BM / 4, RPP = NTHREADS / TPR;
#pragma unroll
      for (int i = 0; i < BM / 64; i++)
        c.voff_a[i] = (int)(((long long)(tid / TPR + i * RPP) * lda + row0 + (tid % TPR) * 4) * 4);
    }
    if (B_IS_KC) {
#pragma unroll
      for (int i = 0; i < BN / 64; i++) {
        int cc = col0 + (tid >> 2) + i * 64;
        cc = cc < p.n ? cc : p.n - 1;
        c.voff_b[i] = (int)(((long long)cc * ldb + (tid & 3) * 4) * 4);
      }
    } else if (!IM2COL) {
      constexpr int TPR = BN / 4, RPP = NTHREADS / TPR;
      // B_PIXELS: column = pixel index over the batch; its four pixels share an image
      long long colpos = col0 + (tid % TPR) * 4;
      long long colpos2 = 0;
      if (PIX_S2) {
        // output pixel -> (image, row, column) -> offset of its input pixel; pixels 0,1 and 2,3 of the
        // thread's four are neighbours in a row (rows hold an even number of pixels)
        const unsigned plane = (unsigned)(p.cv.h * p.cv.w), ohw = (unsigned)(p.cv.oh * p.cv.ow);
        auto input_offset = [&](unsigned P) {
          const unsigned img = (unsigned)fdiv((int)P, p.cv.fd_ohw), q = P - img * ohw;
          const unsigned oy = (unsigned)fdiv((int)q, p.cv.fd_ow), ox = q - oy * (unsigned)p.cv.ow;
          return (long long)img * p.cv.c_total * plane + (long long)oy * p.cv.sh * p.cv.w + 2 * ox;
        };
        colpos2 = input_offset((unsigned)colpos + 2);
        colpos = input_offset((unsigned)colpos);
      } else if (PIXELS) {
        const unsigned plane = (unsigned)(p.cv.h * p.cv.w);
        const unsigned img = (unsigned)fdiv((int)colpos, p.cv.fd_plane);
        colpos = (long long)img * p.cv.c_total * plane + ((unsigned)colpos - img * plane);
      }
#pragma unroll
      for (int i = 0; i < BN / 64; i++) {
        c.voff_b[i] = (int)(((long long)(tid / TPR + i * RPP) * ldb + colpos) * 4);
        if (PIX_S2) c.voff_b2[PIX_S2 ? i : 0] = (int)(((long long)(tid / TPR + i * RPP) * ldb + colpos2) * 4);
      }
    }
    c.rsrc_a = make_rsrc(c.A, p.a_bytes);

    // ---- im2col: what this thread's pixel looks like ----------------------------
    c.px = PixelCtx{p.B, 0, 0, 0, 0ull};
    c.pf = PixelFast{0, 0xffffffffu, 0xffffffffu};
    const float *bbase = c.B;  // base of the B descriptor
    if (IM2COL) {
      const unsigned P = (unsigned)col0 + (unsigned)(tid % BN);  // npix < 2^31
      const long long plane = (long long)p.cv.h * p.cv.w;
      const int bias = p.cv.pt * p.cv.w + p.cv.pl;  // makes every corner offset >= 0
      c.px.xbase = p.B + (long long)bz * p.cv.c_in_g * plane;
      bbase = c.px.xbase - bias;
      if (P < (unsigned)p.cv.npix) {
        const unsigned ohw = (unsigned)(p.cv.oh * p.cv.ow);
        const unsigned img = (unsigned)fdiv((int)P, p.cv.fd_ohw);
        const unsigned q = P - img * ohw;
        const int oy = fdiv((int)q, p.cv.fd_ow), ox = (int)q - oy * p.cv.ow;
        const long long img_off = (long long)img * p.cv.c_total * plane;
        c.px.iy0 = oy * p.cv.sh - p.cv.pt;
        c.px.ix0 = ox * p.cv.sw - p.cv.pl;
        c.px.pbase = c.px.iy0 * p.cv.w + c.px.ix0;
        if (IM2COL_FAST) {
          c.pf.valid = (int)((img_off + c.px.pbase + bias) * 4);
          // which taps of this pixel fall inside the input: rows first, then columns
          unsigned long long inside = 0;
          int t = 0;
          for (int ky = 0; ky < p.cv.kh; ky++) {
            const bool row_in = (unsigned)(c.px.iy0 + ky * p.cv.dh) < (unsigned)p.cv.h;
            for (int kx = 0; kx < p.cv.kw; kx++, t++)
              if (row_in && (unsigned)(c.px.ix0 + kx * p.cv.dw) < (unsigned)p.cv.w)
                inside |= 1ull << t;
          }
          c.pf.pad_lo = ~(unsigned)inside;
          c.pf.pad_hi = ~(unsigned)(inside >> 32);
        } else {
          c.px.xbase += img_off;
          c.px.mask = 1ull;
        }
      }
    }
    // conv: p.b_bytes is group 0's window, later groups start further into X
    const int b_window =
        CONV ? p.b_bytes - (int)((long long)bz * p.cv.c_in_g * p.cv.h * p.cv.w * 4) : p.b_bytes;
    c.rsrc_b = make_rsrc(bbase, b_window);
    c.kgroup0 = IM2COL ? __builtin_amdgcn_readfirstlane(tid / BN) * (BK / (NTHREADS / BN)) : 0;
  };
  // A stream launch walks the segments of this workgroup's slab range (see stream_next);
  // any other launch has one tile, or one chunk of a tile, per workgroup.
  StreamPos pos = {};
  if (STREAM) pos = stream_begin(p);
  auto next_segment = [&](Ctx &c) {
    int tm, tn;
    if (STREAM) {
      const Segment sg = stream_next(p, pos);
      c.whole = true;
      c.first = sg.first;
      c.last = sg.last;
      c.tile_begin = sg.tile_begin;
      c.lin = sg.lin;
      c.chunk = 0;
      c.kbeg = sg.sbeg * BK;
      c.kend = sg.send * BK < p.k ? sg.send * BK : p.k;
      c.bz = fdiv(c.lin, p.fd_tiles_per_z);
      tile_coords(p, c.lin - c.bz * (p.tiles_m * p.tiles_n), &tm, &tn);
    } else {
      const TileWork tw = decode_work(p);
      c.whole = tw.whole;
      c.first = c.last = true;
      c.tile_begin = 0;
      c.lin = tw.lin; c.chunk = tw.chunk; c.bz = tw.bz; tm = tw.tm; tn = tw.tn;
      // this workgroup's share of K
      c.kbeg = c.whole ? 0 : c.chunk * p.kchunk;
      c.kend = c.whole ? p.k : (c.kbeg + p.kchunk < p.k ? c.kbeg + p.kchunk : p.k);
    }
    setup(c, tm, tn);
  };

  // Registers that carry one fetched K slab from global memory to LDS.
  struct Staged {
    f32x4 a[BM / 64], b[BN / 64];
    f32x4 b2[PIX_S2 ? BN / 64 : 1];  // B_PIXELS_S2: the second 16 bytes of each piece
    unsigned ok;  // flat im2col only: which fetched taps lie inside the input
  };
  // B_PIXELS_S2: two pieces of four consecutive input floats, of which elements 0 and 2 are pixels
  auto fetch_b_s2 = [&](const Ctx &c, int k0, Staged &st) {
    const int soff = (int)(k0 * c.ldb * 4);
#pragma unroll
    for (int i = 0; i < BN / 64; i++) {
      st.b[i] = buf_load4(c.rsrc_b, c.voff_b[i], soff);
      st.b2[PIX_S2 ? i : 0] = buf_load4(c.rsrc_b, c.voff_b2[PIX_S2 ? i : 0], soff);
    }
  };
  // Descriptor-only fetch: legal for a slab that lies fully inside K when
  // both operands qualify (all_fast).
  auto fetch_fast = [&](const Ctx &c, int k0, Staged &st) {
    fetch_rows_fast<BM, VEC>(c.rsrc_a, c.voff_a, A_KC ? k0 * 4 : (int)(k0 * c.lda * 4), st.a);
    if (IM2COL_FAST)
      fetch_im2col_fast<BN, BMODE_ == B_IM2COL64>(c.rsrc_b, p.cv.ktab, c.pf, k0 + c.kgroup0, st.b);
    else if (PIX_S2)
      fetch_b_s2(c, k0, st);
    else if (!IM2COL)
      fetch_rows_fast<BN, VEC>(c.rsrc_b, c.voff_b, B_IS_KC ? k0 * 4 : (int)(k0 * c.ldb * 4), st.b);
  };
  // Fetch that copes with everything: ragged last slab, edge tiles, huge operands.
  auto fetch_any = [&](const Ctx &c, int k0, Staged &st) {
    const bool full = k0 + BK <= c.kend;
    if (a_fast && full) {
      fetch_rows_fast<BM, VEC>(c.rsrc_a, c.voff_a, A_KC ? k0 * 4 : (int)(k0 * c.lda * 4), st.a);
    } else if (A_KC) {
      fetch_kc<BM, VEC>(c.A, c.lda, c.row0, p.m, k0, c.kend, tid, st.a);
    } else {
      fetch_mc<BM, VEC>(c.A, c.lda, c.row0, p.m, k0, c.kend, tid, st.a);
    }
    if (IM2COL_FAST) {
      // padding entries of the tap table read as 0, so a ragged K needs no care
      fetch_im2col_fast<BN, BMODE_ == B_IM2COL64>(c.rsrc_b, p.cv.ktab, c.pf, k0 + c.kgroup0, st.b);
    } else if (IM2COL) {
      st.ok = fetch_im2col<BN>(p.cv, c.px, k0, c.kend, tid, st.b);
    } else if (PIX_S2) {
      fetch_b_s2(c, k0, st);
    } else if ((b_fast && full) || PIXELS) {
      fetch_rows_fast<BN, VEC>(c.rsrc_b, c.voff_b, B_IS_KC ? k0 * 4 : (int)(k0 * c.ldb * 4), st.b);
    } else if (B_IS_KC) {
      fetch_kc<BN, VEC>(c.B, c.ldb, c.col0, p.n, k0, c.kend, tid, st.b);
    } else {
      fetch_mc<BN, VEC>(c.B, c.ldb, c.col0, p.n, k0, c.kend, tid, st.b);
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
    else if (PIX_S2) {
      f32x4 even[BN / 64];
#pragma unroll
      for (int i = 0; i < BN / 64; i++)
        even[i] = f32x4{st.b[i].x, st.b[i].z, st.b2[PIX_S2 ? i : 0].x, st.b2[PIX_S2 ? i : 0].z};
      stash_mc<BN>(lds_b[buf], tid, even);
    } else
      stash_mc<BN>(lds_b[buf], tid, st.b);
  };

  f32x16 acc[MT][NT];
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

  Ctx c;
  Staged st0;
  if (STREAM && pos.cur_end <= pos.u0) return;  // (an XCD without tiles)
  next_segment(c);
  fetch_any(c, c.kbeg, st0);
  for (;;) {
#pragma unroll
    for (int a = 0; a < MT; a++)
#pragma unroll
      for (int b = 0; b < NT; b++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[a][b][r] = 0.0f;

    // Slab s+1 travels global -> registers while slab s runs through the matrix
    // cores, then goes to the other LDS buffer.  (A second slab in flight was
    // measured and bought nothing.)  The main loop takes two slabs per trip, so
    // that LDS buffer indices are compile-time constants, and contains
    // descriptor fetches only; the few slabs it leaves over (and every slab of a
    // workgroup that cannot use descriptors) run in the general loop below it.  (Two slabs
    // in flight, requested two trips ahead, were measured again on the ResNet-50 layers, same box,
    // alternating builds: 2966 against 2957 us over the 54 launches -- nothing.)
    const int kbeg = c.kbeg;
    const int nslabs = (c.kend - kbeg + BK - 1) / BK;
    const int nfull = (c.kend - kbeg) / BK;
    const bool all_fast = a_fast && b_fast && !(IM2COL && !IM2COL_FAST);
    const int nfast = all_fast ? nfull - 1 : 0;  // steps whose next slab is a full one
    stash(0, st0);
    __syncthreads();
    int s = 0;
    // The scheduling fences keep the compiler from sinking the loads below the
    // matrix-core work they are meant to overlap.
    for (; s + 2 <= nfast; s += 2) {
      fetch_fast(c, kbeg + (s + 1) * BK, st0);
      __builtin_amdgcn_sched_barrier(0);
      compute(0);
      stash(1, st0);
      __syncthreads();
      fetch_fast(c, kbeg + (s + 2) * BK, st0);
      __builtin_amdgcn_sched_barrier(0);
      compute(1);
      stash(0, st0);
      __syncthreads();
    }
    for (; s < nslabs; s++) {
      const int cur = s & 1;
      if (s + 1 < nslabs) fetch_any(c, kbeg + (s + 1) * BK, st0);
      compute(cur);
      if (s + 1 < nslabs) stash(cur ^ 1, st0);
      __syncthreads();
    }

    // what the epilogue needs of this segment; c moves on to the next one, whose first slab
    // is requested before the epilogue so that it travels while the results are stored
    const bool whole = c.whole, first = c.first, last = c.last;
    const int lin = c.lin, chunk = c.chunk, bz = c.bz, row0 = c.row0, col0 = c.col0;
    Segment sg;
    sg.tile_begin = c.tile_begin;
    const bool more = STREAM && pos.cur_end > pos.u0;
    if (more) {
      next_segment(c);
      fetch_any(c, c.kbeg, st0);
    }
    static_assert(2 * A_FLOATS >= 2 * STAGE_FLOATS && 2 * B_FLOATS >= 2 * STAGE_FLOATS, "epilogue staging");
    if (STREAM && !last) {
      stream_hand_on<MT, NT>(p, acc);
    } else {
      if (STREAM && !first) stream_collect<MT, NT>(p, pos, sg, acc);
      finish_tile<BM, BN, WM, WN, CONV>(p, acc, whole, lin, chunk, bz, row0, col0,
                                        (wave < 2 ? &lds_a[0][0] : &lds_b[0][0]) + (wave & 1) * STAGE_FLOATS);
    }
    if (!more) break;
    __syncthreads();  // the epilogue has finished with the LDS
  }
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

// workgroups of the LDS-tile conv a CU holds (LDS and registers)
constexpr int halo_blocks(int bm, int bn) { return bm == 64 ? (bn == 64 ? 4 : (bn == 128 ? 3 : 2)) : 2; }

template <int BM, int BN, int WM, int WN, int VECW, bool STREAM>
__global__ __launch_bounds__(NTHREADS, halo_blocks(BM, BN)) void conv3x3_halo_kernel(Params p) {
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

  const ConvGeom &cv = p.cv;
  const int plane_in = cv.h * cv.w;
  const int pg = cv.pitch / VECW;       // pieces per row
  const int upc = cv.slots * pg;        // pieces per channel
  const int xu = cv.units;              // pieces per thread this geometry needs (<= XU)

  // ---- weights: piece (row r0 + 14 i, k 4q .. 4q+3) of the block -----------------
  // (threads 252..255 repeat pieces of row 13: same values to the same cells)
  const int q = tid % 18, r0 = tid / 18 < HALO_AROWS ? tid / 18 : HALO_AROWS - 1;
  const int lds_a_w = (r0 * HALO_ROWA + 4 * q) * 4;
  // ---- where a lane finds its weights in LDS --------------------------------------
  int lds_a_r[MT];
#pragma unroll
  for (int mt = 0; mt < MT; mt++)
    lds_a_r[mt] = ((wrow + mt * 32 + li) * HALO_ROWA + 36 * half) * 4;

  // What the loops need to know about one segment of work (a tile, a range of K blocks).
  struct Ctx {
    TileWork t;
    bool first, last;
    int tile_begin, row0, col0, kbeg, kend;
    int voff_a[AU], voff_x[XU], lds_x_w[XU];
    rsrc_t rsrc_a, rsrc_x;
    int lds_b_r[NT][9];   // where a lane finds tap t of its pixel of block nt in LDS
  };
  // (a stream launch walks the segments of this workgroup's range of K blocks: see stream_next)
  StreamPos pos = {};
  if (STREAM) pos = stream_begin(p);
  auto next_segment = [&](Ctx &c) {
    TileWork &t = c.t;
    if (STREAM) {
      const Segment sg = stream_next(p, pos);
      c.first = sg.first;
      c.last = sg.last;
      c.tile_begin = sg.tile_begin;
      t.whole = true;
      t.lin = sg.lin;
      t.chunk = 0;
      t.bz = fdiv(t.lin, p.fd_tiles_per_z);
      tile_coords(p, t.lin - t.bz * (p.tiles_m * p.tiles_n), &t.tm, &t.tn);
      c.kbeg = sg.sbeg * HALO_KB;
      c.kend = sg.send * HALO_KB < p.k ? sg.send * HALO_KB : p.k;
    } else {
      t = decode_work(p);
      c.first = c.last = true;
      c.tile_begin = 0;
      c.kbeg = t.whole ? 0 : t.chunk * p.kchunk;
      c.kend = t.whole ? p.k : (c.kbeg + p.kchunk < p.k ? c.kbeg + p.kchunk : p.k);
    }
    const int row0 = c.row0 = t.tm * BM, col0 = c.col0 = t.tn * BN;
    // first output row of the tile (rows numbered through the batch) and its image
    const int R0 = fdiv(col0, cv.fd_ow);
    const int img0 = fdiv(R0, cv.fd_oh);
#pragma unroll
    for (int i = 0; i < AU; i++) {
      int r = row0 + r0 + HALO_AROWS * i;
      r = r < p.m ? r : p.m - 1;  // rows past the edge are never stored
      c.voff_a[i] = (r * p.k + 4 * q) * 4;
    }
    c.rsrc_a = make_rsrc(p.A + (long long)t.bz * p.sAb, p.a_bytes);

    // ---- input rows: piece u = tid + 256 i -> (channel, slot, column group) ---------
    const int first_rows = (img0 + 1) * cv.oh - R0;  // output rows from R0 to the end of its image
#pragma unroll
    for (int i = 0; i < XU; i++) {
      const int u = tid + NTHREADS * i;
      const int ch = fdiv(u, cv.fd_upc), rem = u - ch * upc;
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
      const bool live = ch < HALO_CB;
      const bool data = live && (long long)img * cv.oh * cv.ow < cv.npix && iy >= 0 && iy < cv.h &&
                        ix >= 0 && ix + VECW <= cv.w;
      c.voff_x[i] = data ? (((img * cv.c_total + ch) * cv.h + iy) * cv.w + ix) * 4 : BUF_OOB;
    }
    const long long group_off = (long long)t.bz * cv.c_in_g * plane_in;
    c.rsrc_x = make_rsrc(p.B + group_off, p.b_bytes - (int)(group_off * 4));
  };
  // The LDS side of a segment's plan: where the fetched pieces go and where a lane finds its
  // taps.  Computed after the previous segment's epilogue (it is not needed to request the
  // first block, and the epilogue needs the registers).
  auto lds_plan = [&](Ctx &c) {
    const int col0 = c.col0;
    const int R0 = fdiv(col0, cv.fd_ow);
    const int img0 = fdiv(R0, cv.fd_oh);
#pragma unroll
    for (int i = 0; i < XU; i++) {
      const int u = tid + NTHREADS * i;
      const int ch = fdiv(u, cv.fd_upc), rem = u - ch * upc;
      const int slot = fdiv(rem, cv.fd_pg), cg = rem - slot * pg;
      c.lds_x_w[i] = ch < HALO_CB ? (ch * PLANE + slot * cv.pitch + cg * VECW) * 4 : HALO_CB * PLANE * 4;
    }
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      int P = col0 + wcol + nt * 32 + li;
      P = P < (int)cv.npix ? P : (int)cv.npix - 1;  // lanes past the edge are never stored
      const int R = fdiv(P, cv.fd_ow), ox = P - R * cv.ow;
      const int slot0 = (R - R0) + 2 * (fdiv(R, cv.fd_oh) - img0);
      const int corner = (4 * half * PLANE + slot0 * cv.pitch + cv.col0 - cv.pl + ox) * 4;
#pragma unroll
      for (int tap = 0; tap < 9; tap++)
        c.lds_b_r[nt][tap] = corner + ((tap / 3) * cv.pitch + tap % 3) * 4;
    }
  };

  f32x16 acc[MT][NT];
  f32x4 ra[AU];
  xpiece rx[XU];
  auto fetch = [&](const Ctx &c, int k0) {
    const int soff_a = k0 * 4;
    const int soff_x = (k0 / 9) * plane_in * 4;
#pragma unroll
    for (int i = 0; i < AU; i++) ra[i] = buf_load4(c.rsrc_a, c.voff_a[i], soff_a);
#pragma unroll
    for (int i = 0; i < XU; i++)
      if (i < xu) rx[i] = HaloPiece<VECW>::load(c.rsrc_x, c.voff_x[i], soff_x);
  };
  auto stash = [&](const Ctx &c) {
    char *const as_b = reinterpret_cast<char *>(as);
    char *const xs_b = reinterpret_cast<char *>(xs);
#pragma unroll
    for (int i = 0; i < AU; i++)
      *reinterpret_cast<f32x4 *>(as_b + lds_a_w + i * (HALO_AROWS * HALO_ROWA * 4)) = ra[i];
#pragma unroll
    for (int i = 0; i < XU; i++)
      if (i < xu) *reinterpret_cast<xpiece *>(xs_b + c.lds_x_w[i]) = rx[i];
  };
  auto compute = [&](const Ctx &c) {
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
        const int kk = 4 * j + e, ch = kk / 9, tap = kk % 9;
        float b_el[NT];
#pragma unroll
        for (int nt = 0; nt < NT; nt++)
          b_el[nt] = *reinterpret_cast<const float *>(xs_b + c.lds_b_r[nt][tap] + ch * (PLANE * 4));
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
          for (int nt = 0; nt < NT; nt++)
            acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[mt][e], b_el[nt], acc[mt][nt], 0, 0, 0);
      }
    }
  };

  if (STREAM && pos.cur_end <= pos.u0) return;  // (an XCD without tiles)
  Ctx c;
  next_segment(c);
  fetch(c, c.kbeg);
  for (;;) {
    lds_plan(c);
#pragma unroll
    for (int a = 0; a < MT; a++)
#pragma unroll
      for (int b = 0; b < NT; b++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[a][b][r] = 0.0f;

    // One LDS buffer: block b+1 travels global -> registers while block b runs through
    // the matrix cores, and is written to LDS once every wavefront has finished reading.
    for (int k0 = c.kbeg; k0 < c.kend; k0 += HALO_KB) {
      if (k0 != c.kbeg) __syncthreads();
      stash(c);
      __syncthreads();
      if (k0 + HALO_KB < c.kend) fetch(c, k0 + HALO_KB);
      __builtin_amdgcn_sched_barrier(0);
      compute(c);
    }
    // what the epilogue needs of this segment; c moves on to the next one, whose first block
    // is requested before the epilogue so that it travels while the results are stored
    const TileWork t = c.t;
    const bool first = c.first, last = c.last;
    const int row0 = c.row0, col0 = c.col0;
    Segment sg;
    sg.tile_begin = c.tile_begin;
    const bool more = STREAM && pos.cur_end > pos.u0;
    if (more) {
      next_segment(c);
      fetch(c, c.kbeg);
    }
    static_assert(AU * HALO_AROWS * HALO_ROWA >= 4 * STAGE_FLOATS, "epilogue staging");
    if (STREAM && !last) {
      stream_hand_on<MT, NT>(p, acc);
    } else {
      if (STREAM && !first) stream_collect<MT, NT>(p, pos, sg, acc);
      finish_tile<BM, BN, WM, WN, true>(p, acc, t.whole, t.lin, t.chunk, t.bz, row0, col0,
                                        as + (threadIdx.x >> 6) * STAGE_FLOATS);
    }
    if (!more) break;
    __syncthreads();  // the epilogue has finished with the LDS
  }
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
static __global__ void contraction_strided_kernel(Params p) {
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

// ---- state and planning shared by the translation units (defined in gemm.hip) -------------
extern int g_forced_tile;    // >= 0: overrides the tile choice (tuning hook)
extern int g_tile_hint;      // >= 0: tile for the next Gemm / MatMul launch, set by a caller inside the library
extern int g_forced_split;   // >= 1: overrides the split-K heuristic
extern int g_last_form;
extern bool g_static_scratch;  // set for the duration of a wdh_gemm_static call
// what launch_planned decided for the most recent launch (wdh_last_plan)
struct LastPlan { int bm, bn, split, form; long long full, tail; };
extern LastPlan g_last_plan;
extern int g_stream_spin;
extern unsigned *g_stream_error_dev;
float *static_scratch();     // device address of the static workspace on the current device, or null
float *stream_workspace();   // slots and flags of stream launches on the current lane: the static workspace on lane 0
TileId pick_tile(int m, int n, int nz);

// How the tiles of one launch are spread over the chip.
struct WorkPlan {
  long long full;   // tiles computed by one workgroup each
  long long tail;   // tiles cut along K
  int split;        // chunks per tail tile
  int kchunk;       // K elements per chunk (a multiple of 16)
};
WorkPlan plan_work(long long tiles, int k, int bm, int bn, bool gather, int kgran = BK);
// Whether (and how wide) a launch runs as a stream of K slabs: workgroups per XCD, 0 = not.
int stream_width(long long tiles, int slabs, int kgran, const WorkPlan &w, int tile_floats, int max_wgs_per_cu);

// Plans the work of one launch, provides the partial-sum workspace, starts the main
// kernel through `start(grid)` and, if tiles were cut along K, the reduce pass.
// max_wgs_per_cu: how many workgroups of this kernel a CU holds (its launch bounds).
// (max_wgs_per_cu = 0: this kernel has no stream form.)
template <int BM, int BN, typename Start>
int launch_planned(Params &p, int nz, bool conv, int kgran, int max_wgs_per_cu, Start start) {
  p.tiles_m = (p.m + BM - 1) / BM;
  p.tiles_n = (p.n + BN - 1) / BN;
  const long long tiles = (long long)p.tiles_m * p.tiles_n * nz;
  const WorkPlan w = plan_work(tiles, p.k, BM, BN, conv, kgran);
  p.nz = nz;
  p.fd_tiles_per_z = make_fastdiv((long long)p.tiles_m * p.tiles_n);
  p.fd_group = make_fastdiv((long long)TILE_GROUP * p.tiles_n);
  p.fd_last_rows = make_fastdiv(p.tiles_m % TILE_GROUP ? p.tiles_m % TILE_GROUP : 1);
  const int slabs = (p.k + kgran - 1) / kgran;
  if (const int wgs = tiles <= 0x7fffffffLL && max_wgs_per_cu > 0
                          ? stream_width(tiles, slabs, kgran, w, BM * BN, max_wgs_per_cu) : 0) {
    float *base = stream_workspace();
    p.stream = 1;
    p.sk_wgs = wgs;
    p.sk_slabs = slabs;
    p.sk_tiles = (int)tiles;
    p.fd_sk_slabs = make_fastdiv(slabs);
    p.fd_sk_wgs = make_fastdiv(wgs);
    p.sk_partial = base;
    p.sk_flags = reinterpret_cast<unsigned *>(base + SK_PARTIAL_FLOATS);
    p.sk_error = g_stream_error_dev;
    p.sk_spin_limit = g_stream_spin;
    p.full_tiles = (int)tiles;
    p.tail_tiles = 0;
    p.tail_split = 1;
    p.fd_tail_tiles = make_fastdiv(1);
    g_last_plan = {BM, BN, 0, g_last_form, tiles, (long long)wgs * XCDS};
    start(dim3((unsigned)(wgs * XCDS)), true);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess)
      return wdh::fail(WDH_EHIP, "contraction launch failed: %s", hipGetErrorString(e));
    return WDH_OK;
  }
  const long long blocks = w.full + w.tail * w.split;
  if (blocks > 0x7fffffffLL)
    return wdh::fail(WDH_EINVAL, "contraction: %lld workgroups exceed the grid limit", blocks);
  p.full_tiles = (int)w.full;
  p.tail_tiles = (int)w.tail;
  p.tail_split = w.split;
  p.kchunk = w.kchunk;
  g_last_plan = {BM, BN, w.split, g_last_form, w.full, w.tail};
  p.fd_tail_tiles = make_fastdiv(w.tail > 0 ? w.tail : 1);
  wdh_buf pooled = 0;
  if (w.tail > 0) {
    const size_t need = (size_t)w.tail * w.split * BM * BN * sizeof(float);
    if (g_static_scratch) {
      // the caller cannot allocate: the chunks' sums go to the library's static workspace,
      // through its device address (every element a reduce pass reads is written first by
      // the launch before it, so nothing has to be cleared between calls)
      if (need > (size_t)SK_PARTIAL_FLOATS * 4)
        return wdh::fail(WDH_EINVAL,
                         "wdh_gemm_static: this problem is cut into %lld x %d partial tiles of %d x %d, "
                         "%zu bytes; the static workspace holds %zu (set split_k to 1 to run it unsplit)",
                         w.tail, w.split, BM, BN, need, (size_t)SK_PARTIAL_FLOATS * 4);
      p.partial = static_scratch();
      if (!p.partial) return wdh::fail(WDH_ESTATE, "wdh_gemm_static: no static workspace on device %d", wdh::device());
    } else {
      pooled = wdh_alloc(need);
      if (!pooled) return WDH_ENOMEM;
      p.partial = (float *)wdh::resolve(pooled, nullptr);
    }
  }
  start(dim3((unsigned)blocks), false);
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
// Which (tile, B mode, load width) combinations have a stream form built: all but the 64x256 tile,
// the flat-load gather and operands that are not 16-byte aligned (those keep one tile or chunk per
// workgroup).
constexpr bool stream_built(int bm, int bn, int bmode) { return !(bm == 64 && bn == 256) && bmode != B_IM2COL_BIG; }

template <int BM, int BN, int WM, int WN, bool A_KC, int BMODE>
int launch_tile(Params &p, int nz, bool vec) {
  g_last_form = BMODE;
  constexpr bool HAS_STREAM = stream_built(BM, BN, BMODE);
  return launch_planned<BM, BN>(p, nz, BMODE >= B_IM2COL32, BK, HAS_STREAM && vec ? stream_blocks(BM, BN) : 0,
                                [&](dim3 grid, bool stream) {
    if constexpr (HAS_STREAM) {
      if (stream) {
        hipLaunchKernelGGL((contraction_kernel<BM, BN, WM, WN, A_KC, BMODE, true, true>), grid,
                           dim3(NTHREADS), 0, wdh::stream(), p);
        return;
      }
    }
    if (vec)
      hipLaunchKernelGGL((contraction_kernel<BM, BN, WM, WN, A_KC, BMODE, true, false>), grid,
                         dim3(NTHREADS), 0, wdh::stream(), p);
    else
      hipLaunchKernelGGL((contraction_kernel<BM, BN, WM, WN, A_KC, BMODE, false, false>), grid,
                         dim3(NTHREADS), 0, wdh::stream(), p);
  });
}

template <int BM, int BN, int WM, int WN, int VECW>
void start_halo(const Params &p, dim3 grid, bool stream) {
  if (stream)
    hipLaunchKernelGGL((conv3x3_halo_kernel<BM, BN, WM, WN, VECW, true>), grid, dim3(NTHREADS), 0, wdh::stream(), p);
  else
    hipLaunchKernelGGL((conv3x3_halo_kernel<BM, BN, WM, WN, VECW, false>), grid, dim3(NTHREADS), 0, wdh::stream(), p);
}

template <int BM, int BN, int WM, int WN>
int launch_halo_tile(Params &p, int nz, int vecw) {
  g_last_form = WDH_FORM_CONV3X3_LDS;
  return launch_planned<BM, BN>(p, nz, true, HALO_KB, halo_blocks(BM, BN), [&](dim3 grid, bool stream) {
    if (vecw == 4) start_halo<BM, BN, WM, WN, 4>(p, grid, stream);
    else if (vecw == 2) start_halo<BM, BN, WM, WN, 2>(p, grid, stream);
    else start_halo<BM, BN, WM, WN, 1>(p, grid, stream);
  });
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
                                : (conv ? conv_tile : (g_tile_hint >= 0 ? (TileId)g_tile_hint : pick_tile(p.m, p.n, nz)));
  switch (t) {
    case T128x128: return launch_tile<128, 128, 2, 2, A_KC, BMODE>(p, nz, vec);
    case T64x256: return launch_tile<64, 256, 1, 4, A_KC, BMODE>(p, nz, vec);
    case T64x128: return launch_tile<64, 128, 1, 4, A_KC, BMODE>(p, nz, vec);
    case T128x64: return launch_tile<128, 64, 2, 2, A_KC, BMODE>(p, nz, vec);
    default: return launch_tile<64, 64, 2, 2, A_KC, BMODE>(p, nz, vec);
  }
}

// ---- one entry per kernel family, each defined in a translation unit of its own -----------
int launch_gemm_a_kc(bool b_kc, Params &p, int nz, bool vec);     // contraction_gemm_akc.hip
int launch_gemm_a_mc(bool b_kc, Params &p, int nz, bool vec);     // contraction_gemm_amc.hip
int launch_conv_gather(int mode, Params &p, int nz, bool vec);    // contraction_conv_gather.hip
int launch_conv_pixels(Params &p, int nz, bool vec, bool stride2);  // contraction_conv_pixels.hip
int launch_conv3x3(int tile, Params &p, int nz, int vecw);        // contraction_conv3x3.hip

}  // namespace wdhc
