// MaxPool (2-D, NCHW), Transpose (rank <= 6 gather-copy) and Gather.
// All three move bytes without arithmetic on them, so results are bit-exact.
//
// Reference semantics:
//   MaxPool   : src/descriptor_runner/operators/cpu/operators/standard/maxpool.ts:58-112
//   Transpose : src/descriptor_runner/operators/cpu/operators/standard/transpose.ts:46-168
//   Gather    : src/descriptor_runner/operators/cpu/operators/standard/gather.ts:20-33
#include <math.h>

#include "common.h"
#include "fastdiv.h"
#include "plane_walk.h"

namespace {

constexpr int MAXD = 6;

// ---- max pooling -------------------------------------------------------------
// One thread per output cell, consecutive threads along ow, so stores are
// coalesced and the overlapping input windows of neighbouring threads are
// served by the vector L1.  blockIdx.x is the (n, c) plane, blockIdx.y a run of
// blockDim.x cells of it: one division per thread.  For windows of up to 3x3 (KH, KW
// > 0) the taps are unrolled and read without branches, so all of a thread's
// loads are in flight together; taps that fall in the padding read a clamped
// address and are replaced by -inf, which the strict comparison never selects.
struct PoolParams {
  const float *X;
  float *Y;
  int h, w, oh, ow, kh, kw, pt, pl, sh, sw, dh, dw;
};

template <int KH, int KW>
__global__ __launch_bounds__(256) void maxpool2d_kernel(PoolParams p) {
  const unsigned cell = blockIdx.y * blockDim.x + threadIdx.x;
  if (cell >= (unsigned)(p.oh * p.ow)) return;
  const int oy = (int)(cell / (unsigned)p.ow);
  const int ox = (int)(cell - (unsigned)oy * (unsigned)p.ow);
  const float *x = p.X + (long long)blockIdx.x * p.h * p.w;
  float *y = p.Y + (long long)blockIdx.x * p.oh * p.ow;
  float mv = -INFINITY;
  if constexpr (KH > 0) {
    float v[KH * KW];
#pragma unroll
    for (int ky = 0; ky < KH; ky++) {
      const int iy = oy * p.sh - p.pt + ky * p.dh;
      const bool rok = (unsigned)iy < (unsigned)p.h;
      const int cy = rok ? iy : 0;
#pragma unroll
      for (int kx = 0; kx < KW; kx++) {
        const int ix = ox * p.sw - p.pl + kx * p.dw;
        const bool ok = rok && (unsigned)ix < (unsigned)p.w;
        const float t = x[cy * p.w + (ok ? ix : 0)];
        v[ky * KW + kx] = ok ? t : -INFINITY;
      }
    }
#pragma unroll
    for (int i = 0; i < KH * KW; i++)
      if (v[i] > mv) mv = v[i];  // strict, NaN never selected: maxpool.ts:98-101
  } else {
    for (int ky = 0; ky < p.kh; ky++) {
      const int iy = oy * p.sh - p.pt + ky * p.dh;
      if ((unsigned)iy >= (unsigned)p.h) continue;
      for (int kx = 0; kx < p.kw; kx++) {
        const int ix = ox * p.sw - p.pl + kx * p.dw;
        if ((unsigned)ix >= (unsigned)p.w) continue;
        const float t = x[iy * p.w + ix];
        if (t > mv) mv = t;
      }
    }
  }
  y[cell] = mv;
}

// Band variant: a workgroup owns `rows` output rows of one plane.  The input
// rows they touch are whole rows, hence one contiguous span; it is copied to
// LDS with coalesced (16-byte where VEC) loads, and the window taps are read
// from there.  Global memory then sees every input element about once per
// band instead of once per tap.
struct PoolBand {
  int rows;     // output rows per workgroup
  int in_rows;  // input rows one band can touch: (rows-1)*sh + (kh-1)*dh + 1
  int tx_log2;  // threads along ow = 2^tx_log2 (at most one wavefront)
};

template <int KH, int KW, bool VEC>
__global__ __launch_bounds__(256) void maxpool2d_band_kernel(PoolParams p, PoolBand b) {
  extern __shared__ float band[];
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  const int oy0 = blockIdx.y * b.rows;
  const int iy0 = oy0 * p.sh - p.pt;                // may lie in the top padding
  const int lo = iy0 < 0 ? 0 : iy0;
  const int hi = iy0 + b.in_rows < p.h ? iy0 + b.in_rows : p.h;
  const float *x = p.X + (long long)blockIdx.x * p.h * p.w + (long long)lo * p.w;
  const int count = (hi - lo) * p.w;                // floats of rows lo..hi-1
  if (VEC) {
    for (int i = threadIdx.x * 4; i < count; i += 1024)
      *reinterpret_cast<f32x4 *>(band + i) = *reinterpret_cast<const f32x4 *>(x + i);
  } else {
    for (int i = threadIdx.x; i < count; i += 256) band[i] = x[i];
  }
  __syncthreads();
  const int nrows = p.oh - oy0 < b.rows ? p.oh - oy0 : b.rows;
  float *y = p.Y + ((long long)blockIdx.x * p.oh + oy0) * p.ow;
  // threads: 2^tx_log2 along ow, the rest along the band's rows
  const int tx_n = 1 << b.tx_log2;
  for (int r = threadIdx.x >> b.tx_log2; r < nrows; r += 256 >> b.tx_log2) {
    const int iyb = (oy0 + r) * p.sh - p.pt;
    for (int ox = threadIdx.x & (tx_n - 1); ox < p.ow; ox += tx_n) {
      const int ixb = ox * p.sw - p.pl;
      float mv = -INFINITY;
      auto tap = [&](int ky, int kx) {
        const int iy = iyb + ky * p.dh, ix = ixb + kx * p.dw;
        // rows outside [lo, hi) and columns outside [0, w) are padding
        const bool ok = iy >= lo && iy < hi && (unsigned)ix < (unsigned)p.w;
        const float t = band[ok ? (iy - lo) * p.w + ix : 0];
        if (ok && t > mv) mv = t;                   // strict, NaN never selected: maxpool.ts:98-101
      };
      if constexpr (KH > 0) {
#pragma unroll
        for (int ky = 0; ky < KH; ky++)
#pragma unroll
          for (int kx = 0; kx < KW; kx++) tap(ky, kx);
      } else {
        for (int ky = 0; ky < p.kh; ky++)
          for (int kx = 0; kx < p.kw; kx++) tap(ky, kx);
      }
      y[r * p.ow + ox] = mv;
    }
  }
}

// 3x3 window, stride 2, one cell of padding on top and left, rows a multiple of four
// wide (the pool after a ResNet stem).  A thread owns two neighbouring output cells:
// their five input columns are one aligned 16-byte piece plus the column before it, so
// a thread issues three 16-byte and three 4-byte loads (all before the first compare)
// and one 8-byte store.  Neighbouring output rows share an input row; the vector L1
// serves the second reader.  No LDS and no barrier.
__global__ __launch_bounds__(256) void maxpool3x3s2_pairs(PoolParams p, unsigned pairs_per_row,
                                                           unsigned total_pairs) {
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  const unsigned id = blockIdx.x * 256u + threadIdx.x;
  if (id >= total_pairs) return;
  const unsigned rowid = id / pairs_per_row;          // plane * oh + oy
  const unsigned pair = id - rowid * pairs_per_row;
  const unsigned plane = rowid / (unsigned)p.oh;
  const int oy = (int)(rowid - plane * (unsigned)p.oh);
  const float *x = p.X + (long long)plane * p.h * p.w;
  const int c0 = 4 * (int)pair;                       // first column of the 16-byte piece
  f32x4 mid[3];
  float left[3];
#pragma unroll
  for (int ky = 0; ky < 3; ky++) {
    const int iy = 2 * oy - 1 + ky;
    const bool rok = (unsigned)iy < (unsigned)p.h;
    const float *row = x + (long long)(rok ? iy : 0) * p.w;
    const f32x4 m = *reinterpret_cast<const f32x4 *>(row + c0);
    const float l = row[c0 > 0 ? c0 - 1 : 0];
    const float ninf = -INFINITY;
    mid[ky] = rok ? m : f32x4{ninf, ninf, ninf, ninf};
    left[ky] = rok && c0 > 0 ? l : ninf;
  }
  float a = -INFINITY, b = -INFINITY;   // cells 2*pair and 2*pair + 1
#pragma unroll
  for (int ky = 0; ky < 3; ky++) {
    // strict comparisons, NaN never selected: maxpool.ts:98-101
    if (left[ky] > a) a = left[ky];
    if (mid[ky][0] > a) a = mid[ky][0];
    if (mid[ky][1] > a) a = mid[ky][1];
    if (mid[ky][1] > b) b = mid[ky][1];
    if (mid[ky][2] > b) b = mid[ky][2];
    if (mid[ky][3] > b) b = mid[ky][3];
  }
  float *y = p.Y + (long long)rowid * p.ow + 2 * pair;
  *reinterpret_cast<f32x2 *>(y) = f32x2{a, b};
}

// ---- transpose -----------------------------------------------------------------
// Strided copy (Slice, Concat, Split): both sides addressed through strides.
struct StridedCopyParams {
  const uint32_t *X;
  uint32_t *Y;
  long long total;
  int ndim;
  unsigned shape[MAXD];
  long long sx[MAXD];
  long long sy[MAXD];
};

// Thread per element, innermost axis fastest: coalesced wherever the innermost
// stride is 1 (always on the dense side of a Slice/Concat/Split).
template <typename IDX>
__global__ __launch_bounds__(256) void strided_copy_kernel(StridedCopyParams p) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < p.total;
       i += stride) {
    IDX rem = (IDX)i;
    long long ox = 0, oy = 0;
#pragma unroll
    for (int d = MAXD - 1; d >= 0; d--) {
      if (d < p.ndim) {
        const IDX q = rem / (IDX)p.shape[d];
        const long long r = (long long)(rem - q * (IDX)p.shape[d]);
        ox += r * p.sx[d];
        oy += r * p.sy[d];
        rem = q;
      }
    }
    p.Y[oy] = p.X[ox];
  }
}

// Strided copy through the workgroup-tiled walk of plane_walk.h: no division
// per thread, and 16 bytes per access (UNIT = 4) when both sides step by 1
// along the innermost axis and every other stride and both bases are
// multiples of 4 elements.  A thread issues its four loads before its stores.
template <int UNIT>
__global__ __launch_bounds__(256) void copy_plane(StridedCopyParams p, wdh::PlaneWalk w) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  const wdh::PlanePos q = wdh::plane_position(w);
  long long bx = 0, by = 0;
#pragma unroll
  for (int d = 0; d < MAXD - 2; d++) {
    if (d < w.nd - 2) {
      bx += (long long)q.oc[d] * p.sx[d];
      by += (long long)q.oc[d] * p.sy[d];
    }
  }
  const unsigned inner = w.shape[w.nd - 1], second = w.shape[w.nd - 2];
  const long long sx2 = p.sx[w.nd - 2], sy2 = p.sy[w.nd - 2];
  const long long sx1 = p.sx[w.nd - 1] * UNIT, sy1 = p.sy[w.nd - 1] * UNIT;
  u32x4 v4[4];
  uint32_t v1[4];
  bool ok[4];
#pragma unroll
  for (int k = 0; k < 4; k++) {
    const unsigned x = q.x0 + k * q.dx, y = q.y0 + k * q.dy;
    ok[k] = x < inner && y < second;
    if (ok[k]) {
      const uint32_t *src = p.X + bx + (long long)y * sx2 + (long long)x * sx1;
      if (UNIT == 4) v4[k] = *reinterpret_cast<const u32x4 *>(src);
      else v1[k] = *src;
    }
  }
#pragma unroll
  for (int k = 0; k < 4; k++) {
    if (ok[k]) {
      const unsigned x = q.x0 + k * q.dx, y = q.y0 + k * q.dy;
      uint32_t *dst = p.Y + by + (long long)y * sy2 + (long long)x * sy1;
      if (UNIT == 4) *reinterpret_cast<u32x4 *>(dst) = v4[k];
      else *dst = v1[k];
    }
  }
}

// Rows of the input gathered into a result whose last two axes are dense (a Slice or Split of
// feature maps, a Concat input's mirror image): a workgroup walks a chunk of the contiguous
// result plane with consecutive threads on consecutive result elements, whatever the row length,
// and finds each element's row with one multiply-high.  The tiled walk above would leave a
// quarter of its lanes idle on rows of 50 elements; here only a plane's last wavefront is ragged.
struct FlatCopyParams {
  const uint32_t *X;
  uint32_t *Y;
  wdh::FastDiv fd_inner;
  long long sx2;        // input stride between rows
  long long osx[MAXD], osy[MAXD];
};
__global__ __launch_bounds__(256) void copy_rows_flat(FlatCopyParams p, wdh::FlatWalk f) {
  const wdh::FlatPos q = wdh::flat_position(f);
  long long bx = 0, by = 0;
#pragma unroll
  for (int d = 0; d < MAXD - 2; d++) {
    if (d < f.n_outer) {
      bx += (long long)q.oc[d] * p.osx[d];
      by += (long long)q.oc[d] * p.osy[d];
    }
  }
  const uint32_t *x = p.X + bx;
  uint32_t *y = p.Y + by;
  for (unsigned f0 = q.begin + threadIdx.x; f0 < q.end; f0 += 1024) {
    uint32_t v[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const unsigned u = f0 + 256 * k;
      if (u < q.end) {
        const unsigned row = (unsigned)wdh::fdiv((int)u, p.fd_inner);
        v[k] = x[(long long)row * p.sx2 + (u - row * f.inner)];
      }
    }
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const unsigned u = f0 + 256 * k;
      if (u < q.end) y[u] = v[k];
    }
  }
}

// Tiled: when the input-contiguous axis `a` is not the last output axis, a
// workgroup moves a 4096-element tile spanned by (axis a, last axis) through LDS:
// reads run along axis a (contiguous in X), writes along the last axis
// (contiguous in Y).  The odd row pitch keeps both phases free of bank
// conflicts.  All remaining axes are folded into blockIdx.z.
struct TileParams {
  const uint32_t *X;
  uint32_t *Y;
  int ndim;               // number of "outer" axes (excluding a and last)
  unsigned oshape[MAXD];  // extents of the outer axes
  long long osin[MAXD];   // their input strides
  long long osout[MAXD];  // their output strides
  unsigned na, nl;        // extents of axis a and of the last axis
  long long a_out;        // output stride of axis a (its input stride is 1)
  long long l_in;         // input stride of the last axis (its output stride is 1)
};

// TA x TL tile (TA along axis a, TL = 4096 / TA along the last axis): the
// narrower TA shapes keep all threads busy when axis a is short.
template <int TA>
__global__ __launch_bounds__(256) void transpose_tiled_kernel(TileParams p) {
  constexpr int TL = 4096 / TA;
  __shared__ uint32_t tile[TL][TA + 1];
  long long rem = blockIdx.z, in_off = 0, out_off = 0;
#pragma unroll
  for (int d = MAXD - 1; d >= 0; d--) {
    if (d < p.ndim) {
      long long q = rem / p.oshape[d];
      long long c = rem - q * p.oshape[d];
      rem = q;
      in_off += c * p.osin[d];
      out_off += c * p.osout[d];
    }
  }
  const unsigned a0 = blockIdx.x * TA, l0 = blockIdx.y * TL;
  {  // read: consecutive threads run along axis a
    const unsigned ta = threadIdx.x % TA, a = a0 + ta;
    for (unsigned r = threadIdx.x / TA; r < TL; r += 256 / TA) {
      const unsigned l = l0 + r;
      if (a < p.na && l < p.nl) tile[r][ta] = p.X[in_off + (long long)l * p.l_in + a];
    }
  }
  __syncthreads();
  {  // write: consecutive threads run along the last axis
    const unsigned tl = threadIdx.x & 63;
    for (unsigned r = threadIdx.x >> 6; r < TA; r += 4) {
      const unsigned a = a0 + r;
      for (unsigned c = tl; c < TL; c += 64) {
        const unsigned l = l0 + c;
        if (a < p.na && l < p.nl) p.Y[out_off + (long long)a * p.a_out + l] = tile[c][r];
      }
    }
  }
}

// The same exchange with wider accesses, for inputs whose rows along axis a are 16-byte
// aligned multiples of four: a thread reads four neighbouring elements of axis a at once
// and writes two neighbouring elements of the last axis at once (rows of the result start
// on 8-byte boundaries far more often than on 16-byte ones: 850-float rows do).  12 memory
// instructions per thread instead of 32; the LDS tile and its odd pitch are unchanged.
template <int TA>
__global__ __launch_bounds__(256) void transpose_tiled_wide(TileParams p) {
  constexpr int TL = 4096 / TA;
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
  __shared__ uint32_t tile[TL][TA + 1];
  long long rem = blockIdx.z, in_off = 0, out_off = 0;
#pragma unroll
  for (int d = MAXD - 1; d >= 0; d--) {
    if (d < p.ndim) {
      long long q = rem / p.oshape[d];
      long long c = rem - q * p.oshape[d];
      rem = q;
      in_off += c * p.osin[d];
      out_off += c * p.osout[d];
    }
  }
  const unsigned a0 = blockIdx.x * TA, l0 = blockIdx.y * TL;
  {  // read: TA/4 threads cover a row of the tile along axis a
    constexpr unsigned TPR = TA / 4;
    const unsigned ta = (threadIdx.x % TPR) * 4, a = a0 + ta;
    for (unsigned r = threadIdx.x / TPR; r < TL; r += 256 / TPR) {
      const unsigned l = l0 + r;
      if (a < p.na && l < p.nl) {  // na is a multiple of 4: a + 3 < na
        const u32x4 v = *reinterpret_cast<const u32x4 *>(p.X + in_off + (long long)l * p.l_in + a);
        tile[r][ta] = v.x; tile[r][ta + 1] = v.y; tile[r][ta + 2] = v.z; tile[r][ta + 3] = v.w;
      }
    }
  }
  __syncthreads();
  {  // write: TL/2 threads cover a row of the result, two elements each
    constexpr unsigned PPR = TL / 2;
    const unsigned c = (threadIdx.x % PPR) * 2, l = l0 + c;
    for (unsigned r = threadIdx.x / PPR; r < TA; r += 256 / PPR) {
      const unsigned a = a0 + r;
      if (a >= p.na || l >= p.nl) continue;
      uint32_t *dst = p.Y + out_off + (long long)a * p.a_out + l;
      const uint32_t v0 = tile[c][r];
      if (l + 1 < p.nl) {
        const uint32_t v1 = tile[c + 1][r];
        if ((reinterpret_cast<uintptr_t>(dst) & 7) == 0) {
          *reinterpret_cast<u32x2 *>(dst) = u32x2{v0, v1};
        } else {
          dst[0] = v0;
          dst[1] = v1;
        }
      } else {
        dst[0] = v0;
      }
    }
  }
}

__global__ __launch_bounds__(256) void gather_axis_kernel(
    const uint32_t *__restrict__ D, const int *__restrict__ Idx,
    uint32_t *__restrict__ Y, long long outer, int axis_len, long long inner,
    long long n_idx) {
  const long long total = outer * n_idx * inner;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += stride) {
    long long in = i % inner;
    long long t = i / inner;
    long long j = t % n_idx;
    long long o = t / n_idx;
    int ix = Idx[j];
    if (ix < 0) ix += axis_len;
    // out-of-range indices read element 0 rather than stray memory
    if (ix < 0 || ix >= axis_len) ix = 0;
    Y[i] = D[(o * axis_len + ix) * inner + in];
  }
}

unsigned grid_for(long long items) {
  long long blocks = (items + 255) / 256;
  long long cap = (long long)wdh::compute_units() * 16;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  return (unsigned)blocks;
}

// Launches the copy described by `g` (axes merged, total > 0).
int launch_strided_copy(const StridedCopyParams &g) {
  hipStream_t st = wdh::stream();
  const int nd = g.ndim;
  bool vec = g.shape[nd - 1] % 4 == 0 && g.sx[nd - 1] == 1 && g.sy[nd - 1] == 1 &&
             (((uintptr_t)g.X | (uintptr_t)g.Y) & 15) == 0;
  for (int d = 0; d + 1 < nd && vec; d++) vec = g.sx[d] % 4 == 0 && g.sy[d] % 4 == 0;
  wdh::PlaneWalk w;
  const bool walk = wdh::plan_plane_walk(&w, nd, g.shape, vec ? g.shape[nd - 1] / 4 : g.shape[nd - 1]);
  // a dense result plane whose rows the tiled walk would cover badly: the flat walk
  wdh::FlatWalk fw;
  if (!vec && nd >= 2 && g.sx[nd - 1] == 1 && g.sy[nd - 1] == 1 && g.sy[nd - 2] == (long long)g.shape[nd - 1] &&
      (!walk || wdh::plane_walk_fill(w) < 0.9) && wdh::plan_flat_walk(&fw, nd, g.shape, g.shape[nd - 1])) {
    FlatCopyParams f = {};
    f.X = g.X; f.Y = g.Y;
    f.fd_inner = wdh::make_fastdiv(fw.inner);
    f.sx2 = g.sx[nd - 2];
    for (int d = 0; d < nd - 2; d++) { f.osx[d] = g.sx[d]; f.osy[d] = g.sy[d]; }
    hipLaunchKernelGGL(copy_rows_flat, dim3(fw.outer * fw.chunks), dim3(256), 0, st, f, fw);
    WDH_LAUNCH_CHECK();
    return WDH_OK;
  }
  if (walk) {
    StridedCopyParams s = g;
    if (w.nd != nd) {  // rank 1: the walk adds a leading axis of extent 1
      for (int d = nd; d > 0; d--) { s.sx[d] = g.sx[d - 1]; s.sy[d] = g.sy[d - 1]; }
      s.sx[0] = s.sy[0] = 0;
    }
    if (vec) hipLaunchKernelGGL(copy_plane<4>, wdh::plane_grid(w), dim3(256), 0, st, s, w);
    else hipLaunchKernelGGL(copy_plane<1>, wdh::plane_grid(w), dim3(256), 0, st, s, w);
  } else if (g.total <= 0xffffffffLL) {
    hipLaunchKernelGGL(strided_copy_kernel<unsigned>, dim3(grid_for(g.total)), dim3(256), 0, st, g);
  } else {
    hipLaunchKernelGGL(strided_copy_kernel<long long>, dim3(grid_for(g.total)), dim3(256), 0, st, g);
  }
  WDH_LAUNCH_CHECK();
  return WDH_OK;
}

}  // namespace

using wdh::fail;

extern "C" int wdh_maxpool2d(wdh_buf hX, wdh_buf hY, int n, int c, int h, int w,
                             int oh, int ow, int kh, int kw, int pt, int pl, int sh,
                             int sw, int dh, int dw) {
  WDH_REQUIRE_INIT();
  WDH_REQUIRE_COMPUTE_LANE();
  if (n < 0 || c < 0 || h <= 0 || w <= 0 || oh < 0 || ow < 0 || kh <= 0 || kw <= 0 ||
      sh <= 0 || sw <= 0 || dh <= 0 || dw <= 0 || pt < 0 || pl < 0)
    return fail(WDH_EINVAL, "wdh_maxpool2d: bad geometry");
  // every input read is bounds-checked in the kernel, so an (oh, ow) larger than
  // the geometry implies only yields windows that lie in the padding (-inf)
  const long long planes = (long long)n * c, cells = (long long)oh * ow;
  if (planes == 0 || cells == 0) return WDH_OK;
  if (planes > 0x7fffffffLL || cells > 65535LL * 256 || (long long)h * w > 0x7fffffffLL)
    return fail(WDH_EINVAL, "wdh_maxpool2d: %lld planes of %lld cells exceed the launch grid",
                planes, cells);
  PoolParams p;
  void *px, *py;
  if (!wdh::operand(hX, (size_t)planes * h * w * 4, "wdh_maxpool2d: X", &px)) return WDH_EINVAL;
  if (!wdh::operand(hY, (size_t)planes * cells * 4, "wdh_maxpool2d: Y", &py)) return WDH_EINVAL;
  p.X = (const float *)px; p.Y = (float *)py;
  p.h = h; p.w = w; p.oh = oh; p.ow = ow; p.kh = kh; p.kw = kw;
  p.pt = pt; p.pl = pl; p.sh = sh; p.sw = sw; p.dh = dh; p.dw = dw;
  hipStream_t st = wdh::stream();
  // the stem's pool: two cells per thread straight from global memory
  if (kh == 3 && kw == 3 && sh == 2 && sw == 2 && dh == 1 && dw == 1 && pt == 1 && pl == 1 &&
      w % 4 == 0 && 2 * ow == w && 2 * (oh - 1) - 1 < h && ((uintptr_t)px & 15) == 0 &&
      ((uintptr_t)py & 7) == 0 && planes * oh * (ow / 2) < 0xffffffffLL) {
    const unsigned pairs_per_row = (unsigned)(ow / 2);
    const unsigned total = (unsigned)(planes * oh * pairs_per_row);
    hipLaunchKernelGGL(maxpool3x3s2_pairs, dim3((total + 255) / 256), dim3(256), 0, st, p, pairs_per_row, total);
    WDH_LAUNCH_CHECK();
    return WDH_OK;
  }
  // band variant: enough rows for two cells per thread, the span within 32 KB of LDS
  {
    PoolBand b;
    b.tx_log2 = 0;
    while (b.tx_log2 < 6 && (1 << b.tx_log2) < ow) b.tx_log2++;
    const int rows_per_pass = 256 >> b.tx_log2;
    b.rows = ((512 + ow - 1) / ow + rows_per_pass - 1) / rows_per_pass * rows_per_pass;
    if (b.rows > oh) b.rows = oh;
    const long long in_rows = (long long)(b.rows - 1) * sh + (long long)(kh - 1) * dh + 1;
    const long long bands = (oh + b.rows - 1) / b.rows;
    if (cells >= 256 && in_rows * w <= 8192 && bands <= 65535) {
      b.in_rows = (int)in_rows;
      const bool vec = w % 4 == 0 && ((long long)h * w) % 4 == 0 && ((uintptr_t)px & 15) == 0;
      const dim3 grid((unsigned)planes, (unsigned)bands);
      const size_t lds = (size_t)in_rows * w * 4;
#define WDH_POOL_BAND(KH, KW)                                                                     \
  do {                                                                                            \
    if (vec) hipLaunchKernelGGL((maxpool2d_band_kernel<KH, KW, true>), grid, dim3(256), lds, st, p, b); \
    else hipLaunchKernelGGL((maxpool2d_band_kernel<KH, KW, false>), grid, dim3(256), lds, st, p, b);    \
  } while (0)
      if (kh == 3 && kw == 3) WDH_POOL_BAND(3, 3);
      else if (kh == 2 && kw == 2) WDH_POOL_BAND(2, 2);
      else WDH_POOL_BAND(0, 0);
#undef WDH_POOL_BAND
      WDH_LAUNCH_CHECK();
      return WDH_OK;
    }
  }
  const unsigned threads = cells <= 64 ? 64 : cells <= 128 ? 128 : 256;
  const dim3 grid((unsigned)planes, (unsigned)((cells + threads - 1) / threads)), block(threads);
  if (kh == 3 && kw == 3) hipLaunchKernelGGL((maxpool2d_kernel<3, 3>), grid, block, 0, st, p);
  else if (kh == 2 && kw == 2) hipLaunchKernelGGL((maxpool2d_kernel<2, 2>), grid, block, 0, st, p);
  else hipLaunchKernelGGL((maxpool2d_kernel<0, 0>), grid, block, 0, st, p);
  WDH_LAUNCH_CHECK();
  return WDH_OK;
}

extern "C" int wdh_transpose(wdh_buf hX, wdh_buf hY, int ndim,
                             const int32_t *out_shape, const int64_t *in_strides) {
  WDH_REQUIRE_INIT();
  WDH_REQUIRE_COMPUTE_LANE();
  if (ndim < 0 || ndim > MAXD)
    return fail(WDH_EINVAL, "wdh_transpose: ndim %d outside 0..%d", ndim, MAXD);
  if (ndim > 0 && (!out_shape || !in_strides))
    return fail(WDH_EINVAL, "wdh_transpose: NULL shape or strides");
  // drop extent-1 axes; merge neighbours that are contiguous in the input
  unsigned shape[MAXD];
  long long sin[MAXD];
  int nd = 0;
  long long total = 1, span = 1;
  for (int d = 0; d < ndim; d++) {
    if (out_shape[d] < 0 || in_strides[d] < 0)
      return fail(WDH_EINVAL, "wdh_transpose: negative extent or stride");
    total *= out_shape[d];
    if (out_shape[d] == 1) continue;
    span += (long long)(out_shape[d] - 1) * in_strides[d];
    if (nd > 0 && sin[nd - 1] == in_strides[d] * out_shape[d] &&
        (unsigned long long)shape[nd - 1] * out_shape[d] <= 0xffffffffULL) {
      shape[nd - 1] *= out_shape[d];
      sin[nd - 1] = in_strides[d];
    } else {
      shape[nd] = out_shape[d];
      sin[nd] = in_strides[d];
      nd++;
    }
  }
  if (total == 0) return WDH_OK;
  void *px, *py;
  if (!wdh::operand(hX, (size_t)span * 4, "wdh_transpose: X", &px)) return WDH_EINVAL;
  if (!wdh::operand(hY, (size_t)total * 4, "wdh_transpose: Y", &py)) return WDH_EINVAL;
  hipStream_t st = wdh::stream();
  if (nd <= 1 && (nd == 0 || sin[0] == 1)) {  // identity permutation
    WDH_HIP_CHECK(hipMemcpyAsync(py, px, (size_t)total * 4, hipMemcpyDeviceToDevice, st));
    return WDH_OK;
  }
  // output strides of the collapsed axes
  long long sout[MAXD];
  {
    long long acc = 1;
    for (int d = nd - 1; d >= 0; d--) { sout[d] = acc; acc *= shape[d]; }
  }
  int a = -1;
  for (int d = 0; d < nd; d++)
    if (sin[d] == 1) a = d;
  if (a >= 0 && a != nd - 1 && shape[a] >= 16 && shape[nd - 1] >= 16) {
    TileParams t = {};
    t.X = (const uint32_t *)px; t.Y = (uint32_t *)py;
    long long nouter = 1;
    for (int d = 0; d < nd - 1; d++) {
      if (d == a) continue;
      t.oshape[t.ndim] = shape[d];
      t.osin[t.ndim] = sin[d];
      t.osout[t.ndim] = sout[d];
      t.ndim++;
      nouter *= shape[d];
    }
    t.na = shape[a]; t.nl = shape[nd - 1];
    t.a_out = sout[a]; t.l_in = sin[nd - 1];
    // Result rows that do not end on a 128-byte line (850 floats) make every run of a tile's writes
    // touch a partial line: runs of 128 floats instead of 64 halve that share, as long as the reads
    // stay whole lines (input rows that are multiples of 32 floats).  11.96 -> 10.15 us on
    // [32,850,256] -> [32,256,850]; square tiles are better everywhere else.
    const bool long_runs = t.nl >= 128 && t.nl % 32 != 0 && t.na % 32 == 0;
    const unsigned ta = (t.na <= 16 && t.nl >= 256) ? 16 : ((t.na <= 32 && t.nl >= 128) || long_runs) ? 32 : 64;
    const unsigned tl = 4096 / ta;
    const unsigned gx = (t.na + ta - 1) / ta, gy = (t.nl + tl - 1) / tl;
    if (nouter <= 65535 && gy <= 65535) {
      const dim3 grid(gx, gy, (unsigned)nouter);
      bool wide = t.na % 4 == 0 && t.l_in % 4 == 0 && ((uintptr_t)px & 15) == 0;
      for (int d = 0; d < t.ndim; d++) wide = wide && t.osin[d] % 4 == 0;
      if (wide) {
        if (ta == 16) hipLaunchKernelGGL(transpose_tiled_wide<16>, grid, dim3(256), 0, st, t);
        else if (ta == 32) hipLaunchKernelGGL(transpose_tiled_wide<32>, grid, dim3(256), 0, st, t);
        else hipLaunchKernelGGL(transpose_tiled_wide<64>, grid, dim3(256), 0, st, t);
      } else if (ta == 16) hipLaunchKernelGGL(transpose_tiled_kernel<16>, grid, dim3(256), 0, st, t);
      else if (ta == 32) hipLaunchKernelGGL(transpose_tiled_kernel<32>, grid, dim3(256), 0, st, t);
      else hipLaunchKernelGGL(transpose_tiled_kernel<64>, grid, dim3(256), 0, st, t);
      WDH_LAUNCH_CHECK();
      return WDH_OK;
    }
  }
  // no tile to exchange: a strided read into the dense output
  StridedCopyParams g = {};
  g.X = (const uint32_t *)px; g.Y = (uint32_t *)py;
  g.total = total; g.ndim = nd;
  for (int d = 0; d < nd; d++) { g.shape[d] = shape[d]; g.sx[d] = sin[d]; g.sy[d] = sout[d]; }
  return launch_strided_copy(g);
}

extern "C" int wdh_gather(wdh_buf hD, wdh_buf hI, wdh_buf hY, int64_t outer,
                          int axis_len, int64_t inner, int64_t n_idx) {
  WDH_REQUIRE_INIT();
  WDH_REQUIRE_COMPUTE_LANE();
  if (outer < 0 || axis_len < 0 || inner < 0 || n_idx < 0)
    return fail(WDH_EINVAL, "wdh_gather: negative extent");
  const long long total = (long long)outer * n_idx * inner;
  if (total == 0) return WDH_OK;
  if (axis_len == 0) return fail(WDH_EINVAL, "wdh_gather: empty axis");
  void *pd, *pi, *py;
  if (!wdh::operand(hD, (size_t)outer * axis_len * inner * 4, "wdh_gather: Data", &pd)) return WDH_EINVAL;
  if (!wdh::operand(hI, (size_t)n_idx * 4, "wdh_gather: Indices", &pi)) return WDH_EINVAL;
  if (!wdh::operand(hY, (size_t)total * 4, "wdh_gather: Y", &py)) return WDH_EINVAL;
  hipLaunchKernelGGL(gather_axis_kernel, dim3(grid_for(total)), dim3(256), 0,
                     wdh::stream(), (const uint32_t *)pd, (const int *)pi,
                     (uint32_t *)py, (long long)outer, axis_len, (long long)inner,
                     (long long)n_idx);
  WDH_LAUNCH_CHECK();
  return WDH_OK;
}

extern "C" int wdh_strided_copy(wdh_buf hX, int64_t x_offset, wdh_buf hY, int64_t y_offset,
                                int ndim, const int32_t *shape, const int64_t *x_strides,
                                const int64_t *y_strides) {
  WDH_REQUIRE_INIT();
  WDH_REQUIRE_COMPUTE_LANE();
  if (ndim < 0 || ndim > MAXD)
    return fail(WDH_EINVAL, "wdh_strided_copy: ndim %d outside 0..%d", ndim, MAXD);
  if (ndim > 0 && (!shape || !x_strides || !y_strides))
    return fail(WDH_EINVAL, "wdh_strided_copy: NULL shape or strides");
  if (x_offset < 0 || y_offset < 0)
    return fail(WDH_EINVAL, "wdh_strided_copy: negative offset");
  // Negative strides are allowed on the X side (a Slice with a negative step);
  // the lowest and highest element touched on each side are bounds-checked.
  StridedCopyParams g = {};
  long long total = 1, x_lo = x_offset, x_hi = x_offset, y_hi = y_offset;
  int nd = 0;
  for (int d = 0; d < ndim; d++) {
    if (shape[d] < 0 || y_strides[d] < 0)
      return fail(WDH_EINVAL, "wdh_strided_copy: negative extent or Y stride");
    total *= shape[d];
    if (shape[d] <= 1) continue;
    const long long reach = (long long)(shape[d] - 1) * x_strides[d];
    if (reach < 0) x_lo += reach; else x_hi += reach;
    y_hi += (long long)(shape[d] - 1) * y_strides[d];
    // merge with the previous axis when both sides step contiguously across it
    if (nd > 0 && g.sx[nd - 1] == x_strides[d] * shape[d] &&
        g.sy[nd - 1] == y_strides[d] * shape[d] &&
        (unsigned long long)g.shape[nd - 1] * shape[d] <= 0xffffffffULL) {
      g.shape[nd - 1] *= shape[d];
      g.sx[nd - 1] = x_strides[d];
      g.sy[nd - 1] = y_strides[d];
    } else {
      g.shape[nd] = shape[d];
      g.sx[nd] = x_strides[d];
      g.sy[nd] = y_strides[d];
      nd++;
    }
  }
  if (total == 0) return WDH_OK;
  if (x_lo < 0) return fail(WDH_EINVAL, "wdh_strided_copy: X view starts before the buffer");
  void *px, *py;
  if (!wdh::operand(hX, (size_t)(x_hi + 1) * 4, "wdh_strided_copy: X", &px)) return WDH_EINVAL;
  if (!wdh::operand(hY, (size_t)(y_hi + 1) * 4, "wdh_strided_copy: Y", &py)) return WDH_EINVAL;
  g.X = (const uint32_t *)px + x_offset;
  g.Y = (uint32_t *)py + y_offset;
  g.total = total;
  g.ndim = nd;
  if (nd == 0 || (nd == 1 && g.sx[0] == 1 && g.sy[0] == 1)) {
    WDH_HIP_CHECK(hipMemcpyAsync(g.Y, g.X, (size_t)total * 4, hipMemcpyDeviceToDevice,
                                 wdh::stream()));
    return WDH_OK;
  }
  return launch_strided_copy(g);
}
