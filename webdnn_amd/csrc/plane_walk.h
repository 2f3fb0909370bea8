// Index walk shared by the strided elementwise and copy kernels.
//
// A strided tensor view of rank <= 6 (axes already merged on the host) is cut
// into workgroup tiles over its last two axes; the coordinates on all outer
// axes come from the workgroup index alone, so they are decomposed once per
// workgroup (wavefront-uniform arithmetic) and a thread needs no division.
// Threads run along the innermost axis first: TX = 2^tx_log2 of them, the
// remaining 256 / TX along the second axis.  Each thread owns four items:
//   wide   (long innermost axis) : x0 + k*TX on one row,
//   narrow (short innermost axis): one x on rows y0 + k*TY.
// The innermost extent is counted in units of UNIT elements (4 for 16-byte
// accesses, 1 otherwise).
#pragma once
#include <stdint.h>

namespace wdh {

constexpr int WALK_MAXD = 6;

struct PlaneWalk {
  int nd;                     // rank after merging, >= 2 (a leading 1 is added to rank 1)
  unsigned shape[WALK_MAXD];  // extents, outermost first; shape[nd-1] in units
  unsigned tx_log2;
  unsigned xchunks, ychunks;  // workgroups along the innermost / the second axis
  bool wide;
  bool grid3d;                // launch grid (xchunks, ychunks, outer) instead of one folded axis
  unsigned blocks;            // xchunks * ychunks * product of the outer extents
  unsigned outer;             // product of the outer extents
};

// Fills `w` for a view of `nd` merged axes whose innermost extent is
// `inner_units` units.  Returns false when the walk would waste more than half
// of its threads or needs more workgroups than a grid holds; the caller then
// uses its per-element kernel.
inline bool plan_plane_walk(PlaneWalk *w, int nd, const unsigned *shape, unsigned inner_units) {
  if (nd < 1 || nd > WALK_MAXD || inner_units == 0 || inner_units > 0x7fffffffu) return false;
  unsigned s[WALK_MAXD];
  int n = 0;
  if (nd == 1) s[n++] = 1;
  for (int d = 0; d < nd; d++) s[n++] = shape[d];
  if (n > WALK_MAXD) return false;
  s[n - 1] = inner_units;
  if (s[n - 2] > 0x7fffffffu) return false;
  w->nd = n;
  for (int d = 0; d < n; d++) w->shape[d] = s[d];
  // TX: the power of two that covers a short innermost axis; for longer ones
  // whichever of 64 / 128 / 256 leaves the fewest threads without an item
  unsigned lg_lo = 0;
  while (lg_lo < 8 && (1u << lg_lo) < inner_units) lg_lo++;
  if (lg_lo > 6) lg_lo = 6;
  const unsigned lg_hi = inner_units > 64 ? 8 : lg_lo;
  double best = -1.0;
  unsigned long long xc = 0, yc = 0;
  for (unsigned lg = lg_hi; lg >= lg_lo; lg--) {
    const unsigned tx = 1u << lg, ty = 256u >> lg;
    const bool wide = inner_units >= 4 * tx;
    const unsigned long long px = wide ? 4ull * tx : tx, py = wide ? ty : 4ull * ty;
    const unsigned long long cx = (inner_units + px - 1) / px, cy = (s[n - 2] + py - 1) / py;
    const double eff = (double)inner_units * s[n - 2] / ((double)cx * px * (double)cy * py);
    if (eff > best + 1e-9) {
      best = eff; w->tx_log2 = lg; w->wide = wide;
      xc = cx; yc = cy;
    }
    if (lg == 0) break;
  }
  unsigned long long outer = 1;
  for (int d = 0; d + 2 < n; d++) {
    outer *= s[d];
    if (outer > 0x7fffffffULL) return false;
  }
  const unsigned long long blocks = xc * yc * outer;
  if (blocks > 0x7fffffffULL) return false;
  if (best < 0.5) return false;
  w->xchunks = (unsigned)xc;
  w->ychunks = (unsigned)yc;
  w->blocks = (unsigned)blocks;
  w->outer = (unsigned)outer;
  w->grid3d = yc <= 65535 && outer <= 65535;
  return true;
}

// Share of the walk's thread items that fall inside the plane of the last two axes.
inline double plane_walk_fill(const PlaneWalk &w) {
  const unsigned tx = 1u << w.tx_log2, ty = 256u >> w.tx_log2;
  const double px = w.wide ? 4.0 * tx : tx, py = w.wide ? ty : 4.0 * ty;
  return (double)w.shape[w.nd - 1] * w.shape[w.nd - 2] / ((double)w.xchunks * px * (double)w.ychunks * py);
}

// The other walk over the same view, for rows the tiles above fit badly (784 or 50 units
// leave a quarter of a power-of-two tile empty): the plane of the last two axes is taken
// as one run of second * inner units, cut into chunks of a workgroup each, thread t of
// which takes units t, t + 256, ...; a unit's row is one multiply-high away.  Only a
// plane's last wavefront is ragged.  The result must be dense over the plane.
struct FlatWalk {
  unsigned plane;    // second * inner, in units
  unsigned inner;    // units per row
  unsigned chunk;    // units per workgroup
  unsigned chunks;   // workgroups per plane
  unsigned outer;    // product of the outer extents
  int n_outer;
  unsigned oshape[WALK_MAXD];
};

inline bool plan_flat_walk(FlatWalk *f, int nd, const unsigned *shape, unsigned inner_units) {
  if (nd < 2 || nd > WALK_MAXD || inner_units == 0) return false;
  const unsigned long long plane = (unsigned long long)shape[nd - 2] * inner_units;
  if (plane < 256 || plane >= 0x7fffffffULL) return false;
  unsigned long long outer = 1;
  for (int d = 0; d + 2 < nd; d++) {
    outer *= shape[d];
    if (outer > 0x7fffffffULL) return false;
    f->oshape[d] = shape[d];
  }
  f->plane = (unsigned)plane;
  f->inner = inner_units;
  f->chunk = plane <= 8192 ? (unsigned)plane : 4096u;
  f->chunks = (unsigned)((plane + f->chunk - 1) / f->chunk);
  f->outer = (unsigned)outer;
  f->n_outer = nd - 2;
  return outer * f->chunks <= 0x7fffffffULL;
}

#ifdef __HIPCC__
// Where a workgroup of a flat walk works: its coordinates on the outer axes, their linear
// index, and the range [begin, end) of the plane's units it covers.
struct FlatPos {
  unsigned oc[WALK_MAXD];
  unsigned outer_linear, begin, end;
};
__device__ __forceinline__ FlatPos flat_position(const FlatWalk &f) {
  FlatPos q;
  unsigned b = blockIdx.x;
  const unsigned c = b % f.chunks;
  b /= f.chunks;
  q.outer_linear = b;
#pragma unroll
  for (int d = WALK_MAXD - 3; d >= 0; d--) {
    q.oc[d] = 0;
    if (d < f.n_outer) {
      const unsigned t = b / f.oshape[d];
      q.oc[d] = b - t * f.oshape[d];
      b = t;
    }
  }
  q.begin = c * f.chunk;
  q.end = q.begin + f.chunk < f.plane ? q.begin + f.chunk : f.plane;
  return q;
}

// The launch grid of a planned walk.  The three-axis form hands the kernel its
// tile and outer index without any division; extents beyond a grid axis's
// limit fall back to one folded axis.
inline dim3 plane_grid(const PlaneWalk &w) {
  return w.grid3d ? dim3(w.xchunks, w.ychunks, w.outer) : dim3(w.blocks);
}

// Position of the calling thread: coordinates on the outer axes (oc[0..nd-3]),
// the linear index over those axes, the first item (x0, y0) and the step
// between a thread's four items (dx along the innermost axis, dy along the second).
struct PlanePos {
  unsigned oc[WALK_MAXD];
  unsigned outer_linear;
  unsigned x0, y0, dx, dy;
};

__device__ __forceinline__ PlanePos plane_position(const PlaneWalk &w) {
  PlanePos q;
  unsigned b, cx, cy;
  if (w.grid3d) {
    cx = blockIdx.x; cy = blockIdx.y; b = blockIdx.z;
  } else {
    b = blockIdx.x;
    cx = b % w.xchunks;
    b /= w.xchunks;
    cy = b % w.ychunks;
    b /= w.ychunks;
  }
  q.outer_linear = b;
#pragma unroll
  for (int d = WALK_MAXD - 3; d >= 1; d--) {
    q.oc[d] = 0;
    if (d < w.nd - 2) {
      const unsigned t = b / w.shape[d];
      q.oc[d] = b - t * w.shape[d];
      b = t;
    }
  }
  q.oc[0] = w.nd > 2 ? b : 0;  // the outermost coordinate is what remains
  const unsigned tx_n = 1u << w.tx_log2, ty_n = 256u >> w.tx_log2;
  const unsigned tx = threadIdx.x & (tx_n - 1), ty = threadIdx.x >> w.tx_log2;
  if (w.wide) {
    q.x0 = cx * tx_n * 4 + tx; q.dx = tx_n;
    q.y0 = cy * ty_n + ty;     q.dy = 0;
  } else {
    q.x0 = cx * tx_n + tx;     q.dx = 0;
    q.y0 = cy * ty_n * 4 + ty; q.dy = ty_n;
  }
  return q;
}
#endif

}  // namespace wdh
