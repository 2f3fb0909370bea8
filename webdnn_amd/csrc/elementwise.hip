// Bandwidth-bound elementwise kernels: broadcasting binary ops and unary ops.
//
// Semantics follow the reference CPU operators, which evaluate every element
// in JavaScript double arithmetic and store into the typed output array:
//   Binary7  : src/descriptor_runner/operators/cpu/operators/standard/binary7.ts:16-68,257-291
//   CPUUnary : src/descriptor_runner/operators/cpu/operators/standard/unary.ts:10-32
// For fp32 +,-,*,/ the double-then-round result equals the IEEE fp32 result,
// so those are single fp32 instructions here (compiled with contraction off).
#include <math.h>

#include <type_traits>

#include "common.h"
#include "fastdiv.h"
#include "plane_walk.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
constexpr int MAXD = 6;

struct BinaryParams {
  const void *L;
  const void *R;
  void *Y;
  long long total;          // number of output elements
  int ndim;                 // after collapsing, >= 1
  unsigned shape[MAXD];     // output shape, outermost first
  long long sl[MAXD];       // element strides of L (0 on broadcast axes)
  long long sr[MAXD];
};

// JavaScript ToInt32 of a double (what storing into an Int32Array does).
__device__ __forceinline__ int js_to_int32(double d) {
  if (!(d == d) || isinf(d)) return 0;
  double t = trunc(d);
  double m = fmod(t, 4294967296.0);
  if (m < 0) m += 4294967296.0;
  return (int)(unsigned)m;
}

template <int OP>
__device__ __forceinline__ float apply_f(float l, float r) {
  if (OP == WDH_BIN_ADD) return l + r;
  if (OP == WDH_BIN_SUB) return l - r;
  if (OP == WDH_BIN_MUL) return l * r;
  if (OP == WDH_BIN_DIV) return l / r;
  return (float)pow((double)l, (double)r);
}

template <int OP>
__device__ __forceinline__ int apply_i(int l, int r) {
  double a = (double)l, b = (double)r;
  if (OP == WDH_BIN_ADD) return js_to_int32(a + b);
  if (OP == WDH_BIN_SUB) return js_to_int32(a - b);
  if (OP == WDH_BIN_MUL) return js_to_int32(a * b);
  if (OP == WDH_BIN_DIV) return js_to_int32(a / b);
  return js_to_int32(pow(a, b));
}

// Dense fast path: both inputs have the output's shape.  16-byte accesses,
// grid-stride; the tail (total % 4) is handled by the first few threads.
template <int OP>
__global__ __launch_bounds__(256) void binary_dense_f32(const float *__restrict__ L,
                                                        const float *__restrict__ R,
                                                        float *__restrict__ Y,
                                                        long long total) {
  const long long nvec = total >> 2;
  const long long stride = (long long)gridDim.x * blockDim.x;
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const f32x4 *L4 = reinterpret_cast<const f32x4 *>(L);
  const f32x4 *R4 = reinterpret_cast<const f32x4 *>(R);
  f32x4 *Y4 = reinterpret_cast<f32x4 *>(Y);
  for (long long v = i; v < nvec; v += stride) {
    f32x4 a = L4[v], b = R4[v], y;
    y.x = apply_f<OP>(a.x, b.x);
    y.y = apply_f<OP>(a.y, b.y);
    y.z = apply_f<OP>(a.z, b.z);
    y.w = apply_f<OP>(a.w, b.w);
    Y4[v] = y;
  }
  const long long tail = (nvec << 2) + i;
  if (i < (total & 3)) Y[tail] = apply_f<OP>(L[tail], R[tail]);
}

// Broadcast path: the workgroup-tiled walk of plane_walk.h.  UNIT = 4 when the
// innermost axis can be moved in 16-byte pieces: an operand whose innermost
// stride is 1 is read with one 16-byte load, one whose stride is 0 with one
// scalar load.  A thread issues the loads of its four items before it uses any.
template <int OP, typename T, int UNIT>
__global__ __launch_bounds__(256) void binary_plane(BinaryParams p, wdh::PlaneWalk w) {
  const wdh::PlanePos q = wdh::plane_position(w);
  long long bl = 0, br = 0;
#pragma unroll
  for (int d = 0; d < MAXD - 2; d++) {
    if (d < w.nd - 2) {
      bl += (long long)q.oc[d] * p.sl[d];
      br += (long long)q.oc[d] * p.sr[d];
    }
  }
  const unsigned inner = w.shape[w.nd - 1], second = w.shape[w.nd - 2];
  const long long sl2 = p.sl[w.nd - 2], sr2 = p.sr[w.nd - 2];
  const long long sl1 = p.sl[w.nd - 1], sr1 = p.sr[w.nd - 1];
  const T *L = (const T *)p.L, *R = (const T *)p.R;
  T *Y = (T *)p.Y;
  const long long row0 = (long long)q.outer_linear * second;
  if (UNIT == 4) {
    f32x4 a[4], b[4];
    bool ok[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const unsigned x = q.x0 + k * q.dx, y = q.y0 + k * q.dy;
      ok[k] = x < inner && y < second;
      if (ok[k]) {
        const float *l = (const float *)L + bl + (long long)y * sl2 + (long long)x * 4 * sl1;
        const float *r = (const float *)R + br + (long long)y * sr2 + (long long)x * 4 * sr1;
        if (sl1) a[k] = *reinterpret_cast<const f32x4 *>(l);
        else { const float s = *l; a[k] = f32x4{s, s, s, s}; }
        if (sr1) b[k] = *reinterpret_cast<const f32x4 *>(r);
        else { const float s = *r; b[k] = f32x4{s, s, s, s}; }
      }
    }
#pragma unroll
    for (int k = 0; k < 4; k++) {
      if (ok[k]) {
        const unsigned x = q.x0 + k * q.dx, y = q.y0 + k * q.dy;
        f32x4 v;
        v.x = apply_f<OP>(a[k].x, b[k].x);
        v.y = apply_f<OP>(a[k].y, b[k].y);
        v.z = apply_f<OP>(a[k].z, b[k].z);
        v.w = apply_f<OP>(a[k].w, b[k].w);
        *reinterpret_cast<f32x4 *>((float *)Y + ((row0 + y) * inner + x) * 4) = v;
      }
    }
  } else {
    T a[4], b[4];
    bool ok[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const unsigned x = q.x0 + k * q.dx, y = q.y0 + k * q.dy;
      ok[k] = x < inner && y < second;
      if (ok[k]) {
        a[k] = L[bl + (long long)y * sl2 + (long long)x * sl1];
        b[k] = R[br + (long long)y * sr2 + (long long)x * sr1];
      }
    }
#pragma unroll
    for (int k = 0; k < 4; k++) {
      if (ok[k]) {
        const unsigned x = q.x0 + k * q.dx, y = q.y0 + k * q.dy;
        const long long o = (row0 + y) * inner + x;
        if (__is_same(T, float))
          ((float *)Y)[o] = apply_f<OP>((float)a[k], (float)b[k]);
        else
          ((int *)Y)[o] = apply_i<OP>((int)a[k], (int)b[k]);
      }
    }
  }
}

// The flat walk of plane_walk.h over the same views, for rows that fill the tiles above
// badly (a bias added to planes of 56x56 = 784 units): consecutive threads take
// consecutive units of the result whatever the row length.
template <int OP, typename T, int UNIT>
__global__ __launch_bounds__(256) void binary_flat(BinaryParams p, wdh::FlatWalk f, wdh::FastDiv fd_inner) {
  const wdh::FlatPos q = wdh::flat_position(f);
  long long bl = 0, br = 0;
#pragma unroll
  for (int d = 0; d < MAXD - 2; d++) {
    if (d < f.n_outer) {
      bl += (long long)q.oc[d] * p.sl[d];
      br += (long long)q.oc[d] * p.sr[d];
    }
  }
  const int nd = f.n_outer + 2;
  const long long sl2 = p.sl[nd - 2], sr2 = p.sr[nd - 2];
  const long long sl1 = p.sl[nd - 1] * UNIT, sr1 = p.sr[nd - 1] * UNIT;
  const T *L = (const T *)p.L + bl, *R = (const T *)p.R + br;
  T *Y = (T *)p.Y + (long long)q.outer_linear * f.plane * UNIT;
  typedef typename std::conditional<UNIT == 4, f32x4, T>::type V;
  for (unsigned u0 = q.begin + threadIdx.x; u0 < q.end; u0 += 1024) {
    V a[4], b[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const unsigned u = u0 + 256 * k;
      if (u < q.end) {
        const unsigned row = (unsigned)wdh::fdiv((int)u, fd_inner), col = u - row * f.inner;
        const T *l = L + (long long)row * sl2 + (long long)col * sl1;
        const T *r = R + (long long)row * sr2 + (long long)col * sr1;
        if constexpr (UNIT == 4) {
          if (sl1) a[k] = *reinterpret_cast<const f32x4 *>(l);
          else { const float s = *l; a[k] = f32x4{s, s, s, s}; }
          if (sr1) b[k] = *reinterpret_cast<const f32x4 *>(r);
          else { const float s = *r; b[k] = f32x4{s, s, s, s}; }
        } else {
          a[k] = *l;
          b[k] = *r;
        }
      }
    }
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const unsigned u = u0 + 256 * k;
      if (u < q.end) {
        if constexpr (UNIT == 4) {
          f32x4 v;
          v.x = apply_f<OP>(a[k].x, b[k].x);
          v.y = apply_f<OP>(a[k].y, b[k].y);
          v.z = apply_f<OP>(a[k].z, b[k].z);
          v.w = apply_f<OP>(a[k].w, b[k].w);
          *reinterpret_cast<f32x4 *>(Y + (long long)u * 4) = v;
        } else if constexpr (__is_same(T, float)) {
          Y[u] = apply_f<OP>(a[k], b[k]);
        } else {
          Y[u] = apply_i<OP>(a[k], b[k]);
        }
      }
    }
  }
}

// General path: one output element per thread per step, any strides.
template <int OP, typename T, typename IDX>
__global__ __launch_bounds__(256) void binary_general(BinaryParams p) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  const T *L = (const T *)p.L, *R = (const T *)p.R;
  T *Y = (T *)p.Y;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
       i < p.total; i += stride) {
    IDX rem = (IDX)i;
    long long ol = 0, orr = 0;
#pragma unroll
    for (int d = MAXD - 1; d >= 0; d--) {
      if (d < p.ndim) {
        const IDX q = rem / (IDX)p.shape[d];
        const long long c = (long long)(rem - q * (IDX)p.shape[d]);
        rem = q;
        ol += c * p.sl[d];
        orr += c * p.sr[d];
      }
    }
    if (sizeof(T) == 4 && __is_same(T, float))
      ((float *)Y)[i] = apply_f<OP>(((const float *)L)[ol], ((const float *)R)[orr]);
    else
      ((int *)Y)[i] = apply_i<OP>(((const int *)L)[ol], ((const int *)R)[orr]);
  }
}

unsigned grid_for(long long work_items, int per_block) {
  long long blocks = (work_items + per_block - 1) / per_block;
  long long cap = (long long)wdh::compute_units() * 16;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  return (unsigned)blocks;
}

// Shifts the strides of a rank-1 view by the leading axis the walk adds.
BinaryParams for_walk(const BinaryParams &p, const wdh::PlaneWalk &w) {
  if (w.nd == p.ndim) return p;
  BinaryParams s = p;
  for (int d = p.ndim; d > 0; d--) { s.sl[d] = p.sl[d - 1]; s.sr[d] = p.sr[d - 1]; }
  s.sl[0] = s.sr[0] = 0;
  return s;
}

template <int OP>
int launch_binary(const BinaryParams &p, int dtype, bool dense, bool vec) {
  hipStream_t st = wdh::stream();
  const bool small = p.total <= 0xffffffffLL;
  wdh::PlaneWalk w;
  wdh::FlatWalk fw;
  const bool vec4 = dtype == 0 && vec;
  const unsigned inner_units = vec4 ? p.shape[p.ndim - 1] / 4 : p.shape[p.ndim - 1];
  if (dtype == 0 && dense) {
    hipLaunchKernelGGL(binary_dense_f32<OP>, dim3(grid_for((p.total + 3) / 4, 256)),
                       dim3(256), 0, st, (const float *)p.L, (const float *)p.R,
                       (float *)p.Y, p.total);
  } else if (p.ndim >= 2 &&
             (!wdh::plan_plane_walk(&w, p.ndim, p.shape, inner_units) || wdh::plane_walk_fill(w) < 0.9) &&
             wdh::plan_flat_walk(&fw, p.ndim, p.shape, inner_units)) {
    const dim3 grid(fw.outer * fw.chunks);
    const wdh::FastDiv fd = wdh::make_fastdiv(fw.inner);
    if (vec4)
      hipLaunchKernelGGL((binary_flat<OP, float, 4>), grid, dim3(256), 0, st, p, fw, fd);
    else if (dtype == 0)
      hipLaunchKernelGGL((binary_flat<OP, float, 1>), grid, dim3(256), 0, st, p, fw, fd);
    else
      hipLaunchKernelGGL((binary_flat<OP, int, 1>), grid, dim3(256), 0, st, p, fw, fd);
  } else if (dtype == 0 && vec &&
             wdh::plan_plane_walk(&w, p.ndim, p.shape, p.shape[p.ndim - 1] / 4)) {
    hipLaunchKernelGGL((binary_plane<OP, float, 4>), wdh::plane_grid(w), dim3(256), 0, st,
                       for_walk(p, w), w);
  } else if (wdh::plan_plane_walk(&w, p.ndim, p.shape, p.shape[p.ndim - 1])) {
    if (dtype == 0)
      hipLaunchKernelGGL((binary_plane<OP, float, 1>), wdh::plane_grid(w), dim3(256), 0, st,
                         for_walk(p, w), w);
    else
      hipLaunchKernelGGL((binary_plane<OP, int, 1>), wdh::plane_grid(w), dim3(256), 0, st,
                         for_walk(p, w), w);
  } else if (dtype == 0) {
    const dim3 grid(grid_for(p.total, 256));
    if (small)
      hipLaunchKernelGGL((binary_general<OP, float, unsigned>), grid, dim3(256), 0, st, p);
    else
      hipLaunchKernelGGL((binary_general<OP, float, long long>), grid, dim3(256), 0, st, p);
  } else {
    const dim3 grid(grid_for(p.total, 256));
    if (small)
      hipLaunchKernelGGL((binary_general<OP, int, unsigned>), grid, dim3(256), 0, st, p);
    else
      hipLaunchKernelGGL((binary_general<OP, int, long long>), grid, dim3(256), 0, st, p);
  }
  WDH_LAUNCH_CHECK();
  return WDH_OK;
}

// ---- unary ---------------------------------------------------------------

__device__ __forceinline__ float relu_js(float v) {
  // Math.max(v, 0): NaN stays NaN (the comparison is false for it), -0 becomes +0.
  return v <= 0.0f ? 0.0f : v;
}

template <int OP>
__device__ __forceinline__ float unary_f(float v) {
  if (OP == WDH_UN_RELU) return relu_js(v);
  if (OP == WDH_UN_SIGMOID) return (float)((tanh((double)v / 2.0) + 1.0) / 2.0);
  if (OP == WDH_UN_SQRT) return (float)sqrt((double)v);
  if (OP == WDH_UN_EXP) return (float)exp((double)v);
  if (OP == WDH_UN_TANH) return (float)tanh((double)v);
  if (OP == WDH_UN_ABS) return fabsf(v);
  if (OP == WDH_UN_NEG) return -v;
  return (float)(1.0 / (double)v);
}

template <int OP>
__global__ __launch_bounds__(256) void unary_f32(const float *__restrict__ X,
                                                 float *__restrict__ Y,
                                                 long long total, bool vec) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (vec) {
    const long long nvec = total >> 2;
    const f32x4 *X4 = reinterpret_cast<const f32x4 *>(X);
    f32x4 *Y4 = reinterpret_cast<f32x4 *>(Y);
    for (long long v = i; v < nvec; v += stride) {
      f32x4 a = X4[v], y;
      y.x = unary_f<OP>(a.x);
      y.y = unary_f<OP>(a.y);
      y.z = unary_f<OP>(a.z);
      y.w = unary_f<OP>(a.w);
      Y4[v] = y;
    }
    const long long tail = (nvec << 2) + i;
    if (i < (total & 3)) Y[tail] = unary_f<OP>(X[tail]);
  } else {
    for (long long e = i; e < total; e += stride) Y[e] = unary_f<OP>(X[e]);
  }
}

__global__ __launch_bounds__(256) void unary_i32(int op, const int *__restrict__ X,
                                                 int *__restrict__ Y, long long total) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total;
       e += stride) {
    int v = X[e];
    int y;
    if (op == WDH_UN_RELU) y = v > 0 ? v : 0;
    else if (op == WDH_UN_ABS) y = js_to_int32(fabs((double)v));
    else y = js_to_int32(-(double)v);
    Y[e] = y;
  }
}

// Cast between the two data types the runner has: storing a float into an
// Int32Array applies ToInt32, storing an int into a Float32Array rounds to nearest.
__global__ __launch_bounds__(256) void cast_f32_i32(const float *__restrict__ X,
                                                    int *__restrict__ Y, long long total) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += stride)
    Y[e] = js_to_int32((double)X[e]);
}
__global__ __launch_bounds__(256) void cast_i32_f32(const int *__restrict__ X,
                                                    float *__restrict__ Y, long long total) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += stride)
    Y[e] = (float)X[e];
}

template <int OP>
int launch_unary(const float *X, float *Y, long long total) {
  bool vec = (((uintptr_t)X | (uintptr_t)Y) & 15) == 0;
  hipLaunchKernelGGL(unary_f32<OP>, dim3(grid_for((total + 3) / 4, 256)), dim3(256),
                     0, wdh::stream(), X, Y, total, vec);
  WDH_LAUNCH_CHECK();
  return WDH_OK;
}

}  // namespace

using wdh::fail;

extern "C" int wdh_binary(int op, int dtype, wdh_buf hL, wdh_buf hR, wdh_buf hY,
                          int ndim, const int32_t *out_shape,
                          const int64_t *strides_l, const int64_t *strides_r) {
  WDH_REQUIRE_INIT();
  WDH_REQUIRE_COMPUTE_LANE();
  if (op < WDH_BIN_ADD || op > WDH_BIN_POW)
    return fail(WDH_EINVAL, "wdh_binary: unknown op %d", op);
  if (dtype != 0 && dtype != 1)
    return fail(WDH_EINVAL, "wdh_binary: unknown dtype %d", dtype);
  if (ndim < 0 || ndim > MAXD)
    return fail(WDH_EINVAL, "wdh_binary: ndim %d outside 0..%d", ndim, MAXD);
  if (ndim > 0 && (!out_shape || !strides_l || !strides_r))
    return fail(WDH_EINVAL, "wdh_binary: NULL shape or strides");

  // Collapse: drop extent-1 axes, merge neighbours that are jointly contiguous
  // (or jointly broadcast) in both operands.
  BinaryParams p = {};
  long long total = 1, span_l = 1, span_r = 1;
  int nd = 0;
  for (int d = 0; d < ndim; d++) {
    if (out_shape[d] < 0 || strides_l[d] < 0 || strides_r[d] < 0)
      return fail(WDH_EINVAL, "wdh_binary: negative extent or stride");
    total *= out_shape[d];
    if (out_shape[d] == 1) continue;
    span_l += (long long)(out_shape[d] - 1) * strides_l[d];
    span_r += (long long)(out_shape[d] - 1) * strides_r[d];
    if (nd > 0 && p.sl[nd - 1] == strides_l[d] * out_shape[d] &&
        p.sr[nd - 1] == strides_r[d] * out_shape[d] &&
        (unsigned long long)p.shape[nd - 1] * out_shape[d] <= 0xffffffffULL) {
      p.shape[nd - 1] *= out_shape[d];
      p.sl[nd - 1] = strides_l[d];
      p.sr[nd - 1] = strides_r[d];
    } else {
      p.shape[nd] = out_shape[d];
      p.sl[nd] = strides_l[d];
      p.sr[nd] = strides_r[d];
      nd++;
    }
  }
  if (total == 0) return WDH_OK;
  if (nd == 0) {  // scalar result
    p.shape[0] = 1;
    p.sl[0] = p.sr[0] = 0;
    nd = 1;
  }
  p.ndim = nd;
  p.total = total;
  void *ptr;
  if (!wdh::operand(hL, (size_t)span_l * 4, "wdh_binary: L", &ptr)) return WDH_EINVAL;
  p.L = ptr;
  if (!wdh::operand(hR, (size_t)span_r * 4, "wdh_binary: R", &ptr)) return WDH_EINVAL;
  p.R = ptr;
  if (!wdh::operand(hY, (size_t)total * 4, "wdh_binary: Y", &ptr)) return WDH_EINVAL;
  p.Y = ptr;

  const bool aligned =
      (((uintptr_t)p.L | (uintptr_t)p.R | (uintptr_t)p.Y) & 15) == 0;
  const bool dense = aligned && nd == 1 && p.sl[0] == 1 && p.sr[0] == 1;
  // 16-byte accesses: the output always; an operand that steps by 1 along the
  // innermost axis needs an aligned base and outer strides that are multiples
  // of 4; one that does not step there (stride 0) is read with scalar loads
  auto vec_ok = [&](const void *base, const long long *st) {
    if (st[nd - 1] == 0) return true;
    if (st[nd - 1] != 1 || ((uintptr_t)base & 15)) return false;
    for (int d = 0; d + 1 < nd; d++)
      if (st[d] % 4) return false;
    return true;
  };
  const bool vec = ((uintptr_t)p.Y & 15) == 0 && p.shape[nd - 1] % 4 == 0 &&
                   vec_ok(p.L, p.sl) && vec_ok(p.R, p.sr);
  switch (op) {
    case WDH_BIN_ADD: return launch_binary<WDH_BIN_ADD>(p, dtype, dense, vec);
    case WDH_BIN_SUB: return launch_binary<WDH_BIN_SUB>(p, dtype, dense, vec);
    case WDH_BIN_MUL: return launch_binary<WDH_BIN_MUL>(p, dtype, dense, vec);
    case WDH_BIN_DIV: return launch_binary<WDH_BIN_DIV>(p, dtype, dense, vec);
    default: return launch_binary<WDH_BIN_POW>(p, dtype, dense, vec);
  }
}

extern "C" int wdh_unary(int op, int dtype, wdh_buf hX, wdh_buf hY, size_t length) {
  WDH_REQUIRE_INIT();
  WDH_REQUIRE_COMPUTE_LANE();
  if (op < WDH_UN_RELU || op > WDH_UN_RECIPROCAL)
    return fail(WDH_EINVAL, "wdh_unary: unknown op %d", op);
  if (dtype != 0 && dtype != 1)
    return fail(WDH_EINVAL, "wdh_unary: unknown dtype %d", dtype);
  if (dtype == 1 && op != WDH_UN_RELU && op != WDH_UN_ABS && op != WDH_UN_NEG)
    return fail(WDH_EINVAL, "wdh_unary: op %d does not accept int32", op);
  if (length == 0) return WDH_OK;
  void *px, *py;
  if (!wdh::operand(hX, length * 4, "wdh_unary: X", &px)) return WDH_EINVAL;
  if (!wdh::operand(hY, length * 4, "wdh_unary: Y", &py)) return WDH_EINVAL;
  const long long total = (long long)length;
  if (dtype == 1) {
    hipLaunchKernelGGL(unary_i32, dim3(grid_for(total, 256)), dim3(256), 0,
                       wdh::stream(), op, (const int *)px, (int *)py, total);
    WDH_LAUNCH_CHECK();
    return WDH_OK;
  }
  const float *X = (const float *)px;
  float *Y = (float *)py;
  switch (op) {
    case WDH_UN_RELU: return launch_unary<WDH_UN_RELU>(X, Y, total);
    case WDH_UN_SIGMOID: return launch_unary<WDH_UN_SIGMOID>(X, Y, total);
    case WDH_UN_SQRT: return launch_unary<WDH_UN_SQRT>(X, Y, total);
    case WDH_UN_EXP: return launch_unary<WDH_UN_EXP>(X, Y, total);
    case WDH_UN_TANH: return launch_unary<WDH_UN_TANH>(X, Y, total);
    case WDH_UN_ABS: return launch_unary<WDH_UN_ABS>(X, Y, total);
    case WDH_UN_NEG: return launch_unary<WDH_UN_NEG>(X, Y, total);
    default: return launch_unary<WDH_UN_RECIPROCAL>(X, Y, total);
  }
}

extern "C" int wdh_cast(int from_dtype, int to_dtype, wdh_buf hX, wdh_buf hY, size_t length) {
  WDH_REQUIRE_INIT();
  WDH_REQUIRE_COMPUTE_LANE();
  if ((from_dtype != 0 && from_dtype != 1) || (to_dtype != 0 && to_dtype != 1))
    return fail(WDH_EINVAL, "wdh_cast: dtype %d -> %d (0 = float32, 1 = int32)", from_dtype,
                to_dtype);
  if (length == 0) return WDH_OK;
  void *px, *py;
  if (!wdh::operand(hX, length * 4, "wdh_cast: X", &px)) return WDH_EINVAL;
  if (!wdh::operand(hY, length * 4, "wdh_cast: Y", &py)) return WDH_EINVAL;
  const long long total = (long long)length;
  if (from_dtype == to_dtype) {
    WDH_HIP_CHECK(hipMemcpyAsync(py, px, length * 4, hipMemcpyDeviceToDevice, wdh::stream()));
    return WDH_OK;
  }
  if (from_dtype == 0)
    hipLaunchKernelGGL(cast_f32_i32, dim3(grid_for(total, 256)), dim3(256), 0, wdh::stream(),
                       (const float *)px, (int *)py, total);
  else
    hipLaunchKernelGGL(cast_i32_f32, dim3(grid_for(total, 256)), dim3(256), 0, wdh::stream(),
                       (const int *)px, (float *)py, total);
  WDH_LAUNCH_CHECK();
  return WDH_OK;
}
