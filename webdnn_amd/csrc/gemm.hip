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
// Tiling: one 256-thread workgroup (4 wavefronts of 64) owns a 128x128 tile of
// the result; each wavefront owns 64x64 = 2x2 v_mfma_f32_32x32x2_f32 tiles
// (64 accumulator registers per lane).  K advances 16 at a time through two
// LDS buffers; the next K slab is fetched from global memory into registers
// while the current one feeds the matrix cores, so there is one barrier per
// slab.
//
// Operand layouts in LDS depend on which index is contiguous in global memory:
//   "KC" (k contiguous, e.g. A of a non-transposed Gemm, conv weights):
//        tile[row][k], row stride 20 floats; a lane reads 4 consecutive k with
//        one ds_read_b128.  The 16 k of a slab are consumed in the order
//        k = 8*(s/4) + 4*half + s%4 for MFMA step s and lane half (lane/32);
//        both operands use the same order, so the sum is over the same set.
//   "MC" (row/column index contiguous, e.g. B of a non-transposed Gemm, the
//        im2col view of a conv input): tile[k][col], row stride 136 floats;
//        a lane reads one float per step, lanes 0..31 hit consecutive banks.
#include <string.h>

#include <map>
#include <vector>

#include "common.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int BM = 128;
constexpr int BN = 128;
constexpr int BK = 16;
constexpr int NTHREADS = 256;
constexpr int LDK = BK + 4;    // KC tile row stride (floats)
constexpr int LDM = 128 + 8;   // MC tile row stride (floats)
constexpr int TILE_FLOATS = (BM * LDK > BK * LDM) ? BM * LDK : BK * LDM;

enum BMode { B_KC = 0, B_MC = 1, B_IM2COL = 2 };

struct ConvGeom {
  int c_in_g;        // input channels per group
  int h, w;          // input spatial size
  int oh, ow;        // output spatial size
  int kh, kw;
  int pt, pl;        // top / left padding
  int sh, sw;        // strides
  int c_total;       // input channels (all groups)
  int cout_total;    // output channels (all groups)
  int cout_g;        // output channels per group
  int64_t npix;      // batch * oh * ow
  const int2 *ktab;  // per k: {offset ci*h*w + ky*dh*w + kx*dw, (ky*dh)<<16 | kx*dw}
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
  float alpha, beta;
  int epilogue;
  int tiles_m, tiles_n;
  ConvGeom cv;
};

__device__ __forceinline__ float relu_js(float v) {
  // Math.max(v, 0): NaN stays NaN, -0 becomes +0.
  return v > 0.0f ? v : (v != v ? v : 0.0f);
}

// Maps the linear workgroup id to a tile so that (1) each XCD (ids are dealt
// round-robin over the 8 XCDs) works on a contiguous range of tiles and
// (2) within that range tiles are visited in groups of 8 tile-rows, which
// keeps the A and B panels a group touches resident in that XCD's L2.
__device__ __forceinline__ void tile_of_block(int pid, int tiles_m, int tiles_n,
                                              int *tm, int *tn) {
  const int total = tiles_m * tiles_n;
  constexpr int XCDS = 8;
  int xcd = pid % XCDS, local = pid / XCDS;
  int base = total / XCDS, rem = total % XCDS;
  int start = xcd * base + (xcd < rem ? xcd : rem);
  int id = start + local;
  constexpr int GROUP = 8;
  int per_group = GROUP * tiles_n;
  int group = id / per_group;
  int first_m = group * GROUP;
  int rows = tiles_m - first_m < GROUP ? tiles_m - first_m : GROUP;
  int in_group = id % per_group;
  *tm = first_m + in_group % rows;
  *tn = in_group / rows;
}

// ---- global -> register fetch of one K slab ------------------------------
// KC operand: thread t fetches rows (t>>2) and (t>>2)+64, k offsets 4*(t&3)..+3.
template <bool VEC>
__device__ __forceinline__ void fetch_kc(const float *__restrict__ base,
                                         long long ld_row, int row0, int nrows,
                                         int k0, int kdim, int tid,
                                         f32x4 (&reg)[2]) {
  const int kq = (tid & 3) * 4;
  const int k = k0 + kq;
#pragma unroll
  for (int i = 0; i < 2; i++) {
    int r = row0 + (tid >> 2) + i * 64;
    r = r < nrows ? r : nrows - 1;  // rows past the edge are never stored
    const float *p = base + (long long)r * ld_row + k;
    if (VEC && k + 3 < kdim) {
      reg[i] = *reinterpret_cast<const f32x4 *>(p);
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

// MC operand: thread t fetches k rows (t>>5) and (t>>5)+8, columns 4*(t&31)..+3.
template <bool VEC>
__device__ __forceinline__ void fetch_mc(const float *__restrict__ base,
                                         long long ld_k, int col0, int ncols,
                                         int k0, int kdim, int tid,
                                         f32x4 (&reg)[2]) {
  const int c = col0 + (tid & 31) * 4;
#pragma unroll
  for (int i = 0; i < 2; i++) {
    int k = k0 + (tid >> 5) + i * 8;
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

// im2col view of X: thread t owns output pixel (t&127) of the tile and k rows
// (t>>7) + 2*i, i = 0..7.  The k row index is uniform across a wavefront.
struct PixelCtx {
  const float *xbase;  // X + (n*c_total + g*c_in_g)*h*w, or null when past the edge
  int iy0, ix0;
};

__device__ __forceinline__ void fetch_im2col(const ConvGeom &cv,
                                             const PixelCtx &px, int k0,
                                             int kdim, int tid,
                                             f32x4 (&reg)[2]) {
  const int khalf = __builtin_amdgcn_readfirstlane(tid >> 7);
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; i++) {
    int k = k0 + khalf + 2 * i;
    float val = 0.0f;
    if (k < kdim) {
      int2 e = cv.ktab[k];
      int iy = px.iy0 + (e.y >> 16);
      int ix = px.ix0 + (e.y & 0xffff);
      if (px.xbase && (unsigned)iy < (unsigned)cv.h &&
          (unsigned)ix < (unsigned)cv.w)
        val = px.xbase[e.x + iy * cv.w + ix];
    }
    v[i] = val;
  }
  reg[0] = f32x4{v[0], v[1], v[2], v[3]};
  reg[1] = f32x4{v[4], v[5], v[6], v[7]};
}

// ---- register -> LDS -------------------------------------------------------
__device__ __forceinline__ void stash_kc(float *tile, int tid,
                                         const f32x4 (&reg)[2]) {
#pragma unroll
  for (int i = 0; i < 2; i++)
    *reinterpret_cast<f32x4 *>(tile + ((tid >> 2) + i * 64) * LDK +
                               (tid & 3) * 4) = reg[i];
}
__device__ __forceinline__ void stash_mc(float *tile, int tid,
                                         const f32x4 (&reg)[2]) {
#pragma unroll
  for (int i = 0; i < 2; i++)
    *reinterpret_cast<f32x4 *>(tile + ((tid >> 5) + i * 8) * LDM +
                               (tid & 31) * 4) = reg[i];
}
__device__ __forceinline__ void stash_im2col(float *tile, int tid,
                                             const f32x4 (&reg)[2]) {
  const int khalf = tid >> 7, pix = tid & 127;
#pragma unroll
  for (int i = 0; i < 8; i++)
    tile[(khalf + 2 * i) * LDM + pix] = reg[i >> 2][i & 3];
}

// ---- the kernel -------------------------------------------------------------
template <bool A_KC, int BMODE, bool VEC>
__global__ __launch_bounds__(NTHREADS) void contraction_kernel(Params p) {
  __shared__ __attribute__((aligned(16))) float lds_a[2][TILE_FLOATS];
  __shared__ __attribute__((aligned(16))) float lds_b[2][TILE_FLOATS];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;  // 2x2 wavefronts
  const int li = lane & 31, half = lane >> 5;

  int tm, tn;
  tile_of_block(blockIdx.x, p.tiles_m, p.tiles_n, &tm, &tn);
  const int row0 = tm * BM, col0 = tn * BN;
  const int bz = blockIdx.y;  // batch (gemm) or group (conv)

  const float *A = p.A + (long long)bz * p.sAb;
  const float *B = p.B + (long long)bz * p.sBb;
  const long long lda = A_KC ? p.sA0 : p.sA1;
  const long long ldb = (BMODE == B_KC) ? p.sB1 : p.sB0;

  PixelCtx px = {nullptr, 0, 0};
  if (BMODE == B_IM2COL) {
    long long P = (long long)col0 + (tid & 127);
    if (P < p.cv.npix) {
      int ohw = p.cv.oh * p.cv.ow;
      int img = (int)(P / ohw);
      int q = (int)(P - (long long)img * ohw);
      int oy = q / p.cv.ow, ox = q - oy * p.cv.ow;
      px.xbase = p.B + ((long long)img * p.cv.c_total + (long long)bz * p.cv.c_in_g) *
                           p.cv.h * p.cv.w;
      px.iy0 = oy * p.cv.sh - p.cv.pt;
      px.ix0 = ox * p.cv.sw - p.cv.pl;
    }
  }

  f32x16 acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; a++)
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[a][b][r] = 0.0f;

  f32x4 ra[2], rb[2];
  auto fetch = [&](int k0) {
    if (A_KC)
      fetch_kc<VEC>(A, lda, row0, p.m, k0, p.k, tid, ra);
    else
      fetch_mc<VEC>(A, lda, row0, p.m, k0, p.k, tid, ra);
    if (BMODE == B_KC)
      fetch_kc<VEC>(B, ldb, col0, p.n, k0, p.k, tid, rb);
    else if (BMODE == B_MC)
      fetch_mc<VEC>(B, ldb, col0, p.n, k0, p.k, tid, rb);
    else
      fetch_im2col(p.cv, px, k0, p.k, tid, rb);
  };
  auto stash = [&](int buf) {
    if (A_KC)
      stash_kc(lds_a[buf], tid, ra);
    else
      stash_mc(lds_a[buf], tid, ra);
    if (BMODE == B_KC)
      stash_kc(lds_b[buf], tid, rb);
    else if (BMODE == B_MC)
      stash_mc(lds_b[buf], tid, rb);
    else
      stash_im2col(lds_b[buf], tid, rb);
  };

  const int nslabs = (p.k + BK - 1) / BK;
  fetch(0);
  stash(0);
  __syncthreads();

  for (int s = 0; s < nslabs; s++) {
    const int cur = s & 1;
    if (s + 1 < nslabs) fetch((s + 1) * BK);

    const float *ta = lds_a[cur];
    const float *tb = lds_b[cur];
    f32x4 av[2][2], bv[2][2];
    if (A_KC) {
#pragma unroll
      for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int j = 0; j < 2; j++)
          av[mt][j] = *reinterpret_cast<const f32x4 *>(
              ta + (wm * 64 + mt * 32 + li) * LDK + 8 * j + 4 * half);
    }
    if (BMODE == B_KC) {
#pragma unroll
      for (int nt = 0; nt < 2; nt++)
#pragma unroll
        for (int j = 0; j < 2; j++)
          bv[nt][j] = *reinterpret_cast<const f32x4 *>(
              tb + (wn * 64 + nt * 32 + li) * LDK + 8 * j + 4 * half);
    }
#pragma unroll
    for (int st = 0; st < 8; st++) {
      const int kk = 8 * (st >> 2) + 4 * half + (st & 3);
      float a_el[2], b_el[2];
#pragma unroll
      for (int mt = 0; mt < 2; mt++)
        a_el[mt] = A_KC ? av[mt][st >> 2][st & 3]
                        : ta[kk * LDM + wm * 64 + mt * 32 + li];
#pragma unroll
      for (int nt = 0; nt < 2; nt++)
        b_el[nt] = (BMODE == B_KC) ? bv[nt][st >> 2][st & 3]
                                   : tb[kk * LDM + wn * 64 + nt * 32 + li];
#pragma unroll
      for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int nt = 0; nt < 2; nt++)
          acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(
              a_el[mt], b_el[nt], acc[mt][nt], 0, 0, 0);
    }

    if (s + 1 < nslabs) stash(cur ^ 1);
    __syncthreads();
  }

  // ---- epilogue: lane holds column (li) of each 32x32 tile, rows
  // 8*(r/4) + 4*half + r%4 for accumulator register r.
#pragma unroll
  for (int nt = 0; nt < 2; nt++) {
    const int col = col0 + wn * 64 + nt * 32 + li;
    if (col >= p.n) continue;
    long long ybase;     // offset of (row 0, this column) in Y
    long long ystride;   // distance between consecutive rows in Y
    if (BMODE == B_IM2COL) {
      int ohw = p.cv.oh * p.cv.ow;
      int img = col / ohw;
      int q = col - img * ohw;
      ybase = ((long long)img * p.cv.cout_total + (long long)bz * p.cv.cout_g) * ohw + q;
      ystride = ohw;
    } else {
      ybase = (long long)bz * p.m * p.n + col;
      ystride = p.n;
    }
#pragma unroll
    for (int mt = 0; mt < 2; mt++) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int row = row0 + wm * 64 + mt * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
        if (row >= p.m) continue;
        float y = p.alpha * acc[mt][nt][r];
        if (p.C) {
          float c = (BMODE == B_IM2COL)
                        ? p.C[bz * p.cv.cout_g + row]
                        : p.C[(long long)row * p.sC0 + (long long)col * p.sC1];
          y = __builtin_fmaf(c, p.beta, y);
        }
        const long long off = ybase + (long long)row * ystride;
        if (p.R) y = y + p.R[off];
        if (p.epilogue == WDH_EPI_RELU) y = relu_js(y);
        p.Y[off] = y;
      }
    }
  }
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
  long long off = (long long)bz * total + idx;
  if (p.R) y = y + p.R[off];
  if (p.epilogue == WDH_EPI_RELU) y = relu_js(y);
  p.Y[off] = y;
}

template <bool A_KC, int BMODE>
int launch(const Params &p, int nz, bool vec) {
  dim3 grid((unsigned)(p.tiles_m * p.tiles_n), (unsigned)nz);
  if (vec)
    hipLaunchKernelGGL((contraction_kernel<A_KC, BMODE, true>), grid,
                       dim3(NTHREADS), 0, wdh::stream(), p);
  else
    hipLaunchKernelGGL((contraction_kernel<A_KC, BMODE, false>), grid,
                       dim3(NTHREADS), 0, wdh::stream(), p);
  WDH_LAUNCH_CHECK();
  return WDH_OK;
}

bool aligned16(const void *ptr) { return ((uintptr_t)ptr & 15) == 0; }

// Largest element offset the strided view touches, for bounds checking.
long long span(long long nb, long long sb, long long n0, long long s0,
               long long n1, long long s1) {
  return (nb - 1) * sb + (n0 - 1) * s0 + (n1 - 1) * s1 + 1;
}

}  // namespace

using wdh::fail;

extern "C" int wdh_gemm(wdh_buf hA, wdh_buf hB, wdh_buf hC, wdh_buf hY,
                        int batch, int m, int n, int k, int64_t sAb,
                        int64_t sA0, int64_t sA1, int64_t sBb, int64_t sB0,
                        int64_t sB1, int64_t sC0, int64_t sC1, float alpha,
                        float beta, int epilogue, wdh_buf hR) {
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
    if (!wdh::operand(hR, (size_t)out_elems * 4, "wdh_gemm: R", &ptr)) return WDH_EINVAL;
    p.R = (const float *)ptr;
  }
  if (!wdh::operand(hY, (size_t)out_elems * 4, "wdh_gemm: Y", &ptr)) return WDH_EINVAL;
  p.Y = (float *)ptr;
  p.m = m; p.n = n; p.k = k;
  p.sAb = sAb; p.sA0 = sA0; p.sA1 = sA1;
  p.sBb = sBb; p.sB0 = sB0; p.sB1 = sB1;
  p.sC0 = sC0; p.sC1 = sC1;
  p.alpha = alpha; p.beta = beta; p.epilogue = epilogue;
  p.tiles_m = (m + BM - 1) / BM;
  p.tiles_n = (n + BN - 1) / BN;

  // Which index of each operand is contiguous?  An extent of 1 makes the
  // stride along it irrelevant.
  const bool a_kc = (sA1 == 1 || k == 1), a_mc = (sA0 == 1 || m == 1);
  const bool b_kc = (sB0 == 1 || k == 1), b_mc = (sB1 == 1 || n == 1);
  if (!(a_kc || a_mc) || !(b_kc || b_mc) ||
      (long long)p.tiles_m * p.tiles_n > 0x7fffffffLL) {
    dim3 grid((unsigned)(((long long)m * n + 255) / 256), (unsigned)batch);
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
  if (useA_kc && useB_kc) return launch<true, B_KC>(p, batch, vec);
  if (useA_kc && !useB_kc) return launch<true, B_MC>(p, batch, vec);
  if (!useA_kc && useB_kc) return launch<false, B_KC>(p, batch, vec);
  return launch<false, B_MC>(p, batch, vec);
}

// ---- conv ----------------------------------------------------------------

namespace {

// One lookup table per conv geometry, built on the host once and kept on the
// device for the life of the library: entry k = (ci, ky, kx) holds the offset
// of that tap relative to the (iy0, ix0) corner of the receptive field and
// the tap's (dy, dx).
struct KtabKey {
  int c_in_g, kh, kw, dh, dw, h, w;
  bool operator<(const KtabKey &o) const {
    return memcmp(this, &o, sizeof(*this)) < 0;
  }
};

std::map<KtabKey, int2 *> g_ktabs;

}  // namespace

namespace wdh {
void release_conv_tables() {
  for (auto &kv : g_ktabs) (void)hipFree(kv.second);
  g_ktabs.clear();
}
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

  KtabKey key;
  memset(&key, 0, sizeof(key));
  key.c_in_g = c_in_g; key.kh = kh; key.kw = kw; key.dh = dh; key.dw = dw;
  key.h = h; key.w = w;
  auto it = g_ktabs.find(key);
  if (it == g_ktabs.end()) {
    std::vector<int2> tab((size_t)kdim);
    size_t idx = 0;
    for (int ci = 0; ci < c_in_g; ci++)
      for (int ky = 0; ky < kh; ky++)
        for (int kx = 0; kx < kw; kx++) {
          tab[idx].x = ci * h * w;
          tab[idx].y = ((ky * dh) << 16) | (kx * dw);
          idx++;
        }
    int2 *dev = nullptr;
    if (hipMalloc(&dev, tab.size() * sizeof(int2)) != hipSuccess) {
      (void)hipGetLastError();
      return fail(WDH_ENOMEM, "wdh_conv2d: tap table allocation failed");
    }
    // synchronous copy: the host vector dies at the end of this scope
    WDH_HIP_CHECK(hipMemcpy(dev, tab.data(), tab.size() * sizeof(int2),
                            hipMemcpyHostToDevice));
    it = g_ktabs.emplace(key, dev).first;
  }

  p.m = cout_g; p.n = (int)npix; p.k = (int)kdim;
  p.sAb = (long long)cout_g * kdim; p.sA0 = kdim; p.sA1 = 1;
  p.sBb = 0; p.sB0 = 0; p.sB1 = 0;
  p.alpha = 1.0f; p.beta = 1.0f; p.epilogue = epilogue;
  p.tiles_m = (p.m + BM - 1) / BM;
  p.tiles_n = (p.n + BN - 1) / BN;
  p.cv.c_in_g = c_in_g; p.cv.h = h; p.cv.w = w; p.cv.oh = oh; p.cv.ow = ow;
  p.cv.kh = kh; p.cv.kw = kw; p.cv.pt = pt; p.cv.pl = pl; p.cv.sh = sh; p.cv.sw = sw;
  p.cv.c_total = c; p.cv.cout_total = cout; p.cv.cout_g = cout_g;
  p.cv.npix = npix; p.cv.ktab = it->second;
  const bool vec = aligned16(p.A) && kdim % 4 == 0;
  return launch<true, B_IM2COL>(p, group, vec);
}
