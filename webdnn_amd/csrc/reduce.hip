// Row-reduction kernels: Softmax, LayerNormalization, ReduceMean /
// GlobalAveragePool.  All view the input as [outer, len] with len contiguous.
//
// Reference semantics:
//   Softmax           : src/descriptor_runner/operators/cpu/operators/standard/softmax.ts:34-57
//   ReduceMean        : src/descriptor_runner/operators/cpu/operators/standard/reduce.ts:369-405
//   GlobalAveragePool : src/descriptor_runner/operators/cpu/operators/standard/globalaveragepool.ts:12-41,
//                       src/descriptor_runner/operators/cpu/rawcomputation/averagepool.ts:1-46
// LayerNormalization has no reference operator; it follows ONNX opset 17 with
// the rounding points of the decomposed ReduceMean/Sub/Mul/ReduceMean/Add/
// Sqrt/Div/Mul/Add subgraph, except that the Div is a multiplication by the
// row's reciprocal (within an ulp of the quotient).
//
// One wavefront owns one row: lanes read consecutive floats (256-byte
// coalesced requests), keep the row in registers when it fits (len <= 64*NV),
// and reduce across lanes (single-precision values through DPP operands, double-precision
// sums through lane shuffles); no LDS tile, no barriers.  Rows longer than
// the register budget are re-read from cache in further passes.
#include <math.h>

#include "common.h"
#include "rowmath.h"

namespace {

using namespace wdh::rowmath;

constexpr int WAVES_PER_BLOCK = 4;

__device__ __forceinline__ double wave_sum_d(double v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// Register-resident rows.  VW = 4: rows are 16-byte aligned and a multiple of 4
// long, and lane l holds elements 4l..4l+3 of every 256-element segment (one
// 16-byte access each); VW = 2: the same with 8-byte pieces of every 128-element segment
// (rows of an even length, 850 say, start on 8-byte boundaries); VW = 1: lane l holds
// elements l, l+64, ...
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

template <int VW>
__device__ __forceinline__ int elem_index(int lane, int i) {
  return VW == 4 ? lane * 4 + 256 * (i >> 2) + (i & 3) : (VW == 2 ? lane * 2 + 128 * (i >> 1) + (i & 1) : lane + 64 * i);
}

template <int NV, int VW>
__device__ __forceinline__ void load_row(const float *x, int len, int lane, float fill,
                                         float (&v)[NV]) {
  if constexpr (VW == 2) {
#pragma unroll
    for (int i = 0; i < NV; i += 2) {
      const int idx = lane * 2 + 64 * i;
      f32x2 t = {fill, fill};
      if (idx < len) t = *reinterpret_cast<const f32x2 *>(x + idx);
      v[i] = t.x; v[i + 1] = t.y;
    }
  } else if constexpr (VW == 4) {
#pragma unroll
    for (int i = 0; i < NV; i += 4) {
      const int idx = lane * 4 + 64 * i;
      f32x4 t = {fill, fill, fill, fill};
      if (idx < len) t = *reinterpret_cast<const f32x4 *>(x + idx);
      v[i] = t.x; v[i + 1] = t.y; v[i + 2] = t.z; v[i + 3] = t.w;
    }
  } else {
#pragma unroll
    for (int i = 0; i < NV; i++) {
      const int idx = lane + 64 * i;
      v[i] = idx < len ? x[idx] : fill;
    }
  }
}

template <int NV, int VW>
__device__ __forceinline__ void store_row(float *y, int len, int lane, const float (&v)[NV]) {
  if constexpr (VW == 2) {
#pragma unroll
    for (int i = 0; i < NV; i += 2) {
      const int idx = lane * 2 + 64 * i;
      if (idx < len) *reinterpret_cast<f32x2 *>(y + idx) = f32x2{v[i], v[i + 1]};
    }
  } else if constexpr (VW == 4) {
#pragma unroll
    for (int i = 0; i < NV; i += 4) {
      const int idx = lane * 4 + 64 * i;
      if (idx < len) *reinterpret_cast<f32x4 *>(y + idx) = f32x4{v[i], v[i + 1], v[i + 2], v[i + 3]};
    }
  } else {
#pragma unroll
    for (int i = 0; i < NV; i++) {
      const int idx = lane + 64 * i;
      if (idx < len) y[idx] = v[i];
    }
  }
}

// ---- softmax ---------------------------------------------------------------
template <int NV, int VW>
__global__ __launch_bounds__(64 * WAVES_PER_BLOCK) void softmax_rows_reg(
    const float *__restrict__ X, float *__restrict__ Y, long long outer, int len) {
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * WAVES_PER_BLOCK + (threadIdx.x >> 6);
  if (row >= outer) return;
  float v[NV];
  load_row<NV, VW>(X + row * len, len, lane, -INFINITY, v);
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < NV; i++) mx = fmaxf(mx, v[i]);  // fmaxf skips NaN, like `if (v > max)`
  mx = wave_max(mx);
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    // (cells past the row's end hold -inf: e^(-inf - max) is 0 for any finite or +inf max, and a
    // row whose max is -inf sums to NaN with or without them)
    const float e = exp_f32(v[i] - mx);
    v[i] = e;
    sum += e;
  }
  sum = wave_sum(sum);
  // one division per row; e * (1/sum) is within an ulp of e / sum
  const float inv = 1.0f / sum;
#pragma unroll
  for (int i = 0; i < NV; i++) v[i] = v[i] * inv;
  store_row<NV, VW>(Y + row * len, len, lane, v);
}

__global__ __launch_bounds__(64 * WAVES_PER_BLOCK) void softmax_rows_stream(
    const float *__restrict__ X, float *__restrict__ Y, long long outer, int len) {
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * WAVES_PER_BLOCK + (threadIdx.x >> 6);
  if (row >= outer) return;
  const float *x = X + row * len;
  float *y = Y + row * len;
  float mx = -INFINITY;
  for (int idx = lane; idx < len; idx += 64) mx = fmaxf(mx, x[idx]);
  mx = wave_max(mx);
  float sum = 0.0f;
  for (int idx = lane; idx < len; idx += 64) {
    float e = exp_f32(x[idx] - mx);
    y[idx] = e;
    sum += e;
  }
  sum = wave_sum(sum);
  for (int idx = lane; idx < len; idx += 64) y[idx] = y[idx] / sum;
}

// ---- layer normalisation -----------------------------------------------------
template <int NV, bool VEC>
__global__ __launch_bounds__(64 * WAVES_PER_BLOCK) void layernorm_rows_reg(
    const float *__restrict__ X, const float *__restrict__ G,
    const float *__restrict__ Bt, float *__restrict__ Y, long long outer, int len,
    float eps, const float *__restrict__ P, float *__restrict__ Y2) {
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * WAVES_PER_BLOCK + (threadIdx.x >> 6);
  if (row >= outer) return;
  float v[NV], g[NV], bt[NV];
  load_row<NV, VEC ? 4 : 1>(X + row * len, len, lane, 0.0f, v);
  if (G) load_row<NV, VEC ? 4 : 1>(G, len, lane, 0.0f, g);
  if (Bt) load_row<NV, VEC ? 4 : 1>(Bt, len, lane, 0.0f, bt);
  double s = 0.0;
#pragma unroll
  for (int i = 0; i < NV; i++) s += (double)v[i];
  const float mean = (float)(wave_sum_d(s) / (double)len);
  double q = 0.0;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const float d = v[i] - mean;
    v[i] = d;
    const float sq = d * d;
    q += elem_index<VEC ? 4 : 1>(lane, i) < len ? (double)sq : 0.0;
  }
  const float var = (float)(wave_sum_d(q) / (double)len);
  const float inv = 1.0f / (float)sqrt((double)(var + eps));
#pragma unroll
  for (int i = 0; i < NV; i++) {
    float t = v[i] * inv;
    if (G) t = t * g[i];
    if (Bt) t = t + bt[i];
    v[i] = t;
  }
  store_row<NV, VEC ? 4 : 1>(Y + row * len, len, lane, v);
  if (P) {  // second output: the normalised row plus a row of P (the Add that follows in the graph)
    float pv[NV];
    load_row<NV, VEC ? 4 : 1>(P + row * len, len, lane, 0.0f, pv);
#pragma unroll
    for (int i = 0; i < NV; i++) v[i] = v[i] + pv[i];
    store_row<NV, VEC ? 4 : 1>(Y2 + row * len, len, lane, v);
  }
}

// Short rows (len <= 256, 16-byte aligned): a wavefront owns 64/SUB rows, SUB lanes each.
// Lane s of a row holds elements 4s .. 4s+3 of every segment of 4*SUB elements, so the
// sums cross log2(SUB) lane distances instead of six and the per-row divisions and the
// square root are paid once per 64/SUB rows.  Same rounding points as layernorm_rows_reg.
template <int SUB>
__device__ __forceinline__ double sub_sum_d(double v) {
#pragma unroll
  for (int off = SUB / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
// FULL: the rows are exactly 256 long, so no piece and no element needs a range test.
template <int SUB, bool FULL>
__global__ __launch_bounds__(64 * WAVES_PER_BLOCK) void layernorm_rows_part(
    const float *__restrict__ X, const float *__restrict__ G,
    const float *__restrict__ Bt, float *__restrict__ Y, long long outer, int len,
    float eps, const float *__restrict__ P, float *__restrict__ Y2) {
  constexpr int NJ = 256 / (4 * SUB);  // 16-byte pieces per lane
  constexpr int SEG = 4 * SUB;
  const int lane = threadIdx.x & 63, sub = lane & (SUB - 1);
  long long row = ((long long)blockIdx.x * WAVES_PER_BLOCK + (threadIdx.x >> 6)) * (64 / SUB) + (lane / SUB);
  const bool live = row < outer;
  if (!live) row = outer - 1;  // idle lanes repeat the last row and store nothing
  const float *x = X + row * len;
  f32x4 v[NJ];
#pragma unroll
  for (int j = 0; j < NJ; j++) {
    const int idx = 4 * sub + SEG * j;
    v[j] = FULL || idx < len ? *reinterpret_cast<const f32x4 *>(x + idx) : f32x4{0.f, 0.f, 0.f, 0.f};
  }
  double s = 0.0;
#pragma unroll
  for (int j = 0; j < NJ; j++)
#pragma unroll
    for (int e = 0; e < 4; e++) s += (double)v[j][e];
  const float mean = (float)(sub_sum_d<SUB>(s) / (double)len);
  double q = 0.0;
#pragma unroll
  for (int j = 0; j < NJ; j++) {
    const bool in = FULL || 4 * sub + SEG * j < len;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const float d = v[j][e] - mean;
      v[j][e] = d;
      const float sq = d * d;
      q += in ? (double)sq : 0.0;
    }
  }
  const float var = (float)(sub_sum_d<SUB>(q) / (double)len);
  // one division per row: d * (1/denom) is within an ulp of d / denom
  const float inv = 1.0f / (float)sqrt((double)(var + eps));
  float *y = Y + row * len;
#pragma unroll
  for (int j = 0; j < NJ; j++) {
    const int idx = 4 * sub + SEG * j;
    if (!(live && (FULL || idx < len))) continue;
    f32x4 t = v[j];
#pragma unroll
    for (int e = 0; e < 4; e++) t[e] = t[e] * inv;
    if (G) {
      const f32x4 g = *reinterpret_cast<const f32x4 *>(G + idx);
#pragma unroll
      for (int e = 0; e < 4; e++) t[e] = t[e] * g[e];
    }
    if (Bt) {
      const f32x4 bt = *reinterpret_cast<const f32x4 *>(Bt + idx);
#pragma unroll
      for (int e = 0; e < 4; e++) t[e] = t[e] + bt[e];
    }
    *reinterpret_cast<f32x4 *>(y + idx) = t;
    if (P) {
      const f32x4 pv = *reinterpret_cast<const f32x4 *>(P + row * len + idx);
#pragma unroll
      for (int e = 0; e < 4; e++) t[e] = t[e] + pv[e];
      *reinterpret_cast<f32x4 *>(Y2 + row * len + idx) = t;
    }
  }
}

__global__ __launch_bounds__(64 * WAVES_PER_BLOCK) void layernorm_rows_stream(
    const float *__restrict__ X, const float *__restrict__ G,
    const float *__restrict__ Bt, float *__restrict__ Y, long long outer, int len,
    float eps, const float *__restrict__ P, float *__restrict__ Y2) {
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * WAVES_PER_BLOCK + (threadIdx.x >> 6);
  if (row >= outer) return;
  const float *x = X + row * len;
  float *y = Y + row * len;
  double s = 0.0;
  for (int idx = lane; idx < len; idx += 64) s += (double)x[idx];
  const float mean = (float)(wave_sum_d(s) / (double)len);
  double q = 0.0;
  for (int idx = lane; idx < len; idx += 64) {
    float d = x[idx] - mean;
    q += (double)(d * d);
  }
  const float var = (float)(wave_sum_d(q) / (double)len);
  const float inv = 1.0f / (float)sqrt((double)(var + eps));
  for (int idx = lane; idx < len; idx += 64) {
    float t = (x[idx] - mean) * inv;
    if (G) t = t * G[idx];
    if (Bt) t = t + Bt[idx];
    y[idx] = t;
    if (P) Y2[row * len + idx] = t + P[row * len + idx];
  }
}

// ---- mean over trailing elements ------------------------------------------------
// Short rows (len <= 64, e.g. the 7x7 = 49 cells of ResNet's final pooling):
// a wavefront owns 64 consecutive rows, which are one contiguous span of
// 64*len floats.  It copies them row by row into LDS (each load instruction
// reads one row: contiguous, coalesced), then every lane sums its own row from
// LDS in the reference's order.  The odd row pitch keeps the lanes' LDS reads
// on distinct banks.
constexpr int SMALL_ROW_WAVES = 2;
__global__ __launch_bounds__(64 * SMALL_ROW_WAVES) void mean_rows_small(
    const float *__restrict__ X, float *__restrict__ Y, long long outer, int len) {
  __shared__ float stage[SMALL_ROW_WAVES][64 * 65];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long long row0 = ((long long)blockIdx.x * SMALL_ROW_WAVES + wave) * 64;
  if (row0 >= outer) return;
  const int rows = outer - row0 < 64 ? (int)(outer - row0) : 64;
  const int pitch = len | 1;
  float *mine = stage[wave];
  const float *x = X + row0 * len;
  if (lane < len) {
#pragma unroll 8
    for (int r = 0; r < rows; r++) mine[r * pitch + lane] = x[(long long)r * len + lane];
  }
  // the wavefront reads back only what it wrote itself
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  if (lane < rows) {
    double s = 0.0;
    for (int i = 0; i < len; i++) s += (double)mine[lane * pitch + i];
    Y[row0 + lane] = (float)(s / (double)len);
  }
}

__global__ __launch_bounds__(64 * WAVES_PER_BLOCK) void mean_rows_wave(
    const float *__restrict__ X, float *__restrict__ Y, long long outer, int len) {
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * WAVES_PER_BLOCK + (threadIdx.x >> 6);
  if (row >= outer) return;
  const float *x = X + row * len;
  double s = 0.0;
  for (int idx = lane; idx < len; idx += 64) s += (double)x[idx];
  s = wave_sum_d(s);
  if (lane == 0) Y[row] = (float)(s / (double)len);
}

// ---- sum over one inner axis -----------------------------------------------------
// X viewed as [outer, red, inner] with inner > 1: thread (o, i) adds its `red` elements,
// which lie `inner` apart, in index order in double; neighbouring threads read
// neighbouring addresses.  Rows along a middle axis are short in the graphs this
// serves (channel or head axes), so one thread per result is the whole schedule.
__global__ __launch_bounds__(256) void sum_axis_kernel(const float *__restrict__ X,
                                                       float *__restrict__ Y, long long outer,
                                                       int red, long long inner, double divisor) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= outer * inner) return;
  const long long o = idx / inner, i = idx - o * inner;
  const float *x = X + o * red * inner + i;
  double s = 0.0;
  for (int r = 0; r < red; r++) s += (double)x[(long long)r * inner];
  Y[idx] = (float)(s / divisor);
}

// the last axis with a divisor that is not its length (a pass of a multi-axis mean)
__global__ __launch_bounds__(64 * WAVES_PER_BLOCK) void sum_rows_wave(
    const float *__restrict__ X, float *__restrict__ Y, long long outer, int len, double divisor) {
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * WAVES_PER_BLOCK + (threadIdx.x >> 6);
  if (row >= outer) return;
  const float *x = X + row * len;
  double s = 0.0;
  for (int idx = lane; idx < len; idx += 64) s += (double)x[idx];
  s = wave_sum_d(s);
  if (lane == 0) Y[row] = (float)(s / divisor);
}

unsigned row_blocks(long long outer) {
  return (unsigned)((outer + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK);
}

int check_rows(const char *fn, long long outer, int len) {
  if (outer < 0 || len < 0) return wdh::fail(WDH_EINVAL, "%s: negative extent", fn);
  if ((outer + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK > 0x7fffffffLL)
    return wdh::fail(WDH_EINVAL, "%s: too many rows", fn);
  return WDH_OK;
}

}  // namespace

using wdh::fail;

extern "C" int wdh_softmax(wdh_buf hX, wdh_buf hY, int64_t outer, int len) {
  WDH_REQUIRE_INIT();
  WDH_REQUIRE_COMPUTE_LANE();
  if (int rc = check_rows("wdh_softmax", outer, len)) return rc;
  if (outer == 0 || len == 0) return WDH_OK;
  void *px, *py;
  const size_t bytes = (size_t)outer * len * 4;
  if (!wdh::operand(hX, bytes, "wdh_softmax: X", &px)) return WDH_EINVAL;
  if (!wdh::operand(hY, bytes, "wdh_softmax: Y", &py)) return WDH_EINVAL;
  const float *X = (const float *)px;
  float *Y = (float *)py;
  dim3 grid(row_blocks(outer)), block(64 * WAVES_PER_BLOCK);
  hipStream_t st = wdh::stream();
  const bool vec = len % 4 == 0 && (((uintptr_t)px | (uintptr_t)py) & 15) == 0;
  const bool vec2 = !vec && len % 2 == 0 && (((uintptr_t)px | (uintptr_t)py) & 7) == 0;
  if (len <= 64 * 2)
    hipLaunchKernelGGL((softmax_rows_reg<2, 1>), grid, block, 0, st, X, Y, outer, len);
  else if (len <= 64 * 8 && vec)
    hipLaunchKernelGGL((softmax_rows_reg<8, 4>), grid, block, 0, st, X, Y, outer, len);
  else if (len <= 64 * 8 && vec2)
    hipLaunchKernelGGL((softmax_rows_reg<8, 2>), grid, block, 0, st, X, Y, outer, len);
  else if (len <= 64 * 8)
    hipLaunchKernelGGL((softmax_rows_reg<8, 1>), grid, block, 0, st, X, Y, outer, len);
  else if (len <= 64 * 16 && vec)
    hipLaunchKernelGGL((softmax_rows_reg<16, 4>), grid, block, 0, st, X, Y, outer, len);
  else if (len <= 64 * 16 && vec2)
    hipLaunchKernelGGL((softmax_rows_reg<16, 2>), grid, block, 0, st, X, Y, outer, len);
  else if (len <= 64 * 16)
    hipLaunchKernelGGL((softmax_rows_reg<16, 1>), grid, block, 0, st, X, Y, outer, len);
  else if (len <= 64 * 32 && vec)
    hipLaunchKernelGGL((softmax_rows_reg<32, 4>), grid, block, 0, st, X, Y, outer, len);
  else if (len <= 64 * 32 && vec2)
    hipLaunchKernelGGL((softmax_rows_reg<32, 2>), grid, block, 0, st, X, Y, outer, len);
  else if (len <= 64 * 32)
    hipLaunchKernelGGL((softmax_rows_reg<32, 1>), grid, block, 0, st, X, Y, outer, len);
  else
    hipLaunchKernelGGL(softmax_rows_stream, grid, block, 0, st, X, Y, outer, len);
  WDH_LAUNCH_CHECK();
  return WDH_OK;
}

namespace {
int layernorm_launch(const char *who, wdh_buf hX, wdh_buf hG, wdh_buf hB, wdh_buf hY, wdh_buf hP, wdh_buf hY2,
                     int64_t outer, int len, float eps) {
  if (int rc = check_rows(who, outer, len)) return rc;
  if (outer == 0 || len == 0) return WDH_OK;
  void *px, *py, *pg = nullptr, *pb = nullptr, *pp = nullptr, *py2 = nullptr;
  const size_t bytes = (size_t)outer * len * 4;
  if (!wdh::operand(hX, bytes, "layernorm: X", &px)) return WDH_EINVAL;
  if (!wdh::operand(hY, bytes, "layernorm: Y", &py)) return WDH_EINVAL;
  if (hG && !wdh::operand(hG, (size_t)len * 4, "layernorm: Gamma", &pg)) return WDH_EINVAL;
  if (hB && !wdh::operand(hB, (size_t)len * 4, "layernorm: Beta", &pb)) return WDH_EINVAL;
  if (hP) {
    if (!wdh::operand(hP, bytes, "layernorm: P", &pp)) return WDH_EINVAL;
    if (!wdh::operand(hY2, bytes, "layernorm: Y2", &py2)) return WDH_EINVAL;
    if (py2 == py || py2 == px || py2 == pp) return fail(WDH_EINVAL, "%s: Y2 aliases another operand", who);
  }
  const float *X = (const float *)px, *G = (const float *)pg, *B = (const float *)pb, *P = (const float *)pp;
  float *Y = (float *)py, *Y2 = (float *)py2;
  dim3 grid(row_blocks(outer)), block(64 * WAVES_PER_BLOCK);
  hipStream_t st = wdh::stream();
  const bool vec = len % 4 == 0 &&
                   (((uintptr_t)px | (uintptr_t)py | (uintptr_t)pg | (uintptr_t)pb | (uintptr_t)pp |
                     (uintptr_t)py2) & 15) == 0;
  if (len <= 256 && vec && outer >= 4096) {  // (fewer rows: a wavefront per row, for four times the wavefronts)
    // (eight lanes per row measured slower: 12.4 us against 10.0 us on 27200 rows of 256)
    const long long per_block = WAVES_PER_BLOCK * 4;
    const dim3 g((unsigned)((outer + per_block - 1) / per_block));
    if (len == 256)
      hipLaunchKernelGGL((layernorm_rows_part<16, true>), g, block, 0, st, X, G, B, Y, outer, len, eps, P, Y2);
    else
      hipLaunchKernelGGL((layernorm_rows_part<16, false>), g, block, 0, st, X, G, B, Y, outer, len, eps, P, Y2);
  } else if (len <= 64 * 4 && vec)
    hipLaunchKernelGGL((layernorm_rows_reg<4, true>), grid, block, 0, st, X, G, B, Y, outer, len, eps, P, Y2);
  else if (len <= 64 * 4)
    hipLaunchKernelGGL((layernorm_rows_reg<4, false>), grid, block, 0, st, X, G, B, Y, outer, len, eps, P, Y2);
  else if (len <= 64 * 16 && vec)
    hipLaunchKernelGGL((layernorm_rows_reg<16, true>), grid, block, 0, st, X, G, B, Y, outer, len, eps, P, Y2);
  else if (len <= 64 * 16)
    hipLaunchKernelGGL((layernorm_rows_reg<16, false>), grid, block, 0, st, X, G, B, Y, outer, len, eps, P, Y2);
  else
    hipLaunchKernelGGL(layernorm_rows_stream, grid, block, 0, st, X, G, B, Y, outer, len, eps, P, Y2);
  WDH_LAUNCH_CHECK();
  return WDH_OK;
}
}  // namespace

extern "C" int wdh_layernorm(wdh_buf hX, wdh_buf hG, wdh_buf hB, wdh_buf hY,
                             int64_t outer, int len, float eps) {
  WDH_REQUIRE_INIT();
  WDH_REQUIRE_COMPUTE_LANE();
  return layernorm_launch("wdh_layernorm", hX, hG, hB, hY, 0, 0, outer, len, eps);
}

extern "C" int wdh_layernorm_add(wdh_buf hX, wdh_buf hG, wdh_buf hB, wdh_buf hY, wdh_buf hP, wdh_buf hY2,
                                 int64_t outer, int len, float eps) {
  WDH_REQUIRE_INIT();
  WDH_REQUIRE_COMPUTE_LANE();
  if (!hP || !hY2) return fail(WDH_EINVAL, "wdh_layernorm_add: P and Y2 are required");
  return layernorm_launch("wdh_layernorm_add", hX, hG, hB, hY, hP, hY2, outer, len, eps);
}

extern "C" int wdh_reduce_mean(wdh_buf hX, wdh_buf hY, int64_t outer, int len) {
  WDH_REQUIRE_INIT();
  WDH_REQUIRE_COMPUTE_LANE();
  if (int rc = check_rows("wdh_reduce_mean", outer, len)) return rc;
  if (outer == 0) return WDH_OK;
  if (len == 0) return fail(WDH_EINVAL, "wdh_reduce_mean: empty reduction");
  void *px, *py;
  if (!wdh::operand(hX, (size_t)outer * len * 4, "wdh_reduce_mean: X", &px)) return WDH_EINVAL;
  if (!wdh::operand(hY, (size_t)outer * 4, "wdh_reduce_mean: Y", &py)) return WDH_EINVAL;
  hipStream_t st = wdh::stream();
  if (len <= 64 && outer >= 4096)
    hipLaunchKernelGGL(mean_rows_small,
                       dim3((unsigned)((outer + 64 * SMALL_ROW_WAVES - 1) / (64 * SMALL_ROW_WAVES))),
                       dim3(64 * SMALL_ROW_WAVES), 0, st, (const float *)px, (float *)py,
                       (long long)outer, len);
  else
    hipLaunchKernelGGL(mean_rows_wave, dim3(row_blocks(outer)),
                       dim3(64 * WAVES_PER_BLOCK), 0, st, (const float *)px,
                       (float *)py, (long long)outer, len);
  WDH_LAUNCH_CHECK();
  return WDH_OK;
}

extern "C" int wdh_reduce_axis(wdh_buf hX, wdh_buf hY, int64_t outer, int red, int64_t inner,
                               int64_t divisor) {
  WDH_REQUIRE_INIT();
  WDH_REQUIRE_COMPUTE_LANE();
  if (outer < 0 || red < 0 || inner < 0) return fail(WDH_EINVAL, "wdh_reduce_axis: negative extent");
  if (divisor <= 0) return fail(WDH_EINVAL, "wdh_reduce_axis: divisor %lld", (long long)divisor);
  const long long results = (long long)outer * inner;
  if (results == 0) return WDH_OK;
  if (red == 0) return fail(WDH_EINVAL, "wdh_reduce_axis: empty reduction");
  if (inner == 1 && divisor == red) return wdh_reduce_mean(hX, hY, outer, red);
  if ((results + 255) / 256 > 0x7fffffffLL || (outer + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK > 0x7fffffffLL)
    return fail(WDH_EINVAL, "wdh_reduce_axis: too many results");
  void *px, *py;
  if (!wdh::operand(hX, (size_t)results * red * 4, "wdh_reduce_axis: X", &px)) return WDH_EINVAL;
  if (!wdh::operand(hY, (size_t)results * 4, "wdh_reduce_axis: Y", &py)) return WDH_EINVAL;
  if (inner == 1)
    hipLaunchKernelGGL(sum_rows_wave, dim3(row_blocks(outer)), dim3(64 * WAVES_PER_BLOCK), 0, wdh::stream(),
                       (const float *)px, (float *)py, (long long)outer, red, (double)divisor);
  else
    hipLaunchKernelGGL(sum_axis_kernel, dim3((unsigned)((results + 255) / 256)), dim3(256), 0, wdh::stream(),
                       (const float *)px, (float *)py, (long long)outer, red, (long long)inner,
                       (double)divisor);
  WDH_LAUNCH_CHECK();
  return WDH_OK;
}

extern "C" int wdh_global_avgpool(wdh_buf hX, wdh_buf hY, int64_t nc, int hw) {
  return wdh_reduce_mean(hX, hY, nc, hw);
}
