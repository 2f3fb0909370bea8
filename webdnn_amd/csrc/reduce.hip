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
// Sqrt/Div/Mul/Add subgraph.
//
// One wavefront owns one row: lanes read consecutive floats (256-byte
// coalesced requests), keep the row in registers when it fits (len <= 64*NV),
// and reduce with cross-lane shuffles; no LDS, no barriers.  Rows longer than
// the register budget are re-read from cache in further passes.
#include <math.h>

#include "common.h"

namespace {

constexpr int WAVES_PER_BLOCK = 4;

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ double wave_sum_d(double v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// ---- softmax ---------------------------------------------------------------
template <int NV>
__global__ __launch_bounds__(64 * WAVES_PER_BLOCK) void softmax_rows_reg(
    const float *__restrict__ X, float *__restrict__ Y, long long outer, int len) {
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * WAVES_PER_BLOCK + (threadIdx.x >> 6);
  if (row >= outer) return;
  const float *x = X + row * len;
  float *y = Y + row * len;
  float v[NV];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    int idx = lane + 64 * i;
    v[i] = idx < len ? x[idx] : -INFINITY;
    mx = fmaxf(mx, v[i]);  // fmaxf skips NaN, like `if (v > max)`
  }
  mx = wave_max(mx);
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    int idx = lane + 64 * i;
    float e = idx < len ? expf(v[i] - mx) : 0.0f;
    v[i] = e;
    sum += e;
  }
  sum = wave_sum(sum);
#pragma unroll
  for (int i = 0; i < NV; i++) {
    int idx = lane + 64 * i;
    if (idx < len) y[idx] = v[i] / sum;
  }
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
    float e = expf(x[idx] - mx);
    y[idx] = e;
    sum += e;
  }
  sum = wave_sum(sum);
  for (int idx = lane; idx < len; idx += 64) y[idx] = y[idx] / sum;
}

// ---- layer normalisation -----------------------------------------------------
template <int NV>
__global__ __launch_bounds__(64 * WAVES_PER_BLOCK) void layernorm_rows_reg(
    const float *__restrict__ X, const float *__restrict__ G,
    const float *__restrict__ Bt, float *__restrict__ Y, long long outer, int len,
    float eps) {
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * WAVES_PER_BLOCK + (threadIdx.x >> 6);
  if (row >= outer) return;
  const float *x = X + row * len;
  float *y = Y + row * len;
  float v[NV];
  double s = 0.0;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    int idx = lane + 64 * i;
    v[i] = idx < len ? x[idx] : 0.0f;
    s += (double)v[i];
  }
  const float mean = (float)(wave_sum_d(s) / (double)len);
  double q = 0.0;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    int idx = lane + 64 * i;
    float d = v[i] - mean;
    v[i] = d;
    float sq = d * d;
    q += idx < len ? (double)sq : 0.0;
  }
  const float var = (float)(wave_sum_d(q) / (double)len);
  const float denom = (float)sqrt((double)(var + eps));
#pragma unroll
  for (int i = 0; i < NV; i++) {
    int idx = lane + 64 * i;
    if (idx < len) {
      float t = v[i] / denom;
      if (G) t = t * G[idx];
      if (Bt) t = t + Bt[idx];
      y[idx] = t;
    }
  }
}

__global__ __launch_bounds__(64 * WAVES_PER_BLOCK) void layernorm_rows_stream(
    const float *__restrict__ X, const float *__restrict__ G,
    const float *__restrict__ Bt, float *__restrict__ Y, long long outer, int len,
    float eps) {
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
  const float denom = (float)sqrt((double)(var + eps));
  for (int idx = lane; idx < len; idx += 64) {
    float t = (x[idx] - mean) / denom;
    if (G) t = t * G[idx];
    if (Bt) t = t + Bt[idx];
    y[idx] = t;
  }
}

// ---- mean over trailing elements ------------------------------------------------
// Short rows (len <= 64, e.g. the 7x7 = 49 cells of ResNet's final pooling):
// one thread per row, summing in the reference's order.  Neighbouring threads
// own neighbouring rows, so a wavefront's loads together cover one contiguous
// span of 64*len floats that stays in the vector L1 between iterations.
__global__ __launch_bounds__(256) void mean_rows_small(const float *__restrict__ X,
                                                       float *__restrict__ Y,
                                                       long long outer, int len) {
  const long long row = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= outer) return;
  const float *x = X + row * len;
  double s = 0.0;
  for (int i = 0; i < len; i++) s += (double)x[i];
  Y[row] = (float)(s / (double)len);
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
  if (len <= 64 * 2)
    hipLaunchKernelGGL(softmax_rows_reg<2>, grid, block, 0, st, X, Y, outer, len);
  else if (len <= 64 * 8)
    hipLaunchKernelGGL(softmax_rows_reg<8>, grid, block, 0, st, X, Y, outer, len);
  else if (len <= 64 * 16)
    hipLaunchKernelGGL(softmax_rows_reg<16>, grid, block, 0, st, X, Y, outer, len);
  else if (len <= 64 * 32)
    hipLaunchKernelGGL(softmax_rows_reg<32>, grid, block, 0, st, X, Y, outer, len);
  else
    hipLaunchKernelGGL(softmax_rows_stream, grid, block, 0, st, X, Y, outer, len);
  WDH_LAUNCH_CHECK();
  return WDH_OK;
}

extern "C" int wdh_layernorm(wdh_buf hX, wdh_buf hG, wdh_buf hB, wdh_buf hY,
                             int64_t outer, int len, float eps) {
  WDH_REQUIRE_INIT();
  if (int rc = check_rows("wdh_layernorm", outer, len)) return rc;
  if (outer == 0 || len == 0) return WDH_OK;
  void *px, *py, *pg = nullptr, *pb = nullptr;
  const size_t bytes = (size_t)outer * len * 4;
  if (!wdh::operand(hX, bytes, "wdh_layernorm: X", &px)) return WDH_EINVAL;
  if (!wdh::operand(hY, bytes, "wdh_layernorm: Y", &py)) return WDH_EINVAL;
  if (hG && !wdh::operand(hG, (size_t)len * 4, "wdh_layernorm: Gamma", &pg)) return WDH_EINVAL;
  if (hB && !wdh::operand(hB, (size_t)len * 4, "wdh_layernorm: Beta", &pb)) return WDH_EINVAL;
  const float *X = (const float *)px, *G = (const float *)pg, *B = (const float *)pb;
  float *Y = (float *)py;
  dim3 grid(row_blocks(outer)), block(64 * WAVES_PER_BLOCK);
  hipStream_t st = wdh::stream();
  if (len <= 64 * 4)
    hipLaunchKernelGGL(layernorm_rows_reg<4>, grid, block, 0, st, X, G, B, Y, outer, len, eps);
  else if (len <= 64 * 16)
    hipLaunchKernelGGL(layernorm_rows_reg<16>, grid, block, 0, st, X, G, B, Y, outer, len, eps);
  else
    hipLaunchKernelGGL(layernorm_rows_stream, grid, block, 0, st, X, G, B, Y, outer, len, eps);
  WDH_LAUNCH_CHECK();
  return WDH_OK;
}

extern "C" int wdh_reduce_mean(wdh_buf hX, wdh_buf hY, int64_t outer, int len) {
  WDH_REQUIRE_INIT();
  if (int rc = check_rows("wdh_reduce_mean", outer, len)) return rc;
  if (outer == 0) return WDH_OK;
  if (len == 0) return fail(WDH_EINVAL, "wdh_reduce_mean: empty reduction");
  void *px, *py;
  if (!wdh::operand(hX, (size_t)outer * len * 4, "wdh_reduce_mean: X", &px)) return WDH_EINVAL;
  if (!wdh::operand(hY, (size_t)outer * 4, "wdh_reduce_mean: Y", &py)) return WDH_EINVAL;
  hipStream_t st = wdh::stream();
  if (len <= 64 && outer >= 4096)
    hipLaunchKernelGGL(mean_rows_small, dim3((unsigned)((outer + 255) / 256)), dim3(256),
                       0, st, (const float *)px, (float *)py, (long long)outer, len);
  else
    hipLaunchKernelGGL(mean_rows_wave, dim3(row_blocks(outer)),
                       dim3(64 * WAVES_PER_BLOCK), 0, st, (const float *)px,
                       (float *)py, (long long)outer, len);
  WDH_LAUNCH_CHECK();
  return WDH_OK;
}

extern "C" int wdh_global_avgpool(wdh_buf hX, wdh_buf hY, int64_t nc, int hw) {
  return wdh_reduce_mean(hX, hY, nc, hw);
}
