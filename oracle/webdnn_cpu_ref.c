/*
 * TEST INFRASTRUCTURE ONLY — CPU restatement of the WebDNN reference CPU
 * operators on the Gemm/MatMul/Conv hot path and their companions.
 *
 * Nothing in the product (webdnn_amd/) links, loads or calls this file.  It is
 * the checker used by tests/, by __graft_entry__.smoke() and by the
 * cpu_baseline leg of bench.py.
 *
 * Every function restates one reference routine, loop for loop, with the same
 * accumulator type (JavaScript numbers are IEEE doubles) and the same points
 * at which a value is rounded to fp32 (a store into a Float32Array).  Paths
 * are relative to src/descriptor_runner/ in the reference tree.
 *
 * Shapes are computed here from ONNX-level arguments (dims + attributes), as
 * the reference's operators/base classes do, so that the oracle does not
 * depend on the product's host-side shape code.
 *
 * Outer loops may run on several OpenMP threads (ref_set_threads); every
 * output element is still produced by one thread with the reference's
 * summation order, so results do not depend on the thread count.
 *
 * Parity status: every function is pinned by tests/test_oracle_*.py against
 * closed forms, brute force on tiny inputs or the reference's own vectors,
 * except the last ulp (in double) of exp/tanh/pow, which V8 and libm may round
 * differently: softmax, sigmoid, exp, tanh and pow are pinned to 1e-6 relative
 * only ("parity unpinned" below that).
 *
 * Return value: 0 on success, a negative number where the reference throws.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define REF_OK 0
#define REF_ETHROW (-1) /* the reference operator would throw */
#define REF_ENOMEM (-2)

static int g_threads = 1;

void ref_set_threads(int n) { g_threads = n > 0 ? n : 1; }
int ref_get_threads(void) { return g_threads; }

/* operators/operatorUtil.ts:169-176 (calcStrides) */
static void calc_strides(const int64_t *dims, int ndim, int64_t *strides) {
  int64_t length = 1;
  for (int i = ndim - 1; i >= 0; i--) {
    strides[i] = length;
    length *= dims[i];
  }
}

/* operators/operatorUtil.ts:178-209 (broadcastUni): strides of B broadcast to A */
static int broadcast_uni(const int64_t *dimsA, int ndimA, const int64_t *dimsB,
                         int ndimB, int64_t *stridesB) {
  int64_t expanded[8];
  if (ndimA < ndimB || ndimA > 8) return REF_ETHROW;
  int pad = ndimA - ndimB;
  for (int i = 0; i < ndimA; i++) expanded[i] = i < pad ? 1 : dimsB[i - pad];
  calc_strides(expanded, ndimA, stridesB);
  for (int i = 0; i < ndimA; i++) {
    if (dimsA[i] != expanded[i]) {
      if (expanded[i] == 1) stridesB[i] = 0;
      else return REF_ETHROW;
    }
  }
  return REF_OK;
}

/* operators/operatorUtil.ts:211-245 (broadcastMulti) for two inputs */
int ref_broadcast_multi(const int64_t *dimsA, int ndimA, const int64_t *dimsB,
                        int ndimB, int64_t *outDims, int64_t *stridesA,
                        int64_t *stridesB) {
  int nd = ndimA > ndimB ? ndimA : ndimB;
  int64_t ea[8], eb[8];
  if (nd > 8) return REF_ETHROW;
  for (int i = 0; i < nd; i++) {
    ea[i] = i < nd - ndimA ? 1 : dimsA[i - (nd - ndimA)];
    eb[i] = i < nd - ndimB ? 1 : dimsB[i - (nd - ndimB)];
    outDims[i] = ea[i] > eb[i] ? ea[i] : eb[i];
  }
  calc_strides(ea, nd, stridesA);
  calc_strides(eb, nd, stridesB);
  for (int i = 0; i < nd; i++) {
    if (ea[i] != outDims[i]) {
      if (ea[i] == 1) stridesA[i] = 0; else return REF_ETHROW;
    }
    if (eb[i] != outDims[i]) {
      if (eb[i] == 1) stridesB[i] = 0; else return REF_ETHROW;
    }
  }
  return nd;
}

/* ---- Gemm --------------------------------------------------------------
 * operators/base/gemm.ts:28-61 (calcShape) and
 * operators/cpu/operators/standard/gemm.ts:21-61 (run).
 * Y must hold m*n floats; *out_m / *out_n receive the result shape. */
int ref_gemm(const float *dA, const int64_t *dimsA, int ndimA, const float *dB,
             const int64_t *dimsB, int ndimB, const float *dC,
             const int64_t *dimsC, int ndimC, double alpha, double beta,
             int transA, int transB, float *Y, int64_t *out_m, int64_t *out_n) {
  int64_t m, n, k, kcheck, sA0, sA1, sB0, sB1;
  if (ndimA != 2 || ndimB != 2) return REF_ETHROW;
  if (transA) { k = dimsA[0]; m = dimsA[1]; sA0 = 1; sA1 = m; }
  else { m = dimsA[0]; k = dimsA[1]; sA0 = k; sA1 = 1; }
  if (transB) { n = dimsB[0]; kcheck = dimsB[1]; sB0 = 1; sB1 = kcheck; }
  else { kcheck = dimsB[0]; n = dimsB[1]; sB0 = n; sB1 = 1; }
  if (k != kcheck) return REF_ETHROW;
  if (out_m) *out_m = m;
  if (out_n) *out_n = n;
  if (!Y) return REF_OK; /* shape query */
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t i = 0; i < m; i++) {
    for (int64_t j = 0; j < n; j++) {
      double sum = 0;
      for (int64_t x = 0; x < k; x++)
        sum += (double)dA[i * sA0 + x * sA1] * (double)dB[x * sB0 + j * sB1];
      sum *= alpha;
      Y[i * n + j] = (float)sum;
    }
  }
  if (dC) {
    int64_t mn[2] = {m, n}, sC[2];
    if (broadcast_uni(mn, 2, dimsC, ndimC, sC) != REF_OK) return REF_ETHROW;
    for (int64_t i = 0; i < m; i++)
      for (int64_t j = 0; j < n; j++)
        Y[i * n + j] =
            (float)((double)Y[i * n + j] + (double)dC[i * sC[0] + j * sC[1]] * beta);
  }
  return REF_OK;
}

/* ---- MatMul --------------------------------------------------------------
 * operators/base/matmul.ts:6-91 (calcShape) and
 * operators/cpu/operators/standard/matmul.ts:11-111 (run, calcDim2, calcDim3).
 * outDims receives resultDimsAfterSqueeze; returns its rank (>= 0) or < 0.
 * Y == NULL asks for the shape only. */
int ref_matmul(const float *dA, const int64_t *dimsA, int ndimA, const float *dB,
               const int64_t *dimsB, int ndimB, float *Y, int64_t *outDims) {
  int total = ndimA > ndimB ? ndimA : ndimB;
  if (total < 2) total = 2;
  if (ndimA == 0 || ndimB == 0 || total > 8) return REF_ETHROW;
  int64_t ea[8], eb[8], sa[8], sb[8], rd[8], rs[8];
  /* A: a 1-D input gets a leading 1, then both are left-padded with 1s */
  {
    int64_t tmp[8]; int nt = 0;
    if (ndimA == 1) tmp[nt++] = 1;
    for (int i = 0; i < ndimA; i++) tmp[nt++] = dimsA[i];
    int pad = total - nt;
    for (int i = 0; i < total; i++) ea[i] = i < pad ? 1 : tmp[i - pad];
  }
  {
    int64_t tmp[8]; int nt = 0;
    for (int i = 0; i < ndimB; i++) tmp[nt++] = dimsB[i];
    if (ndimB == 1) tmp[nt++] = 1;
    int pad = total - nt;
    for (int i = 0; i < total; i++) eb[i] = i < pad ? 1 : tmp[i - pad];
  }
  int64_t inner = ea[total - 1];
  if (inner != eb[total - 2]) return REF_ETHROW;
  calc_strides(ea, total, sa);
  calc_strides(eb, total, sb);
  rd[total - 2] = ea[total - 2];
  rd[total - 1] = eb[total - 1];
  for (int i = total - 3; i >= 0; i--) {
    rd[i] = ea[i] > eb[i] ? ea[i] : eb[i];
    if (ea[i] == 1) sa[i] = 0;
    if (eb[i] == 1) sb[i] = 0;
  }
  calc_strides(rd, total, rs);
  int nout = 0;
  for (int i = 0; i < total; i++) {
    if (ndimA == 1 && i == total - 2) continue;
    if (ndimB == 1 && i == total - 1) continue;
    outDims[nout++] = rd[i];
  }
  if (!Y) return total <= 3 ? nout : REF_ETHROW;
  if (total == 2) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t m = 0; m < rd[0]; m++)
      for (int64_t n = 0; n < rd[1]; n++) {
        double sum = 0;
        for (int64_t k = 0; k < inner; k++)
          sum += (double)dA[m * sa[0] + k * sa[1]] * (double)dB[k * sb[0] + n * sb[1]];
        Y[m * rs[0] + n * rs[1]] = (float)sum;
      }
  } else if (total == 3) {
#pragma omp parallel for num_threads(g_threads) schedule(static) collapse(2)
    for (int64_t o = 0; o < rd[0]; o++)
      for (int64_t m = 0; m < rd[1]; m++)
        for (int64_t n = 0; n < rd[2]; n++) {
          double sum = 0;
          for (int64_t k = 0; k < inner; k++)
            sum += (double)dA[o * sa[0] + m * sa[1] + k * sa[2]] *
                   (double)dB[o * sb[0] + k * sb[1] + n * sb[2]];
          Y[o * rs[0] + m * rs[1] + n * rs[2]] = (float)sum;
        }
  } else {
    return REF_ETHROW; /* matmul.ts:50-53: rank >= 4 results are not supported */
  }
  return nout;
}

/* ---- Conv ----------------------------------------------------------------
 * operators/base/conv.ts:31-79 (calcShape; `pads`, `strides`, `dilations`,
 * `kernel_shape` are passed with n_* = 0 when the attribute is absent) and
 * operators/cpu/operators/standard/conv.ts:134-333: im2col -> matmul ->
 * transpose -> bias, four passes with an fp32 store between them.
 * (runSplitBatch, conv.ts:16-132, processes the batch in slices when the
 * im2col buffer would exceed 511 Mi elements; each output element goes
 * through the same arithmetic, so it is not restated separately.)
 * outDims[4] receives [batch, chOut, oh, ow].  Y == NULL: shape only. */
static int64_t floor_div(int64_t a, int64_t b) {
  int64_t q = a / b;
  if ((a % b != 0) && ((a < 0) != (b < 0))) q--;
  return q;
}

int ref_conv(const float *dX, const int64_t *dimsX, int ndimX, const float *dW,
             const int64_t *dimsW, const float *dB, const int64_t *dilations_,
             int n_dil, int64_t group, const int64_t *kernel_shape_, int n_ks,
             const int64_t *pads_, int n_pads, const int64_t *strides_, int n_str,
             float *Y, int64_t *outDims) {
  if (ndimX != 4) return REF_ETHROW;
  int64_t batch = dimsX[0];
  int64_t dil[2] = {1, 1}, ks[2] = {dimsW[2], dimsW[3]}, pads[4] = {0, 0, 0, 0},
          str[2] = {1, 1};
  if (n_dil > 0) { dil[0] = dilations_[0]; dil[1] = dilations_[1]; }
  if (n_ks > 0) { ks[0] = kernel_shape_[0]; ks[1] = kernel_shape_[1]; }
  if (n_pads > 0) { for (int i = 0; i < 4; i++) pads[i] = pads_[i]; }
  if (n_str > 0) { str[0] = strides_[0]; str[1] = strides_[1]; }
  int64_t inS[2] = {dimsX[2], dimsX[3]};
  int64_t outS[2];
  for (int a = 0; a < 2; a++)
    outS[a] = floor_div(inS[a] + pads[a] + pads[a + 2] - dil[a] * (ks[a] - 1) - 1, str[a]) + 1;
  int64_t chIn = dimsX[1], chInG = chIn / group, chOut = dimsW[0], chOutG = chOut / group;
  outDims[0] = batch; outDims[1] = chOut; outDims[2] = outS[0]; outDims[3] = outS[1];
  if (!Y) return REF_OK;
  int64_t bout = batch * outS[0] * outS[1];
  int64_t cinkhkw = chInG * ks[0] * ks[1];
  int64_t outarea = outS[0] * outS[1];
  float *dI = (float *)malloc(sizeof(float) * (size_t)(group * bout * cinkhkw > 0 ? group * bout * cinkhkw : 1));
  float *dT = (float *)malloc(sizeof(float) * (size_t)(group * bout * chOutG > 0 ? group * bout * chOutG : 1));
  if (!dI || !dT) { free(dI); free(dT); return REF_ENOMEM; }
  /* im2col, conv.ts:223-270 */
#pragma omp parallel for num_threads(g_threads) schedule(static) collapse(2)
  for (int64_t g = 0; g < group; g++)
    for (int64_t b = 0; b < batch; b++) {
      int64_t idx = (g * batch + b) * outarea * cinkhkw;
      for (int64_t oy = 0; oy < outS[0]; oy++)
        for (int64_t ox = 0; ox < outS[1]; ox++)
          for (int64_t ci = 0; ci < chInG; ci++)
            for (int64_t ky = 0; ky < ks[0]; ky++)
              for (int64_t kx = 0; kx < ks[1]; kx++) {
                float v = 0;
                int64_t iny = oy * str[0] - pads[0] + ky * dil[0];
                int64_t inx = ox * str[1] - pads[1] + kx * dil[1];
                if (iny >= 0 && iny < inS[0] && inx >= 0 && inx < inS[1])
                  v = dX[((b * chIn + g * chInG + ci) * inS[0] + iny) * inS[1] + inx];
                dI[idx++] = v;
              }
    }
  /* matmul, conv.ts:272-295 */
#pragma omp parallel for num_threads(g_threads) schedule(static) collapse(2)
  for (int64_t g = 0; g < group; g++)
    for (int64_t y = 0; y < bout; y++)
      for (int64_t x = 0; x < chOutG; x++) {
        double s = 0;
        const float *pi = dI + (g * bout + y) * cinkhkw;
        const float *pw = dW + (g * chOutG + x) * cinkhkw;
        for (int64_t ip = 0; ip < cinkhkw; ip++) s += (double)pi[ip] * (double)pw[ip];
        dT[(g * bout + y) * chOutG + x] = (float)s;
      }
  /* transpose, conv.ts:297-316 */
  {
    int64_t idx = 0;
    for (int64_t b = 0; b < batch; b++)
      for (int64_t g = 0; g < group; g++)
        for (int64_t c = 0; c < chOutG; c++)
          for (int64_t x = 0; x < outarea; x++)
            Y[idx++] = dT[((g * batch + b) * outarea + x) * chOutG + c];
  }
  /* bias, conv.ts:318-333: fp32 store of (double)y + (double)b */
  if (dB) {
    int64_t idx = 0;
    for (int64_t b = 0; b < batch; b++)
      for (int64_t c = 0; c < chOut; c++)
        for (int64_t x = 0; x < outarea; x++) {
          Y[idx] = (float)((double)Y[idx] + (double)dB[c]);
          idx++;
        }
  }
  free(dI);
  free(dT);
  return REF_OK;
}

/* ---- Binary7 -----------------------------------------------------------------
 * operators/cpu/operators/standard/binary7.ts:16-68 (run) and :70-254 (op0d..op6d):
 * op(l, r) in double, stored into the typed output array.
 * op: 0 add 1 sub 2 mul 3 div 4 pow.  dtype: 0 float32, 1 int32. */
static int32_t js_to_int32(double d) {
  if (isnan(d) || isinf(d)) return 0;
  double t = trunc(d);
  double m = fmod(t, 4294967296.0);
  if (m < 0) m += 4294967296.0;
  return (int32_t)(uint32_t)m;
}

static double binop(int op, double l, double r) {
  switch (op) {
    case 0: return l + r;
    case 1: return l - r;
    case 2: return l * r;
    case 3: return l / r;
    default: return pow(l, r);
  }
}

int ref_binary(int op, int dtype, const void *L, const int64_t *dimsL, int ndimL,
               const void *R, const int64_t *dimsR, int ndimR, void *Y,
               int64_t *outDims) {
  int64_t sl[8], sr[8];
  if (op < 0 || op > 4) return REF_ETHROW;
  int nd = ref_broadcast_multi(dimsL, ndimL, dimsR, ndimR, outDims, sl, sr);
  if (nd < 0) return REF_ETHROW;
  if (nd > 6) return REF_ETHROW; /* binary7.ts:63-66 */
  if (!Y) return nd;
  int64_t total = 1;
  for (int i = 0; i < nd; i++) total *= outDims[i];
  int64_t os[8];
  calc_strides(outDims, nd, os);
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t i = 0; i < total; i++) {
    int64_t rem = i, ol = 0, orr = 0;
    for (int d = 0; d < nd; d++) {
      int64_t c = rem / os[d];
      rem -= c * os[d];
      ol += c * sl[d];
      orr += c * sr[d];
    }
    if (dtype == 0) {
      double v = binop(op, (double)((const float *)L)[ol], (double)((const float *)R)[orr]);
      ((float *)Y)[i] = (float)v;
    } else {
      double v = binop(op, (double)((const int32_t *)L)[ol], (double)((const int32_t *)R)[orr]);
      ((int32_t *)Y)[i] = js_to_int32(v);
    }
  }
  return nd;
}

/* ---- CPUUnary ------------------------------------------------------------------
 * operators/cpu/operators/standard/unary.ts:10-32 (run) and the op table
 * :36-230.  op ids match include/webdnn_hip.h:
 * 0 relu 1 sigmoid 2 sqrt 3 exp 4 tanh 5 abs 6 neg 7 reciprocal. */
static double js_max0(double v) {
  /* Math.max(v, 0): NaN -> NaN, -0 -> +0 */
  if (isnan(v)) return v;
  return v > 0 ? v : 0.0;
}

int ref_unary(int op, int dtype, const void *X, void *Y, int64_t length) {
  if (op < 0 || op > 7) return REF_ETHROW;
  if (dtype == 1 && !(op == 0 || op == 5 || op == 6)) return REF_ETHROW;
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t i = 0; i < length; i++) {
    double v = dtype == 0 ? (double)((const float *)X)[i] : (double)((const int32_t *)X)[i];
    double y;
    switch (op) {
      case 0: y = js_max0(v); break;
      case 1: y = (tanh(v / 2) + 1) / 2; break;
      case 2: y = sqrt(v); break;
      case 3: y = exp(v); break;
      case 4: y = tanh(v); break;
      case 5: y = fabs(v); break;
      case 6: y = -v; break;
      default: y = 1 / v; break;
    }
    if (dtype == 0) ((float *)Y)[i] = (float)y;
    else ((int32_t *)Y)[i] = js_to_int32(y);
  }
  return REF_OK;
}

/* ---- Softmax --------------------------------------------------------------------
 * operators/cpu/operators/standard/softmax.ts:21-58.  `axis` as given by the
 * attribute (default -1); anything but the last axis throws (:28-32). */
int ref_softmax(const float *dI, const int64_t *dims, int ndim, int64_t axis, float *dO) {
  if (axis < 0) axis += ndim;
  if (axis != ndim - 1) return REF_ETHROW;
  int64_t length = 1;
  for (int i = 0; i < ndim; i++) length *= dims[i];
  int64_t red = dims[axis];
  int64_t outer = red ? length / red : 0;
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t o = 0; o < outer; o++) {
    double max = -INFINITY;
    for (int64_t r = 0; r < red; r++) {
      double v = dI[o * red + r];
      if (v > max) max = v;
    }
    double expsum = 0;
    for (int64_t r = 0; r < red; r++) {
      double v = dI[o * red + r], e = exp(v - max);
      dO[o * red + r] = (float)e;
      expsum += e;
    }
    for (int64_t r = 0; r < red; r++)
      dO[o * red + r] = (float)((double)dO[o * red + r] / expsum);
  }
  return REF_OK;
}

/* ---- MaxPool ----------------------------------------------------------------------
 * operators/base/maxpool.ts:32-137 (calcShape) and
 * operators/cpu/operators/standard/maxpool.ts:12-112.
 * auto_pad: 0 NOTSET, 1 SAME_UPPER, 2 SAME_LOWER, 3 VALID.
 * outDims[4]; padsOut[4] receives the pads in effect.  Y == NULL: shape only. */
static int64_t ceil_div_d(double a, double b) { return (int64_t)ceil(a / b); }
static int64_t floor_div_d(double a, double b) { return (int64_t)floor(a / b); }

int ref_maxpool(const float *dX, const int64_t *dimsX, int ndimX, int auto_pad,
                int ceil_mode, const int64_t *dilations_, int n_dil,
                const int64_t *kernel_shape, const int64_t *pads_, int n_pads,
                const int64_t *strides_, int n_str, int n_outputs, float *Y,
                int64_t *outDims, int64_t *padsOut) {
  if (n_outputs != 1) return REF_ETHROW;
  if (ndimX != 4) return REF_ETHROW;
  int64_t batch = dimsX[0], ch = dimsX[1];
  int64_t dil[2] = {1, 1}, str[2] = {1, 1}, pads[4] = {0, 0, 0, 0};
  if (n_dil > 0) { dil[0] = dilations_[0]; dil[1] = dilations_[1]; }
  if (n_str > 0) { str[0] = strides_[0]; str[1] = strides_[1]; }
  const int64_t *ks = kernel_shape;
  int64_t inS[2] = {dimsX[2], dimsX[3]}, outS[2];
  if (auto_pad == 0) {
    if (n_pads > 0) for (int i = 0; i < 4; i++) pads[i] = pads_[i];
    for (int a = 0; a < 2; a++) {
      double num = (double)(inS[a] + pads[a] + pads[a + 2] - dil[a] * (ks[a] - 1) - 1);
      outS[a] = (ceil_mode ? ceil_div_d(num, (double)str[a]) : floor_div_d(num, (double)str[a])) + 1;
    }
  } else if (auto_pad == 1 || auto_pad == 2) {
    for (int a = 0; a < 2; a++) {
      outS[a] = ceil_div_d((double)inS[a], (double)str[a]);
      int64_t sum = (outS[a] - 1) * str[a] + ((ks[a] - 1) * dil[a] + 1) - inS[a];
      int64_t lo = floor_div_d((double)sum, 2.0), hi = ceil_div_d((double)sum, 2.0);
      if (auto_pad == 1) { pads[a] = lo; pads[a + 2] = hi; }
      else { pads[a] = hi; pads[a + 2] = lo; }
    }
  } else if (auto_pad == 3) {
    for (int a = 0; a < 2; a++)
      outS[a] = ceil_div_d((double)(inS[a] - dil[a] * (ks[a] - 1)), (double)str[a]);
  } else {
    return REF_ETHROW;
  }
  outDims[0] = batch; outDims[1] = ch; outDims[2] = outS[0]; outDims[3] = outS[1];
  if (padsOut) for (int i = 0; i < 4; i++) padsOut[i] = pads[i];
  if (!Y) return REF_OK;
#pragma omp parallel for num_threads(g_threads) schedule(static) collapse(2)
  for (int64_t b = 0; b < batch; b++)
    for (int64_t c = 0; c < ch; c++) {
      int64_t idx = (b * ch + c) * outS[0] * outS[1];
      for (int64_t oy = 0; oy < outS[0]; oy++)
        for (int64_t ox = 0; ox < outS[1]; ox++) {
          float mv = -INFINITY;
          for (int64_t ky = 0; ky < ks[0]; ky++)
            for (int64_t kx = 0; kx < ks[1]; kx++) {
              int64_t iny = oy * str[0] - pads[0] + ky * dil[0];
              int64_t inx = ox * str[1] - pads[1] + kx * dil[1];
              if (iny >= 0 && iny < inS[0] && inx >= 0 && inx < inS[1]) {
                float v = dX[((b * ch + c) * inS[0] + iny) * inS[1] + inx];
                if (v > mv) mv = v;
              }
            }
          Y[idx++] = mv;
        }
    }
  return REF_OK;
}

/* ---- GlobalAveragePool ------------------------------------------------------------------
 * operators/cpu/operators/standard/globalaveragepool.ts:12-41 calling
 * operators/cpu/rawcomputation/averagepool.ts:1-46 with kernel = input size,
 * pads 0, strides 1, countIncludePad = true. */
int ref_global_average_pool(const float *dX, const int64_t *dimsX, int ndimX, float *Y) {
  if (ndimX != 4) return REF_ETHROW;
  int64_t batch = dimsX[0], ch = dimsX[1], h = dimsX[2], w = dimsX[3];
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t bc = 0; bc < batch * ch; bc++) {
    double sum = 0;
    for (int64_t ky = 0; ky < h; ky++)
      for (int64_t kx = 0; kx < w; kx++) sum += (double)dX[(bc * h + ky) * w + kx];
    Y[bc] = (float)(sum / (double)(h * w));
  }
  return REF_OK;
}

/* ---- Transpose ------------------------------------------------------------------------
 * operators/base/transpose.ts:16-34 (calcShape; n_perm = 0 means reversed)
 * and operators/cpu/operators/standard/transpose.ts:12-168 (copy1d..copy6d).
 * Elements are 4 bytes of any type.  outDims receives the output shape. */
int ref_transpose(const uint32_t *dI, const int64_t *dims, int ndim,
                  const int64_t *perm_, int n_perm, uint32_t *dO, int64_t *outDims) {
  int64_t perm[8], strides[8], inStrides[8], os[8];
  if (ndim < 1 || ndim > 6) return REF_ETHROW;
  if (n_perm > 0) {
    if (n_perm != ndim) return REF_ETHROW;
    for (int i = 0; i < ndim; i++) perm[i] = perm_[i];
  } else {
    for (int i = 0; i < ndim; i++) perm[i] = ndim - 1 - i;
  }
  calc_strides(dims, ndim, strides);
  int64_t total = 1;
  for (int i = 0; i < ndim; i++) {
    outDims[i] = dims[perm[i]];
    inStrides[i] = strides[perm[i]];
    total *= outDims[i];
  }
  if (!dO) return REF_OK;
  calc_strides(outDims, ndim, os);
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t i = 0; i < total; i++) {
    int64_t rem = i, off = 0;
    for (int d = 0; d < ndim; d++) {
      int64_t c = rem / os[d];
      rem -= c * os[d];
      off += c * inStrides[d];
    }
    dO[i] = dI[off];
  }
  return REF_OK;
}

/* ---- ReduceMean ------------------------------------------------------------------------
 * operators/cpu/operators/standard/reduce.ts:369-405 restricted to a reduction
 * over the single last axis: X viewed as [outer, len]; sum in double in index
 * order, divided by len, stored as fp32.  (Several axes are reduced one after
 * the other there with an fp32 store in between: ref_reduce_axis below.) */
int ref_reduce_mean_trailing(const float *X, int64_t outer, int64_t len, float *Y) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t o = 0; o < outer; o++) {
    double s = 0;
    for (int64_t r = 0; r < len; r++) s += (double)X[o * len + r];
    Y[o] = (float)(s / (double)len);
  }
  return REF_OK;
}

/* One pass of the general form (ReduceOp.runCore, reduce.ts:40-100, with the ReduceMean
 * kernels of reduce.ts:369-405): X viewed as [outer, red, inner]; every result is the sum
 * of its `red` elements in index order in double, divided by `divisor` (1 for every pass
 * but the last, the product of all reduced extents for the last) and stored as fp32. */
int ref_reduce_axis(const float *X, int64_t outer, int64_t red, int64_t inner, double divisor, float *Y) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t o = 0; o < outer; o++) {
    for (int64_t n = 0; n < inner; n++) {
      double s = 0;
      for (int64_t r = 0; r < red; r++) s += (double)X[(o * red + r) * inner + n];
      Y[o * inner + n] = divisor == 1.0 ? (float)s : (float)(s / divisor);
    }
  }
  return REF_OK;
}

/* ---- Gather ------------------------------------------------------------------------------
 * operators/cpu/operators/standard/gather.ts:20-33: only the scalar pick
 * (data rank 1, indices rank 0, axis 0) is accepted. */
int ref_gather(const uint32_t *data, int ndimData, const int32_t *indices,
               int ndimIndices, int64_t axis, uint32_t *Y) {
  if (!(ndimData == 1 && ndimIndices == 0 && axis == 0)) return REF_ETHROW;
  Y[0] = data[indices[0]];
  return REF_OK;
}

/* ---- LayerNormalization -----------------------------------------------------------------
 * Not a reference operator.  This is the decomposed subgraph executed with
 * the restated reference ops above, each node storing fp32:
 *   mean = ReduceMean(x); d = Sub(x, mean); sq = Mul(d, d); var = ReduceMean(sq)
 *   s = Sqrt(Add(var, eps)); y = Add(Mul(Div(d, s), gamma), beta)
 * gamma / beta may be NULL (the Mul / Add node is then absent). */
int ref_layernorm_decomposed(const float *X, int64_t outer, int64_t len,
                             const float *gamma, const float *beta, float eps,
                             float *Y) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t o = 0; o < outer; o++) {
    const float *x = X + o * len;
    float *y = Y + o * len;
    double s = 0;
    for (int64_t r = 0; r < len; r++) s += (double)x[r];
    float mean = (float)(s / (double)len);
    double q = 0;
    for (int64_t r = 0; r < len; r++) {
      float d = (float)((double)x[r] - (double)mean);
      float sq = (float)((double)d * (double)d);
      q += (double)sq;
    }
    float var = (float)(q / (double)len);
    float ve = (float)((double)var + (double)eps);
    float sd = (float)sqrt((double)ve);
    for (int64_t r = 0; r < len; r++) {
      float d = (float)((double)x[r] - (double)mean);
      float t = (float)((double)d / (double)sd);
      if (gamma) t = (float)((double)t * (double)gamma[r]);
      if (beta) t = (float)((double)t + (double)beta[r]);
      y[r] = t;
    }
  }
  return REF_OK;
}
