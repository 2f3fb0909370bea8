/*
 * webdnn_hip.node — N-API binding of libwebdnn_hip.so for the Node.js host.
 *
 * A 1:1 mapping of include/webdnn_hip.h: numbers in, numbers out, typed arrays
 * for bulk data.  Plain C against node_api.h (N-API is ABI-stable, so the
 * addon built against the Node 12 headers loads in later Node versions).
 *
 * Error convention: a negative status from the C ABI becomes a thrown
 * JavaScript Error carrying wdh_last_error(), so that the runner's per-node
 * error handling (reference: src/descriptor_runner/core/runnerImpl.ts:511-520)
 * sees hip failures like any other operator exception.
 *
 * It stands where the reference's WASM backend has worker.postMessage +
 * src/shader/wasm/pre.js:4-91; here the calls are direct and synchronous on the
 * JavaScript thread (they only enqueue GPU work, except read/sync).
 */
#include <node_api.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "webdnn_hip.h"

#define MAX_ARGS 24

static napi_value throw_last(napi_env env, const char *fn, int rc) {
  char msg[640];
  snprintf(msg, sizeof(msg), "%s failed (%d): %s", fn, rc, wdh_last_error());
  napi_throw_error(env, "WDH_ERROR", msg);
  return NULL;
}

static napi_value throw_arg(napi_env env, const char *fn, const char *what) {
  char msg[256];
  snprintf(msg, sizeof(msg), "%s: %s", fn, what);
  napi_throw_type_error(env, "WDH_BAD_ARGUMENT", msg);
  return NULL;
}

/* Fetches exactly `want` arguments. */
static int get_args(napi_env env, napi_callback_info info, const char *fn, size_t want,
                    napi_value *argv) {
  size_t argc = MAX_ARGS;
  if (napi_get_cb_info(env, info, &argc, argv, NULL, NULL) != napi_ok || argc != want) {
    char what[64];
    snprintf(what, sizeof(what), "expected %zu arguments, got %zu", want, argc);
    throw_arg(env, fn, what);
    return 0;
  }
  return 1;
}

static int to_i64(napi_env env, napi_value v, int64_t *out) {
  double d;
  if (napi_get_value_double(env, v, &d) != napi_ok) return 0;
  if (d != d || d > 9007199254740992.0 || d < -9007199254740992.0) return 0;
  *out = (int64_t)d;
  return (double)*out == d; /* integers only */
}

static int to_f64(napi_env env, napi_value v, double *out) {
  return napi_get_value_double(env, v, out) == napi_ok;
}

/* Any TypedArray / DataView-free view: pointer + byte length. */
static int to_bytes(napi_env env, napi_value v, void **data, size_t *nbytes) {
  bool is_ta = false;
  if (napi_is_typedarray(env, v, &is_ta) != napi_ok || !is_ta) return 0;
  napi_typedarray_type type;
  size_t length, offset;
  napi_value ab;
  if (napi_get_typedarray_info(env, v, &type, &length, data, &ab, &offset) != napi_ok) return 0;
  size_t elem = 1;
  switch (type) {
    case napi_int16_array: case napi_uint16_array: elem = 2; break;
    case napi_int32_array: case napi_uint32_array: case napi_float32_array: elem = 4; break;
    case napi_float64_array: case napi_bigint64_array: case napi_biguint64_array: elem = 8; break;
    default: elem = 1; break;
  }
  *nbytes = length * elem;
  return 1;
}

/* JS array (or typed array) of integers -> C array of at most `cap` entries. */
static int to_i64_list(napi_env env, napi_value v, int64_t *out, int cap, int *n) {
  uint32_t len = 0;
  bool is_arr = false, is_ta = false;
  napi_is_array(env, v, &is_arr);
  napi_is_typedarray(env, v, &is_ta);
  if (!is_arr && !is_ta) return 0;
  napi_value lenv;
  if (napi_get_named_property(env, v, "length", &lenv) != napi_ok) return 0;
  if (napi_get_value_uint32(env, lenv, &len) != napi_ok || (int)len > cap) return 0;
  for (uint32_t i = 0; i < len; i++) {
    napi_value e;
    if (napi_get_element(env, v, i, &e) != napi_ok || !to_i64(env, e, &out[i])) return 0;
  }
  *n = (int)len;
  return 1;
}

static napi_value make_undefined(napi_env env) {
  napi_value u;
  napi_get_undefined(env, &u);
  return u;
}

#define FN(name) static napi_value name(napi_env env, napi_callback_info info)
#define ARGS(fn, n)                                   \
  napi_value argv[MAX_ARGS];                          \
  static const char *const FNAME = fn;                \
  if (!get_args(env, info, FNAME, n, argv)) return NULL
#define I64(i, var)                                                          \
  int64_t var;                                                               \
  if (!to_i64(env, argv[i], &var)) return throw_arg(env, FNAME, "argument " #i " (" #var ") must be an integer")
#define F64(i, var)                                                          \
  double var;                                                                \
  if (!to_f64(env, argv[i], &var)) return throw_arg(env, FNAME, "argument " #i " (" #var ") must be a number")
#define CHECK(rc)                                     \
  do {                                                \
    int rc_ = (rc);                                   \
    if (rc_ < 0) return throw_last(env, FNAME, rc_);  \
  } while (0)

FN(js_init) {
  ARGS("wdh_init", 1);
  I64(0, device);
  CHECK(wdh_init((int)device));
  return make_undefined(env);
}

FN(js_shutdown) {
  (void)info;
  wdh_shutdown();
  return make_undefined(env);
}

FN(js_device_info) {
  ARGS("wdh_device_info", 0);
  char name[64] = "";
  int cu = 0, mhz = 0;
  uint64_t hbm = 0;
  CHECK(wdh_device_info(name, sizeof(name), &cu, &mhz, &hbm));
  napi_value obj, v;
  napi_create_object(env, &obj);
  napi_create_string_utf8(env, name, NAPI_AUTO_LENGTH, &v);
  napi_set_named_property(env, obj, "name", v);
  napi_create_int32(env, cu, &v);
  napi_set_named_property(env, obj, "computeUnits", v);
  napi_create_int32(env, mhz, &v);
  napi_set_named_property(env, obj, "clockMHz", v);
  napi_create_double(env, (double)hbm, &v);
  napi_set_named_property(env, obj, "hbmBytes", v);
  return obj;
}

FN(js_set_option) {
  ARGS("wdh_set_option", 2);
  char name[64];
  size_t len = 0;
  if (napi_get_value_string_utf8(env, argv[0], name, sizeof(name), &len) != napi_ok)
    return throw_arg(env, FNAME, "option name must be a string");
  I64(1, value);
  CHECK(wdh_set_option(name, (int)value));
  return make_undefined(env);
}

FN(js_alloc) {
  ARGS("wdh_alloc", 1);
  I64(0, bytes);
  if (bytes < 0) return throw_arg(env, FNAME, "negative size");
  wdh_buf h = wdh_alloc((size_t)bytes);
  if (h == 0) return throw_last(env, FNAME, WDH_ENOMEM);
  napi_value v;
  napi_create_double(env, (double)h, &v);
  return v;
}

FN(js_free) {
  ARGS("wdh_free", 1);
  I64(0, h);
  CHECK(wdh_free(h));
  return make_undefined(env);
}

FN(js_write) { /* (handle, dstByteOffset, typedArray) */
  ARGS("wdh_write", 3);
  I64(0, h);
  I64(1, offset);
  void *data;
  size_t nbytes;
  if (!to_bytes(env, argv[2], &data, &nbytes)) return throw_arg(env, FNAME, "data must be a TypedArray");
  CHECK(wdh_write(h, (size_t)offset, data, nbytes));
  return make_undefined(env);
}

FN(js_read) { /* (handle, srcByteOffset, typedArray) — fills the array, blocks */
  ARGS("wdh_read", 3);
  I64(0, h);
  I64(1, offset);
  void *data;
  size_t nbytes;
  if (!to_bytes(env, argv[2], &data, &nbytes)) return throw_arg(env, FNAME, "data must be a TypedArray");
  CHECK(wdh_read(h, (size_t)offset, data, nbytes));
  return make_undefined(env);
}

FN(js_copy) {
  ARGS("wdh_copy", 5);
  I64(0, dst); I64(1, doff); I64(2, src); I64(3, soff); I64(4, bytes);
  CHECK(wdh_copy(dst, (size_t)doff, src, (size_t)soff, (size_t)bytes));
  return make_undefined(env);
}

FN(js_sync) {
  ARGS("wdh_sync", 0);
  CHECK(wdh_sync());
  return make_undefined(env);
}

FN(js_set_lane) {
  ARGS("wdh_set_lane", 1);
  I64(0, lane);
  CHECK(wdh_set_lane((int)lane));
  return make_undefined(env);
}

FN(js_branch_begin) {
  ARGS("wdh_branch_begin", 0);
  CHECK(wdh_branch_begin());
  return make_undefined(env);
}

FN(js_branch_end) {
  ARGS("wdh_branch_end", 0);
  CHECK(wdh_branch_end());
  return make_undefined(env);
}

FN(js_branch_join) {
  ARGS("wdh_branch_join", 0);
  CHECK(wdh_branch_join());
  return make_undefined(env);
}

FN(js_mem_stats) {
  ARGS("wdh_mem_stats", 0);
  uint64_t a = 0, b = 0, c = 0;
  CHECK(wdh_mem_stats(&a, &b, &c));
  napi_value obj, v;
  napi_create_object(env, &obj);
  napi_create_double(env, (double)a, &v);
  napi_set_named_property(env, obj, "inUse", v);
  napi_create_double(env, (double)b, &v);
  napi_set_named_property(env, obj, "cached", v);
  napi_create_double(env, (double)c, &v);
  napi_set_named_property(env, obj, "peak", v);
  return obj;
}

FN(js_trim) {
  ARGS("wdh_trim", 1);
  I64(0, keep);
  CHECK(wdh_trim((size_t)keep));
  return make_undefined(env);
}

FN(js_event_record) {
  ARGS("wdh_event_record", 1);
  I64(0, id);
  CHECK(wdh_event_record((int)id));
  return make_undefined(env);
}

FN(js_event_elapsed_ms) {
  ARGS("wdh_event_elapsed_ms", 2);
  I64(0, a); I64(1, b);
  float ms = 0;
  CHECK(wdh_event_elapsed_ms((int)a, (int)b, &ms));
  napi_value v;
  napi_create_double(env, (double)ms, &v);
  return v;
}

FN(js_gemm) {
  ARGS("wdh_gemm", 20);
  I64(0, A); I64(1, B); I64(2, C); I64(3, Y); I64(4, batch); I64(5, m); I64(6, n); I64(7, k);
  I64(8, sAb); I64(9, sA0); I64(10, sA1); I64(11, sBb); I64(12, sB0); I64(13, sB1);
  I64(14, sC0); I64(15, sC1);
  F64(16, alpha); F64(17, beta);
  I64(18, epilogue); I64(19, R);
  CHECK(wdh_gemm(A, B, C, Y, (int)batch, (int)m, (int)n, (int)k, sAb, sA0, sA1, sBb, sB0, sB1, sC0,
                 sC1, (float)alpha, (float)beta, (int)epilogue, R));
  return make_undefined(env);
}

FN(js_gemm_ex) {
  ARGS("wdh_gemm_ex", 22);
  I64(0, A); I64(1, B); I64(2, C); I64(3, Y); I64(4, batch); I64(5, m); I64(6, n); I64(7, k);
  I64(8, sAb); I64(9, sA0); I64(10, sA1); I64(11, sBb); I64(12, sB0); I64(13, sB1);
  I64(14, sC0); I64(15, sC1);
  F64(16, alpha); F64(17, beta);
  I64(18, epilogue); I64(19, R); I64(20, sYb); I64(21, sY0);
  CHECK(wdh_gemm_ex(A, B, C, Y, (int)batch, (int)m, (int)n, (int)k, sAb, sA0, sA1, sBb, sB0, sB1, sC0,
                    sC1, (float)alpha, (float)beta, (int)epilogue, R, sYb, sY0));
  return make_undefined(env);
}

FN(js_linear_group) { /* (A[], W[], Bias[] (0 = none), Y[], m[], n[], k[], epilogue) */
  ARGS("wdh_linear_group", 8);
  int64_t a[16], w[16], b[16], y[16], m64[16], n64[16], k64[16];
  int count = 0, c2 = 0, c3 = 0, c4 = 0, c5 = 0, c6 = 0, c7 = 0;
  if (!to_i64_list(env, argv[0], a, 16, &count) || !to_i64_list(env, argv[1], w, 16, &c2) ||
      !to_i64_list(env, argv[2], b, 16, &c3) || !to_i64_list(env, argv[3], y, 16, &c4) ||
      !to_i64_list(env, argv[4], m64, 16, &c5) || !to_i64_list(env, argv[5], n64, 16, &c6) ||
      !to_i64_list(env, argv[6], k64, 16, &c7) || c2 != count || c3 != count || c4 != count || c5 != count ||
      c6 != count || c7 != count)
    return throw_arg(env, FNAME, "seven integer arrays of one length (<= 16) expected");
  I64(7, epilogue);
  int m[16], n[16], k[16];
  for (int i = 0; i < count; i++) { m[i] = (int)m64[i]; n[i] = (int)n64[i]; k[i] = (int)k64[i]; }
  CHECK(wdh_linear_group(count, a, w, b, y, m, n, k, (int)epilogue));
  return make_undefined(env);
}

FN(js_conv2d) {
  ARGS("wdh_conv2d", 22);
  I64(0, X); I64(1, W); I64(2, Bias); I64(3, Y);
  int64_t g[17];
  for (int i = 0; i < 17; i++)
    if (!to_i64(env, argv[4 + i], &g[i])) return throw_arg(env, FNAME, "geometry arguments must be integers");
  I64(21, R);
  CHECK(wdh_conv2d(X, W, Bias, Y, (int)g[0], (int)g[1], (int)g[2], (int)g[3], (int)g[4], (int)g[5],
                   (int)g[6], (int)g[7], (int)g[8], (int)g[9], (int)g[10], (int)g[11], (int)g[12],
                   (int)g[13], (int)g[14], (int)g[15], (int)g[16], R));
  return make_undefined(env);
}

FN(js_conv2d_ex) {
  ARGS("wdh_conv2d_ex", 23);
  I64(0, X); I64(1, W); I64(2, Bias); I64(3, Y);
  int64_t g[17];
  for (int i = 0; i < 17; i++)
    if (!to_i64(env, argv[4 + i], &g[i])) return throw_arg(env, FNAME, "geometry arguments must be integers");
  I64(21, R); I64(22, flags);
  CHECK(wdh_conv2d_ex(X, W, Bias, Y, (int)g[0], (int)g[1], (int)g[2], (int)g[3], (int)g[4], (int)g[5],
                      (int)g[6], (int)g[7], (int)g[8], (int)g[9], (int)g[10], (int)g[11], (int)g[12],
                      (int)g[13], (int)g[14], (int)g[15], (int)g[16], R, (int)flags));
  return make_undefined(env);
}
FN(js_binary) { /* (op, dtype, L, R, Y, outShape[], stridesL[], stridesR[]) */
  ARGS("wdh_binary", 8);
  I64(0, op); I64(1, dtype); I64(2, L); I64(3, R); I64(4, Y);
  int64_t shape64[8], sl[8], sr[8];
  int nd = 0, n2 = 0, n3 = 0;
  if (!to_i64_list(env, argv[5], shape64, 8, &nd) || !to_i64_list(env, argv[6], sl, 8, &n2) ||
      !to_i64_list(env, argv[7], sr, 8, &n3) || n2 != nd || n3 != nd)
    return throw_arg(env, FNAME, "shape and strides must be integer arrays of equal length (<= 8)");
  int32_t shape[8];
  for (int i = 0; i < nd; i++) shape[i] = (int32_t)shape64[i];
  CHECK(wdh_binary((int)op, (int)dtype, L, R, Y, nd, shape, sl, sr));
  return make_undefined(env);
}

FN(js_unary) {
  ARGS("wdh_unary", 5);
  I64(0, op); I64(1, dtype); I64(2, X); I64(3, Y); I64(4, length);
  CHECK(wdh_unary((int)op, (int)dtype, X, Y, (size_t)length));
  return make_undefined(env);
}

FN(js_softmax) {
  ARGS("wdh_softmax", 4);
  I64(0, X); I64(1, Y); I64(2, outer); I64(3, len);
  CHECK(wdh_softmax(X, Y, outer, (int)len));
  return make_undefined(env);
}

FN(js_layernorm_add) {
  ARGS("wdh_layernorm_add", 9);
  I64(0, X); I64(1, G); I64(2, B); I64(3, Y); I64(4, P); I64(5, Y2); I64(6, outer); I64(7, len);
  F64(8, eps);
  CHECK(wdh_layernorm_add(X, G, B, Y, P, Y2, outer, (int)len, (float)eps));
  return make_undefined(env);
}

FN(js_attention) { /* (Q, K, V, Y, batch, tq, tk, d, sQb, sQi, sKb, sKj, sVb, sVj, sYb, sYi, alpha) */
  ARGS("wdh_attention", 17);
  I64(0, Q); I64(1, K); I64(2, V); I64(3, Y); I64(4, batch); I64(5, tq); I64(6, tk); I64(7, d);
  I64(8, sQb); I64(9, sQi); I64(10, sKb); I64(11, sKj); I64(12, sVb); I64(13, sVj); I64(14, sYb); I64(15, sYi);
  F64(16, alpha);
  CHECK(wdh_attention(Q, K, V, Y, (int)batch, (int)tq, (int)tk, (int)d, sQb, sQi, sKb, sKj, sVb, sVj, sYb, sYi,
                      (float)alpha));
  return make_undefined(env);
}

FN(js_layernorm) {
  ARGS("wdh_layernorm", 7);
  I64(0, X); I64(1, G); I64(2, B); I64(3, Y); I64(4, outer); I64(5, len);
  F64(6, eps);
  CHECK(wdh_layernorm(X, G, B, Y, outer, (int)len, (float)eps));
  return make_undefined(env);
}

FN(js_reduce_mean) {
  ARGS("wdh_reduce_mean", 4);
  I64(0, X); I64(1, Y); I64(2, outer); I64(3, len);
  CHECK(wdh_reduce_mean(X, Y, outer, (int)len));
  return make_undefined(env);
}

FN(js_reduce_axis) {
  ARGS("wdh_reduce_axis", 6);
  I64(0, X); I64(1, Y); I64(2, outer); I64(3, red); I64(4, inner); I64(5, divisor);
  CHECK(wdh_reduce_axis(X, Y, outer, (int)red, inner, divisor));
  return make_undefined(env);
}

FN(js_maxpool2d) {
  ARGS("wdh_maxpool2d", 16);
  I64(0, X); I64(1, Y);
  int64_t g[14];
  for (int i = 0; i < 14; i++)
    if (!to_i64(env, argv[2 + i], &g[i])) return throw_arg(env, FNAME, "geometry arguments must be integers");
  CHECK(wdh_maxpool2d(X, Y, (int)g[0], (int)g[1], (int)g[2], (int)g[3], (int)g[4], (int)g[5], (int)g[6],
                      (int)g[7], (int)g[8], (int)g[9], (int)g[10], (int)g[11], (int)g[12], (int)g[13]));
  return make_undefined(env);
}

FN(js_global_avgpool) {
  ARGS("wdh_global_avgpool", 4);
  I64(0, X); I64(1, Y); I64(2, nc); I64(3, hw);
  CHECK(wdh_global_avgpool(X, Y, nc, (int)hw));
  return make_undefined(env);
}

FN(js_transpose) { /* (X, Y, outShape[], inStrides[]) */
  ARGS("wdh_transpose", 4);
  I64(0, X); I64(1, Y);
  int64_t shape64[8], strides[8];
  int nd = 0, n2 = 0;
  if (!to_i64_list(env, argv[2], shape64, 8, &nd) || !to_i64_list(env, argv[3], strides, 8, &n2) || n2 != nd)
    return throw_arg(env, FNAME, "shape and strides must be integer arrays of equal length (<= 8)");
  int32_t shape[8];
  for (int i = 0; i < nd; i++) shape[i] = (int32_t)shape64[i];
  CHECK(wdh_transpose(X, Y, nd, shape, strides));
  return make_undefined(env);
}

FN(js_gather) {
  ARGS("wdh_gather", 7);
  I64(0, D); I64(1, I); I64(2, Y); I64(3, outer); I64(4, axis_len); I64(5, inner); I64(6, n_idx);
  CHECK(wdh_gather(D, I, Y, outer, (int)axis_len, inner, n_idx));
  return make_undefined(env);
}

FN(js_cast) {
  ARGS("wdh_cast", 5);
  I64(0, from); I64(1, to); I64(2, X); I64(3, Y); I64(4, length);
  CHECK(wdh_cast((int)from, (int)to, X, Y, (size_t)length));
  return make_undefined(env);
}

FN(js_strided_copy) { /* (X, xOffset, Y, yOffset, shape[], xStrides[], yStrides[]) */
  ARGS("wdh_strided_copy", 7);
  I64(0, X); I64(1, xoff); I64(2, Y); I64(3, yoff);
  int64_t shape64[8], sx[8], sy[8];
  int nd = 0, n2 = 0, n3 = 0;
  if (!to_i64_list(env, argv[4], shape64, 8, &nd) || !to_i64_list(env, argv[5], sx, 8, &n2) ||
      !to_i64_list(env, argv[6], sy, 8, &n3) || n2 != nd || n3 != nd)
    return throw_arg(env, FNAME, "shape and strides must be integer arrays of equal length (<= 8)");
  int32_t shape[8];
  for (int i = 0; i < nd; i++) shape[i] = (int32_t)shape64[i];
  CHECK(wdh_strided_copy(X, xoff, Y, yoff, nd, shape, sx, sy));
  return make_undefined(env);
}

FN(js_graph_begin) {
  ARGS("wdh_graph_begin", 0);
  CHECK(wdh_graph_begin());
  return make_undefined(env);
}

FN(js_graph_end) { /* -> graph id */
  ARGS("wdh_graph_end", 0);
  int id = -1;
  CHECK(wdh_graph_end(&id));
  napi_value out;
  if (napi_create_int32(env, id, &out) != napi_ok) return NULL;
  return out;
}

FN(js_graph_launch) {
  ARGS("wdh_graph_launch", 1);
  I64(0, id);
  CHECK(wdh_graph_launch((int)id));
  return make_undefined(env);
}

FN(js_graph_destroy) {
  ARGS("wdh_graph_destroy", 1);
  I64(0, id);
  CHECK(wdh_graph_destroy((int)id));
  return make_undefined(env);
}

static napi_value init_module(napi_env env, napi_value exports) {
  static const struct {
    const char *name;
    napi_callback fn;
  } table[] = {
      {"init", js_init}, {"shutdown", js_shutdown}, {"deviceInfo", js_device_info},
      {"setOption", js_set_option}, {"alloc", js_alloc}, {"free", js_free}, {"write", js_write},
      {"read", js_read}, {"copy", js_copy}, {"sync", js_sync}, {"memStats", js_mem_stats},
      {"trim", js_trim}, {"eventRecord", js_event_record}, {"eventElapsedMs", js_event_elapsed_ms},
      {"gemm", js_gemm}, {"gemmEx", js_gemm_ex}, {"linearGroup", js_linear_group}, {"conv2d", js_conv2d}, {"conv2dEx", js_conv2d_ex}, {"binary", js_binary}, {"unary", js_unary},
      {"softmax", js_softmax}, {"attention", js_attention}, {"layernorm", js_layernorm}, {"layernormAdd", js_layernorm_add}, {"reduceMean", js_reduce_mean}, {"reduceAxis", js_reduce_axis},
      {"maxpool2d", js_maxpool2d}, {"globalAvgpool", js_global_avgpool},
      {"transpose", js_transpose}, {"gather", js_gather}, {"cast", js_cast},
      {"stridedCopy", js_strided_copy}, {"graphBegin", js_graph_begin}, {"graphEnd", js_graph_end},
      {"graphLaunch", js_graph_launch}, {"graphDestroy", js_graph_destroy},
      {"setLane", js_set_lane}, {"branchBegin", js_branch_begin}, {"branchEnd", js_branch_end},
      {"branchJoin", js_branch_join},
  };
  for (size_t i = 0; i < sizeof(table) / sizeof(table[0]); i++) {
    napi_value fn;
    if (napi_create_function(env, table[i].name, NAPI_AUTO_LENGTH, table[i].fn, NULL, &fn) != napi_ok ||
        napi_set_named_property(env, exports, table[i].name, fn) != napi_ok) {
      napi_throw_error(env, NULL, "webdnn_hip: failed to export a function");
      return NULL;
    }
  }
  return exports;
}

NAPI_MODULE(NODE_GYP_MODULE_NAME, init_module)
