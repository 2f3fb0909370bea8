"use strict";
/*
 * TEST INFRASTRUCTURE — a JavaScript stand-in for the N-API addon (webdnn_hip.node) so
 * that the host side of the hip backend (contexts, tensors, operators, fusion, runner)
 * can be exercised on a machine without a GPU.  It implements the entry points of
 * include/webdnn_hip.h over typed arrays, accumulating in double and rounding where the
 * reference CPU operators round, so a graph run on "hip" through this module must equal
 * the same graph on the cpu path bit for bit.  Never loaded by the product.
 */
const buffers = new Map();
let nextHandle = 1;
let inUse = 0, peak = 0;
const calls = {};
const graphOwned = new Set(); // handles freed while capturing: their memory stays with the graph
const options = {};
let currentLane = 0; // wdh_set_lane: everything here runs at once, so a lane is only remembered

function count(name) {
  calls[name] = (calls[name] || 0) + 1;
}
function buf(h, what) {
  const b = buffers.get(h);
  if (!b) throw new Error(`${what}: unknown buffer handle ${h}`);
  return b;
}
const f32 = (h, what) => new Float32Array(buf(h, what).buffer);
const i32 = (h, what) => new Int32Array(buf(h, what).buffer);
function need(h, bytes, what) {
  if (buf(h, what).byteLength < bytes) throw new Error(`${what}: buffer holds ${buf(h, what).byteLength} bytes, operation needs ${bytes}`);
}
function reluJs(v) {
  return Math.max(v, 0);
}
function toInt32(d) {
  return d | 0; // ToInt32, like a store into an Int32Array
}

function layernormRows(X, G, B, Y, outer, len, eps) {
  const x = f32(X), y = f32(Y), g = G ? f32(G) : null, b = B ? f32(B) : null, t = new Float32Array(4);
  for (let o = 0; o < outer; o++) {
    let s = 0;
    for (let r = 0; r < len; r++) s += x[o * len + r];
    t[0] = s / len; // mean
    let q = 0;
    for (let r = 0; r < len; r++) { t[1] = x[o * len + r] - t[0]; t[2] = t[1] * t[1]; q += t[2]; }
    t[2] = q / len; t[2] = t[2] + Math.fround(eps); t[3] = Math.sqrt(t[2]);
    for (let r = 0; r < len; r++) {
      t[1] = x[o * len + r] - t[0]; t[1] = t[1] / t[3];
      if (g) t[1] = t[1] * g[r];
      if (b) t[1] = t[1] + b[r];
      y[o * len + r] = t[1];
    }
  }
}

const native = {
  init(device) {
    count("init");
    if (device !== 0) throw new Error("wdh_init failed (-1): device out of range");
  },
  shutdown() {},
  deviceInfo() {
    return { name: "fake-gfx950", computeUnits: 256, clockMHz: 2400, hbmBytes: 1 << 30 };
  },
  setOption(name, value) {
    if (name !== "contraction_tile" && name !== "split_k") throw new Error(`wdh_set_option failed (-2): unknown option "${name}"`);
    options[name] = value;
  },
  alloc(bytes) {
    count("alloc");
    const h = nextHandle++;
    buffers.set(h, new Uint8Array(Math.max(bytes, 0)));
    inUse += bytes;
    if (inUse > peak) peak = inUse;
    return h;
  },
  free(h) {
    count("free");
    inUse -= buf(h, "wdh_free").byteLength;
    buffers.delete(h);
  },
  write(h, off, data) {
    count("write");
    const src = new Uint8Array(data.buffer, data.byteOffset, data.byteLength);
    if (off + src.length > buf(h, "wdh_write").byteLength) throw new Error("wdh_write failed (-2): exceeds buffer");
    buf(h).set(src, off);
  },
  read(h, off, data) {
    count("read");
    const dst = new Uint8Array(data.buffer, data.byteOffset, data.byteLength);
    if (off + dst.length > buf(h, "wdh_read").byteLength) throw new Error("wdh_read failed (-2): exceeds buffer");
    dst.set(buf(h).subarray(off, off + dst.length));
  },
  copy(dst, doff, src, soff, bytes) {
    buf(dst).set(buf(src).subarray(soff, soff + bytes), doff);
  },
  sync() {},
  branchBegin() {
    count("branchBegin");
  },
  branchEnd() {
    count("branchEnd");
  },
  branchJoin() {
    count("branchJoin");
  },
  setLane(lane) {
    if (![0, 1, 2, 3].includes(lane)) throw new Error("wdh_set_lane failed (-2): lane " + lane);
    count("setLane");
    currentLane = lane;
  },
  memStats() {
    return { inUse, cached: 0, peak };
  },
  trim() {},
  eventRecord() {},
  eventElapsedMs() {
    return 0;
  },

  gemm(A, B, C, Y, batch, m, n, k, sAb, sA0, sA1, sBb, sB0, sB1, sC0, sC1, alpha, beta, epi, R) {
    native.gemmEx(A, B, C, Y, batch, m, n, k, sAb, sA0, sA1, sBb, sB0, sB1, sC0, sC1, alpha, beta, epi, R, m * n, n);
  },

  gemmEx(A, B, C, Y, batch, m, n, k, sAb, sA0, sA1, sBb, sB0, sB1, sC0, sC1, alpha, beta, epi, R, sYb, sY0) {
    count("gemm");
    need(Y, ((batch - 1) * sYb + (m - 1) * sY0 + n) * 4, "wdh_gemm: Y");
    const a = f32(A, "A"), b = f32(B, "B"), y = f32(Y, "Y");
    const c = C ? f32(C, "C") : null, r = R ? f32(R, "R") : null;
    const out = new Float32Array(1);
    for (let z = 0; z < batch; z++) for (let i = 0; i < m; i++) for (let j = 0; j < n; j++) {
      let sum = 0;
      for (let x = 0; x < k; x++) sum += a[z * sAb + i * sA0 + x * sA1] * b[z * sBb + x * sB0 + j * sB1];
      out[0] = sum; // the device accumulates in fp32: alpha scales an fp32 value
      out[0] = out[0] * alpha;
      if (c) out[0] += c[i * sC0 + j * sC1] * beta;
      const off = z * sYb + i * sY0 + j;
      if (r) out[0] += r[off];
      y[off] = epi === 1 ? reluJs(out[0]) : out[0];
    }
  },

  linearGroup(A, W, Bias, Y, m, n, k, epi) {
    count("linearGroup");
    for (let i = 0; i < A.length; i++) {
      for (let j = 0; j < A.length; j++) {
        if ((j !== i && Y[i] === Y[j]) || Y[i] === A[j] || Y[i] === W[j]) throw new Error("wdh_linear_group failed (-2): result is also an operand");
      }
      native.gemmEx(A[i], W[i], Bias[i], Y[i], 1, m[i], n[i], k[i], 0, k[i], 1, 0, n[i], 1, 0, 1, 1.0, 1.0, epi, 0, m[i] * n[i], n[i]);
      if (--calls.gemm === 0) delete calls.gemm; // counted as one linearGroup call
    }
  },

  // (flags: promises about the operands that let the library keep derived data; nothing to do here)
  conv2dEx(X, W, Bias, Y, n, c, h, w, cout, kh, kw, pt, pl, pb, pr, sh, sw, dh, dw, group, epi, R, flags) {
    if (flags !== 0 && flags !== 1) throw new Error("wdh_conv2d_ex failed (-2): unknown flags");
    return this.conv2d(X, W, Bias, Y, n, c, h, w, cout, kh, kw, pt, pl, pb, pr, sh, sw, dh, dw, group, epi, R);
  },

  conv2d(X, W, Bias, Y, n, c, h, w, cout, kh, kw, pt, pl, pb, pr, sh, sw, dh, dw, group, epi, R) {
    count("conv2d");
    if (c % group || cout % group) throw new Error("wdh_conv2d failed (-2): channels not divisible by group");
    const oh = Math.floor((h + pt + pb - dh * (kh - 1) - 1) / sh) + 1;
    const ow = Math.floor((w + pl + pr - dw * (kw - 1) - 1) / sw) + 1;
    need(Y, n * cout * oh * ow * 4, "wdh_conv2d: Y");
    const x = f32(X), wt = f32(W), y = f32(Y), bias = Bias ? f32(Bias) : null, r = R ? f32(R) : null;
    const cg = c / group, og = cout / group, out = new Float32Array(1);
    for (let b = 0; b < n; b++) for (let co = 0; co < cout; co++) {
      const g = Math.floor(co / og);
      for (let oy = 0; oy < oh; oy++) for (let ox = 0; ox < ow; ox++) {
        let s = 0;
        for (let ci = 0; ci < cg; ci++) for (let ky = 0; ky < kh; ky++) for (let kx = 0; kx < kw; kx++) {
          const iy = oy * sh - pt + ky * dh, ix = ox * sw - pl + kx * dw;
          const v = iy >= 0 && iy < h && ix >= 0 && ix < w ? x[((b * c + g * cg + ci) * h + iy) * w + ix] : 0;
          s += v * wt[((co * cg + ci) * kh + ky) * kw + kx];
        }
        out[0] = s;
        if (bias) out[0] += bias[co];
        const off = ((b * cout + co) * oh + oy) * ow + ox;
        if (r) out[0] += r[off];
        y[off] = epi === 1 ? reluJs(out[0]) : out[0];
      }
    }
  },

  binary(op, dtype, L, R, Y, shape, sl, sr) {
    count("binary");
    const total = shape.reduce((a, b) => a * b, 1);
    need(Y, total * 4, "wdh_binary: Y");
    const view = dtype === 0 ? f32 : i32;
    const l = view(L), r = view(R), y = view(Y);
    const fn = [(a, b) => a + b, (a, b) => a - b, (a, b) => a * b, (a, b) => a / b, (a, b) => a ** b][op];
    if (!fn) throw new Error(`wdh_binary failed (-2): unknown op ${op}`);
    const nd = shape.length, idx = new Array(nd).fill(0);
    let ol = 0, or = 0;
    for (let i = 0; i < total; i++) {
      y[i] = dtype === 0 ? fn(l[ol], r[or]) : toInt32(fn(l[ol], r[or]));
      for (let d = nd - 1; d >= 0; d--) {
        idx[d]++; ol += sl[d]; or += sr[d];
        if (idx[d] < shape[d]) break;
        ol -= sl[d] * shape[d]; or -= sr[d] * shape[d]; idx[d] = 0;
      }
    }
  },

  unary(op, dtype, X, Y, length) {
    count("unary");
    need(Y, length * 4, "wdh_unary: Y");
    const view = dtype === 0 ? f32 : i32, x = view(X), y = view(Y);
    const fn = [reluJs, (v) => (Math.tanh(v / 2) + 1) / 2, Math.sqrt, Math.exp, Math.tanh, Math.abs, (v) => -v, (v) => 1 / v][op];
    if (!fn) throw new Error(`wdh_unary failed (-2): unknown op ${op}`);
    for (let i = 0; i < length; i++) y[i] = fn(x[i]);
  },

  softmax(X, Y, outer, len) {
    count("softmax");
    const x = f32(X), y = f32(Y);
    for (let o = 0; o < outer; o++) {
      let max = -Infinity;
      for (let r = 0; r < len; r++) if (x[o * len + r] > max) max = x[o * len + r];
      let sum = 0;
      for (let r = 0; r < len; r++) { const e = Math.exp(x[o * len + r] - max); y[o * len + r] = e; sum += e; }
      for (let r = 0; r < len; r++) y[o * len + r] /= sum;
    }
  },

  // same limits as the library, so that the operator's choice between the one-launch form and
  // the separate steps is exercised on the CPU tier too
  attention(Q, K, V, Y, batch, tq, tk, d, sQb, sQi, sKb, sKj, sVb, sVj, sYb, sYi, alpha) {
    count("attention");
    if (d !== 32 && d !== 64 && d !== 128) throw new Error(`wdh_attention failed (-2): head dimension ${d}`);
    if (tk > 1024) throw new Error(`wdh_attention failed (-2): ${tk} keys`);
    if ([sQb, sQi, sKb, sKj].some((v) => v % 4 !== 0)) throw new Error("wdh_attention failed (-2): strides of Q and K must be multiples of 4 elements");
    if (batch === 0 || tq === 0) return;
    if (tk === 0) throw new Error("wdh_attention failed (-2): no keys");
    need(Y, ((batch - 1) * sYb + (tq - 1) * sYi + d) * 4, "wdh_attention: Y");
    const q = f32(Q), k = f32(K), v = f32(V), y = f32(Y);
    const s = new Float32Array(tk), out = new Float32Array(1);
    for (let b = 0; b < batch; b++) for (let i = 0; i < tq; i++) {
      let max = -Infinity;
      for (let j = 0; j < tk; j++) {
        let dot = 0;
        for (let x = 0; x < d; x++) dot += q[b * sQb + i * sQi + x] * k[b * sKb + j * sKj + x];
        out[0] = dot;
        s[j] = out[0] * alpha;
        if (s[j] > max) max = s[j];
      }
      let sum = 0;
      for (let j = 0; j < tk; j++) { s[j] = Math.exp(s[j] - max); sum += s[j]; }
      for (let j = 0; j < tk; j++) s[j] /= sum;
      for (let x = 0; x < d; x++) {
        let acc = 0;
        for (let j = 0; j < tk; j++) acc += s[j] * v[b * sVb + j * sVj + x];
        y[b * sYb + i * sYi + x] = acc;
      }
    }
  },

  layernorm(X, G, B, Y, outer, len, eps) {
    count("layernorm");
    layernormRows(X, G, B, Y, outer, len, eps);
  },

  layernormAdd(X, G, B, Y, P, Y2, outer, len, eps) {
    count("layernormAdd");
    layernormRows(X, G, B, Y, outer, len, eps);
    need(Y2, outer * len * 4, "wdh_layernorm_add: Y2");
    const y = f32(Y), p = f32(P), y2 = f32(Y2);
    for (let i = 0; i < outer * len; i++) y2[i] = y[i] + p[i];
  },

  reduceAxis(X, Y, outer, red, inner, divisor) {
    count("reduceAxis");
    const x = f32(X), y = f32(Y);
    for (let o = 0; o < outer; o++) {
      for (let n = 0; n < inner; n++) {
        let s = 0;
        for (let r = 0; r < red; r++) s += x[(o * red + r) * inner + n];
        y[o * inner + n] = s / divisor;
      }
    }
  },

  reduceMean(X, Y, outer, len) {
    count("reduceMean");
    const x = f32(X), y = f32(Y);
    for (let o = 0; o < outer; o++) {
      let s = 0;
      for (let r = 0; r < len; r++) s += x[o * len + r];
      y[o] = s / len;
    }
  },

  maxpool2d(X, Y, n, c, h, w, oh, ow, kh, kw, pt, pl, sh, sw, dh, dw) {
    count("maxpool2d");
    const x = f32(X), y = f32(Y);
    let idx = 0;
    for (let p = 0; p < n * c; p++) for (let oy = 0; oy < oh; oy++) for (let ox = 0; ox < ow; ox++) {
      let mv = -Infinity;
      for (let ky = 0; ky < kh; ky++) for (let kx = 0; kx < kw; kx++) {
        const iy = oy * sh - pt + ky * dh, ix = ox * sw - pl + kx * dw;
        if (iy >= 0 && iy < h && ix >= 0 && ix < w) { const v = x[(p * h + iy) * w + ix]; if (v > mv) mv = v; }
      }
      y[idx++] = mv;
    }
  },

  globalAvgpool(X, Y, nc, hw) {
    count("globalAvgpool");
    native.reduceMean(X, Y, nc, hw);
  },

  transpose(X, Y, shape, strides) {
    count("transpose");
    const x = new Uint32Array(buf(X).buffer), y = new Uint32Array(buf(Y).buffer);
    const total = shape.reduce((a, b) => a * b, 1), nd = shape.length, idx = new Array(nd).fill(0);
    let off = 0;
    for (let i = 0; i < total; i++) {
      y[i] = x[off];
      for (let d = nd - 1; d >= 0; d--) {
        idx[d]++; off += strides[d];
        if (idx[d] < shape[d]) break;
        off -= strides[d] * shape[d]; idx[d] = 0;
      }
    }
  },

  gather(D, I, Y, outer, axisLen, inner, nIdx) {
    count("gather");
    const d = new Uint32Array(buf(D).buffer), ix = i32(I), y = new Uint32Array(buf(Y).buffer);
    let p = 0;
    for (let o = 0; o < outer; o++) for (let j = 0; j < nIdx; j++) {
      let k = ix[j];
      if (k < 0) k += axisLen;
      for (let n = 0; n < inner; n++) y[p++] = d[(o * axisLen + k) * inner + n];
    }
  },

  cast(from, to, X, Y, length) {
    count("cast");
    need(X, length * 4, "wdh_cast: X"); need(Y, length * 4, "wdh_cast: Y");
    const src = from === 0 ? f32(X) : i32(X), dst = to === 0 ? f32(Y) : i32(Y);
    for (let i = 0; i < length; i++) dst[i] = src[i]; // typed-array stores convert like Cast
  },

  stridedCopy(X, xOffset, Y, yOffset, shape, xStrides, yStrides) {
    count("stridedCopy");
    const x = new Uint32Array(buf(X).buffer), y = new Uint32Array(buf(Y).buffer);
    const total = shape.reduce((a, b) => a * b, 1), nd = shape.length, idx = new Array(nd).fill(0);
    for (let n = 0; n < total; n++) {
      let sx = xOffset, sy = yOffset;
      for (let d = 0; d < nd; d++) { sx += idx[d] * xStrides[d]; sy += idx[d] * yStrides[d]; }
      if (sx < 0 || sx >= x.length || sy < 0 || sy >= y.length) throw new Error("wdh_strided_copy failed (-2): view outside the buffer");
      y[sy] = x[sx];
      for (let d = nd - 1; d >= 0; d--) {
        if (++idx[d] < shape[d]) break;
        idx[d] = 0;
      }
    }
  },

  // ---- captured runs: see the wrapper below ----

  // ---- test introspection ----
  __liveBuffers() {
    return buffers.size - graphOwned.size;
  },
  __calls() {
    return Object.assign({}, calls);
  },
  __options() {
    return Object.assign({}, options);
  },
};

// ---- captured runs --------------------------------------------------------------------
// Like the library: between graphBegin and graphEnd compute calls are recorded, not executed;
// alloc/free work, but a buffer freed meanwhile keeps its storage for the graph's lifetime;
// calls that need device data on the host throw and spoil the capture.
const RECORDED = ["copy", "gemm", "gemmEx", "linearGroup", "conv2d", "conv2dEx", "binary", "unary", "softmax", "attention", "layernorm", "layernormAdd", "reduceMean", "reduceAxis", "maxpool2d",
  "globalAvgpool", "transpose", "gather", "cast", "stridedCopy"];
const REFUSED = ["write", "read", "sync", "trim", "eventRecord", "eventElapsedMs"];
const graphs = new Map();
let capture = null, nextGraph = 0;
for (const name of RECORDED) {
  const real = native[name];
  native[name] = function (...args) {
    if (!capture) return real.apply(native, args);
    // arrays are copied: the caller may reuse them
    capture.ops.push([real, args.map((a) => (Array.isArray(a) ? a.slice() : a))]);
    return undefined;
  };
}
for (const name of REFUSED) {
  const real = native[name];
  native[name] = function (...args) {
    if (capture) {
      capture.failed = true;
      throw new Error(`wdh_${name} failed (-5): not possible while a graph is being captured`);
    }
    return real.apply(native, args);
  };
}
const realFree = native.free;
native.free = function (h) {
  if (!capture) return realFree.call(native, h);
  count("free");
  buf(h, "wdh_free");
  capture.freed.push(h);
  graphOwned.add(h);
  return undefined;
};
native.graphBegin = function () {
  count("graphBegin");
  if (capture) throw new Error("wdh_graph_begin failed (-5): a capture is already open");
  capture = { ops: [], freed: [], failed: false };
};
function dropGraphBuffers(g) {
  for (const h of g.freed) {
    graphOwned.delete(h);
    realFree.call(native, h);
  }
}
native.graphEnd = function () {
  if (!capture) throw new Error("wdh_graph_end failed (-5): no capture is open");
  const g = capture;
  capture = null;
  if (g.failed) {
    dropGraphBuffers(g);
    throw new Error("wdh_graph_end failed (-5): the capture was abandoned");
  }
  graphs.set(nextGraph, g);
  return nextGraph++;
};
native.graphLaunch = function (id) {
  count("graphLaunch");
  const g = graphs.get(id);
  if (!g) throw new Error(`wdh_graph_launch failed (-2): unknown graph ${id}`);
  for (const [fn, args] of g.ops) fn.apply(native, args);
};
native.graphDestroy = function (id) {
  const g = graphs.get(id);
  if (!g) throw new Error(`wdh_graph_destroy failed (-2): unknown graph ${id}`);
  graphs.delete(id);
  dropGraphBuffers(g);
};

module.exports = native;
