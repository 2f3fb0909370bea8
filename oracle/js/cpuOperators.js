"use strict";
/*
 * TEST INFRASTRUCTURE ONLY — JavaScript restatement of the WebDNN reference CPU
 * operators on the Gemm/MatMul/Conv hot path and the layout glue around it, behind the reference's own
 * Operator / OperatorEntry interface, so that a model can be run with
 * backendOrder ["cpu"] through the same runner and compared with ["hip"].
 *
 * Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py load this
 * file (through tests/js/*.js and bench's Node driver).  The product never registers
 * these entries: hot-path operators exist in webdnn_amd/js only for the hip backend.
 *
 * Every operator follows the reference file named above it: same loops, same
 * accumulator type (JavaScript numbers are doubles), same stores into typed arrays
 * (the rounding points).  Shape logic is written out here and does not use the
 * product's operators/base classes.  This file and oracle/webdnn_cpu_ref.c are
 * two restatements that must agree bit for bit (tests/test_js_oracle.py), except
 * for exp/tanh/pow whose last ulp may differ between V8 and libm ("parity unpinned"
 * below 1e-6 relative for Softmax, Sigmoid, Exp, Tanh, Pow).
 *
 * Paths are relative to src/descriptor_runner/ in the reference.
 */
const path = require("path");
const JS = path.join(__dirname, "..", "..", "webdnn_amd", "js");
const { OperatorImpl } = require(path.join(JS, "operators", "operatorImpl"));
const { getAttrFloat, getAttrInt, getAttrInts, getAttrString } = require(path.join(JS, "operators", "operatorUtil"));

function prod(v) {
  let x = 1;
  for (let i = 0; i < v.length; i++) x *= v[i];
  return x;
}

function strides(dims) {
  const s = [];
  let len = 1;
  for (let i = dims.length - 1; i >= 0; i--) {
    s.unshift(len);
    len *= dims[i];
  }
  return s;
}

// operators/operatorUtil.ts:178-209
function bcastUni(dimsA, dimsB) {
  if (dimsA.length < dimsB.length) throw new Error(`Unidirectional broadcast error: ${dimsA}, ${dimsB}`);
  const eb = dimsB.slice();
  while (eb.length < dimsA.length) eb.unshift(1);
  const sb = strides(eb);
  for (let i = 0; i < dimsA.length; i++) {
    if (dimsA[i] !== eb[i]) {
      if (eb[i] === 1) sb[i] = 0;
      else throw new Error(`Unidirectional broadcast error: ${dimsA}, ${dimsB}`);
    }
  }
  return sb;
}

// operators/operatorUtil.ts:211-245
function bcastMulti(a, b) {
  const nd = Math.max(a.length, b.length);
  const ea = a.slice(),
    eb = b.slice();
  while (ea.length < nd) ea.unshift(1);
  while (eb.length < nd) eb.unshift(1);
  const dims = ea.map((v, i) => Math.max(v, eb[i]));
  const fix = (e) => {
    const s = strides(e);
    for (let i = 0; i < nd; i++) {
      if (e[i] !== dims[i]) {
        if (e[i] === 1) s[i] = 0;
        else throw new Error(`Multidirectional broadcasting error: ${a}, ${b}`);
      }
    }
    return s;
  };
  return { dims, sa: fix(ea), sb: fix(eb) };
}

// ---- Gemm: operators/base/gemm.ts:20-61, operators/cpu/operators/standard/gemm.ts:21-61
class RefGemm extends OperatorImpl {
  constructor() {
    super("cpu");
  }
  initialize(attribute) {
    this.alpha = getAttrFloat(attribute, "alpha", 1.0);
    this.beta = getAttrFloat(attribute, "beta", 1.0);
    this.transA = getAttrInt(attribute, "transA", 0);
    this.transB = getAttrInt(attribute, "transB", 0);
  }
  async run(context, inputs) {
    context.assertsCPUTensorArray(inputs);
    const [A, B, C] = inputs;
    if (A.ndim !== 2 || B.ndim !== 2) throw new Error();
    let m, n, k, kc, a0, a1, b0, b1;
    if (this.transA) { k = A.dims[0]; m = A.dims[1]; a0 = 1; a1 = m; } else { m = A.dims[0]; k = A.dims[1]; a0 = k; a1 = 1; }
    if (this.transB) { n = B.dims[0]; kc = B.dims[1]; b0 = 1; b1 = kc; } else { kc = B.dims[0]; n = B.dims[1]; b0 = n; b1 = 1; }
    if (k !== kc) throw new Error();
    const dA = A.data, dB = B.data, alpha = this.alpha, Y = new Float32Array(m * n);
    for (let i = 0; i < m; i++) {
      for (let j = 0; j < n; j++) {
        let sum = 0;
        for (let x = 0; x < k; x++) sum += dA[i * a0 + x * a1] * dB[x * b0 + j * b1];
        sum *= alpha;
        Y[i * n + j] = sum;
      }
    }
    if (C) {
      const [c0, c1] = bcastUni([m, n], C.dims), dC = C.data, beta = this.beta;
      for (let i = 0; i < m; i++) for (let j = 0; j < n; j++) Y[i * n + j] += dC[i * c0 + j * c1] * beta;
    }
    return [context.emptyTensor([m, n], "float32", Y)];
  }
}

// ---- MatMul: operators/base/matmul.ts:6-91, operators/cpu/operators/standard/matmul.ts:11-111
class RefMatMul extends OperatorImpl {
  constructor() {
    super("cpu");
  }
  async run(context, inputs) {
    context.assertsCPUTensorArray(inputs);
    const [A, B] = inputs;
    if (A.dataType !== "float32" || B.dataType !== "float32") throw new Error("only float32 is supported");
    const total = Math.max(A.ndim, B.ndim, 2);
    const ea = A.dims.slice(), eb = B.dims.slice();
    if (ea.length === 0 || eb.length === 0) throw new Error();
    if (ea.length === 1) ea.unshift(1);
    while (ea.length < total) ea.unshift(1);
    if (eb.length === 1) eb.push(1);
    while (eb.length < total) eb.unshift(1);
    const inner = ea[total - 1];
    if (inner !== eb[total - 2]) throw new Error();
    const sa = strides(ea), sb = strides(eb);
    const rd = [ea[total - 2], eb[total - 1]];
    for (let i = total - 3; i >= 0; i--) {
      if (ea[i] === 1) sa[i] = 0;
      if (eb[i] === 1) sb[i] = 0;
      rd.unshift(Math.max(ea[i], eb[i]));
    }
    const rs = strides(rd);
    const squeezed = rd.slice();
    if (A.ndim === 1) squeezed.splice(squeezed.length - 2, 1);
    if (B.ndim === 1) squeezed.splice(squeezed.length - 1, 1);
    const dA = A.data, dB = B.data, dC = new Float32Array(prod(rd));
    if (rd.length === 2) {
      for (let m = 0; m < rd[0]; m++) for (let n = 0; n < rd[1]; n++) {
        let sum = 0;
        for (let k = 0; k < inner; k++) sum += dA[m * sa[0] + k * sa[1]] * dB[k * sb[0] + n * sb[1]];
        dC[m * rs[0] + n * rs[1]] = sum;
      }
    } else if (rd.length === 3) {
      for (let o = 0; o < rd[0]; o++) for (let m = 0; m < rd[1]; m++) for (let n = 0; n < rd[2]; n++) {
        let sum = 0;
        for (let k = 0; k < inner; k++) sum += dA[o * sa[0] + m * sa[1] + k * sa[2]] * dB[o * sb[0] + k * sb[1] + n * sb[2]];
        dC[o * rs[0] + m * rs[1] + n * rs[2]] = sum;
      }
    } else {
      throw new Error(); // rank >= 4 is not supported (matmul.ts:50-53)
    }
    return [context.emptyTensor(squeezed, "float32", dC)];
  }
}

// ---- Conv: operators/base/conv.ts:22-79, operators/cpu/operators/standard/conv.ts:134-333
// (runSplitBatch :16-132 slices the batch for very large im2col buffers; same arithmetic)
class RefConv extends OperatorImpl {
  constructor() {
    super("cpu");
  }
  initialize(attribute) {
    this.dilations = getAttrInts(attribute, "dilations", []);
    this.group = getAttrInt(attribute, "group", 1);
    this.kernelShape = getAttrInts(attribute, "kernel_shape", []);
    this.pads = getAttrInts(attribute, "pads", []);
    this.strides = getAttrInts(attribute, "strides", []);
  }
  async run(context, inputs) {
    context.assertsCPUTensorArray(inputs);
    const [X, W, Bias] = inputs;
    if (X.ndim !== 4) throw new Error("Conv other than 2D is not yet supported");
    const batch = X.dims[0], group = this.group;
    const dil = this.dilations.length > 0 ? this.dilations : [1, 1];
    const ks = this.kernelShape.length > 0 ? this.kernelShape : [W.dims[2], W.dims[3]];
    const pads = this.pads.length > 0 ? this.pads : [0, 0, 0, 0];
    const str = this.strides.length > 0 ? this.strides : [1, 1];
    const inS = [X.dims[2], X.dims[3]];
    const outS = [0, 1].map((a) => Math.floor((inS[a] + pads[a] + pads[a + 2] - dil[a] * (ks[a] - 1) - 1) / str[a]) + 1);
    const chIn = X.dims[1], chInG = chIn / group, chOut = W.dims[0], chOutG = chOut / group;
    const bout = batch * outS[0] * outS[1], ckk = chInG * ks[0] * ks[1], area = outS[0] * outS[1];
    const dX = X.data, dW = W.data;
    const dI = new Float32Array(group * bout * ckk);
    const dT = new Float32Array(group * bout * chOutG);
    const dO = new Float32Array(batch * chOut * area);
    // im2col :223-270
    let idx = 0;
    for (let g = 0; g < group; g++) for (let b = 0; b < batch; b++)
      for (let oy = 0; oy < outS[0]; oy++) for (let ox = 0; ox < outS[1]; ox++)
        for (let ci = 0; ci < chInG; ci++) for (let ky = 0; ky < ks[0]; ky++) for (let kx = 0; kx < ks[1]; kx++) {
          let v = 0;
          const iny = oy * str[0] - pads[0] + ky * dil[0], inx = ox * str[1] - pads[1] + kx * dil[1];
          if (iny >= 0 && iny < inS[0] && inx >= 0 && inx < inS[1]) {
            v = dX[((b * chIn + g * chInG + ci) * inS[0] + iny) * inS[1] + inx];
          }
          dI[idx++] = v;
        }
    // matmul :272-295
    for (let g = 0; g < group; g++) for (let y = 0; y < bout; y++) for (let x = 0; x < chOutG; x++) {
      let s = 0;
      for (let ip = 0; ip < ckk; ip++) s += dI[(g * bout + y) * ckk + ip] * dW[(g * chOutG + x) * ckk + ip];
      dT[(g * bout + y) * chOutG + x] = s;
    }
    // transpose :297-316
    idx = 0;
    for (let b = 0; b < batch; b++) for (let g = 0; g < group; g++) for (let c = 0; c < chOutG; c++)
      for (let x = 0; x < area; x++) dO[idx++] = dT[((g * batch + b) * area + x) * chOutG + c];
    // bias :318-333
    if (Bias) {
      const dB = Bias.data;
      idx = 0;
      for (let b = 0; b < batch; b++) for (let c = 0; c < chOut; c++) for (let x = 0; x < area; x++) dO[idx++] += dB[c];
    }
    return [context.emptyTensor([batch, chOut, outS[0], outS[1]], "float32", dO)];
  }
}

// ---- Binary7: operators/cpu/operators/standard/binary7.ts:16-68 (op0d..op6d :70-254 as one index walk)
class RefBinary7 extends OperatorImpl {
  constructor(op, allow) {
    super("cpu");
    this.op = op;
    this.allow = allow;
  }
  async run(context, inputs) {
    context.assertsCPUTensorArray(inputs);
    const [A, B] = inputs;
    if (A.dataType !== B.dataType) throw new Error(`Binary: input dataTypes mismatch: ${A.dataType} !== ${B.dataType}`);
    if (!this.allow.includes(A.dataType)) throw new Error(`Binary: input dataType ${A.dataType} is not supported`);
    const { dims, sa, sb } = bcastMulti(A.dims, B.dims);
    if (dims.length > 6) throw new Error(`Binary: input ndim ${dims.length} > 4 is not yet supported`);
    const out = context.emptyTensor(dims, A.dataType);
    const dA = A.data, dB = B.data, dO = out.data, op = this.op, nd = dims.length, total = prod(dims);
    const idx = new Array(nd).fill(0);
    let oa = 0, ob = 0;
    for (let i = 0; i < total; i++) {
      dO[i] = op(dA[oa], dB[ob]);
      for (let d = nd - 1; d >= 0; d--) {
        idx[d]++;
        oa += sa[d];
        ob += sb[d];
        if (idx[d] < dims[d]) break;
        oa -= sa[d] * dims[d];
        ob -= sb[d] * dims[d];
        idx[d] = 0;
      }
    }
    return [out];
  }
}

// ---- CPUUnary: operators/cpu/operators/standard/unary.ts:10-32 and its op table
class RefUnary extends OperatorImpl {
  constructor(op, allow) {
    super("cpu");
    this.op = op;
    this.allow = allow;
  }
  async run(context, inputs) {
    context.assertsCPUTensorArray(inputs);
    const input = inputs[0];
    if (!this.allow.includes(input.dataType)) throw new Error(`Unary: DataType ${input.dataType} not supported`);
    const out = new input.data.constructor(input.data.length), op = this.op;
    for (let i = 0; i < out.length; i++) out[i] = op(input.data[i]);
    return [context.emptyTensor(input.dims, input.dataType, out)];
  }
}

// ---- Softmax: operators/cpu/operators/standard/softmax.ts:13-59
class RefSoftmax extends OperatorImpl {
  constructor() {
    super("cpu");
  }
  initialize(attribute) {
    this.axis = getAttrInt(attribute, "axis", -1);
  }
  async run(context, inputs) {
    context.assertsCPUTensorArray(inputs);
    const input = inputs[0];
    let axis = this.axis;
    if (axis < 0) axis += input.ndim;
    if (axis !== input.ndim - 1) throw new Error("Softmax: currently only reducing final axis is supported");
    const red = input.dims[axis], outer = input.length / red;
    const output = context.emptyTensor(input.dims, input.dataType), dI = input.data, dO = output.data;
    for (let o = 0; o < outer; o++) {
      let max = -Infinity;
      for (let r = 0; r < red; r++) {
        const v = dI[o * red + r];
        if (v > max) max = v;
      }
      let expsum = 0;
      for (let r = 0; r < red; r++) {
        const e = Math.exp(dI[o * red + r] - max);
        dO[o * red + r] = e;
        expsum += e;
      }
      for (let r = 0; r < red; r++) dO[o * red + r] /= expsum;
    }
    return [output];
  }
}

// ---- MaxPool: operators/base/maxpool.ts:18-137, operators/cpu/operators/standard/maxpool.ts:12-112
class RefMaxPool extends OperatorImpl {
  constructor() {
    super("cpu");
  }
  initialize(attribute) {
    this.autoPad = getAttrString(attribute, "auto_pad", "NOTSET");
    this.ceilMode = getAttrInt(attribute, "ceil_mode", 0) !== 0;
    this.dilations = getAttrInts(attribute, "dilations", []);
    this.kernelShape = getAttrInts(attribute, "kernel_shape", []);
    this.pads = getAttrInts(attribute, "pads", []);
    this.strides = getAttrInts(attribute, "strides", []);
    if (getAttrInt(attribute, "storage_order", 0) !== 0) throw new Error("MaxPool: storage_order !== 0 is not supported.");
  }
  async run(context, inputs, nOutputs) {
    context.assertsCPUTensorArray(inputs);
    const X = inputs[0];
    if (nOutputs !== 1) throw new Error("MaxPool: output indices is not yet supported");
    if (X.ndim !== 4) throw new Error("MaxPool other than 2D is not yet supported");
    const [batch, ch] = X.dims, inS = [X.dims[2], X.dims[3]];
    const dil = this.dilations.length > 0 ? this.dilations : [1, 1];
    const str = this.strides.length > 0 ? this.strides : [1, 1];
    const ks = this.kernelShape;
    let outS, pads;
    if (this.autoPad === "NOTSET") {
      pads = this.pads.length > 0 ? this.pads : [0, 0, 0, 0];
      const rnd = this.ceilMode ? Math.ceil : Math.floor;
      outS = [0, 1].map((a) => rnd((inS[a] + pads[a] + pads[a + 2] - dil[a] * (ks[a] - 1) - 1) / str[a]) + 1);
    } else if (this.autoPad === "SAME_UPPER" || this.autoPad === "SAME_LOWER") {
      outS = [0, 1].map((a) => Math.ceil(inS[a] / str[a]));
      const sum = [0, 1].map((a) => (outS[a] - 1) * str[a] + ((ks[a] - 1) * dil[a] + 1) - inS[a]);
      const lo = sum.map((s) => Math.floor(s / 2)), hi = sum.map((s) => Math.ceil(s / 2));
      pads = this.autoPad === "SAME_UPPER" ? [lo[0], lo[1], hi[0], hi[1]] : [hi[0], hi[1], lo[0], lo[1]];
    } else if (this.autoPad === "VALID") {
      outS = [0, 1].map((a) => Math.ceil((inS[a] - dil[a] * (ks[a] - 1)) / str[a]));
      pads = [0, 0, 0, 0];
    } else {
      throw new Error(`Unknown auto_pad ${this.autoPad} for MaxPool`);
    }
    const dX = X.data, dO = new Float32Array(batch * ch * outS[0] * outS[1]);
    let idx = 0;
    for (let b = 0; b < batch; b++) for (let c = 0; c < ch; c++)
      for (let oy = 0; oy < outS[0]; oy++) for (let ox = 0; ox < outS[1]; ox++) {
        let mv = -Infinity;
        for (let ky = 0; ky < ks[0]; ky++) for (let kx = 0; kx < ks[1]; kx++) {
          const iny = oy * str[0] - pads[0] + ky * dil[0], inx = ox * str[1] - pads[1] + kx * dil[1];
          if (iny >= 0 && iny < inS[0] && inx >= 0 && inx < inS[1]) {
            const v = dX[((b * ch + c) * inS[0] + iny) * inS[1] + inx];
            if (v > mv) mv = v;
          }
        }
        dO[idx++] = mv;
      }
    return [context.emptyTensor([batch, ch, outS[0], outS[1]], "float32", dO)];
  }
}

// ---- GlobalAveragePool: operators/cpu/operators/standard/globalaveragepool.ts:12-41 +
//      operators/cpu/rawcomputation/averagepool.ts:1-46 (kernel = input, countIncludePad)
class RefGlobalAveragePool extends OperatorImpl {
  constructor() {
    super("cpu");
  }
  async run(context, inputs) {
    context.assertsCPUTensorArray(inputs);
    const X = inputs[0];
    if (X.ndim !== 4) throw new Error("MaxPool other than 2D is not yet supported");
    const [batch, ch, h, w] = X.dims, dX = X.data, dO = new Float32Array(batch * ch);
    for (let bc = 0; bc < batch * ch; bc++) {
      let sum = 0;
      for (let ky = 0; ky < h; ky++) for (let kx = 0; kx < w; kx++) sum += dX[(bc * h + ky) * w + kx];
      dO[bc] = sum / (h * w);
    }
    return [context.emptyTensor([batch, ch, 1, 1], "float32", dO)];
  }
}

// ---- Transpose: operators/base/transpose.ts:10-35, operators/cpu/operators/standard/transpose.ts:12-168
class RefTranspose extends OperatorImpl {
  constructor() {
    super("cpu");
  }
  initialize(attribute) {
    this.perm = getAttrInts(attribute, "perm", []);
  }
  async run(context, inputs) {
    context.assertsCPUTensorArray(inputs);
    const input = inputs[0], nd = input.ndim;
    const perm = this.perm.length > 0 ? this.perm : Array.from({ length: nd }, (v, i) => nd - 1 - i);
    if (perm.length !== nd) throw new Error();
    if (nd < 1 || nd > 6) throw new Error(`Transpose: ndim ${nd} > 4 is not yet supported`);
    const outShape = perm.map((p) => input.dims[p]), inStrides = perm.map((p) => input.strides[p]);
    const output = context.emptyTensor(outShape, input.dataType), dI = input.data, dO = output.data;
    const idx = new Array(nd).fill(0), total = prod(outShape);
    let off = 0;
    for (let i = 0; i < total; i++) {
      dO[i] = dI[off];
      for (let d = nd - 1; d >= 0; d--) {
        idx[d]++;
        off += inStrides[d];
        if (idx[d] < outShape[d]) break;
        off -= inStrides[d] * outShape[d];
        idx[d] = 0;
      }
    }
    return [output];
  }
}

// ---- Flatten: operators/base/flatten.ts:7-17, operators/cpu/operators/standard/flatten.ts:11-20
class RefFlatten extends OperatorImpl {
  constructor() {
    super("cpu");
  }
  initialize(attribute) {
    if (getAttrInt(attribute, "axis", 1) !== 1) throw new Error("Flatten: only axis === 1 is supported");
  }
  async run(context, inputs) {
    context.assertsCPUTensorArray(inputs);
    const input = inputs[0];
    return [context.emptyTensor([input.dims[0], prod(input.dims.slice(1))], input.dataType, input.data)];
  }
}

// ---- Reshape: operators/base/reshape5.ts:16-75, operators/cpu/operators/standard/reshape5.ts:8-28
class RefReshape5 extends OperatorImpl {
  constructor() {
    super("cpu");
  }
  initialize(attribute) {
    this.allowzero = getAttrInt(attribute, "allowzero", 0) !== 0;
  }
  getTensorBackendRequirement() {
    return ["cpu", "cpu"];
  }
  async run(context, inputs) {
    context.assertsCPUTensorArray(inputs);
    const [input, shapeTensor] = inputs;
    const shapeInput = Array.from(shapeTensor.data);
    let explicitProd = 1, minusDim = -1;
    shapeInput.forEach((s, i) => {
      if (s > 0) explicitProd *= s;
      else if (s === 0 && !this.allowzero) explicitProd *= input.dims[i];
      else if (s === -1) {
        if (minusDim >= 0) throw new Error("Reshape: multiple -1 dimensions");
        minusDim = i;
      } else if (s < 0 && !this.allowzero) throw new Error();
    });
    if (minusDim >= 0 && explicitProd <= 0) throw new Error();
    const minusDimValue = input.length / explicitProd;
    const shape = shapeInput.map((s, i) => (s > 0 ? s : s === 0 ? (this.allowzero ? 0 : input.dims[i]) : minusDimValue));
    return [context.emptyTensor(shape, input.dataType, input.data)];
  }
}

// ---- Gather: operators/cpu/operators/standard/gather.ts:8-34
class RefGather extends OperatorImpl {
  constructor() {
    super("cpu");
  }
  initialize(attribute) {
    this.axis = getAttrInt(attribute, "axis", 0);
  }
  async run(context, inputs) {
    context.assertsCPUTensorArray(inputs);
    const [data, indices] = inputs;
    if (!(data.ndim === 1 && indices.ndim === 0 && this.axis === 0)) {
      throw new Error("Gather: currently supports data.ndim === 1 && indices.ndim === 0 && axis === 0");
    }
    const output = context.emptyTensor([], data.dataType);
    output.data[0] = data.data[indices.data[0]];
    return [output];
  }
}

// ---- ReduceMean: operators/cpu/operators/standard/reduce.ts:14-140 (runCore, axis by axis) and :369-405
class RefReduceMean extends OperatorImpl {
  constructor() {
    super("cpu");
  }
  initialize(attribute) {
    this.axes = getAttrInts(attribute, "axes", []);
    this.keepdims = getAttrInt(attribute, "keepdims", 1) !== 0;
  }
  async run(context, inputs) {
    context.assertsCPUTensorArray(inputs);
    const input = inputs[0];
    let axes = this.axes.map((a) => (a < 0 ? a + input.ndim : a));
    if (axes.length === 0) axes = input.dims.map((v, i) => i);
    axes.sort((a, b) => a - b);
    let data = input.data, shape = input.dims.slice(), totalRed = 1;
    for (let i = 0; i < axes.length; i++) {
      const axis = axes[i], red = shape[axis];
      totalRed *= red;
      const outer = prod(shape.slice(0, axis)), inner = prod(shape.slice(axis + 1));
      const out = new Float32Array(outer * inner), last = i === axes.length - 1;
      for (let o = 0; o < outer; o++) for (let n = 0; n < inner; n++) {
        let s = 0;
        for (let r = 0; r < red; r++) s += data[(o * red + r) * inner + n];
        out[o * inner + n] = last ? s / totalRed : s;
      }
      shape[axis] = 1;
      data = out;
    }
    const outShape = this.keepdims ? shape : shape.filter((v, i) => !axes.includes(i));
    return [context.emptyTensor(outShape, "float32", data)];
  }
}

// ---- Squeeze / Unsqueeze: operators/base/squeeze.ts:7-43, base/unsqueeze.ts:7-47; the cpu
// operators share the input buffer (cpu/operators/standard/squeeze.ts:12-37, unsqueeze.ts)
class RefSqueeze extends OperatorImpl {
  constructor(axesFromInput) {
    super("cpu");
    this.axesFromInput = axesFromInput;
  }
  initialize(attribute) {
    this.axes = this.axesFromInput ? null : getAttrInts(attribute, "axes", []);
  }
  async run(context, inputs) {
    context.assertsCPUTensorArray(inputs);
    const input = inputs[0];
    const axes = this.axesFromInput ? (inputs[1] ? Array.from(inputs[1].data) : []) : this.axes;
    let shape;
    if (axes.length === 0) shape = input.dims.filter((s) => s !== 1);
    else {
      const nn = axes.map((a) => (a >= 0 ? a : a + input.dims.length));
      shape = input.dims.filter((_, i) => !nn.includes(i));
    }
    return [context.emptyTensor(shape, input.dataType, input.data)];
  }
}

class RefUnsqueeze extends OperatorImpl {
  constructor(axesFromInput) {
    super("cpu");
    this.axesFromInput = axesFromInput;
  }
  initialize(attribute) {
    this.axes = this.axesFromInput ? null : getAttrInts(attribute, "axes", []);
  }
  async run(context, inputs) {
    context.assertsCPUTensorArray(inputs);
    const input = inputs[0];
    const axes = this.axesFromInput ? Array.from(inputs[1].data) : this.axes;
    const nd = input.dims.length + axes.length, nn = axes.map((a) => (a >= 0 ? a : a + nd)), shape = [];
    let src = 0;
    for (let d = 0; d < nd; d++) shape.push(nn.includes(d) ? 1 : input.dims[src++]);
    return [context.emptyTensor(shape, input.dataType, input.data)];
  }
}

// ---- Concat: operators/cpu/operators/standard/concat.ts:9-84
class RefConcat extends OperatorImpl {
  constructor() {
    super("cpu");
  }
  initialize(attribute) {
    this.axis = getAttrInt(attribute, "axis", 0);
  }
  async run(context, inputs) {
    context.assertsCPUTensorArray(inputs);
    const axis = this.axis >= 0 ? this.axis : inputs[0].ndim + this.axis;
    if (axis < 0 || axis >= inputs[0].ndim) throw new Error(`Concat: axis ${axis} out of range`);
    let axisLength = 0;
    const parts = [];
    for (const it of inputs) {
      const st = strides(it.dims);
      parts.push([it, axisLength, it.dims[axis], st[Math.max(axis - 1, 0)], st[axis]]);
      axisLength += it.dims[axis];
    }
    const outShape = inputs[0].dims.slice();
    outShape[axis] = axisLength;
    const outerLength = prod(inputs[0].dims.slice(0, axis)), innerLength = prod(inputs[0].dims.slice(axis + 1));
    const output = context.emptyTensor(outShape, inputs[0].dataType), so = strides(outShape);
    const outOuter = so[Math.max(axis - 1, 0)], outCat = so[axis];
    for (const [it, off, dim, outerS, catS] of parts) {
      for (let c = 0; c < dim; c++) for (let o = 0; o < outerLength; o++) for (let i = 0; i < innerLength; i++) {
        output.data[(c + off) * outCat + o * outOuter + i] = it.data[c * catS + o * outerS + i];
      }
    }
    return [output];
  }
}

// ---- Split: operators/base/split.ts:7-102, operators/cpu/operators/standard/split.ts:7-87
class RefSplit extends OperatorImpl {
  constructor(splitFromInput) {
    super("cpu");
    this.splitFromInput = splitFromInput;
  }
  initialize(attribute) {
    this.axis = getAttrInt(attribute, "axis", 0);
    this.split = this.splitFromInput ? null : getAttrInts(attribute, "split", []);
  }
  async run(context, inputs, nOutputs) {
    context.assertsCPUTensorArray(inputs);
    const input = inputs[0];
    const splitSrc = this.splitFromInput ? (inputs[1] ? Array.from(inputs[1].data) : []) : this.split;
    let axis = this.axis;
    if (axis < 0) axis += input.ndim;
    if (axis < 0 || axis >= input.ndim) throw new Error(`Split: axis ${axis} out of range`);
    const axisLength = input.dims[axis];
    const split = splitSrc.length > 0 ? splitSrc : Array.from({ length: nOutputs }, () => Math.floor(axisLength / nOutputs));
    const outerLength = prod(input.dims.slice(0, axis)), innerLength = prod(input.dims.slice(axis + 1));
    const si = strides(input.dims), inOuter = si[Math.max(axis - 1, 0)], inCat = si[axis];
    const outputs = [];
    let offset = 0;
    for (let n = 0; n < nOutputs; n++) {
      const dim = split[n], outShape = input.dims.slice();
      outShape[axis] = dim;
      const outerS = prod(outShape.slice(Math.max(axis - 1, 0) + 1)), splitS = prod(outShape.slice(axis + 1));
      const ot = context.emptyTensor(outShape, input.dataType);
      for (let c = 0; c < dim; c++) for (let o = 0; o < outerLength; o++) for (let i = 0; i < innerLength; i++) {
        ot.data[c * splitS + o * outerS + i] = input.data[(c + offset) * inCat + o * inOuter + i];
      }
      outputs.push(ot);
      offset += dim;
    }
    return outputs;
  }
}

// ---- Slice (opset >= 10): operators/cpu/operators/standard/slice.ts:12-330; copy1d..copy6d
// are one loop nest here
class RefSlice10 extends OperatorImpl {
  constructor() {
    super("cpu");
  }
  async run(context, inputs) {
    context.assertsCPUTensorArray(inputs);
    const [data, starts, ends, axesTensor, stepsTensor] = inputs;
    if (data.ndim > 6) throw new Error(`Slice: input dimension ${data.ndim} > 6 is not yet supported`);
    const axes = axesTensor ? Array.from(axesTensor.data).map((a) => (a < 0 ? a + data.ndim : a)) : data.dims.map((_, i) => i);
    const steps = stepsTensor ? Array.from(stepsTensor.data) : axes.map(() => 1);
    const ranges = data.dims.map((d) => [0, d, 1, d]);
    for (let i = 0; i < axes.length; i++) ranges[axes[i]] = [starts.data[i], ends.data[i], steps[i], data.dims[axes[i]]];
    const rws = ranges.map(([start, stop, step, srcsize]) => {
      if (start < 0) start += srcsize;
      start = Math.max(Math.min(start, srcsize - 1), 0);
      if (stop < 0) stop += srcsize;
      stop = Math.max(Math.min(stop, srcsize), -1);
      return [start, stop, step, srcsize, Math.max(Math.ceil((stop - start) / step), 0)];
    });
    const outShape = rws.map((r) => r[4]), output = context.emptyTensor(outShape, data.dataType);
    const ss = strides(data.dims), ds = strides(outShape), nd = data.ndim, idx = new Array(nd).fill(0);
    const total = prod(outShape);
    for (let n = 0; n < total; n++) {
      let src = 0, dst = 0;
      for (let d = 0; d < nd; d++) {
        src += (rws[d][0] + idx[d] * rws[d][2]) * ss[d];
        dst += idx[d] * ds[d];
      }
      output.data[dst] = data.data[src];
      for (let d = nd - 1; d >= 0; d--) {
        if (++idx[d] < outShape[d]) break;
        idx[d] = 0;
      }
    }
    return [output];
  }
}

// ---- Cast: operators/cpu/operators/standard/cast.ts:12-52 (typed-array `set` does the conversion)
class RefCast extends OperatorImpl {
  constructor() {
    super("cpu");
  }
  initialize(attribute) {
    this.to = getAttrInt(attribute, "to", 1);
  }
  async run(context, inputs) {
    context.assertsCPUTensorArray(inputs);
    const input = inputs[0];
    let dt;
    if (this.to === 1) dt = "float32";
    else if (this.to === 2 || this.to === 6 || this.to === 7) dt = "int32";
    else throw new Error(`Cast: converting to DataType ${this.to} is not yet supported`);
    const newData = dt === "float32" ? new Float32Array(input.data.length) : new Int32Array(input.data.length);
    newData.set(input.data);
    return [context.emptyTensor(input.dims, dt, newData)];
  }
}

function getOpEntries() {
  const fi = ["float32", "int32"], f = ["float32"];
  const e = (opType, opsetMin, factory) => ({ opType, backend: "cpu", opsetMin, factory });
  return [
    e("Gemm", 1, () => new RefGemm()),
    e("MatMul", 1, () => new RefMatMul()),
    e("Conv", 1, () => new RefConv()),
    e("Add", 7, () => new RefBinary7((l, r) => l + r, fi)),
    e("Sub", 7, () => new RefBinary7((l, r) => l - r, fi)),
    e("Mul", 7, () => new RefBinary7((l, r) => l * r, fi)),
    e("Div", 7, () => new RefBinary7((l, r) => l / r, fi)),
    e("Pow", 7, () => new RefBinary7((l, r) => l ** r, fi)),
    e("Relu", 1, () => new RefUnary((v) => Math.max(v, 0), fi)),
    e("Sigmoid", 1, () => new RefUnary((v) => (Math.tanh(v / 2) + 1) / 2, f)),
    e("Sqrt", 1, () => new RefUnary((v) => Math.sqrt(v), f)),
    e("Exp", 1, () => new RefUnary((v) => Math.exp(v), f)),
    e("Tanh", 1, () => new RefUnary((v) => Math.tanh(v), f)),
    e("Abs", 1, () => new RefUnary((v) => Math.abs(v), fi)),
    e("Neg", 1, () => new RefUnary((v) => -v, fi)),
    e("Reciprocal", 1, () => new RefUnary((v) => 1 / v, f)),
    e("Softmax", 1, () => new RefSoftmax()),
    e("MaxPool", 1, () => new RefMaxPool()),
    e("GlobalAveragePool", 1, () => new RefGlobalAveragePool()),
    e("Transpose", 1, () => new RefTranspose()),
    e("Flatten", 1, () => new RefFlatten()),
    e("Reshape", 5, () => new RefReshape5()),
    e("Gather", 1, () => new RefGather()),
    e("ReduceMean", 1, () => new RefReduceMean()),
    { opType: "Squeeze", backend: "cpu", opsetMin: 13, factory: () => new RefSqueeze(true) },
    { opType: "Squeeze", backend: "cpu", opsetMin: 1, opsetMax: 13, factory: () => new RefSqueeze(false) },
    { opType: "Unsqueeze", backend: "cpu", opsetMin: 13, factory: () => new RefUnsqueeze(true) },
    { opType: "Unsqueeze", backend: "cpu", opsetMin: 1, opsetMax: 13, factory: () => new RefUnsqueeze(false) },
    e("Concat", 1, () => new RefConcat()),
    { opType: "Split", backend: "cpu", opsetMin: 13, factory: () => new RefSplit(true) },
    { opType: "Split", backend: "cpu", opsetMin: 1, opsetMax: 13, factory: () => new RefSplit(false) },
    e("Slice", 10, () => new RefSlice10()),
    e("Cast", 6, () => new RefCast()),
  ];
}

module.exports = { getOpEntries };
