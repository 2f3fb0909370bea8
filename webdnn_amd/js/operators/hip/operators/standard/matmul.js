"use strict";
// MatMul (result rank 2 or 3, as the CPU operator) and its fused forms.
// Semantics: src/descriptor_runner/operators/cpu/operators/standard/matmul.ts:11-111; the
// absorbed Transposes follow CPUTranspose (transpose.ts:12-168).
const { MatMul } = require("../../../base/matmul");
const { broadcastUni, getAttrFloat, getAttrInt, getAttrInts, getAttrString } = require("../../../operatorUtil");
const { permutedView, denseStrides } = require("../../../shapes");
const { addThenActivate } = require("./conv");

// An operand as the product sees it: dims and element strides.  With a permutation absorbed
// from a Transpose the strides are the tensor's own, permuted, and nothing is copied -- unless
// neither of the last two axes ends up contiguous, which the kernel could only serve one
// element at a time: then the Transpose is carried out after all (temp = its result).
function operandView(context, tensor, perm) {
  if (!perm.length) return { dims: tensor.dims, strides: tensor.strides, temp: null };
  const { outShape, inStrides } = permutedView(tensor.dims, tensor.strides, perm);
  const rank = outShape.length;
  const contiguous = (axis) => outShape[axis] === 1 || inStrides[axis] === 1;
  if (rank >= 2 && (contiguous(rank - 1) || contiguous(rank - 2))) return { dims: outShape, strides: inStrides, temp: null };
  const temp = context.emptyTensor(outShape, tensor.dataType);
  context.native.transpose(tensor.handle, temp.handle, outShape, inStrides);
  return { dims: outShape, strides: temp.strides, temp };
}

class HipMatMul extends MatMul {
  // fused: inputs are (A, B[, bias][, residual]) as announced by the node's attributes
  constructor(fused) {
    super("hip");
    this.fused = !!fused;
    this.hasBias = false;
    this.hasResidual = false;
    this.activation = "";
    this.alpha = 1.0;
    this.permA = [];
    this.permB = [];
    this.permY = [];
  }

  initialize(attribute) {
    super.initialize(attribute);
    if (this.fused) {
      this.hasBias = getAttrInt(attribute, "has_bias", 0) !== 0;
      this.hasResidual = getAttrInt(attribute, "has_residual", 0) !== 0;
      this.activation = getAttrString(attribute, "activation", "");
      if (this.activation !== "" && this.activation !== "Relu") {
        throw new Error(`FusedMatMul: activation ${this.activation} is not supported`);
      }
      this.alpha = getAttrFloat(attribute, "alpha", 1.0);
      this.permA = getAttrInts(attribute, "perm_a", []);
      this.permB = getAttrInts(attribute, "perm_b", []);
      this.permY = getAttrInts(attribute, "perm_y", []);
    }
  }

  async run(context, inputs) {
    context.assertsHipTensorArray(inputs);
    let next = 2;
    const bias = this.hasBias ? inputs[next++] : null;
    const residual = this.hasResidual ? inputs[next++] : null;
    for (const t of inputs) if (t.dataType !== "float32") throw new Error("only float32 is supported");
    const viewA = operandView(context, inputs[0], this.permA),
      viewB = operandView(context, inputs[1], this.permB);
    try {
      return [this.product(context, inputs[0], inputs[1], viewA, viewB, bias, residual)];
    } finally {
      if (viewA.temp) viewA.temp.dispose();
      if (viewB.temp) viewB.temp.dispose();
    }
  }

  product(context, tensorA, tensorB, viewA, viewB, bias, residual, activation = this.activation) {
    const plan = this.calcShape(viewA.dims, viewB.dims);
    const { resultDims, resultDimsAfterSqueeze, innerProductLength } = plan;
    const nd = resultDims.length;
    if (nd !== 2 && nd !== 3) throw new Error("MatMul: result rank >= 4 is not supported");
    if (resultDimsAfterSqueeze.length !== nd && (bias || residual)) {
      // A rank-1 operand: the Adds that were absorbed saw the squeezed result ([m] of a matrix-vector
      // product, not [m, 1]), so their broadcasting is not that of the kernel's C term.  They run as
      // the separate nodes they came from.
      let output = this.product(context, tensorA, tensorB, viewA, viewB, null, null, "");
      if (bias) output = addThenActivate(context, output, bias, residual ? "" : activation);
      if (residual) output = addThenActivate(context, output, residual, activation);
      return output;
    }
    // strides of a permuted view replace the dense ones the plan assumes (same broadcasting rule:
    // a batch axis of extent 1 is re-read)
    const stridesOf = (view, planned) => {
      if (view.dims.length !== nd) return planned; // rank-1 / lower-rank operands are never permuted views
      return view.strides.map((s, axis) => (axis < nd - 2 && view.dims[axis] === 1 ? 0 : s));
    };
    const stridesA = stridesOf(viewA, plan.stridesA),
      stridesB = stridesOf(viewB, plan.stridesB);
    let batch = nd === 3 ? resultDims[0] : 1,
      m = resultDims[nd - 2];
    const n = resultDims[nd - 1];
    let sAb = nd === 3 ? stridesA[0] : 0;
    const sBb = nd === 3 ? stridesB[0] : 0;
    const sA0 = stridesA[nd - 2],
      sA1 = stridesA[nd - 1],
      sB0 = stridesB[nd - 2],
      sB1 = stridesB[nd - 1];
    const mergeHeads = this.permY.length === 3 && nd === 3 && resultDimsAfterSqueeze.length === 3;
    // a batch that only broadcasts B over dense rows of A is one tall GEMM
    if (batch > 1 && sBb === 0 && sAb === m * sA0 && !residual && (!bias || bias.ndim <= 1) && !this.permY.length) {
      m *= batch;
      batch = 1;
      sAb = 0;
    }
    let strideC = [0, 0];
    if (bias) strideC = broadcastUni([m, n], bias.dims);
    // a residual of exactly the result's shape rides in the epilogue; a broadcasting Add is
    // run as the separate nodes it came from
    const sameShape = residual && residual.ndim === resultDimsAfterSqueeze.length &&
      residual.dims.every((d, i) => d === resultDimsAfterSqueeze[i]);
    const inEpilogue = !residual || sameShape;
    const epilogue = inEpilogue && activation === "Relu" ? 1 : 0;
    if (mergeHeads) {
      // [batch, m, n] written as [m, batch, n]: what Transpose(1,0,2) would produce
      const output = context.emptyTensor([m, batch, n], "float32");
      context.native.gemmEx(operandHandle(viewA, tensorA), operandHandle(viewB, tensorB), 0, output.handle, batch, m, n,
        innerProductLength, sAb, sA0, sA1, sBb, sB0, sB1, 0, 0, this.alpha, 1.0, 0, 0, n, batch * n);
      return output;
    }
    let output = context.emptyTensor(resultDimsAfterSqueeze, "float32");
    context.native.gemm(operandHandle(viewA, tensorA), operandHandle(viewB, tensorB), bias ? bias.handle : 0,
      output.handle, batch, m, n, innerProductLength, sAb, sA0, sA1, sBb, sB0, sB1, strideC[0], strideC[1],
      this.alpha, 1.0, epilogue, sameShape ? residual.handle : 0);
    if (!inEpilogue) output = addThenActivate(context, output, residual, activation);
    if (this.permY.length) {
      // a result Transpose that could not be folded into the store (rank other than 3)
      const { outShape, inStrides } = permutedView(output.dims, denseStrides(output.dims), this.permY);
      const moved = context.emptyTensor(outShape, "float32");
      context.native.transpose(output.handle, moved.handle, outShape, inStrides);
      output.dispose();
      output = moved;
    }
    return output;
  }
}

// Several independent linear layers (A [m, k] times a [k, n] weight, plus a bias row, then
// Relu or nothing) as one node: what the hip fusion pass makes of neighbouring MatMul(+Add)
// chains that do not read each other, such as the query, key and value projections of an
// attention block.  Rank-2 operands go to the native grouped call, which puts the small
// products into one launch; anything else runs product by product as the separate nodes would.
class HipLinearGroup extends MatMul {
  constructor() {
    super("hip");
  }

  initialize(attribute) {
    super.initialize(attribute);
    this.arity = getAttrInts(attribute, "arity", []);
    this.activation = getAttrString(attribute, "activation", "");
    if (this.activation !== "" && this.activation !== "Relu") {
      throw new Error(`LinearGroup: activation ${this.activation} is not supported`);
    }
    this.single = new HipMatMul(true);
    this.single.initialize([]);
    this.single.activation = this.activation;
  }

  async run(context, inputs, nOutputs) {
    context.assertsHipTensorArray(inputs);
    const problems = [];
    let next = 0;
    for (const count of this.arity) {
      problems.push({ a: inputs[next], w: inputs[next + 1], bias: count === 3 ? inputs[next + 2] : null });
      next += count;
    }
    if (next !== inputs.length || problems.length !== nOutputs) throw new Error("LinearGroup: malformed node");
    for (const t of inputs) if (t.dataType !== "float32") throw new Error("only float32 is supported");
    const plain = problems.length <= 16 && problems.every(({ a, w, bias }) => a.ndim === 2 && w.ndim === 2 &&
      a.dims[1] === w.dims[0] && (!bias || (bias.ndim === 1 && bias.dims[0] === w.dims[1])));
    if (plain) {
      const outputs = problems.map(({ a, w }) => context.emptyTensor([a.dims[0], w.dims[1]], "float32"));
      context.native.linearGroup(problems.map((p) => p.a.handle), problems.map((p) => p.w.handle),
        problems.map((p) => (p.bias ? p.bias.handle : 0)), outputs.map((o) => o.handle), problems.map((p) => p.a.dims[0]),
        problems.map((p) => p.w.dims[1]), problems.map((p) => p.a.dims[1]), this.activation === "Relu" ? 1 : 0);
      return outputs;
    }
    const outputs = [];
    try {
      for (const { a, w, bias } of problems) {
        outputs.push(this.single.product(context, a, w, operandView(context, a, []), operandView(context, w, []), bias, null));
      }
    } catch (e) {
      for (const o of outputs) o.dispose();
      throw e;
    }
    return outputs;
  }
}

// the buffer an operand is read from: the materialised Transpose if there had to be one
function operandHandle(view, tensor) {
  return view.temp ? view.temp.handle : tensor.handle;
}

function getOpEntries() {
  return [
    { opType: "MatMul", backend: "hip", opsetMin: 1, factory: () => new HipMatMul(false) },
    // produced by the hip fusion pass ([Transpose ->] MatMul [* scalar] [+ bias] [+ residual] [+ Relu | -> Transpose])
    { opType: "WebDNNHipFusedMatMul", backend: "hip", opsetMin: 1, factory: () => new HipMatMul(true) },
    { opType: "WebDNNHipLinearGroup", backend: "hip", opsetMin: 1, factory: () => new HipLinearGroup() },
  ];
}
module.exports = { getOpEntries, HipMatMul, operandView };
