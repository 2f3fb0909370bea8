"use strict";
// Conv (2-D) as implicit GEMM, and its fused forms (bias / residual Add / Relu in the epilogue).
// Semantics: src/descriptor_runner/operators/cpu/operators/standard/conv.ts:134-221.
const { Conv } = require("../../../base/conv");
const { getAttrInt, getAttrString, broadcastMulti } = require("../../../operatorUtil");

// y = activation(x + r) with multidirectional broadcasting, as separate kernels; x is consumed.
function addThenActivate(context, x, r, activation) {
  const { dims, allStrides } = broadcastMulti([x.dims, r.dims]);
  let y = context.emptyTensor(dims, "float32");
  context.native.binary(0, 0, x.handle, r.handle, y.handle, dims, allStrides[0], allStrides[1]);
  x.dispose();
  if (activation === "Relu") {
    const z = context.emptyTensor(dims, "float32");
    context.native.unary(0, 0, y.handle, z.handle, y.length);
    y.dispose();
    y = z;
  }
  return y;
}

class HipConv extends Conv {
  constructor(fused) {
    super("hip");
    this.fused = !!fused;
    this.hasBias = null; // null: plain ONNX Conv, bias is inputs[2] when present
    this.hasResidual = false;
    this.activation = "";
  }

  initialize(attribute) {
    super.initialize(attribute);
    if (this.fused) {
      this.hasBias = getAttrInt(attribute, "has_bias", 0) !== 0;
      this.hasResidual = getAttrInt(attribute, "has_residual", 0) !== 0;
      this.activation = getAttrString(attribute, "activation", "");
      if (this.activation !== "" && this.activation !== "Relu") {
        throw new Error(`FusedConv: activation ${this.activation} is not supported`);
      }
    }
  }

  async run(context, inputs) {
    context.assertsHipTensorArray(inputs);
    const inputX = inputs[0],
      inputW = inputs[1];
    let next = 2;
    const hasBias = this.hasBias === null ? inputs.length > 2 : this.hasBias;
    const inputB = hasBias ? inputs[next++] : null;
    const residual = this.hasResidual ? inputs[next++] : null;
    if (inputX.ndim !== 4) throw new Error("Conv other than 2D is not yet supported");
    for (const t of inputs) if (t.dataType !== "float32") throw new Error("Conv: only float32 is supported");
    const s = this.calcShape(inputX.dims, inputW.dims);
    const outDims = [s.batch, s.chOut, s.outShape[0], s.outShape[1]];
    // The epilogue adds a residual of exactly the output's shape; an Add that broadcasts
    // (the fusion pass cannot know shapes) is run as the separate nodes it came from.
    const sameShape = residual && residual.ndim === 4 && residual.dims.every((d, i) => d === outDims[i]);
    const inEpilogue = !residual || sameShape;
    const output = context.emptyTensor(outDims, "float32");
    // flags bit 0: the weights are an initializer's device copy, which nobody writes to while it
    // lives, so the library may keep forms derived from them (transformed filters) across calls
    context.native.conv2dEx(inputX.handle, inputW.handle, inputB ? inputB.handle : 0, output.handle,
      s.batch, s.chIn, s.inShape[0], s.inShape[1], s.chOut, s.kernelShape[0], s.kernelShape[1],
      s.pads[0], s.pads[1], s.pads[2], s.pads[3], s.strides[0], s.strides[1], s.dilations[0], s.dilations[1],
      s.group, inEpilogue && this.activation === "Relu" ? 1 : 0, sameShape ? residual.handle : 0,
      inputW.constant ? 1 : 0);
    if (inEpilogue) return [output];
    return [addThenActivate(context, output, residual, this.activation)];
  }
}

function getOpEntries() {
  return [
    { opType: "Conv", backend: "hip", opsetMin: 1, factory: () => new HipConv(false) },
    // produced by the hip fusion pass (Conv [+ Add residual] [+ Relu])
    { opType: "WebDNNHipFusedConv", backend: "hip", opsetMin: 1, factory: () => new HipConv(true) },
  ];
}
module.exports = { getOpEntries, addThenActivate };
