"use strict";
// MaxPool (2-D).  Semantics: src/descriptor_runner/operators/cpu/operators/standard/maxpool.ts:12-112.
const { MaxPool } = require("../../../base/maxpool");

class HipMaxPool extends MaxPool {
  constructor() {
    super("hip");
  }

  async run(context, inputs, nOutputs) {
    context.assertsHipTensorArray(inputs);
    const inputX = inputs[0];
    if (nOutputs !== 1) throw new Error("MaxPool: output indices is not yet supported");
    if (inputX.ndim !== 4) throw new Error("MaxPool other than 2D is not yet supported");
    if (inputX.dataType !== "float32") throw new Error("MaxPool: only float32 is supported");
    const s = this.calcShape(inputX.dims);
    if (s.pads[0] < 0 || s.pads[1] < 0) throw new Error("MaxPool: negative padding");
    const output = context.emptyTensor([s.batch, s.ch, s.outShape[0], s.outShape[1]], "float32");
    context.native.maxpool2d(inputX.handle, output.handle, s.batch, s.ch, s.inShape[0], s.inShape[1],
      s.outShape[0], s.outShape[1], s.kernelShape[0], s.kernelShape[1], s.pads[0], s.pads[1],
      s.strides[0], s.strides[1], s.dilations[0], s.dilations[1]);
    return [output];
  }
}

function getOpEntries() {
  return [{ opType: "MaxPool", backend: "hip", opsetMin: 1, factory: () => new HipMaxPool() }];
}
module.exports = { getOpEntries };
