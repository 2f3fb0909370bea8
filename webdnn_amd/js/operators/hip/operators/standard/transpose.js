"use strict";
// Transpose (rank 1..6, any 4-byte type).
// Semantics: src/descriptor_runner/operators/cpu/operators/standard/transpose.ts:12-168.
const { Transpose } = require("../../../base/transpose");

class HipTranspose extends Transpose {
  constructor() {
    super("hip");
  }

  async run(context, inputs) {
    context.assertsHipTensorArray(inputs);
    const input = inputs[0];
    if (input.ndim < 1 || input.ndim > 6) throw new Error(`Transpose: ndim ${input.ndim} is not supported`);
    const { outShape, inStrides } = this.calcShape(input);
    const output = context.emptyTensor(outShape, input.dataType);
    context.native.transpose(input.handle, output.handle, outShape, inStrides);
    return [output];
  }
}

function getOpEntries() {
  return [{ opType: "Transpose", backend: "hip", opsetMin: 1, factory: () => new HipTranspose() }];
}
module.exports = { getOpEntries };
