"use strict";
// GlobalAveragePool (2-D).
// Semantics: src/descriptor_runner/operators/cpu/operators/standard/globalaveragepool.ts:12-41.
const { OperatorImpl } = require("../../../operatorImpl");

class HipGlobalAveragePool extends OperatorImpl {
  constructor() {
    super("hip");
  }

  async run(context, inputs) {
    context.assertsHipTensorArray(inputs);
    const inputX = inputs[0];
    if (inputX.ndim !== 4) throw new Error("GlobalAveragePool other than 2D is not yet supported");
    if (inputX.dataType !== "float32") throw new Error("GlobalAveragePool: only float32 is supported");
    const [batch, ch, h, w] = inputX.dims;
    const output = context.emptyTensor([batch, ch, 1, 1], "float32");
    context.native.globalAvgpool(inputX.handle, output.handle, batch * ch, h * w);
    return [output];
  }
}

function getOpEntries() {
  return [{ opType: "GlobalAveragePool", backend: "hip", opsetMin: 1, factory: () => new HipGlobalAveragePool() }];
}
module.exports = { getOpEntries };
