"use strict";
// Shape: reads only the metadata of its input, so the input may live on any backend and
// the int32 result is a cpu tensor (where Reshape / Slice / Unsqueeze want their
// parameter tensors).  The runner always places this operator on the cpu.
// Reference: src/descriptor_runner/operators/cpu/operators/standard/shape.ts:7-27,
// src/descriptor_runner/core/operatorTable.ts:47-50.
const { OperatorImpl } = require("../../../operatorImpl");

class Shape extends OperatorImpl {
  constructor() {
    super("cpu");
  }

  // eslint-disable-next-line no-unused-vars
  getTensorBackendRequirement(nInputs, nOutputs) {
    return [null];
  }

  async run(context, inputs) {
    const shapeData = new Int32Array(inputs[0].dims);
    return [context.emptyTensor([shapeData.length], "int32", shapeData)];
  }
}

function getOpEntries() {
  return [{ opType: "Shape", backend: "cpu", opsetMin: 1, factory: () => new Shape() }];
}
module.exports = { getOpEntries };
