"use strict";
// Reshape (opset >= 5): data on the device, shape tensor on the cpu; zero-copy alias.
// Reference: src/descriptor_runner/operators/wasm/operators/standard/reshape5.ts:12-18 (placement),
// src/descriptor_runner/operators/base/reshape5.ts:16-75 (shape).
const { Reshape5 } = require("../../../base/reshape5");

class HipReshape5 extends Reshape5 {
  constructor() {
    super("hip");
  }

  // eslint-disable-next-line no-unused-vars
  getTensorBackendRequirement(nInputs, nOutputs) {
    return [this.backend, "cpu"];
  }

  async run(context, inputs) {
    const input = inputs[0],
      shapeTensor = inputs[1];
    context.assertsHipTensor(input);
    context.cpuContext.assertsCPUTensor(shapeTensor);
    const computedShape = this.calcShape(input, shapeTensor);
    let length = 1;
    for (const d of computedShape) length *= d;
    if (length !== input.length) throw new Error("Reshape: element count differs");
    return [input.alias(computedShape)];
  }
}

function getOpEntries() {
  return [{ opType: "Reshape", backend: "hip", opsetMin: 5, factory: () => new HipReshape5() }];
}
module.exports = { getOpEntries };
