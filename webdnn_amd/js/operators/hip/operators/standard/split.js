"use strict";
// Split: one strided copy per output.
// Semantics: src/descriptor_runner/operators/cpu/operators/standard/split.ts:7-87.
const { Split2, Split13 } = require("../../../base/split");
const { calcStrides } = require("../../../operatorUtil");

function runSplit(context, input, axis, parts) {
  const inStrides = calcStrides(input.dims),
    outputs = [];
  for (const { offset, outShape } of parts) {
    const ot = context.emptyTensor(outShape, input.dataType);
    if (ot.length > 0) {
      context.native.stridedCopy(input.handle, offset * inStrides[axis], ot.handle, 0, outShape, inStrides, calcStrides(outShape));
    }
    outputs.push(ot);
  }
  return outputs;
}

class HipSplit2 extends Split2 {
  constructor() {
    super("hip");
  }

  async run(context, inputs, nOutputs) {
    context.assertsHipTensor(inputs[0]);
    const { axis, parts } = this.calcShape(inputs[0], nOutputs);
    return runSplit(context, inputs[0], axis, parts);
  }
}

class HipSplit13 extends Split13 {
  constructor() {
    super("hip");
  }

  // eslint-disable-next-line no-unused-vars
  getTensorBackendRequirement(nInputs, nOutputs) {
    return nInputs > 1 ? [this.backend, "cpu"] : [this.backend];
  }

  async run(context, inputs, nOutputs) {
    context.assertsHipTensor(inputs[0]);
    if (inputs[1]) context.cpuContext.assertsCPUTensor(inputs[1]);
    const { axis, parts } = this.calcShape(inputs[0], nOutputs, inputs[1]);
    return runSplit(context, inputs[0], axis, parts);
  }
}

function getOpEntries() {
  return [
    { opType: "Split", backend: "hip", opsetMin: 13, factory: () => new HipSplit13() },
    { opType: "Split", backend: "hip", opsetMin: 1, opsetMax: 13, factory: () => new HipSplit2() },
  ];
}
module.exports = { getOpEntries };
