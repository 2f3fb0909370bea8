"use strict";
// Unsqueeze on the device: a zero-copy alias
// (src/descriptor_runner/operators/cpu/operators/standard/unsqueeze.ts shares the buffer).
const { Unsqueeze1, Unsqueeze13 } = require("../../../base/unsqueeze");

class HipUnsqueeze1 extends Unsqueeze1 {
  constructor() {
    super("hip");
  }

  async run(context, inputs) {
    context.assertsHipTensor(inputs[0]);
    return [inputs[0].alias(this.calcShape(inputs[0]))];
  }
}

class HipUnsqueeze13 extends Unsqueeze13 {
  constructor() {
    super("hip");
  }

  // eslint-disable-next-line no-unused-vars
  getTensorBackendRequirement(nInputs, nOutputs) {
    return [this.backend, "cpu"];
  }

  async run(context, inputs) {
    context.assertsHipTensor(inputs[0]);
    context.cpuContext.assertsCPUTensor(inputs[1]);
    return [inputs[0].alias(this.calcShape(inputs[0], inputs[1]))];
  }
}

function getOpEntries() {
  return [
    { opType: "Unsqueeze", backend: "hip", opsetMin: 13, factory: () => new HipUnsqueeze13() },
    { opType: "Unsqueeze", backend: "hip", opsetMin: 1, opsetMax: 13, factory: () => new HipUnsqueeze1() },
  ];
}
module.exports = { getOpEntries };
