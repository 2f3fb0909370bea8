"use strict";
// Squeeze on the device: a zero-copy alias, as the CPU operator shares its input buffer
// (src/descriptor_runner/operators/cpu/operators/standard/squeeze.ts:12-37).  The axes
// tensor of opset 13 stays on the cpu.
const { Squeeze1, Squeeze13 } = require("../../../base/squeeze");

class HipSqueeze1 extends Squeeze1 {
  constructor() {
    super("hip");
  }

  async run(context, inputs) {
    context.assertsHipTensor(inputs[0]);
    return [inputs[0].alias(this.calcShape(inputs[0]))];
  }
}

class HipSqueeze13 extends Squeeze13 {
  constructor() {
    super("hip");
  }

  // eslint-disable-next-line no-unused-vars
  getTensorBackendRequirement(nInputs, nOutputs) {
    return nInputs > 1 ? [this.backend, "cpu"] : [this.backend];
  }

  async run(context, inputs) {
    context.assertsHipTensor(inputs[0]);
    if (inputs[1]) context.cpuContext.assertsCPUTensor(inputs[1]);
    return [inputs[0].alias(this.calcShape(inputs[0], inputs[1]))];
  }
}

function getOpEntries() {
  return [
    { opType: "Squeeze", backend: "hip", opsetMin: 13, factory: () => new HipSqueeze13() },
    { opType: "Squeeze", backend: "hip", opsetMin: 1, opsetMax: 13, factory: () => new HipSqueeze1() },
  ];
}
module.exports = { getOpEntries };
