"use strict";
// Operator entries for the tests of the runner's per-node cpu retry (core/runnerImpl.ts:511-520
// in the reference): the oracle's cpu operators plus a made-up operator "TestFlaky" whose hip
// implementation always throws (after allocating a tensor, as a real operator would have) and
// whose cpu implementation doubles its input.
const path = require("path");
const oracle = require(path.join(__dirname, "..", "..", "oracle", "js", "cpuOperators"));

class FlakyOnHip {
  constructor() {
    this.backend = "hip";
  }
  initialize() {}
  getTensorBackendRequirement(nInputs) {
    return new Array(nInputs).fill("hip");
  }
  async run(context, inputs) {
    context.emptyTensor(inputs[0].dims, "float32");
    throw new Error("TestFlaky: the hip implementation refuses");
  }
}

class FlakyOnCpu {
  constructor() {
    this.backend = "cpu";
  }
  initialize() {}
  getTensorBackendRequirement(nInputs) {
    return new Array(nInputs).fill("cpu");
  }
  async run(context, inputs) {
    const out = context.emptyTensor(inputs[0].dims, "float32");
    for (let i = 0; i < out.length; i++) out.data[i] = 2 * inputs[0].data[i];
    return [out];
  }
}

function getOpEntries() {
  return oracle.getOpEntries().concat([
    { opType: "TestFlaky", backend: "hip", opsetMin: 1, factory: () => new FlakyOnHip() },
    { opType: "TestFlaky", backend: "cpu", opsetMin: 1, factory: () => new FlakyOnCpu() },
  ]);
}
module.exports = { getOpEntries };
