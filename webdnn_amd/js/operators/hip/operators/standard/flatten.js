"use strict";
// Flatten: a second view of the same device buffer (the CPU operator shares the typed
// array the same way: src/descriptor_runner/operators/cpu/operators/standard/flatten.ts:11-20;
// alias precedent: src/descriptor_runner/operators/webgl/operators/standard/flatten.ts:16).
const { Flatten } = require("../../../base/flatten");

class HipFlatten extends Flatten {
  constructor() {
    super("hip");
  }

  async run(context, inputs) {
    context.assertsHipTensorArray(inputs);
    const input = inputs[0];
    return [input.alias(this.calcShape(input))];
  }
}

function getOpEntries() {
  return [{ opType: "Flatten", backend: "hip", opsetMin: 1, factory: () => new HipFlatten() }];
}
module.exports = { getOpEntries };
