"use strict";
// ReduceMean over the last axis (what decomposed LayerNormalization graphs use).
// Semantics: src/descriptor_runner/operators/cpu/operators/standard/reduce.ts:369-405;
// other axis sets throw, so the runner falls back to the cpu operator for them.
const { OperatorImpl } = require("../../../operatorImpl");
const { getAttrInt, getAttrInts } = require("../../../operatorUtil");

class HipReduceMean extends OperatorImpl {
  constructor() {
    super("hip");
  }

  initialize(attribute) {
    super.initialize(attribute);
    this.axes = getAttrInts(attribute, "axes", []);
    this.keepdims = getAttrInt(attribute, "keepdims", 1) !== 0;
  }

  async run(context, inputs) {
    context.assertsHipTensorArray(inputs);
    const input = inputs[0];
    if (input.dataType !== "float32") throw new Error("ReduceMean: only float32 is supported");
    const axes = this.axes.map((a) => (a < 0 ? a + input.ndim : a));
    if (axes.length !== 1 || axes[0] !== input.ndim - 1) {
      throw new Error("ReduceMean: only a reduction over the last axis is supported on hip");
    }
    const len = input.dims[input.ndim - 1];
    const outDims = input.dims.slice(0, -1);
    if (this.keepdims) outDims.push(1);
    const output = context.emptyTensor(outDims, "float32");
    context.native.reduceMean(input.handle, output.handle, len ? input.length / len : 0, len);
    return [output];
  }
}

function getOpEntries() {
  return [{ opType: "ReduceMean", backend: "hip", opsetMin: 1, opsetMax: 18, factory: () => new HipReduceMean() }];
}
module.exports = { getOpEntries };
