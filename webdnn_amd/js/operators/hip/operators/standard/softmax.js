"use strict";
// Softmax over the last axis.
// Semantics: src/descriptor_runner/operators/cpu/operators/standard/softmax.ts:13-59
// (axis defaults to -1 for every opset there; other axes throw).
const { OperatorImpl } = require("../../../operatorImpl");
const { getAttrInt } = require("../../../operatorUtil");

class HipSoftmax extends OperatorImpl {
  constructor() {
    super("hip");
  }

  initialize(attribute) {
    super.initialize(attribute);
    this.axis = getAttrInt(attribute, "axis", -1);
  }

  async run(context, inputs) {
    context.assertsHipTensorArray(inputs);
    const input = inputs[0];
    if (input.dataType !== "float32") throw new Error("Softmax: only float32 is supported");
    let axis = this.axis;
    if (axis < 0) axis += input.ndim;
    if (axis !== input.ndim - 1) throw new Error("Softmax: currently only reducing final axis is supported");
    const reductionLength = input.dims[axis],
      outerLength = reductionLength ? input.length / reductionLength : 0,
      output = context.emptyTensor(input.dims, input.dataType);
    context.native.softmax(input.handle, output.handle, outerLength, reductionLength);
    return [output];
  }
}

function getOpEntries() {
  return [{ opType: "Softmax", backend: "hip", opsetMin: 1, factory: () => new HipSoftmax() }];
}
module.exports = { getOpEntries };
