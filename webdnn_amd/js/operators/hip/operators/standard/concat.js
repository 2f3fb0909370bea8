"use strict";
// Concat: every input is copied into its band of the output with one strided copy.
// Semantics: src/descriptor_runner/operators/cpu/operators/standard/concat.ts:9-84.
const { OperatorImpl } = require("../../../operatorImpl");
const { getAttrInt, calcStrides } = require("../../../operatorUtil");

class HipConcat extends OperatorImpl {
  constructor() {
    super("hip");
  }

  initialize(attribute) {
    super.initialize(attribute);
    this.axis = getAttrInt(attribute, "axis", 0);
  }

  async run(context, inputs) {
    context.assertsHipTensorArray(inputs);
    const first = inputs[0],
      axis = this.axis >= 0 ? this.axis : first.ndim + this.axis;
    if (axis < 0 || axis >= first.ndim) throw new Error(`Concat: axis ${axis} out of range`);
    let axisLength = 0;
    for (const it of inputs) {
      if (it.ndim !== first.ndim || it.dataType !== first.dataType) throw new Error("Concat: inputs differ in rank or type");
      for (let d = 0; d < first.ndim; d++) {
        if (d !== axis && it.dims[d] !== first.dims[d]) throw new Error("Concat: input shapes differ outside the axis");
      }
      axisLength += it.dims[axis];
    }
    const outputShape = first.dims.slice();
    outputShape[axis] = axisLength;
    const output = context.emptyTensor(outputShape, first.dataType),
      outStrides = calcStrides(outputShape);
    let offset = 0;
    for (const it of inputs) {
      if (it.length > 0) {
        context.native.stridedCopy(it.handle, 0, output.handle, offset * outStrides[axis], it.dims, calcStrides(it.dims), outStrides);
      }
      offset += it.dims[axis];
    }
    return [output];
  }
}

function getOpEntries() {
  return [{ opType: "Concat", backend: "hip", opsetMin: 1, factory: () => new HipConcat() }];
}
module.exports = { getOpEntries };
