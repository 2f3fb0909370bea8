"use strict";
// Gather along one axis with an int32 index tensor (negative indices wrap).  The
// reference's CPU operator accepts only the scalar pick from a 1-D tensor
// (src/descriptor_runner/operators/cpu/operators/standard/gather.ts:20-33); that
// case is included.
const { OperatorImpl } = require("../../../operatorImpl");
const { getAttrInt } = require("../../../operatorUtil");
const { arrayProd } = require("../../../../util");

class HipGather extends OperatorImpl {
  constructor() {
    super("hip");
  }

  initialize(attribute) {
    super.initialize(attribute);
    this.axis = getAttrInt(attribute, "axis", 0);
  }

  async run(context, inputs) {
    context.assertsHipTensorArray(inputs);
    const [data, indices] = inputs;
    if (indices.dataType !== "int32") throw new Error("Gather: indices must be int32");
    let axis = this.axis;
    if (axis < 0) axis += data.ndim;
    if (axis < 0 || axis >= data.ndim) throw new Error("Gather: axis out of range");
    const outer = arrayProd(data.dims.slice(0, axis)),
      inner = arrayProd(data.dims.slice(axis + 1)),
      outDims = data.dims.slice(0, axis).concat(indices.dims, data.dims.slice(axis + 1));
    const output = context.emptyTensor(outDims, data.dataType);
    context.native.gather(data.handle, indices.handle, output.handle, outer, data.dims[axis], inner, indices.length);
    return [output];
  }
}

function getOpEntries() {
  return [{ opType: "Gather", backend: "hip", opsetMin: 1, factory: () => new HipGather() }];
}
module.exports = { getOpEntries };
