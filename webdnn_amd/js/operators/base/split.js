"use strict";
// Split along one axis: part lengths from the `split` attribute (opset < 13) or input
// tensor (opset >= 13); without them every output gets floor(axisLength / nOutputs).
// Reference: src/descriptor_runner/operators/base/split.ts:7-102.
const { OperatorImpl } = require("../operatorImpl");
const { getAttrInt, getAttrInts } = require("../operatorUtil");

class Split extends OperatorImpl {
  // -> {axis, parts: [{dim, offset, outShape}]}
  calcShapeBase(input, nOutputs, splitSrc) {
    let axis = this.axis;
    if (axis < 0) axis += input.ndim;
    if (axis < 0 || axis >= input.ndim) throw new Error(`Split: axis ${axis} out of range`);
    const axisLength = input.dims[axis],
      split = splitSrc.length > 0 ? splitSrc : Array.from({ length: nOutputs }, () => Math.floor(axisLength / nOutputs));
    const parts = [];
    let offset = 0;
    for (let i = 0; i < nOutputs; i++) {
      const dim = split[i],
        outShape = input.dims.slice();
      if (!(dim >= 0)) throw new Error("Split: fewer part lengths than outputs");
      outShape[axis] = dim;
      parts.push({ dim, offset, outShape });
      offset += dim;
    }
    if (offset > axisLength) throw new Error("Split: parts exceed the axis");
    return { axis, parts };
  }
}

class Split2 extends Split {
  initialize(attribute) {
    super.initialize(attribute);
    this.axis = getAttrInt(attribute, "axis", 0);
    this.split = getAttrInts(attribute, "split", []);
  }

  calcShape(input, nOutputs) {
    return this.calcShapeBase(input, nOutputs, this.split);
  }
}

class Split13 extends Split {
  initialize(attribute) {
    super.initialize(attribute);
    this.axis = getAttrInt(attribute, "axis", 0);
  }

  calcShape(input, nOutputs, splitTensor) {
    return this.calcShapeBase(input, nOutputs, splitTensor ? Array.from(splitTensor.data) : []);
  }
}
module.exports = { Split2, Split13 };
