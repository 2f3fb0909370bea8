"use strict";
// Split along one axis: part lengths from the `split` attribute (opset < 13) or input tensor
// (opset >= 13).  Contract after src/descriptor_runner/operators/base/split.ts:7-102.
const { OperatorImpl } = require("../operatorImpl");
const { getAttrInt, getAttrInts } = require("../operatorUtil");
const { splitBands } = require("../shapes");

class Split2 extends OperatorImpl {
  initialize(attribute) {
    super.initialize(attribute);
    this.axis = getAttrInt(attribute, "axis", 0);
    this.split = getAttrInts(attribute, "split", []);
  }

  // -> {axis, parts: [{dim, offset, outShape}]}
  calcShape(input, nOutputs) {
    return splitBands(input.dims, this.axis, nOutputs, this.split);
  }
}

class Split13 extends OperatorImpl {
  initialize(attribute) {
    super.initialize(attribute);
    this.axis = getAttrInt(attribute, "axis", 0);
  }

  calcShape(input, nOutputs, lengthsTensor) {
    return splitBands(input.dims, this.axis, nOutputs, lengthsTensor ? Array.from(lengthsTensor.data) : []);
  }
}
module.exports = { Split2, Split13 };
