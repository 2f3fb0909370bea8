"use strict";
// Squeeze: axes as an attribute (opset < 13) or as an input tensor (opset >= 13).
// Contract after src/descriptor_runner/operators/base/squeeze.ts:7-43.
const { OperatorImpl } = require("../operatorImpl");
const { getAttrInts } = require("../operatorUtil");
const { withoutAxes } = require("../shapes");

class Squeeze1 extends OperatorImpl {
  initialize(attribute) {
    super.initialize(attribute);
    this.axes = getAttrInts(attribute, "axes", []);
  }

  calcShape(input) {
    return withoutAxes(input.dims, this.axes);
  }
}

class Squeeze13 extends OperatorImpl {
  calcShape(input, axesTensor) {
    return withoutAxes(input.dims, axesTensor ? Array.from(axesTensor.data) : []);
  }
}
module.exports = { Squeeze1, Squeeze13, squeezedShape: withoutAxes };
