"use strict";
// Unsqueeze: axes as an attribute (opset < 13) or as an input tensor (opset >= 13).
// Contract after src/descriptor_runner/operators/base/unsqueeze.ts:7-47.
const { OperatorImpl } = require("../operatorImpl");
const { getAttrInts } = require("../operatorUtil");
const { withAxes } = require("../shapes");

class Unsqueeze1 extends OperatorImpl {
  initialize(attribute) {
    super.initialize(attribute);
    this.axes = getAttrInts(attribute, "axes", []);
  }

  calcShape(input) {
    return withAxes(input.dims, this.axes);
  }
}

class Unsqueeze13 extends OperatorImpl {
  calcShape(input, axesTensor) {
    return withAxes(input.dims, Array.from(axesTensor.data));
  }
}
module.exports = { Unsqueeze1, Unsqueeze13, unsqueezedShape: withAxes };
