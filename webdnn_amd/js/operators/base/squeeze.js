"use strict";
// Squeeze: axes as an attribute (opset < 13) or as an input tensor (opset >= 13).
// Reference: src/descriptor_runner/operators/base/squeeze.ts:7-43.
const { OperatorImpl } = require("../operatorImpl");
const { getAttrInts } = require("../operatorUtil");

function squeezedShape(inputShape, axes) {
  if (axes.length === 0) return inputShape.filter((s) => s !== 1); // every extent-1 axis goes
  const nonNegativeAxes = axes.map((a) => (a >= 0 ? a : a + inputShape.length));
  return inputShape.filter((_, i) => !nonNegativeAxes.includes(i));
}

class Squeeze1 extends OperatorImpl {
  initialize(attribute) {
    super.initialize(attribute);
    this.axes = getAttrInts(attribute, "axes", []);
  }

  calcShape(input) {
    return squeezedShape(input.dims, this.axes);
  }
}

class Squeeze13 extends OperatorImpl {
  calcShape(input, axes) {
    return squeezedShape(input.dims, axes ? Array.from(axes.data) : []);
  }
}
module.exports = { Squeeze1, Squeeze13, squeezedShape };
