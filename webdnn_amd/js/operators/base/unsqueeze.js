"use strict";
// Unsqueeze: axes as an attribute (opset < 13) or as an input tensor (opset >= 13);
// negative axes count from the end of the EXPANDED shape.
// Reference: src/descriptor_runner/operators/base/unsqueeze.ts:7-47.
const { OperatorImpl } = require("../operatorImpl");
const { getAttrInts } = require("../operatorUtil");

function unsqueezedShape(inputShape, axes) {
  const expandedNdim = inputShape.length + axes.length,
    nonNegativeAxes = axes.map((a) => (a >= 0 ? a : a + expandedNdim)),
    expandedShape = [];
  let srcIdx = 0;
  for (let d = 0; d < expandedNdim; d++) {
    if (nonNegativeAxes.includes(d)) expandedShape.push(1);
    else expandedShape.push(inputShape[srcIdx++]);
  }
  if (srcIdx !== inputShape.length || expandedShape.some((s) => s === undefined)) {
    throw new Error("Unsqueeze: axes are out of range or repeated");
  }
  return expandedShape;
}

class Unsqueeze1 extends OperatorImpl {
  initialize(attribute) {
    super.initialize(attribute);
    this.axes = getAttrInts(attribute, "axes", []);
  }

  calcShape(input) {
    return unsqueezedShape(input.dims, this.axes);
  }
}

class Unsqueeze13 extends OperatorImpl {
  calcShape(input, axes) {
    return unsqueezedShape(input.dims, Array.from(axes.data));
  }
}
module.exports = { Unsqueeze1, Unsqueeze13, unsqueezedShape };
