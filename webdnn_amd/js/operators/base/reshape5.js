"use strict";
// Reshape, opset >= 5 (shape is an input tensor).
// Reference: src/descriptor_runner/operators/base/reshape5.ts:8-75.
const { OperatorImpl } = require("../operatorImpl");
const { getAttrInt } = require("../operatorUtil");

class Reshape5 extends OperatorImpl {
  initialize(attribute) {
    super.initialize(attribute);
    this.allowzero = getAttrInt(attribute, "allowzero", 0) !== 0;
  }

  calcShape(input, shapeTensor) {
    const shapeInput = Array.from(shapeTensor.data);
    let explicitProd = 1,
      minusDim = -1;
    shapeInput.forEach((s, i) => {
      if (s > 0) {
        explicitProd *= s;
      } else if (s === 0 && !this.allowzero) {
        explicitProd *= input.dims[i];
      } else if (s === -1) {
        if (minusDim >= 0) throw new Error("Reshape: multiple -1 dimensions");
        minusDim = i;
      } else if (s < 0 && !this.allowzero) {
        throw new Error("Reshape: negative dimension");
      }
    });
    if (minusDim >= 0 && explicitProd <= 0) throw new Error("Reshape: cannot infer -1");
    const minusDimValue = input.length / explicitProd;
    return shapeInput.map((s, i) => {
      if (s > 0) return s;
      if (s === 0) return this.allowzero ? 0 : input.dims[i];
      return minusDimValue;
    });
  }
}
module.exports = { Reshape5 };
