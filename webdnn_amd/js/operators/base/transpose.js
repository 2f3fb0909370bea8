"use strict";
// Reference: src/descriptor_runner/operators/base/transpose.ts:7-35.
const { OperatorImpl } = require("../operatorImpl");
const { getAttrInts } = require("../operatorUtil");

class Transpose extends OperatorImpl {
  initialize(attribute) {
    super.initialize(attribute);
    this.perm = getAttrInts(attribute, "perm", []);
  }

  calcShape(input) {
    // default perm: reversed axes
    const perm = this.perm.length > 0 ? this.perm : Array.from({ length: input.ndim }, (v, i) => input.ndim - 1 - i);
    if (perm.length !== input.ndim) throw new Error("Transpose: perm length differs from rank");
    const outShape = new Array(input.ndim),
      inStrides = new Array(input.ndim);
    for (let outAxis = 0; outAxis < input.ndim; outAxis++) {
      const inAxis = perm[outAxis];
      outShape[outAxis] = input.dims[inAxis];
      inStrides[outAxis] = input.strides[inAxis];
    }
    return { outShape, inStrides };
  }
}
module.exports = { Transpose };
