"use strict";
// Contract after src/descriptor_runner/operators/base/transpose.ts:7-35.
const { OperatorImpl } = require("../operatorImpl");
const { getAttrInts } = require("../operatorUtil");
const { permutedView } = require("../shapes");

class Transpose extends OperatorImpl {
  initialize(attribute) {
    super.initialize(attribute);
    this.perm = getAttrInts(attribute, "perm", []);
  }

  // -> {outShape, inStrides}: the output is the input read through permuted strides
  calcShape(input) {
    return permutedView(input.dims, input.strides, this.perm);
  }
}
module.exports = { Transpose };
