"use strict";
// Gemm attributes (alpha, beta = 1.0; transA, transB = 0) and operand strides.
// Contract after src/descriptor_runner/operators/base/gemm.ts:7-61.
const { OperatorImpl } = require("../operatorImpl");
const { getAttrFloat, getAttrInt } = require("../operatorUtil");
const { gemmPlan } = require("../shapes");

class Gemm extends OperatorImpl {
  initialize(attribute) {
    super.initialize(attribute);
    for (const name of ["alpha", "beta"]) this[name] = getAttrFloat(attribute, name, 1.0);
    for (const name of ["transA", "transB"]) this[name] = getAttrInt(attribute, name, 0);
  }

  // -> {m, n, k, strideA: [row, k], strideB: [k, column]}
  calcShape(dimsA, dimsB) {
    return gemmPlan(dimsA, dimsB, this.transA, this.transB);
  }
}
module.exports = { Gemm };
