"use strict";
// numpy-style batched MatMul.  Contract after src/descriptor_runner/operators/base/matmul.ts:5-91.
const { OperatorImpl } = require("../operatorImpl");
const { matmulPlan } = require("../shapes");

class MatMul extends OperatorImpl {
  calcShape(dimsA, dimsB) {
    return matmulPlan(dimsA, dimsB);
  }
}
module.exports = { MatMul };
