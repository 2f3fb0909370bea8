"use strict";
// Reference: src/descriptor_runner/operators/base/gemm.ts:7-61.
const { OperatorImpl } = require("../operatorImpl");
const { getAttrFloat, getAttrInt } = require("../operatorUtil");

class Gemm extends OperatorImpl {
  initialize(attribute) {
    super.initialize(attribute);
    this.alpha = getAttrFloat(attribute, "alpha", 1.0);
    this.beta = getAttrFloat(attribute, "beta", 1.0);
    this.transA = getAttrInt(attribute, "transA", 0);
    this.transB = getAttrInt(attribute, "transB", 0);
  }

  calcShape(dimsA, dimsB) {
    if (dimsA.length !== 2 || dimsB.length !== 2) throw new Error("Gemm: inputs must be 2-D");
    let m, n, k, kcheck, strideA, strideB;
    if (this.transA) {
      k = dimsA[0];
      m = dimsA[1];
      strideA = [1, m];
    } else {
      m = dimsA[0];
      k = dimsA[1];
      strideA = [k, 1];
    }
    if (this.transB) {
      n = dimsB[0];
      kcheck = dimsB[1];
      strideB = [1, kcheck];
    } else {
      kcheck = dimsB[0];
      n = dimsB[1];
      strideB = [n, 1];
    }
    if (k !== kcheck) throw new Error("Gemm: inner dimensions differ");
    return { m, n, k, strideA, strideB };
  }
}
module.exports = { Gemm };
