"use strict";
// numpy-style batched MatMul shapes.  Reference: src/descriptor_runner/operators/base/matmul.ts:5-91.
const { OperatorImpl } = require("../operatorImpl");
const { calcStrides } = require("../operatorUtil");

class MatMul extends OperatorImpl {
  calcShape(dimsA, dimsB) {
    const totalNDims = Math.max(dimsA.length, dimsB.length, 2);
    const expandedDimsA = Array.prototype.slice.call(dimsA);
    if (expandedDimsA.length === 0) throw new Error("MatMul: scalar input");
    if (expandedDimsA.length === 1) expandedDimsA.unshift(1); // (k) -> (1,k)
    while (expandedDimsA.length < totalNDims) expandedDimsA.unshift(1);
    const expandedDimsB = Array.prototype.slice.call(dimsB);
    if (expandedDimsB.length === 0) throw new Error("MatMul: scalar input");
    if (expandedDimsB.length === 1) expandedDimsB.push(1); // (k) -> (k,1)
    while (expandedDimsB.length < totalNDims) expandedDimsB.unshift(1);

    const resultDims = [expandedDimsA[totalNDims - 2], expandedDimsB[totalNDims - 1]];
    const innerProductLength = expandedDimsA[totalNDims - 1];
    if (innerProductLength !== expandedDimsB[totalNDims - 2]) throw new Error("MatMul: inner dimensions differ");
    const stridesA = calcStrides(expandedDimsA),
      stridesB = calcStrides(expandedDimsB);
    for (let i = totalNDims - 3; i >= 0; i--) {
      // a broadcast batch axis is read with stride 0
      if (expandedDimsA[i] === 1) stridesA[i] = 0;
      if (expandedDimsB[i] === 1) stridesB[i] = 0;
      resultDims.unshift(Math.max(expandedDimsA[i], expandedDimsB[i]));
    }
    const resultStrides = calcStrides(resultDims);
    const resultLength = resultDims.reduce((a, b) => a * b, 1);
    const resultDimsAfterSqueeze = resultDims.slice();
    if (dimsA.length === 1) resultDimsAfterSqueeze.splice(resultDimsAfterSqueeze.length - 2, 1);
    if (dimsB.length === 1) resultDimsAfterSqueeze.splice(resultDimsAfterSqueeze.length - 1, 1);
    return { resultLength, resultDims, resultStrides, resultDimsAfterSqueeze, stridesA, stridesB, innerProductLength };
  }
}
module.exports = { MatMul };
