"use strict";
// Shape logic of Gemm, shared by every backend.
// Semantics: src/descriptor_runner/operators/base/gemm.ts:7-61 — attributes alpha, beta (1.0),
// transA, transB (0); both inputs rank 2; a transposed operand is addressed by swapped strides.
const { OperatorImpl } = require("../operatorImpl");
const { getAttrFloat, getAttrInt } = require("../operatorUtil");

// A rank-2 operand seen as [outer, inner] of the product: its two extents and the element strides
// that walk it in that order.  `swapped` = the stored matrix is [inner, outer].
function asProductOperand(dims, swapped) {
  const [d0, d1] = dims;
  return swapped ? { outer: d1, inner: d0, strides: [1, d1] } : { outer: d0, inner: d1, strides: [d1, 1] };
}

class Gemm extends OperatorImpl {
  initialize(attribute) {
    super.initialize(attribute);
    for (const [name, fallback] of [["alpha", 1.0], ["beta", 1.0]]) this[name] = getAttrFloat(attribute, name, fallback);
    for (const name of ["transA", "transB"]) this[name] = getAttrInt(attribute, name, 0);
  }

  // -> {m, n, k, strideA: [row, k], strideB: [k, column]}
  calcShape(dimsA, dimsB) {
    if (dimsA.length !== 2 || dimsB.length !== 2) throw new Error("Gemm: inputs must be 2-D");
    const a = asProductOperand(dimsA, !!this.transA); // rows x k
    const b = asProductOperand(dimsB, !this.transB); //  columns x k when seen from the result
    if (a.inner !== b.inner) throw new Error("Gemm: inner dimensions differ");
    return { m: a.outer, n: b.outer, k: a.inner, strideA: a.strides, strideB: [b.strides[1], b.strides[0]] };
  }
}
module.exports = { Gemm };
