"use strict";
// Gemm on the hip backend: shape logic of the shared base class, arithmetic in wdh_gemm.
// Semantics: src/descriptor_runner/operators/cpu/operators/standard/gemm.ts:21-61.
const { Gemm } = require("../../../base/gemm");
const { broadcastUni } = require("../../../operatorUtil");

class HipGemm extends Gemm {
  constructor() {
    super("hip");
  }

  async run(context, inputs) {
    context.assertsHipTensorArray(inputs);
    const [inputA, inputB, inputC] = inputs;
    for (const t of inputs) if (t.dataType !== "float32") throw new Error("Gemm: only float32 is supported");
    const { m, n, k, strideA, strideB } = this.calcShape(inputA.dims, inputB.dims);
    let strideC = [0, 0];
    if (inputC) strideC = broadcastUni([m, n], inputC.dims);
    const output = context.emptyTensor([m, n], "float32");
    context.native.gemm(inputA.handle, inputB.handle, inputC ? inputC.handle : 0, output.handle, 1, m, n, k,
      0, strideA[0], strideA[1], 0, strideB[0], strideB[1], strideC[0], strideC[1], this.alpha, this.beta, 0, 0);
    return [output];
  }
}

function getOpEntries() {
  return [{ opType: "Gemm", backend: "hip", opsetMin: 1, factory: () => new HipGemm() }];
}
module.exports = { getOpEntries };
