"use strict";
// MatMul (result rank 2 or 3, as the CPU operator) and its fused forms.
// Semantics: src/descriptor_runner/operators/cpu/operators/standard/matmul.ts:11-111.
const { MatMul } = require("../../../base/matmul");
const { broadcastUni, getAttrInt, getAttrString } = require("../../../operatorUtil");
const { addThenActivate } = require("./conv");

class HipMatMul extends MatMul {
  // fused: inputs are (A, B[, bias][, residual]) as announced by the node's attributes
  constructor(fused) {
    super("hip");
    this.fused = !!fused;
    this.hasBias = false;
    this.hasResidual = false;
    this.activation = "";
  }

  initialize(attribute) {
    super.initialize(attribute);
    if (this.fused) {
      this.hasBias = getAttrInt(attribute, "has_bias", 0) !== 0;
      this.hasResidual = getAttrInt(attribute, "has_residual", 0) !== 0;
      this.activation = getAttrString(attribute, "activation", "");
      if (this.activation !== "" && this.activation !== "Relu") {
        throw new Error(`FusedMatMul: activation ${this.activation} is not supported`);
      }
    }
  }

  async run(context, inputs) {
    context.assertsHipTensorArray(inputs);
    const inputA = inputs[0],
      inputB = inputs[1];
    let next = 2;
    const bias = this.hasBias ? inputs[next++] : null;
    const residual = this.hasResidual ? inputs[next++] : null;
    for (const t of inputs) if (t.dataType !== "float32") throw new Error("only float32 is supported");
    const { resultDims, resultDimsAfterSqueeze, stridesA, stridesB, innerProductLength } = this.calcShape(
      inputA.dims,
      inputB.dims
    );
    let batch, m, n, sAb, sBb;
    const nd = resultDims.length;
    if (nd === 2) {
      batch = 1;
      sAb = sBb = 0;
    } else if (nd === 3) {
      batch = resultDims[0];
      sAb = stridesA[0];
      sBb = stridesB[0];
    } else {
      throw new Error("MatMul: result rank >= 4 is not supported");
    }
    m = resultDims[nd - 2];
    n = resultDims[nd - 1];
    const sA0 = stridesA[nd - 2],
      sA1 = stridesA[nd - 1],
      sB0 = stridesB[nd - 2],
      sB1 = stridesB[nd - 1];
    // a batch that only broadcasts B over dense rows of A is one tall GEMM
    if (batch > 1 && sBb === 0 && sAb === m * sA0 && !residual && (!bias || bias.ndim <= 1)) {
      m *= batch;
      batch = 1;
      sAb = 0;
    }
    let strideC = [0, 0];
    if (bias) strideC = broadcastUni([m, n], bias.dims);
    // a residual of exactly the result's shape rides in the epilogue; a broadcasting Add is
    // run as the separate nodes it came from
    const sameShape = residual && residual.ndim === resultDimsAfterSqueeze.length &&
      residual.dims.every((d, i) => d === resultDimsAfterSqueeze[i]);
    const inEpilogue = !residual || sameShape;
    const output = context.emptyTensor(resultDimsAfterSqueeze, "float32");
    context.native.gemm(inputA.handle, inputB.handle, bias ? bias.handle : 0, output.handle, batch, m, n,
      innerProductLength, sAb, sA0, sA1, sBb, sB0, sB1, strideC[0], strideC[1], 1.0, 1.0,
      inEpilogue && this.activation === "Relu" ? 1 : 0, sameShape ? residual.handle : 0);
    if (inEpilogue) return [output];
    return [addThenActivate(context, output, residual, this.activation)];
  }
}

function getOpEntries() {
  return [
    { opType: "MatMul", backend: "hip", opsetMin: 1, factory: () => new HipMatMul(false) },
    // produced by the hip fusion pass (MatMul + Add [+ Relu] / + residual Add)
    { opType: "WebDNNHipFusedMatMul", backend: "hip", opsetMin: 1, factory: () => new HipMatMul(true) },
  ];
}
module.exports = { getOpEntries };
