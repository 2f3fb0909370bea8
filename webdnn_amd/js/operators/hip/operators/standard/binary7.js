"use strict";
// Add / Sub / Mul / Div / Pow with multidirectional broadcasting (opset >= 7).
// Semantics: src/descriptor_runner/operators/cpu/operators/standard/binary7.ts:16-68,257-291.
const { OperatorImpl } = require("../../../operatorImpl");
const { broadcastMulti } = require("../../../operatorUtil");

class HipBinary7 extends OperatorImpl {
  constructor(opId, allowDataTypes) {
    super("hip");
    this.opId = opId;
    this.allowDataTypes = allowDataTypes;
  }

  async run(context, inputs) {
    context.assertsHipTensorArray(inputs);
    const [inputA, inputB] = inputs;
    if (inputA.dataType !== inputB.dataType) {
      throw new Error(`Binary: input dataTypes mismatch: ${inputA.dataType} !== ${inputB.dataType}`);
    }
    if (!this.allowDataTypes.includes(inputA.dataType)) {
      throw new Error(`Binary: input dataType ${inputA.dataType} is not supported`);
    }
    const { dims: outShape, allStrides } = broadcastMulti([inputA.dims, inputB.dims]);
    if (outShape.length > 6) throw new Error(`Binary: input ndim ${outShape.length} > 6 is not supported`);
    const output = context.emptyTensor(outShape, inputA.dataType);
    context.native.binary(this.opId, inputA.dataType === "float32" ? 0 : 1, inputA.handle, inputB.handle,
      output.handle, outShape, allStrides[0], allStrides[1]);
    return [output];
  }
}

function getOpEntries() {
  const both = ["float32", "int32"];
  return [
    { opType: "Add", backend: "hip", opsetMin: 7, factory: () => new HipBinary7(0, both) },
    { opType: "Sub", backend: "hip", opsetMin: 7, factory: () => new HipBinary7(1, both) },
    { opType: "Mul", backend: "hip", opsetMin: 7, factory: () => new HipBinary7(2, both) },
    { opType: "Div", backend: "hip", opsetMin: 7, factory: () => new HipBinary7(3, both) },
    { opType: "Pow", backend: "hip", opsetMin: 7, factory: () => new HipBinary7(4, ["float32"]) },
  ];
}
module.exports = { getOpEntries };
