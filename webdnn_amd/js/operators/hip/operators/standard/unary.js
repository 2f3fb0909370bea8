"use strict";
// Elementwise unary operators.
// Semantics: src/descriptor_runner/operators/cpu/operators/standard/unary.ts:10-32 and its op table.
const { OperatorImpl } = require("../../../operatorImpl");

class HipUnary extends OperatorImpl {
  constructor(opId, allowDataTypes) {
    super("hip");
    this.opId = opId;
    this.allowDataTypes = allowDataTypes;
  }

  async run(context, inputs) {
    context.assertsHipTensorArray(inputs);
    const input = inputs[0];
    if (!this.allowDataTypes.includes(input.dataType)) {
      throw new Error(`Unary: DataType ${input.dataType} not supported`);
    }
    const output = context.emptyTensor(input.dims, input.dataType);
    context.native.unary(this.opId, input.dataType === "float32" ? 0 : 1, input.handle, output.handle, input.length);
    return [output];
  }
}

function getOpEntries() {
  const f = ["float32"],
    fi = ["float32", "int32"];
  const table = [
    ["Relu", 0, fi], ["Sigmoid", 1, f], ["Sqrt", 2, f], ["Exp", 3, f], ["Tanh", 4, f],
    ["Abs", 5, fi], ["Neg", 6, fi], ["Reciprocal", 7, f],
  ];
  return table.map(([opType, id, types]) => ({
    opType, backend: "hip", opsetMin: 1, factory: () => new HipUnary(id, types),
  }));
}
module.exports = { getOpEntries };
