"use strict";
// Cast between float32 and int32 (ONNX UINT8 / INT32 / INT64 all mean int32 here).
// Semantics: src/descriptor_runner/operators/cpu/operators/standard/cast.ts:12-52.
const { OperatorImpl } = require("../../../operatorImpl");
const { getAttrInt } = require("../../../operatorUtil");
const { DataType } = require("../../../../core/onnxProto");

class HipCast extends OperatorImpl {
  constructor() {
    super("hip");
  }

  initialize(attribute) {
    super.initialize(attribute);
    this.to = getAttrInt(attribute, "to", DataType.FLOAT);
  }

  async run(context, inputs) {
    context.assertsHipTensorArray(inputs);
    const input = inputs[0];
    let outputDataType;
    switch (this.to) {
      case DataType.FLOAT:
        outputDataType = "float32";
        break;
      case DataType.UINT8:
      case DataType.INT32:
      case DataType.INT64:
        outputDataType = "int32";
        break;
      default:
        throw new Error(`Cast: converting to DataType ${this.to} is not yet supported`);
    }
    const output = context.emptyTensor(input.dims, outputDataType);
    context.native.cast(input.dataType === "float32" ? 0 : 1, outputDataType === "float32" ? 0 : 1, input.handle, output.handle, input.length);
    return [output];
  }
}

function getOpEntries() {
  return [{ opType: "Cast", backend: "hip", opsetMin: 6, factory: () => new HipCast() }];
}
module.exports = { getOpEntries };
