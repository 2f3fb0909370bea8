"use strict";
// LayerNormalization (ONNX opset 17) over the last axis.  The reference has no such
// operator; exported graphs carry it either as this node or decomposed into
// ReduceMean/Sub/Pow/Sqrt/Div/Mul/Add, which the other hip operators cover.
const { OperatorImpl } = require("../../../operatorImpl");
const { getAttrFloat, getAttrInt } = require("../../../operatorUtil");

class HipLayerNormalization extends OperatorImpl {
  constructor() {
    super("hip");
  }

  initialize(attribute) {
    super.initialize(attribute);
    this.axis = getAttrInt(attribute, "axis", -1);
    this.epsilon = getAttrFloat(attribute, "epsilon", 1e-5);
  }

  async run(context, inputs, nOutputs) {
    context.assertsHipTensorArray(inputs);
    if (nOutputs !== 1) throw new Error("LayerNormalization: Mean / InvStdDev outputs are not supported");
    const [x, scale, bias] = inputs;
    for (const t of inputs) if (t.dataType !== "float32") throw new Error("LayerNormalization: only float32 is supported");
    let axis = this.axis;
    if (axis < 0) axis += x.ndim;
    if (axis !== x.ndim - 1) throw new Error("LayerNormalization: only the last axis is supported");
    const len = x.dims[axis];
    for (const t of [scale, bias]) {
      if (t && t.length !== len) throw new Error("LayerNormalization: scale/bias must have the normalised length");
    }
    const output = context.emptyTensor(x.dims, "float32");
    context.native.layernorm(x.handle, scale ? scale.handle : 0, bias ? bias.handle : 0, output.handle,
      len ? x.length / len : 0, len, this.epsilon);
    return [output];
  }
}

function getOpEntries() {
  return [{ opType: "LayerNormalization", backend: "hip", opsetMin: 17, factory: () => new HipLayerNormalization() }];
}
module.exports = { getOpEntries };
