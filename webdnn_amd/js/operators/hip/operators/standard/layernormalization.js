"use strict";
// LayerNormalization (ONNX opset 17) over the last axis.  The reference has no such
// operator; exported graphs carry it either as this node or decomposed into
// ReduceMean/Sub/Pow/Sqrt/Div/Mul/Add, which the other hip operators cover.
const { OperatorImpl } = require("../../../operatorImpl");
const { getAttrFloat, getAttrInt, broadcastMulti } = require("../../../operatorUtil");

class HipLayerNormalization extends OperatorImpl {
  // withAdd: the node pair LayerNormalization -> Add as the hip fusion pass leaves it
  constructor(withAdd) {
    super("hip");
    this.withAdd = !!withAdd;
  }

  initialize(attribute) {
    super.initialize(attribute);
    this.axis = getAttrInt(attribute, "axis", -1);
    this.epsilon = getAttrFloat(attribute, "epsilon", 1e-5);
  }

  async run(context, inputs, nOutputs) {
    context.assertsHipTensorArray(inputs);
    if (this.withAdd) return this.runWithAdd(context, inputs, nOutputs);
    if (nOutputs !== 1) throw new Error("LayerNormalization: Mean / InvStdDev outputs are not supported");
    return [this.normalise(context, inputs, null)];
  }

  // inputs (x, scale, bias, addend) -> (normalised, normalised + addend).  An addend of the input's
  // shape rides in the same launch; a broadcasting one is added by the Add kernel as the separate
  // node would.
  async runWithAdd(context, inputs, nOutputs) {
    if (nOutputs !== 2) throw new Error("LayerNormalization+Add: two outputs expected");
    const x = inputs[0], addend = inputs[3];
    const sameShape = addend.ndim === x.ndim && addend.dims.every((d, i) => d === x.dims[i]);
    if (sameShape) {
      const second = context.emptyTensor(x.dims, "float32");
      const first = this.normalise(context, inputs.slice(0, 3), { addend, second });
      return [first, second];
    }
    const first = this.normalise(context, inputs.slice(0, 3), null);
    const { dims: outShape, allStrides } = broadcastMulti([first.dims, addend.dims]);
    const second = context.emptyTensor(outShape, "float32");
    context.native.binary(0, 0, first.handle, addend.handle, second.handle, outShape, allStrides[0], allStrides[1]);
    return [first, second];
  }

  normalise(context, inputs, add) {
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
    if (add) {
      if (add.addend.dataType !== "float32") throw new Error("LayerNormalization: only float32 is supported");
      context.native.layernormAdd(x.handle, scale ? scale.handle : 0, bias ? bias.handle : 0, output.handle,
        add.addend.handle, add.second.handle, len ? x.length / len : 0, len, this.epsilon);
    } else {
      context.native.layernorm(x.handle, scale ? scale.handle : 0, bias ? bias.handle : 0, output.handle,
        len ? x.length / len : 0, len, this.epsilon);
    }
    return output;
  }
}

function getOpEntries() {
  return [
    { opType: "LayerNormalization", backend: "hip", opsetMin: 17, factory: () => new HipLayerNormalization(false) },
    { opType: "WebDNNHipLayerNormAdd", backend: "hip", opsetMin: 1, factory: () => new HipLayerNormalization(true) },
  ];
}
module.exports = { getOpEntries };
