"use strict";
// Constant: the tensor in the `value` attribute becomes a cpu tensor; the runner moves it
// to the device when a device operator consumes it.  This is graph metadata, not
// computation, and the reference offers it on the cpu backend only.
// Reference: src/descriptor_runner/operators/cpu/operators/standard/constant.ts:9-43.
const { OperatorImpl } = require("../../../operatorImpl");
const { getAttrTensor } = require("../../../operatorUtil");

class Constant extends OperatorImpl {
  constructor() {
    super("cpu");
  }

  initialize(attribute) {
    super.initialize(attribute);
    const constant = getAttrTensor(attribute, "value");
    if (!constant) throw new Error("value not exist in Constant"); // value_float etc. of opset 12 are not supported
    this.constant = constant;
  }

  // eslint-disable-next-line no-unused-vars
  async run(context, inputs) {
    const output = context.emptyTensor(this.constant.dims, this.constant.dataType);
    output.data.set(this.constant.data);
    return [output];
  }
}

function getOpEntries() {
  return [{ opType: "Constant", backend: "cpu", opsetMin: 1, factory: () => new Constant() }];
}
module.exports = { getOpEntries };
