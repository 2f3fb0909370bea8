"use strict";
// Conv attributes and geometry.  Contract (property names of calcShape's result) after
// src/descriptor_runner/operators/base/conv.ts:7-79; auto_pad is not read there either.
const { OperatorImpl } = require("../operatorImpl");
const { getAttrInt, getAttrInts } = require("../operatorUtil");
const { convGeometry } = require("../shapes");

const LIST_ATTRS = { dilations: "dilations", kernelShape: "kernel_shape", pads: "pads", strides: "strides" };

class Conv extends OperatorImpl {
  initialize(attribute) {
    super.initialize(attribute);
    for (const [field, onnxName] of Object.entries(LIST_ATTRS)) this[field] = getAttrInts(attribute, onnxName, []);
    this.group = getAttrInt(attribute, "group", 1);
  }

  calcShape(dimsX, dimsW) {
    return convGeometry(dimsX, dimsW, this);
  }
}
module.exports = { Conv };
