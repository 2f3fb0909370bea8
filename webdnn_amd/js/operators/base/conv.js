"use strict";
// Reference: src/descriptor_runner/operators/base/conv.ts:7-79 (auto_pad is not read there either).
const { OperatorImpl } = require("../operatorImpl");
const { getAttrInt, getAttrInts } = require("../operatorUtil");

class Conv extends OperatorImpl {
  initialize(attribute) {
    super.initialize(attribute);
    this.dilations = getAttrInts(attribute, "dilations", []);
    this.group = getAttrInt(attribute, "group", 1);
    this.kernelShape = getAttrInts(attribute, "kernel_shape", []);
    this.pads = getAttrInts(attribute, "pads", []);
    this.strides = getAttrInts(attribute, "strides", []);
  }

  calcShape(dimsX, dimsW) {
    const batch = dimsX[0],
      dilations = this.dilations.length > 0 ? this.dilations : [1, 1],
      group = this.group,
      kernelShape = this.kernelShape.length > 0 ? this.kernelShape : [dimsW[2], dimsW[3]],
      pads = this.pads.length > 0 ? this.pads : [0, 0, 0, 0],
      strides = this.strides.length > 0 ? this.strides : [1, 1],
      inShape = [dimsX[2], dimsX[3]],
      outShape = [0, 1].map(
        (a) => Math.floor((inShape[a] + pads[a] + pads[a + 2] - dilations[a] * (kernelShape[a] - 1) - 1) / strides[a]) + 1
      ),
      chIn = dimsX[1],
      chInPerGroup = chIn / group,
      chOut = dimsW[0],
      chOutPerGroup = chOut / group;
    return { batch, dilations, group, kernelShape, pads, strides, inShape, outShape, chIn, chInPerGroup, chOut, chOutPerGroup };
  }
}
module.exports = { Conv };
