"use strict";
// Reference: src/descriptor_runner/operators/base/maxpool.ts:6-137.
const { OperatorImpl } = require("../operatorImpl");
const { getAttrInt, getAttrInts, getAttrString } = require("../operatorUtil");

class MaxPool extends OperatorImpl {
  initialize(attribute) {
    super.initialize(attribute);
    this.autoPad = getAttrString(attribute, "auto_pad", "NOTSET");
    this.ceilMode = getAttrInt(attribute, "ceil_mode", 0) !== 0;
    this.dilations = getAttrInts(attribute, "dilations", []);
    this.kernelShape = getAttrInts(attribute, "kernel_shape", []);
    this.pads = getAttrInts(attribute, "pads", []);
    this.strides = getAttrInts(attribute, "strides", []);
    const storageOrder = getAttrInt(attribute, "storage_order", 0);
    if (storageOrder !== 0) throw new Error("MaxPool: storage_order !== 0 is not supported.");
  }

  calcShape(dimsX) {
    const batch = dimsX[0],
      dilations = this.dilations.length > 0 ? this.dilations : [1, 1],
      kernelShape = this.kernelShape,
      strides = this.strides.length > 0 ? this.strides : [1, 1],
      inShape = [dimsX[2], dimsX[3]];
    let outShape, pads;
    if (this.autoPad === "NOTSET") {
      pads = this.pads.length > 0 ? this.pads : [0, 0, 0, 0];
      const round = this.ceilMode ? Math.ceil : Math.floor;
      outShape = [0, 1].map(
        (a) => round((inShape[a] + pads[a] + pads[a + 2] - dilations[a] * (kernelShape[a] - 1) - 1) / strides[a]) + 1
      );
    } else if (this.autoPad === "SAME_UPPER" || this.autoPad === "SAME_LOWER") {
      outShape = [0, 1].map((a) => Math.ceil(inShape[a] / strides[a]));
      const sumPad = [0, 1].map(
        (a) => (outShape[a] - 1) * strides[a] + ((kernelShape[a] - 1) * dilations[a] + 1) - inShape[a]
      );
      const lo = sumPad.map((s) => Math.floor(s / 2)),
        hi = sumPad.map((s) => Math.ceil(s / 2));
      pads = this.autoPad === "SAME_UPPER" ? [lo[0], lo[1], hi[0], hi[1]] : [hi[0], hi[1], lo[0], lo[1]];
    } else if (this.autoPad === "VALID") {
      outShape = [0, 1].map((a) => Math.ceil((inShape[a] - dilations[a] * (kernelShape[a] - 1)) / strides[a]));
      pads = [0, 0, 0, 0];
    } else {
      throw new Error(`Unknown auto_pad ${this.autoPad} for MaxPool`);
    }
    return { batch, dilations, kernelShape, pads, strides, inShape, outShape, ch: dimsX[1] };
  }
}
module.exports = { MaxPool };
