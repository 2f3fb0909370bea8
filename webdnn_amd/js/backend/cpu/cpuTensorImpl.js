"use strict";
// Host tensor: a typed array plus dims; what runner.run() takes and returns.
// Interface after src/descriptor_runner/backend/cpu/cpuTensorImpl.ts:14-89 (data,
// useExternalBuffer, getData / setData / getDataSync, getValue / setValue, dispose, isCPUTensor).
const { TensorImpl } = require("../../core/tensorImpl");
const { DataArrayConstructor } = require("../../interface/constants");

class CPUTensorImpl extends TensorImpl {
  // `data`: wrap the caller's typed array instead of allocating a zero-filled one
  constructor(dims, dataType, data) {
    super(dims, dataType || "float32", "cpu");
    this.useExternalBuffer = data != null;
    this.data = this.useExternalBuffer ? data : new DataArrayConstructor[this.dataType](this.length);
  }

  static isCPUTensor(tensor) {
    return tensor.backend === "cpu";
  }

  getDataSync() {
    return this.data;
  }

  async getData() {
    return this.data;
  }

  async setData(values) {
    this.data.set(values);
  }

  // Drops the (possibly large) array; the object stays valid but empty.
  dispose() {
    this.data = new Float32Array(1);
  }

  // Position of an element named by one index per axis.
  offsetOf(indices) {
    if (indices.length !== this.ndim) throw new Error("length of idxs does not match tensor.ndim");
    return indices.reduce((offset, index, axis) => offset + index * this.strides[axis], 0);
  }

  getValue(indices) {
    return this.data[this.offsetOf(indices)];
  }

  setValue(value, indices) {
    this.data[this.offsetOf(indices)] = value;
  }
}

module.exports = { CPUTensorImpl };
