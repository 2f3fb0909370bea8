"use strict";
// CPU tensor: a typed array plus dims.  The I/O type of runner.run().
// Reference: src/descriptor_runner/backend/cpu/cpuTensorImpl.ts:14-89.
const { TensorImpl } = require("../../core/tensorImpl");
const { DataArrayConstructor } = require("../../interface/constants");

class CPUTensorImpl extends TensorImpl {
  constructor(dims, dataType, data) {
    super(dims, dataType || "float32", "cpu");
    this.data = data || new DataArrayConstructor[this.dataType](this.length);
    this.useExternalBuffer = !!data;
  }

  async getData() {
    return this.data;
  }

  async setData(data) {
    this.data.set(data);
  }

  dispose() {
    this.data = new Float32Array(1);
  }

  static isCPUTensor(tensor) {
    return tensor.backend === "cpu";
  }

  getDataSync() {
    return this.data;
  }

  getValue(idxs) {
    if (idxs.length !== this.ndim) throw new Error("length of idxs does not match tensor.ndim");
    let ofs = 0;
    for (let i = 0; i < this.ndim; i++) ofs += this.strides[i] * idxs[i];
    return this.data[ofs];
  }

  setValue(value, idxs) {
    if (idxs.length !== this.ndim) throw new Error("length of idxs does not match tensor.ndim");
    let ofs = 0;
    for (let i = 0; i < this.ndim; i++) ofs += this.strides[i] * idxs[i];
    this.data[ofs] = value;
  }
}

module.exports = { CPUTensorImpl };
