"use strict";
// Reference: src/descriptor_runner/backend/cpu/cpuContextImpl.ts:7-50.
const { CPUTensorImpl } = require("./cpuTensorImpl");

class WebDNNCPUContextImpl {
  constructor() {
    this.backend = "cpu";
  }

  async initialize() {}

  isCPUTensor(tensor) {
    return tensor.backend === this.backend;
  }

  assertsCPUTensor(tensor) {
    if (tensor.backend !== this.backend) {
      throw new Error(`Tensor backend ${this.backend} is expected, but ${tensor.backend} is given.`);
    }
  }

  assertsCPUTensorArray(tensors) {
    for (const tensor of tensors) this.assertsCPUTensor(tensor);
  }

  emptyTensor(dims, dataType, data) {
    return new CPUTensorImpl(dims, dataType, data);
  }

  async moveTensor(tensor) {
    return new CPUTensorImpl(tensor.dims, tensor.dataType, await tensor.getData());
  }
}

module.exports = { WebDNNCPUContextImpl };
