"use strict";
// Base of every backend's tensor: dims, row-major strides, length.
// Reference: src/descriptor_runner/core/tensorImpl.ts:4-29.
class TensorImpl {
  constructor(dims, dataType, backend) {
    this.dims = Array.prototype.slice.call(dims); // callers must not be able to alter it
    this.ndim = this.dims.length;
    this.dataType = dataType;
    this.backend = backend;
    let length = 1;
    const strides = [];
    for (let d = this.dims.length - 1; d >= 0; d--) {
      strides.unshift(length);
      length *= this.dims[d];
    }
    this.length = length;
    this.strides = strides;
  }
}
module.exports = { TensorImpl };
