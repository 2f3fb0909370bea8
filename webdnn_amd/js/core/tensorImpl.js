"use strict";
// What every backend's tensor has: dims (a private copy), rank, dense strides, element count.
// Fields after src/descriptor_runner/core/tensorImpl.ts:4-29.
const { denseStrides, elementCount } = require("../operators/shapes");

class TensorImpl {
  constructor(dims, dataType, backend) {
    this.dims = Array.from(dims);
    this.ndim = this.dims.length;
    this.strides = denseStrides(this.dims);
    this.length = elementCount(this.dims);
    this.dataType = dataType;
    this.backend = backend;
  }
}
module.exports = { TensorImpl };
