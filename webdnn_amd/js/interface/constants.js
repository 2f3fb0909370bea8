"use strict";
// Backend names, data types and typed-array constructors.
// Reference: src/descriptor_runner/interface/core/constants.ts:1-15, with "hip"
// added to the closed backend set.
const backendsWithoutCPU = ["hip"];
const backends = ["cpu", "hip"];
const DataArrayConstructor = {
  float32: Float32Array,
  int32: Int32Array,
  bool: Uint8Array,
};
module.exports = { backendsWithoutCPU, backends, DataArrayConstructor };
