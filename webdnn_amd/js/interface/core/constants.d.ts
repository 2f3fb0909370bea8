// Types of ../constants.js.  Reference: src/descriptor_runner/interface/core/constants.ts:1-15,
// with "hip" in the closed backend set (this package carries the cpu and hip backends only).
export type BackendWithoutCPU = "hip";
export type Backend = "cpu" | BackendWithoutCPU;
export const backendsWithoutCPU: BackendWithoutCPU[];
export const backends: Backend[];
export type DataType = "float32" | "int32" | "bool";
export const DataArrayConstructor: {
  float32: Float32ArrayConstructor;
  int32: Int32ArrayConstructor;
  bool: Uint8ArrayConstructor;
};
export type DataArrayTypes = Float32Array | Int32Array | Uint8Array;
