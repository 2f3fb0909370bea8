"use strict";
// Device tensor of the hip backend: a buffer handle of libwebdnn_hip.so plus dims.
// Aliases (zero-copy Reshape/Flatten/Squeeze/Unsqueeze) share one reference-counted
// buffer, as WasmSharedBuffer does in the reference
// (src/descriptor_runner/backend/wasm/wasmTensorImpl.ts:16-99).
const { TensorImpl } = require("../../core/tensorImpl");
const { DataArrayConstructor } = require("../../interface/constants");

class HipSharedBuffer {
  constructor(native, byteLength) {
    this.native = native;
    this.byteLength = byteLength;
    this.handle = native.alloc(byteLength);
    this.refCount = 1;
    this.disposed = false;
  }

  incrementRef() {
    this.refCount++;
  }

  dispose() {
    this.refCount--;
    if (this.refCount <= 0 && !this.disposed) {
      this.disposed = true;
      this.native.free(this.handle);
    }
  }
}

class HipTensorImpl extends TensorImpl {
  constructor(context, dims, dataType, sharedBuffer) {
    super(dims, dataType || "float32", "hip");
    if (this.dataType !== "float32" && this.dataType !== "int32") {
      throw new Error(`HipTensor: dataType ${this.dataType} is not supported`);
    }
    this.context = context;
    if (sharedBuffer) {
      sharedBuffer.incrementRef();
      this.sharedBuffer = sharedBuffer;
    } else {
      this.sharedBuffer = new HipSharedBuffer(context.native, this.length * 4);
    }
    this.disposedFlag = false;
  }

  // The native buffer handle (throws after dispose()).
  get handle() {
    if (this.disposedFlag) throw new Error("HipTensor is already disposed");
    return this.sharedBuffer.handle;
  }

  alias(dims) {
    return new HipTensorImpl(this.context, dims, this.dataType, this.sharedBuffer);
  }

  // Device -> host; a fresh array every time (like wasmTensorImpl.ts:87-90).  Blocks
  // until the stream has produced the data.
  async getData() {
    const data = new DataArrayConstructor[this.dataType](this.length);
    this.context.native.read(this.handle, 0, data);
    return data;
  }

  async setData(data) {
    if (data.length !== this.length) throw new Error("setData: length mismatch");
    const Ctor = DataArrayConstructor[this.dataType];
    const src = data instanceof Ctor ? data : new Ctor(data);
    this.context.native.write(this.handle, 0, src);
  }

  dispose() {
    if (!this.disposedFlag) {
      this.disposedFlag = true;
      this.sharedBuffer.dispose();
    }
  }
}

module.exports = { HipTensorImpl, HipSharedBuffer };
