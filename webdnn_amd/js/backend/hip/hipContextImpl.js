"use strict";
// Context of the hip backend: owns the native library binding.
// Counterpart of WebDNNWasmContextImpl
// (src/descriptor_runner/backend/wasm/wasmContextImpl.ts:13-163): emptyTensor,
// moveTensor, initialize, tensor assertions; the launch primitive is the set of
// wdh_* entry points exposed by the N-API addon (`this.native`).
const path = require("path");
const { HipTensorImpl } = require("./hipTensorImpl");

const ADDON_PATH = path.join(__dirname, "..", "..", "..", "lib", "webdnn_hip.node");

class WebDNNHipContextImpl {
  // option: { device?: number, strict?: boolean, contractionTile?: number, splitK?: number, native?: object }
  constructor(cpuContext, option) {
    this.backend = "hip";
    this.cpuContext = cpuContext;
    this.option = option || {};
    this.native = null;
    this.initialized = false;
    this.tracked = null;
  }

  // Throws when the addon, the library or the GPU is missing; load() then skips
  // this backend (reference: src/descriptor_runner/index.ts:68-79).
  async initialize() {
    // `native` can be injected (host tests without a GPU supply a fake)
    this.native = this.option.native || require(ADDON_PATH);
    this.native.init(this.option.device || 0);
    if (this.option.contractionTile != null) this.native.setOption("contraction_tile", this.option.contractionTile);
    if (this.option.splitK != null) this.native.setOption("split_k", this.option.splitK);
    this.initialized = true;
  }

  isHipTensor(tensor) {
    return tensor.backend === this.backend;
  }

  assertsHipTensor(tensor) {
    if (tensor.backend !== this.backend) {
      throw new Error(`Tensor backend ${this.backend} is expected, but ${tensor.backend} is given.`);
    }
  }

  assertsHipTensorArray(tensors) {
    for (const tensor of tensors) this.assertsHipTensor(tensor);
  }

  emptyTensor(dims, dataType) {
    const t = new HipTensorImpl(this, dims, dataType);
    if (this.tracked) this.tracked.push(t);
    return t;
  }

  // The runner brackets every operator.run with trackAllocations / stopTracking; when the
  // operator throws, releaseTracked frees what it had allocated (its outputs and
  // temporaries), which nobody else holds a reference to.
  trackAllocations() {
    this.tracked = [];
  }

  releaseTracked() {
    for (const t of this.tracked || []) t.dispose();
    this.tracked = null;
  }

  stopTracking() {
    this.tracked = null;
  }

  // eslint-disable-next-line no-unused-vars
  async moveTensor(tensor, option) {
    const dst = new HipTensorImpl(this, tensor.dims, tensor.dataType);
    try {
      await dst.setData(await tensor.getData());
    } catch (error) {
      dst.dispose(); // e.g. an upload attempted while a graph is being captured
      throw error;
    }
    return dst;
  }

  sync() {
    this.native.sync();
  }

  deviceInfo() {
    return this.native.deviceInfo();
  }

  memStats() {
    return this.native.memStats();
  }
}

module.exports = { WebDNNHipContextImpl, ADDON_PATH };
