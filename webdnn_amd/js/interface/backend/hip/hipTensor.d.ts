// Device tensor of the hip backend (backend/hip/hipTensorImpl.js).  Shaped after
// src/descriptor_runner/interface/backend/wasm/wasmTensor.ts; `handle` and `alias` are what the hip
// operators use beyond the Tensor contract.
import { Tensor } from "../../core/contracts";

export interface HipTensor extends Tensor {
  readonly backend: "hip";
  /** Buffer handle of libwebdnn_hip.so (a wdh_buf, > 0).  Throws after dispose(). */
  readonly handle: number;
  /** Another view of the same device buffer with other dims (Reshape, Flatten, Squeeze, Unsqueeze);
   *  the buffer is freed when the last view is disposed. */
  alias(dims: ReadonlyArray<number>): HipTensor;
  /** Set by the runner on the device copy of an initializer: the contents stay as they are for as long as the
   *  tensor lives, so an operator may let the library keep what it derives from them (Conv passes
   *  WDH_CONV_CONSTANT_WEIGHTS). */
  constant?: boolean;
}
