// Context of the hip backend (backend/hip/hipContextImpl.js) and the options that reach it through
// WebDNN.load(directory, {backendOrder: ["hip", "cpu"], backendOptions: {hip: ...}}).  Shaped after
// src/descriptor_runner/interface/backend/wasm/wasmContext.ts.
import { BackendContext, DataType, Tensor } from "../../core/contracts";
import { HipDeviceInfo, HipMemStats, HipNative } from "./hipNative";
import { HipTensor } from "./hipTensor";

export interface WebDNNHipContextOption {
  /** GPU ordinal for wdh_init (default 0) */
  device?: number;
  /** no retry of a failed hip node on the cpu operators, and load() throws if hip is unavailable */
  strict?: boolean;
  /** run the hip fusion passes of core/modelTransform.js (default true) */
  fuse?: boolean;
  /** captured runs: true = record the second run; "auto" (default) = record the third run with inputs
   *  of one signature; false = always the node loop.  runner.run(inputs, {graph}) overrides it per call. */
  graph?: boolean | "auto";
  /** false: keep the graph's node order; by default a convolution whose inputs are ready early (a projection
   *  shortcut) is moved up and recorded as a side branch that a replay may run next to the main chain */
  sideBranches?: boolean;
  /** how many runs runner.submit keeps in flight (lanes it alternates over): 2 (default) to 4 */
  inFlight?: number;
  /** tuning hooks handed to wdh_set_option */
  contractionTile?: number;
  splitK?: number;
  /** another implementation of the addon's interface */
  native?: HipNative;
}

export interface WebDNNHipContext extends BackendContext {
  backend: "hip";
  native: HipNative;
  initialized: boolean;
  initialize(): Promise<void>;
  isHipTensor(tensor: Tensor): tensor is HipTensor;
  assertsHipTensor(tensor: Tensor): asserts tensor is HipTensor;
  assertsHipTensorArray(tensors: Tensor[]): asserts tensors is HipTensor[];
  emptyTensor(dims: ReadonlyArray<number>, dataType?: DataType): HipTensor;
  moveTensor(tensor: Tensor, option: Record<string, any>): Promise<HipTensor>;
  sync(): void;
  deviceInfo(): HipDeviceInfo;
  memStats(): HipMemStats;
}
