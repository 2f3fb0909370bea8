// The contracts between the runner, a backend and its operators, as this package implements them: what a
// caller written against the reference's descriptor runner may rely on, typed.  One file, in dependency
// order.  Each block names the reference declaration it keeps (src/descriptor_runner/interface/core/*.ts);
// the member names are the reference's, because operators and callers written for it must type-check here.

// ---- closed sets (constants.ts:1-15; this package carries the cpu and hip backends only) ----------------
/** Every backend but the host: tensors of these live in device memory. */
export type BackendWithoutCPU = "hip";
export type Backend = "cpu" | BackendWithoutCPU;
/** Element types; "bool" is one byte per element. */
export type DataType = "float32" | "int32" | "bool";
/** What getData() hands back and setData() takes, by DataType. */
export type DataArrayTypes = Float32Array | Int32Array | Uint8Array;
/** Run-time values of ../constants.js. */
export const backends: Backend[];
export const backendsWithoutCPU: BackendWithoutCPU[];
export const DataArrayConstructor: {
  float32: Float32ArrayConstructor;
  int32: Int32ArrayConstructor;
  bool: Uint8ArrayConstructor;
};

// ---- a tensor on any backend (tensor.ts:3-14) ---------------------------------------------------------------
export interface Tensor {
  /** Where the elements live; decides which operators may take the tensor without a move. */
  readonly backend: Backend;
  readonly dataType: DataType;
  readonly dims: ReadonlyArray<number>;
  /** dims.length */
  readonly ndim: number;
  /** Product of dims (1 for a scalar). */
  readonly length: number;
  /** Row-major element strides of dims. */
  readonly strides: ReadonlyArray<number>;
  /** A copy of the elements on the host.  On hip: a download, which waits for the stream. */
  getData(): Promise<DataArrayTypes>;
  /** Overwrites the elements from the host (data.length === length).  On hip: an upload. */
  setData(data: DataArrayTypes): Promise<void>;
  /** Gives the storage back; the tensor must not be used afterwards.  Idempotent. */
  dispose(): void;
}

// ---- what the runner needs from a backend (backendContext.ts:4-8) -------------------------------------------
export interface BackendContext {
  backend: Backend;
  /** A new tensor of this backend with unspecified contents (float32 when dataType is omitted). */
  emptyTensor(dims: ReadonlyArray<number>, dataType?: DataType): Tensor;
  /** The tensor's contents on this backend: the tensor itself when it is already here, else a copy
   * (the source stays valid).  `option` is backend specific; hip ignores it. */
  moveTensor(tensor: Tensor, option: Record<string, any>): Promise<Tensor>;
}

// ---- operators and their registration (operator.ts:6-30) ----------------------------------------------------
/** A decoded onnx.AttributeProto record, as core/onnxProto.js produces it. */
export interface AttributeProto {
  name: string;
  type: number;
  f?: number;
  i?: number | null;
  s?: Uint8Array | null;
  floats: number[];
  ints: number[];
  strings: Uint8Array[];
  t?: unknown;
}

export interface Operator {
  backend: Backend;
  /** Called once per node, before the first run, with the node's attributes. */
  initialize(attribute: AttributeProto[]): void;
  /** Per input (then per output): the backend the tensor must be on, or null for "leave it where it is". */
  getTensorBackendRequirement(nInputs: number, nOutputs: number): (Backend | null)[];
  /** Enqueues the node's work and returns its outputs; inputs stay owned by the runner. */
  run(context: BackendContext, inputs: Tensor[], nOutputs: number): Promise<Tensor[]>;
}

/** One line of an operator table: which factory serves an opType on a backend for a range of opsets. */
export interface OperatorEntry {
  opType: string;
  backend: Backend;
  /** First opset served (inclusive). */
  opsetMin: number;
  /** First opset no longer served (exclusive); absent = no upper bound. */
  opsetMax?: number;
  /** ONNX domain; absent = the default domain. */
  domain?: string;
  factory: () => Operator;
}
