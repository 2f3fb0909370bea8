// Reference: src/descriptor_runner/interface/core/operator.ts:6-30 (unchanged contract).  The attribute
// objects are the decoded onnx.AttributeProto records of core/onnxProto.js.
import { BackendContext } from "./backendContext";
import { Backend } from "./constants";
import { Tensor } from "./tensor";

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
  run(context: BackendContext, inputs: Tensor[], nOutputs: number): Promise<Tensor[]>;
  initialize(attribute: AttributeProto[]): void;
  getTensorBackendRequirement(nInputs: number, nOutputs: number): (Backend | null)[];
}

export interface OperatorEntry {
  opType: string;
  /** inclusive */
  opsetMin: number;
  /** exclusive; undefined = no upper bound */
  opsetMax?: number;
  domain?: string;
  backend: Backend;
  factory: () => Operator;
}
