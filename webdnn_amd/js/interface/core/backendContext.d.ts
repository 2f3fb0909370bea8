// Reference: src/descriptor_runner/interface/core/backendContext.ts:4-8 (unchanged contract).
import { Backend, DataType } from "./constants";
import { Tensor } from "./tensor";

export interface BackendContext {
  backend: Backend;
  emptyTensor(dims: ReadonlyArray<number>, dataType?: DataType): Tensor;
  moveTensor(tensor: Tensor, option: Record<string, any>): Promise<Tensor>;
}
