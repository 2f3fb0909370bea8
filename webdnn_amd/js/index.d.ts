// Entry points of the package (index.js).  Reference: src/descriptor_runner/index.ts:23-149 and
// interface/core/runner.ts; `backendOptions.hip` and the `graph` run option are the additions.
import { Backend, Tensor } from "./interface/core/contracts";
import { WebDNNHipContext, WebDNNHipContextOption } from "./interface/backend/hip/hipContext";

export interface InitOption {
  backendOrder?: Backend[];
  backendOptions?: { hip?: WebDNNHipContextOption };
  /** file name of the graph inside the directory (default model.onnx, or model-<backend>.onnx with `optimized`) */
  onnxBaseName?: string | null;
  /** the directory is an optimized-model directory (graph per backend, WDN2 weight files) */
  optimized?: boolean;
}

export interface RunOption {
  measurePerformance?: boolean;
  graph?: boolean | "auto";
}

export interface RunStats {
  nodesByBackend: Record<string, number>;
  retriedOnCpu: string[];
  nodes: number;
  operatorsCreated: number;
  enqueueMs?: number;
  graphReplay?: boolean;
}

/** What submit() returns and collect() takes; opaque to callers. */
export interface RunTicket {
  readonly lane?: number;
}

export interface Runner {
  readonly backendName: Backend;
  readonly backendContexts: { cpu: unknown; hip?: WebDNNHipContext };
  lastRunStats: RunStats | null;
  lastPerformance: Array<{ name: string; opType: string; backend: Backend; elapsed?: number; deviceElapsed?: number }> | null;
  graphUnsupported: string | null;
  getInputNames(): string[];
  getOutputNames(): string[];
  /** outputs come back as CPU tensors, as in the reference */
  run(inputs?: Tensor[], options?: RunOption): Promise<Tensor[]>;
  /**
   * Several runs in flight -- two unless backendOptions.hip.inFlight says 3 or 4 (no counterpart in the reference).  submit() enqueues a run on one of the library's
   * two lanes and returns without waiting for the device; collect() downloads that run's outputs.  Submit
   * batch i+1 before collecting batch i and the device works on one while the other's data travels.  At
   * most that many runs may be outstanding; collect them in the order of submission, and before calling run().
   * Until the model is captured (or if it cannot be) submit() simply runs and the ticket holds the outputs.
   * Inputs that already live on the device must be complete (uploaded, or produced by work that was waited for).
   */
  submit(inputs: Tensor[], options?: RunOption): Promise<RunTicket>;
  collect(ticket: RunTicket): Promise<Tensor[]>;
  disposeGraph(): void;
}

export function load(directory: string, options?: InitOption): Promise<Runner>;
export const CPUTensor: new (dims: ReadonlyArray<number>, dataType?: "float32" | "int32" | "bool",
                             data?: Float32Array | Int32Array | Uint8Array) => Tensor;
