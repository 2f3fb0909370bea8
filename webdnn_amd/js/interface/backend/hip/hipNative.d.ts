// The N-API addon webdnn_amd/lib/webdnn_hip.node (napi/addon.c): one function per entry point of
// include/webdnn_hip.h, arguments in the order of the C declaration.  Handles, sizes, strides and
// extents are integers passed as numbers; a negative status of the C call becomes a thrown Error
// whose message ends with wdh_last_error().  `backendOptions.hip.native` may supply another object
// of this shape (the host tests run with one that computes on the CPU).
export type Handle = number;
export type IntList = ReadonlyArray<number> | Int32Array;

export interface HipDeviceInfo {
  name: string;
  computeUnits: number;
  clockMHz: number;
  hbmBytes: number;
}
export interface HipMemStats {
  inUse: number;
  cached: number;
  peak: number;
}

export interface HipNative {
  // ---- runtime ----
  init(device: number): void;
  shutdown(): void;
  deviceInfo(): HipDeviceInfo;
  setOption(name: string, value: number): void;
  alloc(bytes: number): Handle;
  free(h: Handle): void;
  /** host -> device; `data` may be reused on return */
  write(h: Handle, dstByteOffset: number, data: ArrayBufferView): void;
  /** device -> host; fills `data`, blocks until the stream has produced it */
  read(h: Handle, srcByteOffset: number, data: ArrayBufferView): void;
  copy(dst: Handle, dstByteOffset: number, src: Handle, srcByteOffset: number, bytes: number): void;
  sync(): void;
  /** wdh_set_lane: 0 = the stream everything runs on by default, 1 = the second stream (two runs in flight). */
  setLane(lane: number): void;
  /** wdh_branch_begin / _end / _join: a side branch of the run being recorded (no-ops outside a recording). */
  branchBegin(): void;
  branchEnd(): void;
  branchJoin(): void;
  memStats(): HipMemStats;
  trim(keepBytes: number): void;
  eventRecord(id: number): void;
  eventElapsedMs(startId: number, stopId: number): number;
  // ---- captured runs ----
  graphBegin(): void;
  graphEnd(): number;
  graphLaunch(graphId: number): void;
  graphDestroy(graphId: number): void;
  // ---- contraction ----
  /** epilogue: 0 none, 1 Relu; C / R: 0 = absent */
  gemm(A: Handle, B: Handle, C: Handle, Y: Handle, batch: number, m: number, n: number, k: number,
       sAb: number, sA0: number, sA1: number, sBb: number, sB0: number, sB1: number, sC0: number, sC1: number,
       alpha: number, beta: number, epilogue: number, R: Handle): void;
  gemmEx(A: Handle, B: Handle, C: Handle, Y: Handle, batch: number, m: number, n: number, k: number,
         sAb: number, sA0: number, sA1: number, sBb: number, sB0: number, sB1: number, sC0: number, sC1: number,
         alpha: number, beta: number, epilogue: number, R: Handle, sYb: number, sY0: number): void;
  /** arrays of one length (<= 16); bias entries may be 0 */
  linearGroup(A: IntList, W: IntList, bias: IntList, Y: IntList, m: IntList, n: IntList, k: IntList, epilogue: number): void;
  conv2d(X: Handle, W: Handle, bias: Handle, Y: Handle, n: number, c: number, h: number, w: number, cout: number,
         kh: number, kw: number, pt: number, pl: number, pb: number, pr: number, sh: number, sw: number,
         dh: number, dw: number, group: number, epilogue: number, R: Handle): void;
  /** flags bit 0: W is not written to while its handle lives (derived forms of it may be kept) */
  conv2dEx(X: Handle, W: Handle, bias: Handle, Y: Handle, n: number, c: number, h: number, w: number, cout: number,
           kh: number, kw: number, pt: number, pl: number, pb: number, pr: number, sh: number, sw: number,
           dh: number, dw: number, group: number, epilogue: number, R: Handle, flags: number): void;
  attention(Q: Handle, K: Handle, V: Handle, Y: Handle, batch: number, tq: number, tk: number, d: number,
            sQb: number, sQi: number, sKb: number, sKj: number, sVb: number, sVj: number, sYb: number, sYi: number,
            alpha: number): void;
  // ---- bandwidth-bound companions ----
  /** op: 0 Add, 1 Sub, 2 Mul, 3 Div, 4 Pow; dtype: 0 float32, 1 int32; strides 0 where an operand broadcasts */
  binary(op: number, dtype: number, L: Handle, R: Handle, Y: Handle, outShape: IntList, stridesL: IntList, stridesR: IntList): void;
  /** op: 0 Relu, 1 Sigmoid, 2 Sqrt, 3 Exp, 4 Tanh, 5 Abs, 6 Neg, 7 Reciprocal */
  unary(op: number, dtype: number, X: Handle, Y: Handle, length: number): void;
  softmax(X: Handle, Y: Handle, outer: number, len: number): void;
  layernorm(X: Handle, gamma: Handle, beta: Handle, Y: Handle, outer: number, len: number, epsilon: number): void;
  /** Y = LayerNormalization(X); Y2 = Y + P (P shaped like X) */
  layernormAdd(X: Handle, gamma: Handle, beta: Handle, Y: Handle, P: Handle, Y2: Handle, outer: number, len: number, epsilon: number): void;
  reduceMean(X: Handle, Y: Handle, outer: number, len: number): void;
  reduceAxis(X: Handle, Y: Handle, outer: number, reduced: number, inner: number, divisor: number): void;
  maxpool2d(X: Handle, Y: Handle, n: number, c: number, h: number, w: number, oh: number, ow: number, kh: number, kw: number,
            pt: number, pl: number, sh: number, sw: number, dh: number, dw: number): void;
  globalAvgpool(X: Handle, Y: Handle, nc: number, hw: number): void;
  /** Y (dense, shape outShape) [i...] = X[sum i_a * inStrides[a]] */
  transpose(X: Handle, Y: Handle, outShape: IntList, inStrides: IntList): void;
  gather(data: Handle, indices: Handle, Y: Handle, outer: number, axisLength: number, inner: number, nIndices: number): void;
  /** from / to: 0 float32, 1 int32 */
  cast(from: number, to: number, X: Handle, Y: Handle, length: number): void;
  stridedCopy(X: Handle, xOffset: number, Y: Handle, yOffset: number, shape: IntList, xStrides: IntList, yStrides: IntList): void;
}
