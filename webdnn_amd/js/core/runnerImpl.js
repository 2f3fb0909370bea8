"use strict";
// The descriptor runner: loads an ONNX model and interprets it node by node.
// Reference: src/descriptor_runner/core/runnerImpl.ts:42-597, with a `hip` slot in
// every place where the reference hard-codes its closed backend set
// (BackendContexts :35-40, tensorsForBackends :323-328, the context switch :470-486,
// end-of-run disposal :574-582).
//
// Additions for the hip backend (none changes what a model computes):
//   * strict mode (backendOptions.hip.strict): the one-time retry of a failed node on
//     the cpu operators (:511-520) is switched off, so a benchmark or parity run cannot
//     silently pass on the fallback;
//   * lastRunStats: how many nodes ran on which backend, and which were retried;
//   * measurePerformance uses HIP events on the library's stream for hip nodes
//     (Date.now() only sees enqueue time there);
//   * run(inputs, {graph: true}) records the device work of one run into a HIP graph
//     and replays it on later calls with inputs of the same shapes: the node loop
//     below (runnerImpl.ts:377-542 in the reference) then runs once, not per call;
//   * callers that pass no option get the same thing by themselves (graph: "auto", the
//     default of backendOptions.hip.graph): two eager runs with inputs of one signature,
//     then the third is recorded and later ones replay it.  A model that cannot be
//     recorded, a change of input shapes or a measurePerformance run falls back to the
//     node loop exactly as {graph: true} does.  backendOptions.hip.graph = false or
//     run(inputs, {graph: false}) keeps every run in the node loop.
const fs = require("fs");
const path = require("path");
const { backends, backendsWithoutCPU } = require("../interface/constants");
const { nonnull, clipToInt32 } = require("../util");
const { findTensorReleaseTiming, modelTransform } = require("./modelTransform");
const { instantiateOperator } = require("./operatorTable");
const { decodeModel, DataType } = require("./onnxProto");
const { tensorProtoToArray } = require("../operators/operatorUtil");
const { getLogger } = require("../logging");

const logger = getLogger("WebDNN.runner");

// What a captured run is specific to: the types and shapes of the inputs.
function inputSignature(inputs) {
  return inputs.map((t) => `${t.dataType}[${t.dims.join(",")}]`).join(";");
}

class RunnerImpl {
  // backendContexts: { cpu, hip? };  options: { strict?, fuse?, graph?: true | false | "auto" }
  constructor(backendOrder, backendContexts, options) {
    this.backendOrder = backendOrder;
    this.backendContexts = backendContexts;
    this.backendName = backendOrder[0];
    this.options = options || {};
    this.loaded = false;
    this.model = null;
    this.tensorMoveOptions = {};
    this.forceOperatorBackendOrder = {};
    this.lastRunStats = null;
    this.lastPerformance = null;
    // captured run: {id, inputs, ownedInputs, outputs, signature, stats}; see runWithGraph
    this.graphState = null;
    // two runs in flight (submit / collect): the captured run of the second lane, built like graphState
    // from the same node loop recorded on the library's lane 1; which lane the next submit takes; and
    // the submitted runs not collected yet, by lane
    this.sideGraphStates = [];        // by lane - 1
    this.submitLane = 0;
    this.inFlight = [];               // by lane
    this.lanes = Math.max(1, Math.min(4, (options && options.inFlight) || 2)); // lanes submit() alternates over
    this.graphWarm = false;
    this.graphUnsupported = null; // reason, once a capture has failed for this model
    this.graphRetries = 0; // captures given up for a reason an eager run cures
    this.autoSeen = { signature: null, runs: 0 }; // graph "auto": eager runs in a row with one input signature
    // Operator instances by node and by where its inputs live.  The reference builds
    // and initializes a new instance per node per run (runnerImpl.ts:441-452);
    // instances here keep no state beyond their attributes, so later runs reuse them.
    this.operatorCache = new Map();
  }

  async loadModel(directory, onnxBasename) {
    this.disposeGraph();
    this.graphWarm = false;
    this.graphUnsupported = null;
    this.graphRetries = 0;
    const bytes = fs.readFileSync(path.join(directory, onnxBasename));
    this.loadModelFromBytes(bytes, directory);
  }

  // `bytes`: the serialized ModelProto; `directory`: where external weight files live
  loadModelFromBytes(bytes, directory) {
    this.model = decodeModel(new Uint8Array(bytes.buffer, bytes.byteOffset, bytes.byteLength));
    this.operatorCache.clear();
    modelTransform(this.model, this.backendOrder, { fuse: this.options.fuse, sideBranches: this.options.sideBranches });
    if (this.model.opsetImport.length !== 1) {
      logger.warn("Specifying multiple opset_import is not supported. Using first one.");
    }
    if (this.model.opsetImport.length === 0) throw new Error("model has no opset_import");
    this.opset = clipToInt32(this.model.opsetImport[0].version);
    this.initializerTensors = new Map();
    for (const [name, tensor] of this.extractInitializerTensor().entries()) {
      this.initializerTensors.set(name, tensor);
    }
    for (const [name, tensor] of this.loadExternalInitializerTensor(directory).entries()) {
      this.initializerTensors.set(name, tensor);
    }
    for (const kv of (this.copiedInitializerTensors || new Map()).values()) {
      for (const t of kv.values()) t.dispose();
    }
    this.copiedInitializerTensors = new Map();
    for (const backend of this.backendOrder) {
      if (backend !== "cpu") this.copiedInitializerTensors.set(backend, new Map());
    }
    this.inputsWithoutInitializer = this.model.graph.input.filter(
      (v) => v.name && !this.initializerTensors.has(v.name)
    );
    for (const md of this.model.metadataProps) {
      if (md.key === "WebDNN2.TensorMoveOptions") this.tensorMoveOptions = JSON.parse(md.value);
      if (md.key === "WebDNN2.ForceOperatorBackendOrder") this.forceOperatorBackendOrder = JSON.parse(md.value);
    }
    this.loaded = true;
  }

  // FLOAT / INT64 (clipped to int32) / INT32 initializers become CPU tensors; anything
  // else throws (runnerImpl.ts:136-233).
  extractInitializerTensor() {
    const tensors = new Map();
    for (const initializer of this.model.graph.initializer) {
      if (![DataType.FLOAT, DataType.INT64, DataType.INT32].includes(initializer.dataType)) {
        throw new Error(`Unsupported initializer dataType ${initializer.dataType}`);
      }
      const { dims, dataType, data } = tensorProtoToArray(initializer);
      tensors.set(initializer.name, this.backendContexts.cpu.emptyTensor(dims, dataType, data));
    }
    return tensors;
  }

  // Optimized models keep their weights in WDN2 tensor files named by metadata
  // (runnerImpl.ts:235-268).
  loadExternalInitializerTensor(directory) {
    for (const md of this.model.metadataProps) {
      if (md.key === "WebDNN2.WeightPaths") {
        const { TensorLoaderImpl } = require("./tensorLoaderImpl");
        const paths = md.value.split(":").map((bn) => path.join(directory || ".", bn));
        return new TensorLoaderImpl(paths, this.backendContexts.cpu).loadAllSync();
      }
    }
    return new Map();
  }

  getInputNames() {
    return this.inputsWithoutInitializer.map((gi) => gi.name);
  }

  getOutputNames() {
    return nonnull(this.model).graph.output.map((gi) => gi.name);
  }

  contextFor(backend) {
    const context = this.backendContexts[backend];
    if (!context) throw new Error(`No context for backend ${backend}`);
    return context;
  }

  async run(inputs, options) {
    const opts = options || {};
    if (!this.model || !this.loaded) throw new Error("not initialized");
    if (!inputs) throw new Error("inputs are required");
    if (this.inFlight.some((t) => t)) throw new Error("run: collect the submitted runs first");
    const hipContext = this.backendContexts.hip;
    let mode = opts.graph !== undefined ? opts.graph : this.options.graph;
    if (mode === undefined || mode === null) mode = "auto";
    const available = hipContext && hipContext.initialized && hipContext.native.graphBegin && !this.graphUnsupported;
    if (mode === "auto" && available) {
      // Per-node timings need the node loop; so does anything seen fewer than twice.
      if (opts.measurePerformance) return this.runEager(inputs, opts);
      const signature = inputSignature(inputs);
      if (this.autoSeen.signature !== signature) this.autoSeen = { signature, runs: 0 };
      if (this.autoSeen.runs < 2) {
        this.autoSeen.runs++;
        this.graphWarm = !this.graphState || this.graphState.signature === signature;
        if (this.graphState && this.graphState.signature !== signature) this.disposeGraph();
        return this.runEager(inputs, opts);
      }
      return this.runWithGraph(inputs, opts);
    }
    if (mode === true && available) return this.runWithGraph(inputs, opts);
    return this.runEager(inputs, opts);
  }

  // Frees the captured runs, if any (their output and input buffers included).
  disposeGraph() {
    const states = this.sideGraphStates.concat([this.graphState]);
    this.sideGraphStates = [];
    this.graphState = null;
    for (const state of states) if (state) this.disposeCapturedRun(state);
    this.inFlight = [];
    this.submitLane = 0;
  }

  disposeCapturedRun(state) {
    for (const t of state.outputs) if (t.backend === "hip") t.dispose();
    for (const t of state.ownedInputs) t.dispose();
    this.backendContexts.hip.native.graphDestroy(state.id);
  }

  // First call: an ordinary run (it uploads the weights, fills the buffer pool and builds
  // the conv tap tables, none of which can happen while capturing).  Second call: the node
  // loop runs once more with the stream in capture mode -- operators record their kernels
  // instead of executing them -- and the resulting graph is launched.  Later calls with
  // inputs of the same shapes and types refill the captured input buffers, launch the graph
  // and read the captured output buffers.  A model whose run needs the host to look at
  // device data (a shape computed on the device, a node that fails over to the cpu) cannot
  // be captured: the capture is dropped, the reason kept in graphUnsupported, and this and
  // all later calls run eagerly.
  async runWithGraph(inputs, opts) {
    const hip = this.backendContexts.hip,
      cpu = this.backendContexts.cpu;
    if (this.inputsWithoutInitializer.length !== inputs.length) throw new Error("length of inputs mismatch");
    const signature = inputSignature(inputs);
    if (this.graphState && this.graphState.signature !== signature) {
      // other shapes: other buffers, maybe conv geometries not seen yet -- warm up again
      this.disposeGraph();
      this.graphWarm = false;
    }
    if (!this.graphState) {
      if (!this.graphWarm) {
        this.graphWarm = true;
        return this.runEager(inputs, opts);
      }
      const state = await this.captureRun(inputs);
      if (!state) return this.runEager(inputs, opts);
      this.graphState = state;
    } else {
      await this.refillGraphInputs(this.graphState, inputs);
    }
    const state = this.graphState;
    if (opts.measurePerformance) hip.native.eventRecord(0);
    hip.native.graphLaunch(state.id);
    if (opts.measurePerformance) hip.native.eventRecord(1);
    const results = await this.readGraphOutputs(state);
    if (opts.measurePerformance) {
      this.lastPerformance = [{ opType: "(captured graph)", name: "graph", backend: "hip", deviceElapsed: hip.native.eventElapsedMs(0, 1) }];
    }
    this.lastRunStats = Object.assign({}, state.stats, { graphReplay: true });
    return results;
  }

  // Records one run of the node loop on the library's current lane.  Returns the captured run
  // {id, inputs, ownedInputs, outputs, signature, stats}, or null when the run cannot be recorded
  // (the reason is logged; graphUnsupported is set unless the cause is transient).
  async captureRun(inputs) {
    const hip = this.backendContexts.hip;
    // The graph reads its inputs from buffers the runner owns: a caller's device tensor
    // is copied in like a host tensor is uploaded, so the caller may overwrite or dispose
    // it afterwards and later replays never write into caller memory.
    const graphInputs = [];
    try {
      for (const t of inputs) {
        if (t.backend === "hip") {
          const own = hip.emptyTensor(t.dims, t.dataType);
          graphInputs.push(own);
          hip.native.copy(own.handle, 0, t.handle, 0, own.length * 4);
        } else {
          graphInputs.push(await hip.moveTensor(t, {}));
        }
      }
    } catch (error) {
      for (const t of graphInputs) t.dispose();
      throw error;
    }
    let outputs = null,
      failure = null;
    hip.native.graphBegin();
    try {
      outputs = await this.runEager(graphInputs, { capture: true });
    } catch (error) {
      failure = error;
    }
    let id = -1;
    try {
      id = hip.native.graphEnd();
    } catch (error) {
      failure = failure || error;
    }
    if (failure) {
      if (id >= 0) hip.native.graphDestroy(id);
      for (const t of outputs || []) if (t.backend === "hip") t.dispose();
      for (const t of graphInputs) t.dispose();
      // A geometry met for the first time while recording (its tables need a blocking
      // copy) is cured by an eager run; anything else will fail the same way again.
      const transient = /run it once before capturing/.test(failure.message) && this.graphRetries < 3;
      if (transient) {
        this.graphRetries++;
      } else {
        this.graphUnsupported = failure.message;
      }
      logger.warn(`run could not be captured into a graph (${failure.message}); running eagerly`);
      return null;
    }
    this.graphRetries = 0;
    return { id, inputs: graphInputs, ownedInputs: graphInputs, outputs, signature: inputSignature(inputs), stats: this.lastRunStats };
  }

  // The caller's inputs go into the captured run's own input buffers (upload or device copy).
  async refillGraphInputs(state, inputs) {
    const hip = this.backendContexts.hip;
    for (let i = 0; i < inputs.length; i++) {
      const src = inputs[i],
        dst = state.inputs[i];
      if (src.backend === "hip") hip.native.copy(dst.handle, 0, src.handle, 0, dst.length * 4);
      else await dst.setData(await src.getData());
    }
  }

  // device -> host, the run's only synchronisation; a cpu output (a constant) is copied
  async readGraphOutputs(state) {
    const cpu = this.backendContexts.cpu;
    const results = [];
    for (const t of state.outputs) results.push(await cpu.moveTensor(t, {}));
    return results;
  }

  // Several runs in flight (two unless the load option inFlight says 3 or 4).  submit() enqueues a run -- inputs uploaded, the captured graph launched -- and
  // returns a ticket without waiting for the device; collect(ticket) downloads that run's outputs.  A
  // caller that submits batch i+1 before it collects batch i keeps the device busy while batch i's
  // results travel and while batch i+1's kernels start: the two runs sit on the library's two lanes
  // (streams) and overlap where the device has room.  Each lane has its own captured run (own input,
  // output and workspace buffers).  Until the model has been captured (the first calls, or a model that
  // cannot be captured, or graph mode off) submit() simply runs and the ticket carries the outputs.
  // An input that already lives on the device must be complete when it is submitted (uploaded -- the
  // library waits for uploads by itself -- or produced by work that has been waited for): the lanes do
  // not wait for each other.
  // At most one run per lane may be outstanding: collect in the order of submission.  A second batch in
  // flight fills most of what one leaves idle (ResNet-50 b32: +11 %, a batch-1 DETR +33 %); a third adds little
  // once recordings have side branches, and four lanes are more than a process has hardware queues for.
  async submit(inputs, options) {
    const opts = options || {};
    if (!this.model || !this.loaded) throw new Error("not initialized");
    const hip = this.backendContexts.hip;
    let mode = opts.graph !== undefined ? opts.graph : this.options.graph;
    if (mode === undefined || mode === null) mode = "auto";
    const lanes = hip && hip.initialized && hip.native.setLane && hip.native.graphBegin && !this.graphUnsupported && mode !== false;
    const signature = lanes ? inputSignature(inputs) : null;
    if (!lanes || opts.measurePerformance || !this.graphState || this.graphState.signature !== signature) {
      // not captured yet (or never will be): an ordinary run, which also does the warming up and capturing
      await this.drainInFlight();
      return { done: await this.run(inputs, opts) };
    }
    const lane = this.submitLane;
    if (this.inFlight[lane]) throw new Error(`submit: ${this.lanes} runs are in flight already; collect the oldest one first`);
    if (this.inputsWithoutInitializer.length !== inputs.length) throw new Error("length of inputs mismatch");
    let state = lane === 0 ? this.graphState : this.sideGraphStates[lane - 1];
    if (state && state.signature !== signature) state = null; // (cannot happen for lane 0: checked above)
    hip.native.setLane(lane);
    try {
      if (!state) {
        if (this.sideGraphStates[lane - 1]) {
          const old = this.sideGraphStates[lane - 1];
          this.sideGraphStates[lane - 1] = null;
          this.disposeCapturedRun(old);
        }
        state = await this.captureRun(inputs);
        if (!state) {
          hip.native.setLane(0);
          await this.drainInFlight();
          return { done: await this.run(inputs, opts) };
        }
        this.sideGraphStates[lane - 1] = state;
      } else {
        await this.refillGraphInputs(state, inputs);
      }
      hip.native.graphLaunch(state.id);
    } finally {
      hip.native.setLane(0);
    }
    const ticket = { lane, state };
    this.inFlight[lane] = ticket;
    this.submitLane = (lane + 1) % this.lanes;
    return ticket;
  }

  async collect(ticket) {
    if (!ticket) throw new Error("collect: no ticket");
    if (ticket.done) return ticket.done;
    if (this.inFlight[ticket.lane] !== ticket) throw new Error("collect: this run has been collected already");
    const hip = this.backendContexts.hip;
    hip.native.setLane(ticket.lane);
    try {
      const results = await this.readGraphOutputs(ticket.state);
      this.lastRunStats = Object.assign({}, ticket.state.stats, { graphReplay: true, lane: ticket.lane });
      return results;
    } finally {
      this.inFlight[ticket.lane] = null;
      hip.native.setLane(0);
    }
  }

  // Waits for the submitted runs (their outputs are dropped).
  async drainInFlight() {
    for (const ticket of this.inFlight) if (ticket) await this.collect(ticket);
  }

  // opts.capture (internal): the stream is recording; keep the outputs where they are and
  // never retry on the cpu.
  async runEager(inputs, options) {
    const opts = options || {};
    const graph = this.model.graph;
    const tensorsForBackends = {};
    for (const backend of backends) tensorsForBackends[backend] = new Map();

    for (const [name, tensor] of this.initializerTensors.entries()) tensorsForBackends.cpu.set(name, tensor);
    for (const [backend, kv] of this.copiedInitializerTensors.entries()) {
      for (const [name, tensor] of kv.entries()) tensorsForBackends[backend].set(name, tensor);
    }

    if (this.inputsWithoutInitializer.length !== inputs.length) throw new Error("length of inputs mismatch");
    // Inputs are CPU tensors in the reference; a tensor that already lives on another
    // backend (uploaded once by the caller, e.g. through context.moveTensor) is taken
    // where it is.  Caller-owned tensors are never disposed by the run.
    const callerOwned = new Set();
    for (let i = 0; i < inputs.length; i++) {
      const name = this.inputsWithoutInitializer[i].name;
      if (!(inputs[i].backend in tensorsForBackends)) throw new Error(`input ${name}: unknown backend ${inputs[i].backend}`);
      tensorsForBackends[inputs[i].backend].set(name, inputs[i]);
      callerOwned.add(inputs[i]);
    }

    const runStart = process.hrtime.bigint();
    const tensorReleaseTiming = findTensorReleaseTiming(this.model, new Set(this.initializerTensors.keys()));
    const nodePerformances = [];
    const stats = { nodesByBackend: {}, retriedOnCpu: [], nodes: graph.node.length, operatorsCreated: 0 };
    const strict = !!this.options.strict || !!opts.capture;
    const hip = this.backendContexts.hip;
    const useEvents = !opts.capture && !!opts.measurePerformance && hip && hip.initialized && graph.node.length + 1 <= 4096;

    try {
      for (let i = 0; i < graph.node.length; i++) {
        const nodeStartTime = Date.now(),
          node = graph.node[i],
          opType = nonnull(node.opType);
        let actualBackend, actualInputDims, actualOutputDims;
        let backendOrderForNode = this.forceOperatorBackendOrder[node.name] || this.backendOrder;
        let firstTry = true;

        // eslint-disable-next-line no-constant-condition
        while (true) {
          try {
            // where does each input live?
            const currentTensorsBackends = [];
            for (const inputName of node.input) {
              const bs = [];
              for (const backend of backendOrderForNode) {
                if (tensorsForBackends[backend].has(inputName)) bs.push(backend);
              }
              if (bs.length === 0) {
                // a forced order such as ["hip"] must still find tensors that sit on the cpu
                for (const backend of backends) {
                  if (tensorsForBackends[backend].has(inputName)) bs.push(backend);
                }
              }
              currentTensorsBackends.push(bs);
            }
            const cacheKey = `${i}:${backendOrderForNode.join()}:${currentTensorsBackends.map((b) => b.join("+")).join("|")}`;
            let operator = this.operatorCache.get(cacheKey);
            if (!operator) {
              operator = instantiateOperator(opType, this.opset, backendOrderForNode, currentTensorsBackends);
              if (!operator) {
                throw new Error(`Operator implementation for ${opType}, opset=${this.opset} does not exist.`);
              }
              operator.initialize(nonnull(node.attribute));
              this.operatorCache.set(cacheKey, operator);
              stats.operatorsCreated++;
            }
            const requirement = operator.getTensorBackendRequirement(node.input.length, node.output.length);
            const operatorInputs = [];
            for (let j = 0; j < node.input.length; j++) {
              const inputName = node.input[j],
                reqBackend = requirement[j];
              if (!reqBackend) {
                // anywhere will do
                const where = currentTensorsBackends[j][0];
                const t = where && tensorsForBackends[where].get(inputName);
                if (!t) throw new Error(`Input ${inputName} not found`);
                operatorInputs.push(t);
                continue;
              }
              const t = tensorsForBackends[reqBackend].get(inputName);
              if (t) {
                operatorInputs.push(t);
                continue;
              }
              let found = false;
              for (const otherBackend of this.backendOrder) {
                const otherT = tensorsForBackends[otherBackend].get(inputName);
                if (otherT) {
                  const movedT = await this.contextFor(reqBackend).moveTensor(
                    otherT,
                    this.tensorMoveOptions[inputName] || {}
                  );
                  // the device copy of an initializer keeps its contents for as long as it lives
                  // (operators may keep forms derived from it: see HipConv)
                  if (this.initializerTensors.has(inputName)) movedT.constant = true;
                  tensorsForBackends[reqBackend].set(inputName, movedT);
                  operatorInputs.push(movedT);
                  found = true;
                  break;
                }
              }
              if (!found) throw new Error(`Input ${inputName} not found`);
            }

            const context = this.contextFor(operator.backend);
            logger.debug(`Running ${node.name}(${opType}) on ${operator.backend}`);
            // side branches of a recorded run (modelTransform.hoistSideBranches); no-ops while executing
            const branches = operator.backend === "hip" && hip && hip.native.branchBegin;
            if (branches && node.hipJoin) hip.native.branchJoin();
            if (branches && node.hipSide) hip.native.branchBegin();
            // one event per node boundary: node i's device time runs from event i to event i+1
            // (every event costs the stream a small bubble, so as few as possible)
            if (useEvents) hip.native.eventRecord(i);
            // tensors an operator allocates before it throws would otherwise never be freed
            if (context.trackAllocations) context.trackAllocations();
            let operatorOutputs;
            try {
              operatorOutputs = await operator.run(context, operatorInputs, node.output.length);
            } catch (error) {
              if (context.releaseTracked) context.releaseTracked();
              throw error;
            } finally {
              if (context.stopTracking) context.stopTracking();
              if (branches && node.hipSide) hip.native.branchEnd();
            }
            actualInputDims = operatorInputs.map((t) => t.dims);
            actualOutputDims = operatorOutputs.map((t) => t.dims);
            for (let j = 0; j < node.output.length; j++) {
              tensorsForBackends[operatorOutputs[j].backend].set(node.output[j], operatorOutputs[j]);
            }
            actualBackend = operator.backend;
            break;
          } catch (error) {
            if (firstTry && !strict && !(backendOrderForNode.length === 1 && backendOrderForNode[0] === "cpu")) {
              logger.warn(`Failed to run ${node.name}. Retrying on cpu.`, error);
              firstTry = false;
              backendOrderForNode = ["cpu"];
              stats.retriedOnCpu.push(node.name);
              continue;
            }
            throw error;
          }
        }

        stats.nodesByBackend[actualBackend] = (stats.nodesByBackend[actualBackend] || 0) + 1;
        for (const name of tensorReleaseTiming.get(node.name) || []) {
          for (const backend of backends) {
            const t = tensorsForBackends[backend].get(name);
            if (t) {
              t.dispose();
              tensorsForBackends[backend].delete(name);
            }
          }
        }
        nodePerformances.push({
          opType: node.opType,
          name: node.name,
          backend: actualBackend,
          inputDims: actualInputDims,
          outputDims: actualOutputDims,
          elapsed: Date.now() - nodeStartTime,
        });
      }

      // host time of the node loop: everything is enqueued, nothing has been waited for yet
      stats.enqueueMs = Number(process.hrtime.bigint() - runStart) / 1e6;
      const outputs = [];
      for (const outputInfo of graph.output) {
        let outputTensor = tensorsForBackends.cpu.get(outputInfo.name);
        if (!outputTensor && opts.capture) {
          // recorded, not computed yet: the tensor stays on the device for the replays
          for (const otherBackend of this.backendOrder) {
            const otherT = tensorsForBackends[otherBackend].get(outputInfo.name);
            if (otherT) {
              outputTensor = otherT;
              callerOwned.add(otherT);
              break;
            }
          }
        }
        if (!outputTensor) {
          for (const otherBackend of this.backendOrder) {
            const otherT = tensorsForBackends[otherBackend].get(outputInfo.name);
            if (otherT) {
              // device -> host: the only point where the run waits for the GPU
              outputTensor = await this.backendContexts.cpu.moveTensor(otherT, {});
              tensorsForBackends.cpu.set(outputInfo.name, outputTensor);
              break;
            }
          }
        }
        if (!outputTensor) throw new Error(`Output ${outputInfo.name} not found`);
        outputs.push(outputTensor);
      }

      if (opts.measurePerformance) {
        if (useEvents) {
          hip.native.eventRecord(nodePerformances.length);
          for (let i = 0; i < nodePerformances.length; i++) {
            if (nodePerformances[i].backend === "hip") {
              nodePerformances[i].deviceElapsed = hip.native.eventElapsedMs(i, i + 1);
            }
          }
        }
        this.lastPerformance = nodePerformances;
        logger.debug("Performance", nodePerformances);
      }
      this.lastRunStats = stats;
      return outputs;
    } finally {
      // device copies of initializers stay for the next run; every other device tensor goes
      for (const backend of backendsWithoutCPU) {
        for (const [name, t] of tensorsForBackends[backend].entries()) {
          if (this.initializerTensors.has(name) && this.copiedInitializerTensors.has(backend)) {
            this.copiedInitializerTensors.get(backend).set(name, t);
          } else if (!callerOwned.has(t)) {
            t.dispose();
          }
        }
      }
    }
  }
}

module.exports = { RunnerImpl };
