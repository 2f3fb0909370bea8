#!/usr/bin/env node
"use strict";
// Runs an ONNX model directory through the descriptor runner from the command line.
//
//   node run_model.js --model DIR [--onnx model.onnx | --optimized] [--backend hip|cpu]
//        --inputs a.bin[,b.bin...] --output out.bin
//        [--strict] [--no-fuse] [--no-side-branches] [--warmup W] [--runs N] [--measure [--queue-ahead MS]] [--measure-all]
//        [--resident-inputs] [--cpu-entries module.js] [--native module.js]
//        [--graph | --no-graph] [--in-flight [N]] [--alt-inputs a2.bin[,b2.bin...]]
//
// Inputs are raw little-endian files (float32, or int32 where the graph input says
// so) in the order of the graph's non-initializer inputs; outputs are written the same
// way, concatenated.  One JSON line on stdout reports output dims, per-run wall times,
// the per-backend node counts of the last run and, with --measure, per-node device
// times.  --cpu-entries registers extra cpu OperatorEntry objects exported by a module
// (getOpEntries()); parity tests and the CPU baseline pass the CPU restatement of the
// reference operators that way, the product itself ships hot-path operators for hip only.
//
// --graph passes {graph: true} to runner.run: the second call records the run into a HIP graph,
// later calls replay it.  --no-graph passes {graph: false}: every run walks the node loop.  With
// neither, runner.run gets no option, as from a caller written for the reference: the runner's
// default ("auto") records the third run with inputs of one signature and replays it afterwards.
// --alt-inputs names a second set of input files used by every other
// run (odd run numbers), so that replays see changing data.
// --in-flight [N] keeps N (2 unless given, at most 4) runs in flight: run i+1 is submitted (runner.submit) before
// the outputs of run i+2-N are collected (runner.collect).  msPerRun[i] is then the time from one submission to the next, the last
// entry including the wait for the last run's outputs; the output file holds the last run's outputs.
//
// Methodology follows the reference's harness (example/benchmark/runner/bench.js:130-167):
// warm-up runs, then timed runner.run() calls.
const fs = require("fs");
const path = require("path");
const WebDNN = require("../index");
const { registerOperators } = require("../core/operatorTable");

function parseArgs(argv) {
  const args = { backend: "hip", warmup: 0, runs: 1, onnx: null };
  for (let i = 2; i < argv.length; i++) {
    const a = argv[i];
    const next = () => {
      if (i + 1 >= argv.length) throw new Error(`${a} needs a value`);
      return argv[++i];
    };
    if (a === "--model") args.model = next();
    else if (a === "--onnx") args.onnx = next();
    else if (a === "--optimized") args.optimized = true;
    else if (a === "--graph") args.graph = true;
    else if (a === "--no-graph") args.graph = false;
    else if (a === "--in-flight") {
      // optional count: --in-flight 3
      args.inFlight = i + 1 < argv.length && /^[0-9]+$/.test(argv[i + 1]) ? parseInt(argv[++i], 10) : 2;
    }
    else if (a === "--alt-inputs") args.altInputs = next().split(",");
    else if (a === "--backend") args.backend = next();
    else if (a === "--inputs") args.inputs = next().split(",").filter((s) => s.length);
    else if (a === "--output") args.output = next();
    else if (a === "--strict") args.strict = true;
    else if (a === "--no-fuse") args.noFuse = true;
    else if (a === "--no-side-branches") args.noSideBranches = true;
    else if (a === "--check-each") args.checkEach = true;
    else if (a === "--warmup") args.warmup = parseInt(next(), 10);
    else if (a === "--runs") args.runs = parseInt(next(), 10);
    else if (a === "--queue-ahead") args.queueAhead = parseFloat(next());
    else if (a === "--measure-all") args.measureAll = true;
    else if (a === "--measure") args.measure = true;
    else if (a === "--cpu-entries") args.cpuEntries = next();
    else if (a === "--tile") args.tile = parseInt(next(), 10);
    else if (a === "--resident-inputs") args.residentInputs = true;
    else if (a === "--native") args.native = next();
    else throw new Error(`unknown argument ${a}`);
  }
  if (!args.model) throw new Error("--model is required");
  return args;
}

async function main() {
  const args = parseArgs(process.argv);
  if (args.cpuEntries) registerOperators(require(path.resolve(args.cpuEntries)).getOpEntries());
  const hipOption = { strict: !!args.strict, fuse: !args.noFuse };
  if (args.tile != null) hipOption.contractionTile = args.tile;
  if (args.inFlight) hipOption.inFlight = args.inFlight;
  if (args.noSideBranches) hipOption.sideBranches = false;
  // --native: another implementation of the addon's interface (host tests without a GPU)
  if (args.native) hipOption.native = require(path.resolve(args.native));
  const runner = await WebDNN.load(args.model, {
    backendOrder: args.backend === "cpu" ? ["cpu"] : ["hip", "cpu"],
    backendOptions: { hip: hipOption },
    onnxBaseName: args.onnx,
    optimized: !!args.optimized,
  });
  if (args.backend === "hip" && runner.backendName !== "hip") {
    throw new Error("hip backend was requested but is not available");
  }
  const graphInputs = runner.inputsWithoutInitializer;
  const files = args.inputs || [];
  if (files.length !== graphInputs.length) {
    throw new Error(`model has ${graphInputs.length} inputs, ${files.length} files given`);
  }
  const readInputs = (paths) => graphInputs.map((gi, idx) => {
    const tt = gi.type.tensorType;
    const dims = tt.shape.dim.map((d) => d.dimValue);
    const dataType = tt.elemType === 1 ? "float32" : "int32";
    const buf = fs.readFileSync(paths[idx]);
    const Ctor = dataType === "float32" ? Float32Array : Int32Array;
    const copy = new Uint8Array(buf.byteLength);
    copy.set(buf);
    const data = new Ctor(copy.buffer, 0, copy.byteLength / 4);
    const expect = dims.reduce((a, b) => a * b, 1);
    if (data.length !== expect) throw new Error(`${paths[idx]}: ${data.length} elements, graph input needs ${expect}`);
    return new WebDNN.CPUTensor(dims, dataType, data);
  });
  const inputs = readInputs(files);
  const altInputs = args.altInputs ? readInputs(args.altInputs) : null;

  // --resident-inputs: upload the inputs once; the timed runs then start with their data in HBM
  let runInputs = inputs,
    runAltInputs = altInputs;
  if (args.residentInputs && runner.backendName === "hip") {
    runInputs = [];
    for (const t of inputs) runInputs.push(await runner.backendContexts.hip.moveTensor(t, {}));
    if (altInputs) {
      runAltInputs = [];
      for (const t of altInputs) runAltInputs.push(await runner.backendContexts.hip.moveTensor(t, {}));
    }
    runner.backendContexts.hip.sync();
  }
  // --check-each: every timed run's outputs are compared, byte for byte, with the first outputs seen for the
  // same input set (even runs: --inputs, odd runs: --alt-inputs); the report counts the runs that differ
  const firstSeen = [null, null];
  let mismatchedRuns = 0, checkedRuns = 0;
  const checkRun = (index, outs) => {
    if (!args.checkEach) return;
    const which = runAltInputs && index % 2 === 1 ? 1 : 0;
    const bytes = outs.map((t) => Buffer.from(t.data.buffer, t.data.byteOffset, t.data.byteLength));
    if (!firstSeen[which]) {
      firstSeen[which] = bytes.map((b) => Buffer.from(b));
      return;
    }
    checkedRuns++;
    if (bytes.length !== firstSeen[which].length || bytes.some((b, k) => !b.equals(firstSeen[which][k]))) mismatchedRuns++;
  };
  const runOptions = (extra) => (args.graph === undefined ? extra : Object.assign({ graph: args.graph }, extra));
  for (let i = 0; i < args.warmup; i++) await runner.run(runInputs, runOptions({}));
  const times = [];
  let outputs = null;
  let queueAhead = null;
  const deviceTimes = [];
  if (args.inFlight) {
    const pending = []; // [run index, ticket] in order of submission, at most args.inFlight - 1 while the next is submitted
    let t0 = process.hrtime.bigint();
    for (let i = 0; i < args.runs; i++) {
      pending.push([i, await runner.submit(runAltInputs && i % 2 === 1 ? runAltInputs : runInputs, runOptions({}))]);
      while (pending.length >= args.inFlight || (i + 1 === args.runs && pending.length)) {
        const [index, ticket] = pending.shift();
        outputs = await runner.collect(ticket);
        checkRun(index, outputs);
      }
      const t1 = process.hrtime.bigint();
      times.push(Number(t1 - t0) / 1e6);
      t0 = t1;
    }
  }
  for (let i = 0; i < (args.inFlight ? 0 : args.runs); i++) {
    // --queue-ahead MS (with --measure): put about MS milliseconds of streaming kernels on the
    // device queue first, so that the measured run's launches are all queued before the device
    // reaches them.  Its kernels then run back to back and the per-node events time the device
    // alone, not the host's enqueue rate.
    if (args.queueAhead && args.measure && i === args.runs - 1 && runner.backendName === "hip") {
      const hip = runner.backendContexts.hip;
      const n = 128 * 1024 * 1024; // floats: 0.5 GiB in, 0.5 GiB out per launch
      const a = hip.emptyTensor([n], "float32"), b = hip.emptyTensor([n], "float32");
      hip.native.unary(0, 0, a.handle, b.handle, n); // touch both buffers once
      hip.sync();
      const reps = Math.max(1, Math.ceil(args.queueAhead / 0.2));
      hip.native.eventRecord(4094);
      for (let r = 0; r < reps; r++) hip.native.unary(0, 0, a.handle, b.handle, n);
      hip.native.eventRecord(4095);
      queueAhead = { launches: reps, tensors: [a, b] };
    }
    const t0 = process.hrtime.bigint();
    outputs = await runner.run(runAltInputs && i % 2 === 1 ? runAltInputs : runInputs,
      runOptions({ measurePerformance: !!args.measureAll || (!!args.measure && i === args.runs - 1) }));
    times.push(Number(process.hrtime.bigint() - t0) / 1e6);
    checkRun(i, outputs);
    // --measure-all: device time of every timed run (HIP events on the library's stream; a replayed
    // graph is bracketed by one pair, an eager run has one event per node boundary)
    if (args.measureAll && runner.lastPerformance) {
      deviceTimes.push(runner.lastPerformance.reduce((acc, p) => acc + (p.deviceElapsed || 0), 0));
    }
  }
  if (args.output) {
    const fd = fs.openSync(args.output, "w");
    for (const t of outputs) {
      const d = t.data;
      fs.writeSync(fd, Buffer.from(d.buffer, d.byteOffset, d.byteLength));
    }
    fs.closeSync(fd);
  }
  const report = {
    backend: runner.backendName,
    outputs: outputs.map((t, i) => ({ name: runner.getOutputNames()[i], dims: t.dims, dataType: t.dataType })),
    msPerRun: times,
    deviceMsPerRun: args.measureAll ? deviceTimes : undefined,
    stats: runner.lastRunStats,
    nodes: runner.model.graph.node.length,
    checkEach: args.checkEach ? { checkedRuns, mismatchedRuns } : undefined,
    node: process.version,
    graph: args.graph !== false ? { captured: !!runner.graphState, lanes: (runner.graphState ? 1 : 0) + runner.sideGraphStates.filter((st) => st).length,
      unsupported: runner.graphUnsupported } : undefined,
  };
  runner.disposeGraph();
  if (queueAhead) {
    // the queued work must have outlasted the host's enqueue of the measured run
    report.queueAhead = { launches: queueAhead.launches, deviceMs: runner.backendContexts.hip.native.eventElapsedMs(4094, 4095) };
    for (const t of queueAhead.tensors) t.dispose();
  }
  if (args.measure && runner.lastPerformance) {
    report.performance = runner.lastPerformance.map((p) => ({
      name: p.name, opType: p.opType, backend: p.backend, outputDims: p.outputDims,
      elapsed: p.elapsed, deviceElapsed: p.deviceElapsed,
    }));
  }
  if (runner.backendContexts.hip && runner.backendContexts.hip.initialized) {
    const hip = runner.backendContexts.hip;
    report.device = hip.deviceInfo();
    report.memory = hip.memStats();
    if (hip.native.__liveBuffers) {
      report.liveBuffers = hip.native.__liveBuffers();
      report.nativeCalls = hip.native.__calls();
      report.initializerCopies = Array.from(runner.copiedInitializerTensors.get("hip").keys()).length;
    }
  }
  // the library gives its device memory, stream and staging buffers back before the process ends
  if (runner.backendContexts.hip && runner.backendContexts.hip.initialized && runner.backendContexts.hip.native.shutdown) {
    runner.backendContexts.hip.native.shutdown();
  }
  process.stdout.write(JSON.stringify(report) + "\n", () => process.exit(0));
}

main().catch((e) => {
  process.stderr.write(`run_model: ${e && e.stack ? e.stack : e}\n`);
  process.exit(1);
});
