"use strict";
// Entry point of the Node.js host: WebDNN.load(directory, options) -> Runner.
// Reference: src/descriptor_runner/index.ts:23-149 with a "hip" case in the backend
// switch and backendOptions.hip; default backendOrder is ["hip", "cpu"].
const { WebDNNCPUContextImpl } = require("./backend/cpu/cpuContextImpl");
const { CPUTensorImpl } = require("./backend/cpu/cpuTensorImpl");
const { WebDNNHipContextImpl } = require("./backend/hip/hipContextImpl");
const { RunnerImpl } = require("./core/runnerImpl");
const { registerOperators } = require("./core/operatorTable");
const { getOpEntries: getOpEntriesCPU } = require("./operators/cpu/opEntriesStandard");
const { getOpEntries: getOpEntriesHip } = require("./operators/hip/opEntriesStandard");
const Logging = require("./logging");

const logger = Logging.getLogger("WebDNN.load");

const defaultContexts = { cpu: null, hip: null };

// options: { backendOrder?, backendOptions?: { hip?: {device, strict, fuse, graph, contractionTile, splitK} },
//            onnxBaseName?, optimized? }
async function load(directory, options) {
  const opts = options || {};
  const backendOrder = opts.backendOrder || ["hip", "cpu"];
  const hipOption = (opts.backendOptions && opts.backendOptions.hip) || {};
  if (!defaultContexts.cpu) {
    defaultContexts.cpu = new WebDNNCPUContextImpl();
    await defaultContexts.cpu.initialize();
    registerOperators(getOpEntriesCPU());
  }
  const cpuContext = defaultContexts.cpu,
    backendContexts = { cpu: cpuContext };
  let succeedBackend = null;
  for (const tryBackend of backendOrder) {
    switch (tryBackend) {
      case "cpu":
        succeedBackend = "cpu";
        break;
      case "hip":
        if (!defaultContexts.hip) {
          try {
            const ctx = new WebDNNHipContextImpl(cpuContext, hipOption);
            await ctx.initialize();
            defaultContexts.hip = ctx;
            registerOperators(getOpEntriesHip());
            succeedBackend = "hip";
            backendContexts.hip = ctx;
          } catch (error) {
            // no GPU / no library: fall through to the next backend, like index.ts:68-79
            logger.info(`hip backend is not available: ${error.message}`);
            if (hipOption.strict) throw error;
          }
        } else {
          succeedBackend = "hip";
          backendContexts.hip = defaultContexts.hip;
        }
        break;
      default:
        throw new Error(`Unknown backend ${tryBackend}`);
    }
    if (succeedBackend) break;
  }
  if (!succeedBackend) throw new Error("No backend available");
  const actualBackendOrder = succeedBackend === "cpu" ? ["cpu"] : [succeedBackend, "cpu"];
  const runner = new RunnerImpl(actualBackendOrder, backendContexts, {
    strict: !!hipOption.strict,
    fuse: hipOption.fuse,
    graph: hipOption.graph, // true | false | "auto" (default): see RunnerImpl.run
    inFlight: hipOption.inFlight, // 2 (default) .. 4: lanes runner.submit alternates over
    sideBranches: hipOption.sideBranches, // false: keep the graph's node order (no side branches in recorded runs)
  });
  // An optimized-model directory holds one graph per backend, named after it, and keeps the
  // weights in WDN2 tensor files (separateBuild/coreOnly.ts:200-204).
  const baseName = opts.onnxBaseName || (opts.optimized ? `model-${succeedBackend}.onnx` : "model.onnx");
  await runner.loadModel(directory, baseName);
  return runner;
}

// Test hook: forget the cached contexts (a fresh load() then initialises again).
function resetDefaultContexts() {
  defaultContexts.cpu = null;
  defaultContexts.hip = null;
}

module.exports = { load, CPUTensor: CPUTensorImpl, Logging, resetDefaultContexts };
