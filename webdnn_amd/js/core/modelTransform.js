"use strict";
// Load-time graph rewrites and tensor release timing.
// Reference: src/descriptor_runner/core/modelTransform.ts:7-82 — modelTransform()
// is the designated (there still empty) hook for backend-specific rewrites; only the
// duplicate-node renaming is implemented there.  Here the hook also carries the hip
// fusion pass, in the manner of the reference's offline unary-chain fusion
// (src/graph_transpiler/webdnn/pass_fusion_unary.py:26-97): chains are replaced by one
// node of a backend-specific op type.
const { getLogger } = require("../logging");
const { AttributeType } = require("./onnxProto");

const logger = getLogger("WebDNN.modelTransform");

function modelTransform(model, backendOrder, options) {
  renameDuplicatedNode(model);
  const opt = options || {};
  if (backendOrder.includes("hip") && opt.fuse !== false) {
    fuseForHip(model);
  }
}

function renameDuplicatedNode(model) {
  const usedNames = new Set();
  for (const node of model.graph.node) {
    let origName = node.name;
    if (!origName) origName = "unnamed";
    if (usedNames.has(origName)) {
      let newName = origName + "_";
      while (usedNames.has(newName)) newName += "_";
      node.name = newName;
      usedNames.add(newName);
      logger.warn(`node name ${origName} is already used: renaming to ${newName}`);
    } else {
      node.name = origName;
      usedNames.add(origName);
    }
  }
}

function intAttr(name, value) {
  return { name, i: value, type: AttributeType.INT, floats: [], ints: [], strings: [] };
}

function stringAttr(name, value) {
  return { name, s: Buffer.from(value, "utf-8"), type: AttributeType.STRING, floats: [], ints: [], strings: [] };
}

// Conv [+ Add(residual)] [+ Relu]  ->  WebDNNHipFusedConv
// MatMul [+ Add(bias | residual)] [+ Relu]  ->  WebDNNHipFusedMatMul
// A link of the chain is absorbed only when its input has no other consumer, so no
// intermediate tensor that something else reads disappears.  The fused node takes the
// place of the chain's last node: everything it reads has been produced by then.
function fuseForHip(model) {
  const graph = model.graph;
  const nodes = graph.node;
  const consumers = new Map(); // tensor name -> number of readers (graph outputs count)
  const bump = (name) => consumers.set(name, (consumers.get(name) || 0) + 1);
  for (const node of nodes) for (const name of node.input) bump(name);
  for (const out of graph.output) bump(out.name);
  const initializers = new Map();
  for (const init of graph.initializer) initializers.set(init.name, init);

  const readerOf = new Map(); // tensor name -> index of its only reader
  nodes.forEach((node, idx) => {
    for (const name of node.input) if (consumers.get(name) === 1) readerOf.set(name, idx);
  });

  const removed = new Set();
  let fusedCount = 0;
  for (let i = 0; i < nodes.length; i++) {
    if (removed.has(i)) continue;
    const head = nodes[i];
    if (head.opType !== "Conv" && head.opType !== "MatMul") continue;
    if (head.output.length !== 1) continue;
    const isConv = head.opType === "Conv";
    const inputs = head.input.slice();
    if (inputs.some((n) => n === "")) continue; // optional input left empty: keep the plain node
    let hasBias = isConv && inputs.length > 2;
    let hasResidual = false;
    let activation = "";
    let tail = i; // index of the last absorbed node
    let cur = head.output[0];
    const absorbed = [];

    // + Add
    let next = readerOf.get(cur);
    if (next !== undefined && !removed.has(next) && nodes[next].opType === "Add" && nodes[next].input.length === 2) {
      const add = nodes[next];
      const other = add.input[0] === cur ? add.input[1] : add.input[0];
      if (other !== cur) {
        const init = initializers.get(other);
        if (!isConv && !hasBias && init && init.dims.length <= 1) {
          // MatMul + constant vector: a bias along the last axis
          inputs.push(other);
          hasBias = true;
          absorbed.push(next);
          tail = next;
          cur = add.output[0];
        } else if (!init) {
          // an activation tensor: residual connection
          inputs.push(other);
          hasResidual = true;
          absorbed.push(next);
          tail = next;
          cur = add.output[0];
        }
      }
    }
    // + Relu
    next = readerOf.get(cur);
    if (next !== undefined && !removed.has(next) && nodes[next].opType === "Relu") {
      activation = "Relu";
      absorbed.push(next);
      tail = next;
      cur = nodes[next].output[0];
    }
    if (absorbed.length === 0) continue;

    const fused = {
      input: inputs,
      output: [cur],
      name: nodes[tail].name,
      opType: isConv ? "WebDNNHipFusedConv" : "WebDNNHipFusedMatMul",
      attribute: head.attribute.concat([
        intAttr("has_bias", hasBias ? 1 : 0),
        intAttr("has_residual", hasResidual ? 1 : 0),
        stringAttr("activation", activation),
      ]),
      domain: "webdnn.hip",
    };
    removed.add(i);
    for (const a of absorbed) removed.add(a);
    removed.delete(tail);
    nodes[tail] = fused;
    fusedCount++;
  }
  if (fusedCount > 0) {
    graph.node = nodes.filter((n, idx) => !removed.has(idx));
    logger.info(`hip fusion: ${fusedCount} chains fused, ${removed.size} nodes removed`);
  }
  return fusedCount;
}

// For every node name, the tensors that can be disposed right after it has run.
function findTensorReleaseTiming(model, initializerTensorNames) {
  const lastReferencedAt = new Map(),
    graph = model.graph;
  for (const node of graph.node) {
    for (const inputName of node.input) lastReferencedAt.set(inputName, node.name);
  }
  // optimized models load tensors from outside graph.initializer: use the names actually loaded
  for (const name of initializerTensorNames) lastReferencedAt.delete(name);
  for (const input of graph.input) lastReferencedAt.delete(input.name);
  for (const output of graph.output) lastReferencedAt.delete(output.name);
  const timing = new Map();
  for (const [name, last] of lastReferencedAt.entries()) {
    const t = timing.get(last) || [];
    t.push(name);
    timing.set(last, t);
  }
  return timing;
}

module.exports = { modelTransform, findTensorReleaseTiming, fuseForHip };
