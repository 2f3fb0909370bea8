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
const { tensorProtoToArray } = require("../operators/operatorUtil");

const logger = getLogger("WebDNN.modelTransform");

function modelTransform(model, backendOrder, options) {
  renameDuplicatedNode(model);
  const opt = options || {};
  if (backendOrder.includes("hip") && opt.fuse !== false) {
    fuseForHip(model);
  }
  if (backendOrder.includes("hip") && opt.sideBranches !== false) {
    hoistSideBranches(model.graph);
  }
}

// Side branches.  A convolution whose inputs are ready well before its turn -- the projection shortcut of a
// residual block reads the block's input, and only the block's last convolution wants its result -- is moved
// up to where its inputs become ready and marked `hipSide`; the first node that reads its result is marked
// `hipJoin`.  The runner brackets a hipSide node with branchBegin / branchEnd and calls branchJoin before a
// hipJoin node, so that a recorded run may execute the shortcut next to the convolutions it used to wait
// behind (one launch then fills what the other leaves idle at its start and its end).  The nodes in between
// come before the moved node in the original order, so none of them reads its result.  One branch at a time.
// An eager run executes the new order on one stream: the same kernels on the same data, the same bits.
const SIDE_BRANCH_OPS = new Set(["Conv", "WebDNNHipFusedConv"]);
function hoistSideBranches(graph) {
  const order = [];
  const producedAt = new Map(); // tensor name -> index in `order` of its producer
  let pending = null; // outputs of the branch waiting for its join
  let barrier = 0; // no branch starts before the last join
  let count = 0;
  const place = (node, at) => {
    order.splice(at, 0, node);
    for (let i = at; i < order.length; i++) for (const name of order[i].output) producedAt.set(name, i);
  };
  for (const node of graph.node) {
    if (pending && node.input.some((name) => pending.has(name))) {
      node.hipJoin = true;
      pending = null;
      barrier = order.length;
    }
    if (!pending && !node.hipJoin && SIDE_BRANCH_OPS.has(node.opType)) {
      let ready = barrier;
      for (const name of node.input) if (producedAt.has(name)) ready = Math.max(ready, producedAt.get(name) + 1);
      const between = order.slice(ready);
      if (between.length >= 2 && between.every((n) => SIDE_BRANCH_OPS.has(n.opType))) {
        node.hipSide = true;
        pending = new Set(node.output);
        place(node, ready);
        count++;
        continue;
      }
    }
    place(node, order.length);
  }
  if (pending) {
    // nobody reads the branch's result (a graph output): it is joined at the end of the run anyway
    for (const n of order) if (n.hipSide && n.output.some((name) => pending.has(name))) delete n.hipSide;
  }
  if (count) {
    graph.node = order;
    logger.info(`hip: ${count} convolutions run as side branches of recorded runs`);
  }
  return count;
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

function intsAttr(name, values) {
  return { name, type: AttributeType.INTS, floats: [], ints: values.slice(), strings: [] };
}

function floatAttr(name, value) {
  return { name, f: value, type: AttributeType.FLOAT, floats: [], ints: [], strings: [] };
}

function stringAttr(name, value) {
  return { name, s: Buffer.from(value, "utf-8"), type: AttributeType.STRING, floats: [], ints: [], strings: [] };
}

// Conv [+ Add(residual)] [+ Relu]  ->  WebDNNHipFusedConv
// [Transpose ->] MatMul [* constant scalar] [+ Add(bias)] [+ Add(residual)] [+ Relu | -> Transpose]
//                                                                        ->  WebDNNHipFusedMatMul
// A link of the chain is absorbed only when the tensor between the two nodes has no other
// reader, so no intermediate tensor that something else reads disappears.  The fused node
// takes the place of the chain's last node: everything it reads has been produced by then.
//
// What the MatMul forms cost nothing to absorb (the kernel already has the means):
//   a Transpose that feeds only this MatMul   -> the operand is read through permuted strides
//   a Mul by a one-element constant           -> the product's alpha (the accumulator is fp32,
//                                                so f32(alpha * acc) is what the Mul would store)
//   a Transpose(1,0,2) of the rank-3 result   -> the rows are written where the Transpose
//                                                would have put them
// which is the whole head split / scale / head merge of an attention block.
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
  const producerOf = new Map(); // tensor name -> index of the node that writes it
  nodes.forEach((node, idx) => {
    for (const name of node.input) if (consumers.get(name) === 1) readerOf.set(name, idx);
    for (const name of node.output) producerOf.set(name, idx);
  });
  const permOf = (node) => {
    const attr = node.attribute.find((a) => a.name === "perm");
    return attr && attr.ints ? attr.ints.map(Number) : [];
  };
  // value of a one-element float constant of rank 0 or 1, or null (a [1,1,1,1] constant would raise
  // the rank of the product it multiplies, which the fused node does not)
  const scalarConstant = (name) => {
    const init = initializers.get(name);
    if (!init || init.dims.length > 1) return null;
    let t;
    try {
      t = tensorProtoToArray(init);
    } catch (e) {
      return null;
    }
    return t.dataType === "float32" && t.data.length === 1 ? t.data[0] : null;
  };

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
    let alpha = null;
    const perms = { a: [], b: [], y: [] };
    let tail = i; // index of the last absorbed node
    let cur = head.output[0];
    const absorbed = [];
    const onlyReader = (name) => {
      const idx = readerOf.get(name);
      return idx !== undefined && !removed.has(idx) ? idx : undefined;
    };

    if (!isConv) {
      // Transpose -> operand
      ["a", "b"].forEach((which, k) => {
        const src = producerOf.get(inputs[k]);
        if (src === undefined || removed.has(src) || consumers.get(inputs[k]) !== 1) return;
        const t = nodes[src];
        const perm = permOf(t);
        if (t.opType !== "Transpose" || perm.length !== 3) return; // rank 3: [batch, rows, columns]
        perms[which] = perm;
        inputs[k] = t.input[0];
        absorbed.push(src);
      });
      // * constant scalar
      const next = onlyReader(cur);
      if (next !== undefined && nodes[next].opType === "Mul" && nodes[next].input.length === 2) {
        const mul = nodes[next];
        const other = mul.input[0] === cur ? mul.input[1] : mul.input[0];
        const value = other !== cur ? scalarConstant(other) : null;
        if (value !== null) {
          alpha = value;
          absorbed.push(next);
          tail = next;
          cur = mul.output[0];
        }
      }
    }
    // + Add (a constant vector after a MatMul: bias; an activation tensor: residual), twice at most:
    // bias first, then the residual, the order in which the epilogue adds them
    for (let round = 0; round < 2 && !hasResidual; round++) {
      const next = onlyReader(cur);
      if (next === undefined || nodes[next].opType !== "Add" || nodes[next].input.length !== 2) break;
      const add = nodes[next];
      const other = add.input[0] === cur ? add.input[1] : add.input[0];
      if (other === cur) break;
      const init = initializers.get(other);
      if (!isConv && !hasBias && init && init.dims.length <= 1) {
        inputs.push(other);
        hasBias = true;
      } else if (!init) {
        inputs.push(other);
        hasResidual = true;
      } else {
        break;
      }
      absorbed.push(next);
      tail = next;
      cur = add.output[0];
    }
    // + Relu
    let next = onlyReader(cur);
    if (next !== undefined && nodes[next].opType === "Relu") {
      activation = "Relu";
      absorbed.push(next);
      tail = next;
      cur = nodes[next].output[0];
    } else if (!isConv && next !== undefined && nodes[next].opType === "Transpose" && !hasBias && !hasResidual &&
      permOf(nodes[next]).join() === "1,0,2") {
      // -> Transpose(1,0,2): heads merged back
      perms.y = [1, 0, 2];
      absorbed.push(next);
      tail = next;
      cur = nodes[next].output[0];
    }
    if (absorbed.length === 0) continue;

    const extra = [
      intAttr("has_bias", hasBias ? 1 : 0),
      intAttr("has_residual", hasResidual ? 1 : 0),
      stringAttr("activation", activation),
    ];
    if (alpha !== null) extra.push(floatAttr("alpha", alpha));
    for (const which of ["a", "b", "y"]) if (perms[which].length) extra.push(intsAttr("perm_" + which, perms[which]));
    const fused = {
      input: inputs,
      output: [cur],
      name: nodes[tail].name,
      opType: isConv ? "WebDNNHipFusedConv" : "WebDNNHipFusedMatMul",
      attribute: head.attribute.concat(extra),
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
  return fusedCount + fuseAttention(graph) + fuseLayerNormAdd(graph) + groupLinears(graph);
}

// Neighbouring linear layers that do not read each other  ->  one WebDNNHipLinearGroup node.
// A linear layer here is a MatMul, or a fused MatMul that carries at most a bias and an
// activation (no operand permutation, scale or residual).  Only nodes that follow each
// other directly are grouped, so the order of everything else stays what it was; the group
// takes the place of its last member.
function groupLinears(graph) {
  const nodes = graph.node;
  const attr = (node, name) => node.attribute.find((a) => a.name === name);
  const flag = (node, name) => {
    const a = attr(node, name);
    return a && a.i !== undefined && a.i !== null ? Number(a.i) : 0;
  };
  const activationOf = (node) => {
    const a = attr(node, "activation");
    return a && a.s ? Buffer.from(a.s).toString("utf-8") : "";
  };
  const isLinear = (node) => {
    if (node.output.length !== 1) return false;
    if (node.opType === "MatMul") return node.input.length === 2 && node.input.every((n) => n !== "");
    if (node.opType !== "WebDNNHipFusedMatMul") return false;
    if (flag(node, "has_residual") || attr(node, "alpha")) return false;
    if (["perm_a", "perm_b", "perm_y"].some((name) => attr(node, name))) return false;
    return node.input.length === 2 + flag(node, "has_bias");
  };
  const result = [];
  let groups = 0;
  let i = 0;
  while (i < nodes.length) {
    if (!isLinear(nodes[i])) {
      result.push(nodes[i++]);
      continue;
    }
    const run = [nodes[i]];
    const produced = new Set(nodes[i].output);
    const activation = activationOf(nodes[i]);
    let j = i + 1;
    while (j < nodes.length && run.length < 16 && isLinear(nodes[j]) && activationOf(nodes[j]) === activation &&
      !nodes[j].input.some((name) => produced.has(name))) {
      run.push(nodes[j]);
      produced.add(nodes[j].output[0]);
      j++;
    }
    if (run.length === 1) {
      result.push(nodes[i++]);
      continue;
    }
    result.push({
      input: [].concat(...run.map((n) => n.input)),
      output: run.map((n) => n.output[0]),
      name: run[run.length - 1].name,
      opType: "WebDNNHipLinearGroup",
      attribute: [intsAttr("arity", run.map((n) => n.input.length)), stringAttr("activation", activation)],
      domain: "webdnn.hip",
    });
    groups++;
    i = j;
  }
  if (groups > 0) {
    graph.node = result;
    logger.info(`hip fusion: ${groups} groups of neighbouring linear layers`);
  }
  return groups;
}

// LayerNormalization -> Add(other)  ->  WebDNNHipLayerNormAdd with two outputs
// (the normalised tensor, which the graph usually reads again, and the sum).  `other` must exist
// before the LayerNormalization runs: an initializer, a graph input or an earlier node's output.
// Of several Adds reading the result the first qualifies.  Float32 Adds only compute fl(y + p),
// which is what the kernel stores, so nothing about the numbers changes.
function fuseLayerNormAdd(graph) {
  const nodes = graph.node;
  const known = new Set(graph.initializer.map((t) => t.name));
  for (const input of graph.input) known.add(input.name);
  const removed = new Set();
  let count = 0;
  nodes.forEach((ln, li) => {
    if (ln.opType === "LayerNormalization" && ln.output.length === 1 && ln.input.length === 3 &&
      ln.input.every((n) => n !== "")) {
      const y = ln.output[0];
      const ai = nodes.findIndex((n, idx) => idx > li && !removed.has(idx) && n.opType === "Add" && n.input.length === 2 &&
        n.input.includes(y) && n.input[0] !== n.input[1] && known.has(n.input[0] === y ? n.input[1] : n.input[0]));
      if (ai >= 0) {
        const add = nodes[ai];
        const other = add.input[0] === y ? add.input[1] : add.input[0];
        nodes[li] = {
          input: ln.input.concat([other]),
          output: [y, add.output[0]],
          name: ln.name,
          opType: "WebDNNHipLayerNormAdd",
          attribute: ln.attribute,
          domain: "webdnn.hip",
        };
        removed.add(ai);
        count++;
      }
    }
    for (const name of nodes[li].output) known.add(name);
  });
  if (count > 0) {
    graph.node = nodes.filter((n, idx) => !removed.has(idx));
    logger.info(`hip fusion: ${count} LayerNormalization + Add pairs fused`);
  }
  return count;
}

// (Fused)MatMul -> Softmax -> (Fused)MatMul  ->  WebDNNHipAttention
// where the first product carries nothing but operand permutations and a scale, the Softmax
// normalises the last axis of its rank-3 result, and the second product takes the
// probabilities as they are (no permutation of its first operand), adds nothing and may
// write the merged-heads layout.  Both intermediate tensors must have no other reader.
// Runs after the MatMul chains have been fused, so the Transposes and the scale are
// already attributes of the two products.
function fuseAttention(graph) {
  const nodes = graph.node;
  const readers = new Map();
  const bump = (name) => readers.set(name, (readers.get(name) || 0) + 1);
  for (const node of nodes) for (const name of node.input) bump(name);
  for (const out of graph.output) bump(out.name);
  const producerOf = new Map();
  nodes.forEach((node, idx) => node.output.forEach((name) => producerOf.set(name, idx)));
  const attr = (node, name) => node.attribute.find((a) => a.name === name);
  const intOf = (node, name, dflt) => {
    const a = attr(node, name);
    return a && a.i !== undefined && a.i !== null ? Number(a.i) : dflt;
  };
  const intsOf = (node, name) => {
    const a = attr(node, name);
    return a && a.ints ? a.ints.map(Number) : [];
  };
  const stringOf = (node, name) => {
    const a = attr(node, name);
    return a && a.s ? Buffer.from(a.s).toString("utf-8") : "";
  };
  const isProduct = (node) => node.opType === "MatMul" || node.opType === "WebDNNHipFusedMatMul";
  const plain = (node) => node.input.length === 2 && intOf(node, "has_bias", 0) === 0 &&
    intOf(node, "has_residual", 0) === 0 && stringOf(node, "activation") === "";

  const removed = new Set();
  let count = 0;
  nodes.forEach((soft, si) => {
    if (soft.opType !== "Softmax" || soft.input.length !== 1 || soft.output.length !== 1) return;
    const axis = intOf(soft, "axis", -1);
    if (axis !== -1 && axis !== 2) return;
    const pi = producerOf.get(soft.input[0]);
    if (pi === undefined || removed.has(pi) || readers.get(soft.input[0]) !== 1) return;
    const scores = nodes[pi];
    if (!isProduct(scores) || !plain(scores) || intsOf(scores, "perm_y").length) return;
    if (readers.get(soft.output[0]) !== 1) return;
    const ci = nodes.findIndex((n, idx) => idx > si && !removed.has(idx) && n.input.includes(soft.output[0]));
    if (ci < 0) return;
    const ctx = nodes[ci];
    if (!isProduct(ctx) || !plain(ctx) || ctx.input[0] !== soft.output[0] || ctx.input[1] === soft.output[0]) return;
    if (intsOf(ctx, "perm_a").length || attr(ctx, "alpha")) return;
    const alphaAttr = attr(scores, "alpha");
    const extra = [intAttr("softmax_axis", axis)];
    if (alphaAttr) extra.push(floatAttr("alpha", alphaAttr.f));
    const perms = { perm_q: intsOf(scores, "perm_a"), perm_k: intsOf(scores, "perm_b"), perm_v: intsOf(ctx, "perm_b"),
      perm_y: intsOf(ctx, "perm_y") };
    for (const name of Object.keys(perms)) if (perms[name].length) extra.push(intsAttr(name, perms[name]));
    nodes[ci] = {
      input: [scores.input[0], scores.input[1], ctx.input[1]],
      output: ctx.output.slice(),
      name: ctx.name,
      opType: "WebDNNHipAttention",
      attribute: extra,
      domain: "webdnn.hip",
    };
    removed.add(pi);
    removed.add(si);
    count++;
  });
  if (count > 0) {
    graph.node = nodes.filter((n, idx) => !removed.has(idx));
    logger.info(`hip fusion: ${count} attention chains fused`);
  }
  return count;
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

module.exports = { modelTransform, findTensorReleaseTiming, fuseForHip, fuseAttention, fuseLayerNormAdd, groupLinears, hoistSideBranches };
