"use strict";
// Operator registry and the choice of an implementation for a node.
// Behaviour after src/descriptor_runner/core/operatorTable.ts:1-69: an entry serves opsets
// [opsetMin, opsetMax); the first backend of the node's order that has a serving entry wins;
// layout operators follow their data; Shape always runs on the cpu.
const registry = new Map(); // opType -> entries in registration order

function registerOperators(entries) {
  for (const entry of entries) {
    if (!registry.has(entry.opType)) registry.set(entry.opType, []);
    registry.get(entry.opType).push(entry);
  }
}

// Test hook: forget every registration.
function clearOperators() {
  registry.clear();
}

// A layout operator (it moves no arithmetic, only indices) runs on a backend that already
// holds its data tensor.  When several do, the one named LAST in the order is taken: the
// reference scans the order without stopping at the first hit (operatorTable.ts:41-46).
function whereTheDataIs(order, holdersOfInput0) {
  const holding = order.filter((backend) => holdersOfInput0.includes(backend));
  return holding.length ? [holding[holding.length - 1]] : order;
}

const PLACEMENT_RULES = {
  Flatten: whereTheDataIs,
  Pad: whereTheDataIs,
  Reshape: whereTheDataIs,
  Squeeze: whereTheDataIs,
  Transpose: whereTheDataIs,
  Unsqueeze: whereTheDataIs,
  Shape: () => ["cpu"], // graph metadata, consumed by the host
};

function serves(entry, opset) {
  return entry.opsetMin <= opset && (entry.opsetMax == null || opset < entry.opsetMax);
}

function build(entries, order, opset) {
  for (const backend of order) {
    const entry = entries.find((e) => e.backend === backend && serves(e, opset));
    if (entry) return entry.factory();
  }
  return null;
}

function instantiateOperator(opType, opset, backendOrder, currentTensorsBackends) {
  const entries = registry.get(opType);
  if (!entries) return null;
  const rule = PLACEMENT_RULES[opType];
  const placed = rule ? rule(backendOrder, currentTensorsBackends[0] || []) : backendOrder;
  // A layout operator whose data sits on a backend without an implementation of it (a model
  // input reshaped before any device operator touched it: this package ships no cpu Reshape) is
  // placed by the ordinary order instead; the runner then moves the tensor.
  return build(entries, placed, opset) || (placed !== backendOrder ? build(entries, backendOrder, opset) : null);
}

module.exports = { registerOperators, instantiateOperator, clearOperators };
