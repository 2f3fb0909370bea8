"use strict";
// Operator registry: opType -> entries; choice of the implementation for a node.
// Reference: src/descriptor_runner/core/operatorTable.ts:1-69.
const registeredOperators = Object.create(null);

function registerOperator(entry) {
  if (!(entry.opType in registeredOperators)) registeredOperators[entry.opType] = [];
  registeredOperators[entry.opType].push(entry);
}

function registerOperators(entries) {
  for (const entry of entries) registerOperator(entry);
}

// Test hook: forget every registration.
function clearOperators() {
  for (const k of Object.keys(registeredOperators)) delete registeredOperators[k];
}

function instantiateOperator(opType, opset, backendOrder, currentTensorsBackends) {
  const entries = registeredOperators[opType];
  if (!entries) return null;

  let localBackendOrder = backendOrder;
  switch (opType) {
    case "Flatten":
    case "Pad":
    case "Reshape":
    case "Squeeze":
    case "Transpose":
    case "Unsqueeze":
      // Layout operators run where their data tensor already lives.  The scan has
      // no early exit, so when the tensor is on several backends the LAST one in
      // backendOrder wins (operatorTable.ts:41-46).
      for (const backend of backendOrder) {
        if (currentTensorsBackends[0].includes(backend)) localBackendOrder = [backend];
      }
      break;
    case "Shape":
      localBackendOrder = ["cpu"];
      break;
    default:
      break;
  }

  const pick = (order) => {
    for (const backend of order) {
      for (const entry of entries) {
        if (entry.backend !== backend) continue;
        if (entry.opsetMin > opset) continue;
        if (entry.opsetMax != null && entry.opsetMax <= opset) continue;
        return entry.factory();
      }
    }
    return null;
  };
  // A layout operator whose data sits on a backend without an implementation of it (a
  // model input reshaped before any device operator touched it: this package ships no cpu
  // Reshape) is placed by the ordinary order instead; the runner then moves the tensor.
  return pick(localBackendOrder) || (localBackendOrder !== backendOrder ? pick(backendOrder) : null);
}

module.exports = { registerOperators, instantiateOperator, clearOperators };
