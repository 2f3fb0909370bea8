"use strict";
// ReduceMean over any set of axes (all axes when none are given).
// Semantics: src/descriptor_runner/operators/cpu/operators/standard/reduce.ts:40-131, 369-405:
// the axes are reduced one after the other in ascending order, every pass a sum in double
// stored as float32, the last pass divided by the product of the reduced extents.
const { OperatorImpl } = require("../../../operatorImpl");
const { getAttrInt, getAttrInts } = require("../../../operatorUtil");
const { elementCount } = require("../../../shapes");

class HipReduceMean extends OperatorImpl {
  constructor() {
    super("hip");
  }

  initialize(attribute) {
    super.initialize(attribute);
    this.axes = getAttrInts(attribute, "axes", []);
    this.keepdims = getAttrInt(attribute, "keepdims", 1) !== 0;
  }

  async run(context, inputs) {
    context.assertsHipTensorArray(inputs);
    const input = inputs[0];
    if (input.dataType !== "float32") throw new Error("ReduceMean: only float32 is supported");
    const rank = input.ndim;
    const axes = (this.axes.length ? this.axes.map((a) => (a < 0 ? a + rank : a)) : input.dims.map((_, i) => i)).sort((a, b) => a - b);
    if (axes.some((a, i) => !(a >= 0 && a < rank) || (i > 0 && a === axes[i - 1]))) {
      throw new Error("ReduceMean: axes out of range or repeated");
    }
    const shape = input.dims.slice();
    let current = input,
      reduced = 1;
    axes.forEach((axis, pass) => {
      const extent = shape[axis];
      reduced *= extent;
      const outer = elementCount(shape.slice(0, axis)),
        inner = elementCount(shape.slice(axis + 1));
      shape[axis] = 1;
      const next = context.emptyTensor(shape, "float32");
      context.native.reduceAxis(current.handle, next.handle, outer, extent, inner, pass === axes.length - 1 ? reduced : 1);
      if (current !== input) current.dispose();
      current = next;
    });
    if (current === input) return [input.alias(input.dims)]; // rank 0
    if (this.keepdims) return [current];
    const squeezed = current.alias(shape.filter((_, i) => !axes.includes(i)));
    current.dispose();
    return [squeezed];
  }
}

function getOpEntries() {
  return [{ opType: "ReduceMean", backend: "hip", opsetMin: 1, opsetMax: 18, factory: () => new HipReduceMean() }];
}
module.exports = { getOpEntries };
