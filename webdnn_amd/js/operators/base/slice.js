"use strict";
// Slice, opset >= 10: starts / ends / axes / steps are input tensors.
// Reference: src/descriptor_runner/operators/cpu/operators/standard/slice.ts:12-58
// (range resolution; the reference has no base class for it).  Its clamping is kept
// as it is: start to [0, size-1] and stop to [-1, size] whatever the sign of the step.
const { OperatorImpl } = require("../operatorImpl");

class Slice10 extends OperatorImpl {
  // -> per axis {start, step, size} of the result
  calcRanges(dims, starts, ends, axesTensor, stepsTensor) {
    const ndim = dims.length;
    if (ndim > 6) throw new Error(`Slice: input dimension ${ndim} > 6 is not yet supported`);
    let axes;
    if (axesTensor) axes = Array.from(axesTensor.data).map((a) => (a < 0 ? a + ndim : a));
    else axes = dims.map((_, i) => i);
    const steps = stepsTensor ? Array.from(stepsTensor.data) : axes.map(() => 1);
    const ranges = dims.map((d) => [0, d, 1]);
    for (let i = 0; i < axes.length; i++) {
      if (!(axes[i] >= 0 && axes[i] < ndim)) throw new Error("Slice: axis out of range");
      if (steps[i] === 0) throw new Error("Slice: step 0");
      ranges[axes[i]] = [starts.data[i], ends.data[i], steps[i]];
    }
    return ranges.map(([start0, stop0, step], d) => {
      const srcsize = dims[d];
      let start = start0 < 0 ? start0 + srcsize : start0;
      start = Math.max(Math.min(start, srcsize - 1), 0);
      let stop = stop0 < 0 ? stop0 + srcsize : stop0;
      stop = Math.max(Math.min(stop, srcsize), -1);
      return { start, step, size: Math.max(Math.ceil((stop - start) / step), 0) };
    });
  }
}
module.exports = { Slice10 };
