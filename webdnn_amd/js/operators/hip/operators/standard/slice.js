"use strict";
// Slice (opset >= 10): data on the device, starts/ends/axes/steps on the cpu; one strided
// copy whose source strides carry the steps.
// Semantics: src/descriptor_runner/operators/cpu/operators/standard/slice.ts:12-330.
const { Slice10 } = require("../../../base/slice");
const { calcStrides } = require("../../../operatorUtil");

class HipSlice10 extends Slice10 {
  constructor() {
    super("hip");
  }

  // eslint-disable-next-line no-unused-vars
  getTensorBackendRequirement(nInputs, nOutputs) {
    const req = [this.backend];
    for (let i = 1; i < nInputs; i++) req.push("cpu");
    return req;
  }

  async run(context, inputs) {
    const data = inputs[0];
    context.assertsHipTensor(data);
    for (let i = 1; i < inputs.length; i++) if (inputs[i]) context.cpuContext.assertsCPUTensor(inputs[i]);
    const ranges = this.calcRanges(data.dims, inputs[1], inputs[2], inputs[3], inputs[4]),
      outShape = ranges.map((r) => r.size),
      output = context.emptyTensor(outShape, data.dataType);
    if (output.length > 0) {
      const inStrides = calcStrides(data.dims);
      let offset = 0;
      ranges.forEach((r, d) => {
        offset += r.start * inStrides[d];
      });
      context.native.stridedCopy(data.handle, offset, output.handle, 0, outShape,
        ranges.map((r, d) => r.step * inStrides[d]), calcStrides(outShape));
    }
    return [output];
  }
}

function getOpEntries() {
  return [{ opType: "Slice", backend: "hip", opsetMin: 10, factory: () => new HipSlice10() }];
}
module.exports = { getOpEntries };
