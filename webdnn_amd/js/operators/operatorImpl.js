"use strict";
// Reference: src/descriptor_runner/operators/operatorImpl.ts:7-29.
class OperatorImpl {
  constructor(backend) {
    this.backend = backend;
  }

  // eslint-disable-next-line no-unused-vars
  initialize(attribute) {}

  // Backend each input must live on (null = anywhere); default: all on this operator's backend.
  // eslint-disable-next-line no-unused-vars
  getTensorBackendRequirement(nInputs, nOutputs) {
    const backends = [];
    for (let i = 0; i < nInputs; i++) backends.push(this.backend);
    return backends;
  }
}
module.exports = { OperatorImpl };
