"use strict";
// Contract after src/descriptor_runner/operators/base/flatten.ts:6-17.
const { OperatorImpl } = require("../operatorImpl");
const { getAttrInt } = require("../operatorUtil");
const { flattened } = require("../shapes");

class Flatten extends OperatorImpl {
  initialize(attribute) {
    super.initialize(attribute);
    if (getAttrInt(attribute, "axis", 1) !== 1) throw new Error("Flatten: only axis === 1 is supported");
  }

  calcShape(input) {
    return flattened(input.dims);
  }
}
module.exports = { Flatten };
