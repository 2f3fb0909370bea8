"use strict";
// Reference: src/descriptor_runner/operators/base/flatten.ts:6-17.
const { OperatorImpl } = require("../operatorImpl");
const { getAttrInt } = require("../operatorUtil");
const { arrayProd } = require("../../util");

class Flatten extends OperatorImpl {
  initialize(attribute) {
    super.initialize(attribute);
    const axis = getAttrInt(attribute, "axis", 1);
    if (axis !== 1) throw new Error("Flatten: only axis === 1 is supported");
  }

  calcShape(input) {
    return [input.dims[0], arrayProd(input.dims.slice(1))];
  }
}
module.exports = { Flatten };
