"use strict";
// Attribute getters, strides and broadcasting shared by every backend's operators.
// Reference: src/descriptor_runner/operators/operatorUtil.ts:8-245.
const { clipToInt32 } = require("../util");
const { DataType } = require("../core/onnxProto");

function getAttr(attribute, name) {
  for (const attr of attribute) if (attr.name === name) return attr;
  return null;
}

function getAttrFloat(attribute, name, defaultValue) {
  const attr = getAttr(attribute, name);
  if (!attr) return defaultValue;
  if (attr.f == null) throw new Error(`Attribute ${name} is not float`);
  return attr.f;
}

function getAttrInt(attribute, name, defaultValue) {
  const attr = getAttr(attribute, name);
  if (!attr) return defaultValue;
  if (attr.i == null) throw new Error(`Attribute ${name} is not int`);
  return clipToInt32(attr.i);
}

function getAttrInts(attribute, name, defaultValue) {
  const attr = getAttr(attribute, name);
  if (!attr) return defaultValue;
  if (attr.ints == null) throw new Error(`Attribute ${name} is not int`);
  return attr.ints.map(clipToInt32);
}

function getAttrString(attribute, name, defaultValue) {
  const attr = getAttr(attribute, name);
  if (!attr) return defaultValue;
  if (attr.s == null) throw new Error(`Attribute ${name} is not string`);
  return Buffer.from(attr.s).toString("utf-8");
}

// TensorProto attribute -> {dims, dataType, data}; FLOAT and INT64 only (operatorUtil.ts:73-125).
function getAttrTensor(attribute, name) {
  const attr = getAttr(attribute, name);
  if (!attr) return null;
  const t = attr.t;
  if (t == null) throw new Error(`Attribute ${name} is not tensor`);
  return tensorProtoToArray(t);
}

// Shared with the runner's initializer extraction (core/runnerImpl.ts:136-233).
function tensorProtoToArray(t) {
  const dims = t.dims.map(clipToInt32);
  const raw = t.rawData;
  switch (t.dataType) {
    case DataType.FLOAT: {
      if (raw && raw.byteLength) {
        // copy: rawData is a view at an arbitrary (unaligned) offset of the model file
        const copy = new Uint8Array(raw.byteLength);
        copy.set(raw);
        return { dims, dataType: "float32", data: new Float32Array(copy.buffer, 0, copy.byteLength / 4) };
      }
      return { dims, dataType: "float32", data: new Float32Array(t.floatData || []) };
    }
    case DataType.INT64: {
      if (raw && raw.byteLength) {
        const view = new DataView(raw.buffer, raw.byteOffset, raw.byteLength);
        const out = new Int32Array(raw.byteLength / 8);
        for (let i = 0; i < out.length; i++) out[i] = clipToInt32(view.getBigInt64(i * 8, true));
        return { dims, dataType: "int32", data: out };
      }
      return { dims, dataType: "int32", data: new Int32Array((t.int64Data || []).map(clipToInt32)) };
    }
    case DataType.INT32: {
      if (raw && raw.byteLength) {
        const view = new DataView(raw.buffer, raw.byteOffset, raw.byteLength);
        const out = new Int32Array(raw.byteLength / 4);
        for (let i = 0; i < out.length; i++) out[i] = view.getInt32(i * 4, true);
        return { dims, dataType: "int32", data: out };
      }
      return { dims, dataType: "int32", data: new Int32Array(t.int32Data || []) };
    }
    default:
      throw new Error(`Unsupported TensorProto dataType ${t.dataType}`);
  }
}

function calcStrides(dims) {
  const strides = [];
  let length = 1;
  for (let i = dims.length - 1; i >= 0; i--) {
    strides.unshift(length);
    length *= dims[i];
  }
  return strides;
}

// Strides of B when broadcast (unidirectionally) to A's shape.
function broadcastUni(dimsA, dimsB) {
  if (dimsA.length < dimsB.length) {
    throw new Error(`Unidirectional broadcast error: ${dimsA}, ${dimsB}`);
  }
  const expandedDimsB = Array.prototype.slice.call(dimsB);
  while (expandedDimsB.length < dimsA.length) expandedDimsB.unshift(1);
  const stridesB = calcStrides(expandedDimsB);
  for (let i = 0; i < dimsA.length; i++) {
    if (dimsA[i] !== expandedDimsB[i]) {
      if (expandedDimsB[i] === 1) stridesB[i] = 0;
      else throw new Error(`Unidirectional broadcast error: ${dimsA}, ${dimsB}`);
    }
  }
  return stridesB;
}

// Multidirectional broadcast of several shapes: result dims + strides of every input.
function broadcastMulti(allDims) {
  const ndim = Math.max(...allDims.map((d) => d.length));
  const expandedAll = allDims.map((dims) => {
    const e = Array.prototype.slice.call(dims);
    while (e.length < ndim) e.unshift(1);
    return e;
  });
  const dims = [];
  for (let i = 0; i < ndim; i++) dims.push(Math.max(...expandedAll.map((e) => e[i])));
  const allStrides = expandedAll.map((e) => {
    const strides = calcStrides(e);
    for (let i = 0; i < ndim; i++) {
      if (e[i] !== dims[i]) {
        if (e[i] === 1) strides[i] = 0;
        else throw new Error(`Multidirectional broadcasting error: ${allDims.map((d) => `[${d}]`)}`);
      }
    }
    return strides;
  });
  return { dims, allStrides };
}

module.exports = {
  getAttrFloat, getAttrInt, getAttrInts, getAttrString, getAttrTensor, tensorProtoToArray,
  calcStrides, broadcastUni, broadcastMulti,
};
