"use strict";
// Attribute getters shared by every backend's operators.
// Reference: src/descriptor_runner/operators/operatorUtil.ts:8-125.
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

// Strides and the two broadcasting rules live with the rest of the shape arithmetic
// (operators/shapes.js); operator files import them from here under the names the
// reference's operators use (operatorUtil.ts:169-245).
const { denseStrides: calcStrides, broadcastOnto: broadcastUni, broadcastTogether: broadcastMulti } = require("./shapes");

module.exports = {
  getAttrFloat, getAttrInt, getAttrInts, getAttrString, getAttrTensor, tensorProtoToArray,
  calcStrides, broadcastUni, broadcastMulti,
};
