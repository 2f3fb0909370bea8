"use strict";
// Minimal ONNX protobuf reader and writer: just the messages the runner touches.
//
// The reference decodes models with protobufjs-generated bindings
// (src/descriptor_runner/onnx/onnx.js, from scripts/onnx.proto); this file reads
// the same wire format directly and yields objects with the same camelCase field
// names, so operator code reads attributes as it does there (attr.f, attr.i,
// attr.ints, tensor.rawData, ...).  Field numbers are those of scripts/onnx.proto:
//   ModelProto:357-400  OperatorSetIdProto:785-794  GraphProto:456-477
//   NodeProto:208-224   AttributeProto:122-185      TensorProto:499-618
// int64 values become JavaScript numbers, saturated to the int32 range when
// they are tensor data or exceed 2^53 (the reference clips them the same way:
// src/descriptor_runner/util.ts:73-92).

const DataType = { FLOAT: 1, UINT8: 2, INT8: 3, INT32: 6, INT64: 7, BOOL: 9 };
const AttributeType = { FLOAT: 1, INT: 2, STRING: 3, TENSOR: 4, FLOATS: 6, INTS: 7, STRINGS: 8 };

// ---- schema ------------------------------------------------------------------
// kind: "int" (varint, signed 64), "float" (fixed32), "string", "bytes", or a message schema.
const Dimension = { 1: ["dimValue", "int"], 2: ["dimParam", "string"] };
const TensorShape = { 1: ["dim", Dimension, "repeated"] };
const TypeTensor = { 1: ["elemType", "int"], 2: ["shape", TensorShape] };
const Type = { 1: ["tensorType", TypeTensor] };
const ValueInfo = { 1: ["name", "string"], 2: ["type", Type] };
const Tensor = {
  1: ["dims", "int", "repeated"],
  2: ["dataType", "int"],
  4: ["floatData", "float", "repeated"],
  5: ["int32Data", "int", "repeated"],
  7: ["int64Data", "int", "repeated"],
  8: ["name", "string"],
  9: ["rawData", "bytes"],
};
const Attribute = {
  1: ["name", "string"],
  2: ["f", "float"],
  3: ["i", "int"],
  4: ["s", "bytes"],
  5: ["t", Tensor],
  7: ["floats", "float", "repeated"],
  8: ["ints", "int", "repeated"],
  9: ["strings", "bytes", "repeated"],
  20: ["type", "int"],
};
const Node = {
  1: ["input", "string", "repeated"],
  2: ["output", "string", "repeated"],
  3: ["name", "string"],
  4: ["opType", "string"],
  5: ["attribute", Attribute, "repeated"],
  7: ["domain", "string"],
};
const Graph = {
  1: ["node", Node, "repeated"],
  2: ["name", "string"],
  5: ["initializer", Tensor, "repeated"],
  11: ["input", ValueInfo, "repeated"],
  12: ["output", ValueInfo, "repeated"],
  13: ["valueInfo", ValueInfo, "repeated"],
};
const OperatorSetId = { 1: ["domain", "string"], 2: ["version", "int"] };
const StringStringEntry = { 1: ["key", "string"], 2: ["value", "string"] };
const Model = {
  1: ["irVersion", "int"],
  2: ["producerName", "string"],
  3: ["producerVersion", "string"],
  7: ["graph", Graph],
  8: ["opsetImport", OperatorSetId, "repeated"],
  14: ["metadataProps", StringStringEntry, "repeated"],
};

// ---- reader --------------------------------------------------------------------
const TWO32 = 4294967296;

class Reader {
  constructor(buf, pos, end) {
    this.buf = buf;
    this.pos = pos;
    this.end = end;
    this.view = new DataView(buf.buffer, buf.byteOffset, buf.byteLength);
  }

  // Unsigned varint as (lo, hi) 32-bit halves.
  varintParts() {
    const buf = this.buf;
    let lo = 0,
      hi = 0,
      shift = 0;
    for (let i = 0; i < 10; i++) {
      if (this.pos >= this.end) throw new Error("onnx: truncated varint");
      const b = buf[this.pos++];
      const v = b & 0x7f;
      if (shift < 28) {
        lo += v * Math.pow(2, shift);
      } else if (shift === 28) {
        lo += (v & 0x0f) * Math.pow(2, 28);
        hi += v >>> 4;
      } else {
        hi += v * Math.pow(2, shift - 32);
      }
      if (!(b & 0x80)) {
        return [lo >>> 0, hi >>> 0];
      }
      shift += 7;
    }
    throw new Error("onnx: varint too long");
  }

  // Signed 64-bit varint as a number; values beyond +-2^53 saturate to int32 limits'
  // direction (they only occur as "to the end" sentinels).
  int64() {
    const [lo, hi] = this.varintParts();
    if (hi & 0x80000000) {
      // negative: two's complement
      const nlo = (~lo + 1) >>> 0;
      const nhi = (~hi + (nlo === 0 ? 1 : 0)) >>> 0;
      if (nhi >= 0x200000) return -Number.MAX_SAFE_INTEGER;
      return -(nhi * TWO32 + nlo);
    }
    if (hi >= 0x200000) return Number.MAX_SAFE_INTEGER;
    return hi * TWO32 + lo;
  }

  uint32() {
    const [lo, hi] = this.varintParts();
    if (hi !== 0) throw new Error("onnx: length too large");
    return lo;
  }

  float32() {
    if (this.pos + 4 > this.end) throw new Error("onnx: truncated float");
    const v = this.view.getFloat32(this.pos, true);
    this.pos += 4;
    return v;
  }

  skip(wireType) {
    switch (wireType) {
      case 0:
        this.varintParts();
        break;
      case 1:
        this.pos += 8;
        break;
      case 2:
        this.pos += this.uint32();
        break;
      case 5:
        this.pos += 4;
        break;
      default:
        throw new Error(`onnx: unsupported wire type ${wireType}`);
    }
    if (this.pos > this.end) throw new Error("onnx: truncated field");
  }
}

const utf8 = new (require("util").TextDecoder)("utf-8");

function newMessage(schema) {
  const msg = {};
  for (const key of Object.keys(schema)) {
    const field = schema[key];
    if (field[2] === "repeated") msg[field[0]] = [];
  }
  return msg;
}

function decodeMessage(schema, buf, pos, end) {
  const r = new Reader(buf, pos, end);
  const msg = newMessage(schema);
  while (r.pos < r.end) {
    const tag = r.uint32();
    const fieldNo = tag >>> 3,
      wireType = tag & 7;
    const field = schema[fieldNo];
    if (!field) {
      r.skip(wireType);
      continue;
    }
    const [name, kind, rep] = field;
    let value;
    if (kind === "int") {
      if (wireType === 2 && rep) {
        // packed
        const len = r.uint32();
        const stop = r.pos + len;
        if (stop > r.end) throw new Error("onnx: truncated packed field");
        while (r.pos < stop) msg[name].push(r.int64());
        continue;
      }
      if (wireType !== 0) throw new Error(`onnx: field ${name}: wire type ${wireType}`);
      value = r.int64();
    } else if (kind === "float") {
      if (wireType === 2 && rep) {
        const len = r.uint32();
        const stop = r.pos + len;
        if (stop > r.end || len % 4) throw new Error("onnx: bad packed float field");
        while (r.pos < stop) msg[name].push(r.float32());
        continue;
      }
      if (wireType !== 5) throw new Error(`onnx: field ${name}: wire type ${wireType}`);
      value = r.float32();
    } else {
      if (wireType !== 2) throw new Error(`onnx: field ${name}: wire type ${wireType}`);
      const len = r.uint32();
      const stop = r.pos + len;
      if (stop > r.end) throw new Error(`onnx: truncated field ${name}`);
      if (kind === "string") value = utf8.decode(buf.subarray(r.pos, stop));
      else if (kind === "bytes") value = buf.subarray(r.pos, stop); // a view, not a copy
      else value = decodeMessage(kind, buf, r.pos, stop);
      r.pos = stop;
    }
    if (rep) msg[name].push(value);
    else msg[name] = value;
  }
  return msg;
}

function decodeModel(bytes) {
  const buf = bytes instanceof Uint8Array ? bytes : new Uint8Array(bytes);
  const model = decodeMessage(Model, buf, 0, buf.length);
  if (!model.graph) throw new Error("onnx: model has no graph");
  return model;
}

// ---- writer (tests and model generators) ------------------------------------------
class Writer {
  constructor() {
    this.chunks = [];
    this.length = 0;
  }

  push(bytes) {
    this.chunks.push(bytes);
    this.length += bytes.length;
  }

  varint(v) {
    // v: non-negative safe integer, or negative (written as 64-bit two's complement)
    const out = [];
    if (v < 0) {
      let big = BigInt.asUintN(64, BigInt(v));
      while (big > 0x7fn) {
        out.push(Number(big & 0x7fn) | 0x80);
        big >>= 7n;
      }
      out.push(Number(big));
    } else {
      while (v > 0x7f) {
        out.push((v % 128) | 0x80);
        v = Math.floor(v / 128);
      }
      out.push(v);
    }
    this.push(Uint8Array.from(out));
  }

  tag(fieldNo, wireType) {
    this.varint(fieldNo * 8 + wireType);
  }

  finish() {
    const out = new Uint8Array(this.length);
    let pos = 0;
    for (const c of this.chunks) {
      out.set(c, pos);
      pos += c.length;
    }
    return out;
  }
}

const utf8enc = new (require("util").TextEncoder)();

function encodeMessage(schema, msg) {
  const w = new Writer();
  for (const key of Object.keys(schema)) {
    const fieldNo = Number(key);
    const [name, kind, rep] = schema[key];
    const raw = msg[name];
    if (raw === undefined || raw === null) continue;
    const values = rep ? raw : [raw];
    if (rep && values.length === 0) continue;
    if (kind === "int" && rep) {
      const inner = new Writer();
      for (const v of values) inner.varint(v);
      w.tag(fieldNo, 2);
      w.varint(inner.length);
      w.push(inner.finish());
      continue;
    }
    if (kind === "float" && rep) {
      const bytes = new Uint8Array(Float32Array.from(values).buffer);
      w.tag(fieldNo, 2);
      w.varint(bytes.length);
      w.push(bytes);
      continue;
    }
    for (const v of values) {
      if (kind === "int") {
        w.tag(fieldNo, 0);
        w.varint(v);
      } else if (kind === "float") {
        w.tag(fieldNo, 5);
        w.push(new Uint8Array(Float32Array.of(v).buffer));
      } else {
        let bytes;
        if (kind === "string") bytes = utf8enc.encode(v);
        else if (kind === "bytes") bytes = v;
        else bytes = encodeMessage(kind, v);
        w.tag(fieldNo, 2);
        w.varint(bytes.length);
        w.push(bytes);
      }
    }
  }
  return w.finish();
}

function encodeModel(model) {
  return encodeMessage(Model, model);
}

module.exports = { decodeModel, encodeModel, DataType, AttributeType };
