"use strict";
// Uncompressed tensor body (compression algorithm 0): little-endian elements; INT64 is
// narrowed to int32 with saturation, like every 64-bit integer the runner meets.
// Reference: src/descriptor_runner/core/tensorDecoder/decodeTensorRaw.ts:6-42.
const { DataType } = require("../onnxProto");
const { INT32_MAX, INT32_MIN } = require("../../util");

function decodeTensorRaw(buf, bodyByteOffset, bodyCompressedLength, dataType, numel) {
  if (dataType === DataType.INT64) {
    if (bodyCompressedLength < numel * 8) throw new Error("Unexpected EOF");
    const data = new Int32Array(numel),
      view = new DataView(buf, bodyByteOffset, numel * 8);
    for (let idx = 0; idx < numel; idx++) {
      const v = view.getBigInt64(idx * 8, true);
      data[idx] = v > BigInt(INT32_MAX) ? INT32_MAX : v < BigInt(INT32_MIN) ? INT32_MIN : Number(v);
    }
    return data;
  }
  let data;
  if (dataType === DataType.FLOAT) data = new Float32Array(numel);
  else if (dataType === DataType.INT32) data = new Int32Array(numel);
  else throw new Error("Unsupported DataType");
  if (bodyCompressedLength < data.byteLength) throw new Error("Unexpected EOF");
  // byte-wise: the body sits at an arbitrary offset of the file
  new Uint8Array(data.buffer).set(new Uint8Array(buf, bodyByteOffset, data.byteLength));
  return data;
}
module.exports = { decodeTensorRaw };
