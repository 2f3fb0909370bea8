"use strict";
// 8-bit table coding (compression algorithm 1): body = u32 length of the deflate stream,
// f32 scale, deflate stream of one code byte per element.  Bit 7 of a code is the sign,
// bits 0..6 index a fixed table of magnitudes in [0, 1] (the dynamic-tree 8-bit format of
// T. Dettmers, "8-Bit Approximations for Parallelism in Deep Learning"); the element is
// table[code & 127] * scale, negated when bit 7 is set, every product rounded to fp32.
// Reference: src/descriptor_runner/core/tensorDecoder/decodeTensorEightbit.ts:5-61
// (the table is the format's definition; the encoder's copy is
// src/graph_transpiler/webdnn/constant_codec_eightbit.py:9-30).
const zlib = require("zlib");
const { DataType } = require("../onnxProto");
const { MAGNITUDES } = require("./eightbitTable");

function decodeTensorEightbit(buf, bodyByteOffset, bodyCompressedLength, dataType, numel) {
  if (dataType !== DataType.FLOAT) throw new Error("Unsupported DataType");
  if (bodyCompressedLength < 8) throw new Error("Unexpected EOF");
  const view = new DataView(buf, bodyByteOffset, bodyCompressedLength),
    codeByteLength = view.getUint32(0, true),
    scale = view.getFloat32(4, true);
  if (8 + codeByteLength > bodyCompressedLength) throw new Error("Unexpected EOF");
  const codes = zlib.inflateSync(Buffer.from(buf, bodyByteOffset + 8, codeByteLength));
  if (codes.length < numel) throw new Error("8-bit tensor body is shorter than the tensor");
  const scaledTable = new Float32Array(256);
  for (let i = 0; i < 256; i++) scaledTable[i] = MAGNITUDES[i & 0x7f] * scale * (i < 128 ? 1.0 : -1.0);
  const data = new Float32Array(numel);
  for (let i = 0; i < numel; i++) data[i] = scaledTable[codes[i]];
  return data;
}
module.exports = { decodeTensorEightbit };
