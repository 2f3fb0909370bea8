"use strict";
// Reader of WDN2 tensor files, the container "optimized model" directories keep their
// weights in.  The files named by the model's WebDNN2.WeightPaths metadata are
// concatenated (a container may be cut anywhere into pieces) and parsed:
//
//   "WDN2"
//   chunk*:  u32 signature, u32 bodyLength, body          (little endian)
//     "TENS" body: u8 compression (0 raw, 1 8-bit table + deflate), u32 dataLength,
//                  u8 dataType (ONNX TensorProto.DataType), u8 ndim, u32 dims[ndim],
//                  u32 nameLength, name (utf-8), u32 extraLength, extra, data
//     "CLOS" ends the container; chunks with other signatures are skipped.
//
// Reference: src/descriptor_runner/core/tensorLoaderImpl.ts:10-207 (reader),
// src/graph_transpiler/webdnn/tensor_export.py:8-68 (writer).
const fs = require("fs");
const { DataType } = require("./onnxProto");
const { arrayProd } = require("../util");
const { decodeTensorRaw } = require("./tensorDecoder/decodeTensorRaw");
const { decodeTensorEightbit } = require("./tensorDecoder/decodeTensorEightbit");

const signatureFile = 0x324e4457, // "WDN2"
  signatureTensor = 0x534e4554, // "TENS"
  signatureClose = 0x534f4c43; // "CLOS"

class TensorLoaderImpl {
  constructor(path, cpuContext) {
    this.paths = typeof path === "string" ? [path] : path;
    this.cpuContext = cpuContext;
  }

  async loadAll(progressCallback) {
    return this.loadAllSync(progressCallback);
  }

  // -> Map name -> CPU tensor
  loadAllSync(progressCallback) {
    const fileArray = this.readAllFiles(progressCallback),
      buf = fileArray.buffer,
      base = fileArray.byteOffset,
      end = base + fileArray.byteLength;
    if (fileArray.byteLength < 4 || new DataView(buf, base, 4).getUint32(0, true) !== signatureFile) {
      throw new Error("Unexpected file signature");
    }
    const tensors = new Map();
    let offset = base + 4;
    for (;;) {
      if (end - offset < 8) throw new Error("Unexpected EOF");
      const head = new DataView(buf, offset, 8),
        signature = head.getUint32(0, true),
        bodyByteLength = head.getUint32(4, true),
        bodyByteOffset = offset + 8;
      if (end - bodyByteOffset < bodyByteLength) throw new Error("Unexpected EOF");
      if (signature === signatureClose) break;
      if (signature === signatureTensor) {
        const { name, tensor } = this.parseTensorChunk(buf, bodyByteOffset, bodyByteLength);
        tensors.set(name, tensor);
      }
      offset = bodyByteOffset + bodyByteLength;
    }
    return tensors;
  }

  readAllFiles(progressCallback) {
    const parts = [];
    let loadedBytes = 0;
    if (progressCallback) progressCallback(loadedBytes);
    for (const p of this.paths) {
      const part = fs.readFileSync(p);
      parts.push(part);
      loadedBytes += part.byteLength;
      if (progressCallback) progressCallback(loadedBytes);
    }
    // one private ArrayBuffer (small Buffers share a pool with unrelated data)
    const all = new Uint8Array(loadedBytes);
    let ofs = 0;
    for (const part of parts) {
      all.set(part, ofs);
      ofs += part.byteLength;
    }
    return all;
  }

  parseTensorChunk(buf, bodyByteOffset, bodyByteLength) {
    const view = new DataView(buf, bodyByteOffset, bodyByteLength);
    const needBytes = (n) => {
      if (ofs + n > bodyByteLength) throw new Error("Unexpected EOF");
    };
    let ofs = 0;
    needBytes(7);
    const compressionAlgorithm = view.getUint8(ofs);
    ofs += 1;
    const dataByteLength = view.getUint32(ofs, true);
    ofs += 4;
    const dataType = view.getUint8(ofs);
    ofs += 1;
    const ndim = view.getUint8(ofs);
    ofs += 1;
    needBytes(4 * ndim + 4);
    const dims = [];
    for (let i = 0; i < ndim; i++) {
      dims.push(view.getUint32(ofs, true));
      ofs += 4;
    }
    const numel = arrayProd(dims),
      nameLength = view.getUint32(ofs, true);
    ofs += 4;
    needBytes(nameLength + 4);
    const name = Buffer.from(buf, bodyByteOffset + ofs, nameLength).toString("utf-8");
    ofs += nameLength;
    const extraLength = view.getUint32(ofs, true);
    ofs += 4 + extraLength; // nothing defined yet lives in the extra field
    needBytes(dataByteLength);
    let data;
    switch (compressionAlgorithm) {
      case 0:
        data = decodeTensorRaw(buf, bodyByteOffset + ofs, dataByteLength, dataType, numel);
        break;
      case 1:
        data = decodeTensorEightbit(buf, bodyByteOffset + ofs, dataByteLength, dataType, numel);
        break;
      default:
        throw new Error("Unexpected compression algorithm");
    }
    let dataTypeString;
    switch (dataType) {
      case DataType.FLOAT:
        dataTypeString = "float32";
        break;
      case DataType.INT32:
        dataTypeString = "int32";
        break;
      default:
        // INT64 bodies decode (to int32) but the reference does not accept the chunk
        throw new Error("Unsupported DataType");
    }
    return { name, tensor: this.cpuContext.emptyTensor(dims, dataTypeString, data) };
  }
}
module.exports = { TensorLoaderImpl };
