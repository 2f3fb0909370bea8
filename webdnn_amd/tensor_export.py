"""Writer (and a reader, for tests and tools) of WDN2 tensor files, the container that
"optimized model" directories keep their weights in.

Layout (little endian):  b"WDN2", then chunks `signature[4] u32 bodyLength body`:
  b"TENS": u8 compression, u32 dataLength, u8 dataType (ONNX), u8 ndim, u32 dims[ndim],
           u32 nameLength, name utf-8, u32 extraLength, extra, data[dataLength]
  b"CLOS": empty body, ends the container.
compression 0 = raw elements; 1 = 8-bit table code per element, deflated, preceded by
`u32 streamLength, f32 scale` (float32 tensors only; anything else is stored raw).

Reference: src/graph_transpiler/webdnn/tensor_export.py:8-88 (writer),
src/graph_transpiler/webdnn/constant_codec_eightbit.py:32-66 (8-bit coder),
src/descriptor_runner/core/tensorLoaderImpl.ts:10-207 (reader).
"""
import os
import struct
import zlib

import numpy as np

from .eightbit_table import MAGNITUDES

_ONNX_TYPE = {np.dtype(np.float32): 1, np.dtype(np.int32): 6, np.dtype(np.int64): 7}
_NUMPY_TYPE = {v: k for k, v in _ONNX_TYPE.items()}

# Decision thresholds between neighbouring magnitudes, as float32 like the reference's
# (constant_codec_eightbit.py:34-52): below 1.5e-6 -> code 0, then midpoints between table
# entries, and everything above 0.995703 -> code 127 (magnitude 1).
_TABLE = np.array(MAGNITUDES, dtype=np.float64)
_THRESHOLDS = np.array([1.5e-6] + [(_TABLE[i + 1] + _TABLE[i]) / 2.0 for i in range(1, 126)] + [0.995703],
                       dtype=np.float32)


def encode_eightbit(data):
    """float32 array -> body of a compression-1 tensor."""
    data = np.asarray(data)
    if data.dtype != np.float32:
        raise TypeError("8-bit coding is defined for float32 tensors")
    flat = data.reshape(-1)
    scale = np.float32(max(float(np.max(np.abs(flat))) if flat.size else 0.0, 1e-20))
    code = np.searchsorted(_THRESHOLDS, np.abs(flat) / scale).astype(np.int32)
    code += (flat < 0.0).astype(np.int32) * 128
    stream = zlib.compress(code.astype(np.uint8).tobytes(), 9)
    return struct.pack("<If", len(stream), float(scale)) + stream


def decode_eightbit(body, numel):
    """Inverse of encode_eightbit with the reader's arithmetic (float32 products)."""
    length, scale = struct.unpack_from("<If", body, 0)
    codes = np.frombuffer(zlib.decompress(body[8:8 + length]), dtype=np.uint8)[:numel]
    table = np.array(MAGNITUDES, dtype=np.float64)
    signed = np.concatenate([table, -table])
    # decodeTable[i] * scale * (+-1.0) in double, stored to a Float32Array
    scaled = (signed * float(np.float32(scale))).astype(np.float32)
    return scaled[codes]


def _tensor_chunk(name, data, compression):
    data = np.ascontiguousarray(data)
    if data.dtype not in _ONNX_TYPE:
        raise TypeError("tensor %s: dtype %s cannot be stored" % (name, data.dtype))
    if data.dtype != np.float32:
        compression = 0
    if compression == 0:
        body = data.astype(data.dtype.newbyteorder("<")).tobytes()
    elif compression == 1:
        body = encode_eightbit(data)
    else:
        raise ValueError("unknown compression algorithm %d" % compression)
    name_bytes = name.encode("utf-8")
    chunk = struct.pack("<BIBB", compression, len(body), _ONNX_TYPE[data.dtype], data.ndim)
    chunk += struct.pack("<%dI" % data.ndim, *data.shape)
    chunk += struct.pack("<I", len(name_bytes)) + name_bytes
    chunk += struct.pack("<I", 0)          # no extra data
    chunk += body
    return b"TENS" + struct.pack("<I", len(chunk)) + chunk


def serialize_tensors(path_template, tensors, split_size=0, compression_algorithm=0):
    """Writes {name: array} as one container, cut into files of `split_size` bytes when that is
    positive (`path_template` is then formatted with the piece number).  Returns the paths."""
    blob = b"WDN2" + b"".join(_tensor_chunk(n, a, compression_algorithm) for n, a in tensors.items())
    blob += b"CLOS" + struct.pack("<I", 0)
    if split_size <= 0:
        with open(path_template, "wb") as f:
            f.write(blob)
        return [path_template]
    paths = []
    for i in range((len(blob) + split_size - 1) // split_size):
        paths.append(path_template.format(i))
        with open(paths[-1], "wb") as f:
            f.write(blob[i * split_size:(i + 1) * split_size])
    return paths


def load_tensors(paths):
    """Reads a container (one path or the list of its pieces) back: {name: array}.  INT64 data
    comes back as int64 here; the JavaScript reader narrows it to int32."""
    if isinstance(paths, str):
        paths = [paths]
    blob = b"".join(open(p, "rb").read() for p in paths)
    if blob[:4] != b"WDN2":
        raise ValueError("Unexpected file signature")
    out, pos = {}, 4
    while True:
        if len(blob) - pos < 8:
            raise ValueError("Unexpected EOF")
        sig, length = blob[pos:pos + 4], struct.unpack_from("<I", blob, pos + 4)[0]
        body = blob[pos + 8:pos + 8 + length]
        if len(body) < length:
            raise ValueError("Unexpected EOF")
        pos += 8 + length
        if sig == b"CLOS":
            return out
        if sig != b"TENS":
            continue
        compression, data_len, dtype, ndim = struct.unpack_from("<BIBB", body, 0)
        o = 7
        dims = struct.unpack_from("<%dI" % ndim, body, o)
        o += 4 * ndim
        name_len = struct.unpack_from("<I", body, o)[0]
        o += 4
        name = body[o:o + name_len].decode("utf-8")
        o += name_len
        o += 4 + struct.unpack_from("<I", body, o)[0]
        data = body[o:o + data_len]
        numel = int(np.prod(dims, dtype=np.int64)) if ndim else 1
        if compression == 0:
            arr = np.frombuffer(data, dtype=_NUMPY_TYPE[dtype].newbyteorder("<"), count=numel).astype(_NUMPY_TYPE[dtype])
        elif compression == 1:
            arr = decode_eightbit(data, numel)
        else:
            raise ValueError("Unexpected compression algorithm")
        out[name] = arr.reshape(dims)


def export_model_directory(directory, model_bytes, backend="hip", split_size=4 * 1024 * 1024,
                           compression_algorithm=0):
    """Turns a self-contained ONNX model into the directory layout of an optimized model:
    `model-<backend>.onnx` without initializers, `weight-<backend>-<i>.bin` holding them, and the
    WebDNN2.WeightPaths / WebDNN2.WeightSizes metadata that lead the runner to the files
    (src/graph_transpiler/webdnn/optimize_model.py:27-35).  Returns (model path, weight paths)."""
    from . import modelgen

    os.makedirs(directory, exist_ok=True)
    stripped, tensors = modelgen.strip_initializers(model_bytes)
    paths = serialize_tensors(os.path.join(directory, "weight-%s-{}.bin" % backend), tensors, split_size,
                              compression_algorithm)
    metadata = {"WebDNN2.WeightPaths": ":".join(os.path.basename(p) for p in paths),
                "WebDNN2.WeightSizes": ":".join(str(os.path.getsize(p)) for p in paths),
                "WebDNN2.TensorMoveOptions": "{}"}
    model_path = os.path.join(directory, "model-%s.onnx" % backend)
    with open(model_path, "wb") as f:
        f.write(modelgen.add_metadata(stripped, metadata))
    return model_path, paths
