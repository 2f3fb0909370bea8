"""WDN2 tensor files: the JavaScript reader (webdnn_amd/js/core/tensorLoaderImpl.js) against
containers assembled byte by byte from the documented layout, against the Python writer
(webdnn_amd/tensor_export.py), and through WebDNN.load() on an optimized-model directory.

The reference holds no sample container; the hand-assembled bytes below are the pin: they are
written from the chunk layout (tensorLoaderImpl.ts:118-166), not with the writer under test."""
import json
import os
import struct
import subprocess
import zlib

import numpy as np
import pytest

import node_runner
from util import assert_bit_exact
from webdnn_amd import modelgen, tensor_export
from webdnn_amd.eightbit_table import MAGNITUDES

HERE = os.path.dirname(os.path.abspath(__file__))


def js_load(paths):
    out = subprocess.run(["node", os.path.join(HERE, "js", "load_tensors.js"), ",".join(paths)],
                         stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    rep = json.loads(out.stdout.strip().splitlines()[-1])
    if not rep["ok"]:
        raise RuntimeError(rep["error"])
    tensors = {}
    for name, t in rep["tensors"].items():
        bits = np.array(t["bits"], dtype=np.uint32)
        tensors[name] = bits.view(np.float32 if t["dataType"] == "float32" else np.int32).reshape(t["dims"])
    return tensors, rep["progress"]


def chunk(sig, body):
    return sig + struct.pack("<I", len(body)) + body


def tens(name, compression, dtype, dims, data, extra=b""):
    nb = name.encode()
    body = struct.pack("<BIBB", compression, len(data), dtype, len(dims))
    body += b"".join(struct.pack("<I", d) for d in dims)
    body += struct.pack("<I", len(nb)) + nb + struct.pack("<I", len(extra)) + extra + data
    return chunk(b"TENS", body)


def test_hand_assembled_container(tmp_path):
    f = np.array([[1.5, -2.0, 3.25], [0.0, -0.0, 1e-30]], np.float32)
    i = np.array([7, -8, 2 ** 31 - 1], np.int32)
    scalar = np.array(42.0, np.float32)
    # 8-bit body: codes 0, 1, 127, 128+1, 128+127, 64 with scale 2.5
    codes = bytes([0, 1, 127, 129, 255, 64])
    stream = zlib.compress(codes)
    eight = struct.pack("<If", len(stream), 2.5) + stream
    blob = (b"WDN2" + tens("w/f", 0, 1, f.shape, f.tobytes()) + chunk(b"JUNK", b"\x01\x02\x03")
            + tens("idx", 0, 6, i.shape, i.tobytes(), extra=b"ignored")
            + tens("s", 0, 1, (), scalar.tobytes())
            + tens("q", 1, 1, (2, 3), eight)
            + tens("empty", 0, 1, (0, 4), b"")
            + chunk(b"CLOS", b"") + b"trailing bytes are never read")
    # cut the container at awkward places: inside the signature, inside a header, inside data
    cuts = [0, 2, 9, 31, 60, len(blob)]
    paths = []
    for n in range(len(cuts) - 1):
        p = tmp_path / ("part%d.bin" % n)
        p.write_bytes(blob[cuts[n]:cuts[n + 1]])
        paths.append(str(p))
    got, progress = js_load(paths)
    assert list(got) == ["w/f", "idx", "s", "q", "empty"]
    assert_bit_exact(got["w/f"], f)
    assert_bit_exact(got["idx"], i)
    assert_bit_exact(got["s"], scalar)
    assert got["empty"].shape == (0, 4)
    m = MAGNITUDES
    want_q = np.array([[0.0, m[1] * 2.5, 2.5], [-(m[1] * 2.5), -2.5, m[64] * 2.5]], np.float64).astype(np.float32)
    assert_bit_exact(got["q"], want_q)
    assert np.signbit(got["q"][0, 0]) == False and m[0] == 0.0 and m[127] == 1.0 and len(m) == 128   # noqa: E712
    assert progress == [0] + list(np.cumsum([cuts[n + 1] - cuts[n] for n in range(len(cuts) - 1)]))


@pytest.mark.parametrize("blob,msg", [
    (b"WDN3" + chunk(b"CLOS", b""), "signature"),
    (b"WDN2", "EOF"),                                                       # no CLOS
    (b"WDN2" + b"TENS" + struct.pack("<I", 100) + b"\0" * 10, "EOF"),        # chunk longer than the file
    (b"WDN2" + tens("x", 2, 1, (1,), b"\0\0\0\0") + chunk(b"CLOS", b""), "compression"),
    (b"WDN2" + tens("x", 0, 11, (1,), b"\0" * 8) + chunk(b"CLOS", b""), "DataType"),   # DOUBLE
    (b"WDN2" + tens("x", 0, 7, (1,), b"\0" * 8) + chunk(b"CLOS", b""), "DataType"),    # INT64 chunk (reader refuses)
    (b"WDN2" + tens("x", 1, 6, (1,), b"\0" * 12) + chunk(b"CLOS", b""), "DataType"),   # 8-bit coding of ints
    (b"WDN2" + tens("x", 0, 1, (4,), b"\0" * 8) + chunk(b"CLOS", b""), "EOF"),         # data shorter than dims say
])
def test_malformed_containers_throw(tmp_path, blob, msg):
    p = tmp_path / "bad.bin"
    p.write_bytes(blob)
    with pytest.raises(RuntimeError) as err:
        js_load([str(p)])
    assert msg in str(err.value)


def test_python_writer_to_js_reader(tmp_path):
    rng = np.random.default_rng(5)
    tensors = {"conv.weight": rng.standard_normal((16, 8, 3, 3)).astype(np.float32),
               "shape": np.array([1, -1, 256], np.int32),
               "bias": np.zeros(16, np.float32),
               "日本語": rng.uniform(-3, 3, (5,)).astype(np.float32)}
    for compression in (0, 1):
        paths = tensor_export.serialize_tensors(str(tmp_path / ("c%d-{}.bin" % compression)), tensors, 1000, compression)
        assert len(paths) > 1
        got, _ = js_load(paths)
        back = tensor_export.load_tensors(paths)
        assert list(got) == list(tensors)
        for name, want in tensors.items():
            assert_bit_exact(got[name], back[name], name + ": JS reader vs Python reader")
            if compression == 0 or want.dtype != np.float32:
                assert_bit_exact(got[name], want, name)
            else:
                # 8-bit coding: every value lands on a neighbouring table entry
                scale = np.abs(want).max()
                if scale == 0:
                    assert not got[name].any()
                    continue
                assert np.abs(got[name] - want).max() <= 0.02 * scale
                assert np.array_equal(np.sign(got[name])[np.abs(want) > 1e-3 * scale],
                                      np.sign(want)[np.abs(want) > 1e-3 * scale])


def test_eightbit_coder_picks_the_nearest_table_entry():
    m = np.array(MAGNITUDES)
    # exact table values (scaled) survive a round trip; values just beside a midpoint go to the right side
    vals = np.concatenate([m, -m[1:]]).astype(np.float32) * np.float32(4.0)
    body = tensor_export.encode_eightbit(vals)
    back = tensor_export.decode_eightbit(body, vals.size)
    assert_bit_exact(back, (np.concatenate([m, -m[1:]]) * 4.0).astype(np.float32))
    mid = (m[40] + m[41]) / 2
    probe = np.array([1.0, mid * 0.999, mid * 1.001, 1e-7, 0.9958], np.float32)
    back = tensor_export.decode_eightbit(tensor_export.encode_eightbit(probe), probe.size)
    assert_bit_exact(back, np.array([1.0, m[40], m[41], 0.0, 1.0]).astype(np.float32))
    assert struct.unpack_from("<f", tensor_export.encode_eightbit(np.zeros(3, np.float32)), 4)[0] == np.float32(1e-20)


def test_optimized_model_directory_through_load(tmp_path):
    data, _ = modelgen.resnet50_model(batch=2, image=32, width=8, blocks=(1, 1, 1, 1), classes=10)
    X = np.random.default_rng(2).standard_normal((2, 3, 32, 32)).astype(np.float32)
    plain = tmp_path / "plain"
    plain.mkdir()
    (plain / "model.onnx").write_bytes(data)
    want, _ = node_runner.run_model(str(plain), [X], "hip", strict=True, fake_native=True)
    opt = tmp_path / "opt"
    model_path, weights = tensor_export.export_model_directory(str(opt), data, split_size=40000)
    assert os.path.basename(model_path) == "model-hip.onnx" and len(weights) > 3
    assert not modelgen.parse_model(open(model_path, "rb").read())["initializers"]
    got, rep = node_runner.run_model(str(opt), [X], "hip", strict=True, fake_native=True, extra=["--optimized"])
    assert_bit_exact(got[0], want[0], "optimized directory vs self-contained model")
    assert list(rep["stats"]["nodesByBackend"]) == ["hip"]
