"""The JavaScript oracle (oracle/js/cpuOperators.js), run through the product's runner with
backendOrder ["cpu"], against the C oracle interpreting the same graph: the two restatements of the
reference CPU operators must agree bit for bit (exp/tanh aside).  This also exercises, without a
GPU, the host path every model takes: ONNX decoding, initializers, the node loop, tensor release."""
import numpy as np
import pytest

import graph_ref
import node_runner
from util import assert_bit_exact
from webdnn_amd import modelgen


def check(tmp_path, model_bytes, feeds):
    (tmp_path / "model.onnx").write_bytes(model_bytes)
    model = modelgen.parse_model(model_bytes)
    want = graph_ref.run_graph(model, feeds)
    outs, report = node_runner.run_model(str(tmp_path), [feeds[n] for n, _ in model["inputs"]], "cpu",
                                         oracle_cpu=True)
    assert report["backend"] == "cpu" and report["stats"]["nodesByBackend"] == {"cpu": len(model["nodes"])}
    for (name, _), got in zip(model["outputs"], outs):
        assert_bit_exact(got, want[name], name)
    return report


def test_gemm_config1(tmp_path):
    data, _ = modelgen.gemm_model()
    A = np.random.default_rng(1).uniform(-1, 1, (256, 512)).astype(np.float32)
    check(tmp_path, data, {"A": A})


def test_ffn_small(tmp_path):
    data, _ = modelgen.ffn_model(batch=2, seq=16, d=48, hidden=96)
    X = np.random.default_rng(2).standard_normal((2, 16, 48)).astype(np.float32)
    check(tmp_path, data, {"X": X})


def test_conv_relu_small(tmp_path):
    data, _ = modelgen.conv_model(batch=2, cin=8, hw=12, cout=6)
    X = np.random.default_rng(3).uniform(0, 1, (2, 8, 12, 12)).astype(np.float32)
    check(tmp_path, data, {"X": X})


def test_resnet_tiny(tmp_path):
    """The ResNet-50 graph at reduced width/size: every node type of config 4 on the cpu path."""
    data, g = modelgen.resnet50_model(batch=2, image=32, classes=10, width=8, blocks=(1, 1, 1, 1))
    X = np.random.default_rng(4).standard_normal((2, 3, 32, 32)).astype(np.float32)
    report = check(tmp_path, data, {"input": X})
    assert report["nodes"] == len(modelgen.parse_model(data)["nodes"])
