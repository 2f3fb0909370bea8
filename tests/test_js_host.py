"""Host side of the hip backend without a GPU: the real contexts, tensors, operators, fusion pass and
runner, with the N-API addon replaced by tests/js/fake_native.js (same entry points over typed arrays,
reference rounding).  Whatever the hip host code gets wrong — a stride, a shape, an argument order, a
fused chain, a tensor freed too early — shows up as a difference from the cpu path, which must be
bit-exact here."""
import json
import os
import subprocess

import numpy as np
import pytest

import graph_ref
import node_runner
from oracle import ref
from util import assert_bit_exact
from webdnn_amd import modelgen

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def both_paths(tmp_path, data, feeds, fuse=True, strict=True):
    (tmp_path / "model.onnx").write_bytes(data)
    model = modelgen.parse_model(data)
    ordered = [feeds[n] for n, _ in model["inputs"]]
    hip, rep = node_runner.run_model(str(tmp_path), ordered, "hip", strict=strict, fuse=fuse, fake_native=True,
                                     oracle_cpu=not strict, runs=2)
    cpu, _ = node_runner.run_model(str(tmp_path), ordered, "cpu", oracle_cpu=True)
    return model, hip, cpu, rep


def test_every_config_graph_on_the_hip_host_path(tmp_path):
    cases = [
        (modelgen.gemm_model(m=9, k=20, n=13)[0], {"A": (9, 20)}),
        (modelgen.ffn_model(batch=2, seq=5, d=12, hidden=20)[0], {"X": (2, 5, 12)}),
        (modelgen.conv_model(batch=2, cin=4, hw=7, cout=6)[0], {"X": (2, 4, 7, 7)}),
        (modelgen.resnet50_model(batch=1, image=32, classes=7, width=4, blocks=(2, 1, 1, 1))[0], {"input": (1, 3, 32, 32)}),
    ]
    rng = np.random.default_rng(0)
    for i, (data, shapes) in enumerate(cases):
        d = tmp_path / str(i)
        d.mkdir()
        feeds = {k: rng.standard_normal(s).astype(np.float32) for k, s in shapes.items()}
        for fuse in (True, False):
            model, hip, cpu, rep = both_paths(d, data, feeds, fuse=fuse)
            assert list(rep["stats"]["nodesByBackend"]) == ["hip"]
            for got, want, (name, _) in zip(hip, cpu, model["outputs"]):
                assert_bit_exact(got, want, "case %d fuse=%s %s" % (i, fuse, name))
            # nothing but the device copies of the initializers survives a run
            assert rep["liveBuffers"] == rep["initializerCopies"], rep


def test_operator_instances_are_reused_across_runs(tmp_path):
    """The first run creates one instance per node; the second may create some again (weights that were
    on the cpu now have device copies, so the inputs' placement differs); from the third on, none."""
    data, _ = modelgen.resnet50_model(batch=1, image=32, classes=7, width=4, blocks=(1, 1, 1, 1))
    (tmp_path / "model.onnx").write_bytes(data)
    X = np.random.default_rng(0).standard_normal((1, 3, 32, 32)).astype(np.float32)
    created = []
    outs = []
    for runs in (1, 2, 3, 4):
        out, rep = node_runner.run_model(str(tmp_path), [X], "hip", fake_native=True, runs=runs, extra=["--no-graph"])
        created.append(rep["stats"]["operatorsCreated"])
        outs.append(out[0])
        nodes = rep["stats"]["nodes"]
    assert created[0] == nodes and created[1] <= nodes and created[2] == 0 and created[3] == 0
    for o in outs[1:]:
        assert_bit_exact(o, outs[0], "same result whichever run is reported")


def test_fusion_rewrites_the_expected_chains(tmp_path):
    data, _ = modelgen.resnet50_model(batch=1, image=32, classes=7, width=4, blocks=(2, 1, 1, 1))
    feeds = {"input": np.random.default_rng(1).standard_normal((1, 3, 32, 32)).astype(np.float32)}
    _, _, _, fused = both_paths(tmp_path, data, feeds, fuse=True)
    _, _, _, plain = both_paths(tmp_path, data, feeds, fuse=False)
    n_conv = plain["nativeCalls"]["conv2d"]
    assert fused["nativeCalls"]["conv2d"] == n_conv
    assert "binary" not in fused["nativeCalls"] and "unary" not in fused["nativeCalls"]   # all Add/Relu absorbed
    assert plain["nativeCalls"]["binary"] == 2 * 5 and plain["nativeCalls"]["unary"] == 2 * (1 + 3 * 5)
    assert fused["nodes"] == plain["nodes"] - 5 - 16


def test_a_tensor_with_two_readers_is_not_fused_away(tmp_path):
    g = modelgen.GraphBuilder(0)
    g.const("W", g.rng().standard_normal((4, 3, 1, 1)).astype(np.float32))
    g.op("Conv", ["X", "W"], "c")          # read by Relu AND by the final Add -> must stay a tensor
    g.op("Relu", ["c"], "r")
    g.op("Add", ["r", "c"], "Y")
    data = g.finish([("X", [1, 3, 5, 5])], [("Y", [1, 4, 5, 5])])
    feeds = {"X": np.random.default_rng(2).standard_normal((1, 3, 5, 5)).astype(np.float32)}
    model, hip, cpu, rep = both_paths(tmp_path, data, feeds)
    assert rep["nodes"] == 3
    assert_bit_exact(hip[0], cpu[0], "shared tensor")


def test_broadcasting_add_after_conv_falls_back_to_separate_kernels(tmp_path):
    g = modelgen.GraphBuilder(0)
    g.const("W", g.rng().standard_normal((4, 3, 3, 3)).astype(np.float32))
    g.op("Conv", ["X", "W"], "c", pads=[1, 1, 1, 1])
    g.op("Add", ["c", "S"], "a")           # S is [1,4,1,1]: not a same-shape residual
    g.op("Relu", ["a"], "Y")
    data = g.finish([("X", [2, 3, 5, 5]), ("S", [1, 4, 1, 1])], [("Y", [2, 4, 5, 5])])
    rng = np.random.default_rng(3)
    feeds = {"X": rng.standard_normal((2, 3, 5, 5)).astype(np.float32), "S": rng.standard_normal((1, 4, 1, 1)).astype(np.float32)}
    model, hip, cpu, rep = both_paths(tmp_path, data, feeds)
    assert rep["nodes"] == 1 and rep["nativeCalls"]["binary"] == 2 and rep["nativeCalls"]["unary"] == 2
    assert_bit_exact(hip[0], cpu[0], "broadcast residual")


def test_layout_ops_alias_and_attention_shapes(tmp_path):
    """Reshape / Transpose / MatMul / Softmax / LayerNormalization / Gemm as a transformer block uses them."""
    g = modelgen.GraphBuilder(0)
    t, d, h = 10, 16, 4
    g.const("Wq", (g.rng().standard_normal((d, d)) * 0.3).astype(np.float32))
    g.const("split", np.array([t, h, d // h], np.int64))
    g.const("merge", np.array([t, d], np.int64))
    g.const("scale", np.array(0.5, np.float32))
    g.const("gamma", g.rng().standard_normal(d).astype(np.float32))
    g.const("beta", g.rng().standard_normal(d).astype(np.float32))
    g.op("MatMul", ["X", "Wq"], "q")
    g.op("Reshape", ["q", "split"], "q3")
    g.op("Transpose", ["q3"], "qh", perm=[1, 0, 2])       # [h, t, d/h]
    g.op("Transpose", ["q3"], "kt", perm=[1, 2, 0])       # [h, d/h, t]
    g.op("MatMul", ["qh", "kt"], "scores")
    g.op("Mul", ["scores", "scale"], "scaled")
    g.op("Softmax", ["scaled"], "attn", axis=-1)
    g.op("MatMul", ["attn", "qh"], "ctx")
    g.op("Transpose", ["ctx"], "ctx_t", perm=[1, 0, 2])
    g.op("Reshape", ["ctx_t", "merge"], "merged")
    g.op("Add", ["merged", "X"], "res")
    g.op("LayerNormalization", ["res", "gamma", "beta"], "Y", axis=-1, epsilon=1e-5)
    data = g.finish([("X", [t, d])], [("Y", [t, d])], opset=17)
    feeds = {"X": np.random.default_rng(4).standard_normal((t, d)).astype(np.float32)}
    (tmp_path / "model.onnx").write_bytes(data)
    hip, rep = node_runner.run_model(str(tmp_path), [feeds["X"]], "hip", strict=True, fake_native=True)
    assert list(rep["stats"]["nodesByBackend"]) == ["hip"] and rep["liveBuffers"] == rep["initializerCopies"]
    want = graph_ref.run_graph(modelgen.parse_model(data), feeds)["Y"]
    np.testing.assert_allclose(hip[0], want, rtol=0, atol=2e-6)


def test_strict_and_retry(tmp_path):
    g = modelgen.GraphBuilder(0)
    g.op("Relu", ["X"], "r")
    g.op("TestFlaky", ["r"], "m")          # tests/js/retry_entries.js: throws on hip, doubles on cpu
    g.op("Relu", ["m"], "Y")
    data = g.finish([("X", [4, 6])], [("Y", [4, 6])])
    (tmp_path / "model.onnx").write_bytes(data)
    X = np.random.default_rng(5).standard_normal((4, 6)).astype(np.float32)
    retry = ["--cpu-entries", node_runner.RETRY_ENTRIES]
    with pytest.raises(RuntimeError, match="the hip implementation refuses"):
        node_runner.run_model(str(tmp_path), [X], "hip", strict=True, fake_native=True, extra=retry)
    outs, rep = node_runner.run_model(str(tmp_path), [X], "hip", strict=False, fake_native=True, extra=retry)
    assert rep["stats"]["retriedOnCpu"] == ["TestFlaky_1"] and rep["stats"]["nodesByBackend"] == {"hip": 2, "cpu": 1}
    assert_bit_exact(outs[0], 2 * np.maximum(X, 0))
    # the tensor the failing hip operator had allocated is gone; only run-scoped buffers were live
    assert rep["liveBuffers"] == rep["initializerCopies"]
    # without a cpu implementation the retry fails too, and the error surfaces
    g = modelgen.GraphBuilder(0)
    g.op("Softmax", ["X"], "Y", axis=0)   # hip: last axis only; this package registers no cpu Softmax
    data = g.finish([("X", [4, 6])], [("Y", [4, 6])])
    (tmp_path / "model.onnx").write_bytes(data)
    with pytest.raises(RuntimeError, match="does not exist"):
        node_runner.run_model(str(tmp_path), [X], "hip", strict=False, fake_native=True, oracle_cpu=False)


def test_reduce_mean_over_any_axes_on_the_host_path(tmp_path):
    """ReduceMean: one device pass per axis, ascending, fp32 in between (reduce.ts:40-131, 369-405)."""
    X = np.random.default_rng(6).standard_normal((3, 4, 5, 6)).astype(np.float32)
    for axes, keep in (([1], 1), ([0, 2], 0), ([-1], 1), ([], 1), ([3, 0, 1], 0), ([2, 3], 1)):
        g = modelgen.GraphBuilder(0)
        attrs = dict(keepdims=keep)
        if axes:
            attrs["axes"] = axes
        g.op("ReduceMean", ["X"], "Y", **attrs)
        want = ref.reduce_mean(X, axes, keep)
        data = g.finish([("X", list(X.shape))], [("Y", list(want.shape))])
        (tmp_path / "model.onnx").write_bytes(data)
        hip, rep = node_runner.run_model(str(tmp_path), [X], "hip", fake_native=True)
        assert rep["stats"]["nodesByBackend"] == {"hip": 1}
        assert hip[0].shape == want.shape
        assert_bit_exact(hip[0], want, "ReduceMean axes %s" % (axes,))
        cpu, _ = node_runner.run_model(str(tmp_path), [X], "cpu", oracle_cpu=True)
        assert_bit_exact(cpu[0], want, "JS oracle vs C oracle, axes %s" % (axes,))


def test_unit_level_js(tmp_path):
    """tests/js/unit.js: registry rules, CPUTensor, ONNX reader, fusion pass, load() fallbacks."""
    proc = subprocess.run(["node", os.path.join(ROOT, "tests", "js", "unit.js")], stdout=subprocess.PIPE,
                          stderr=subprocess.PIPE, text=True, timeout=120)
    assert proc.returncode == 0, proc.stdout[-3000:] + proc.stderr[-3000:]
    summary = json.loads(proc.stdout.strip().splitlines()[-1])
    assert summary["failed"] == 0 and summary["passed"] >= 14, summary


@pytest.mark.parametrize("hd,one_launch", [(32, True), (8, False)])
def test_attention_chain_becomes_one_node(tmp_path, hd, one_launch):
    """MatMul -> Mul -> Softmax -> MatMul with the head Transposes around it becomes one
    WebDNNHipAttention node.  Head dimensions the kernel is built for take one native call; others
    run the steps one by one inside the node.  Either way the output is the unfused graph's."""
    g = modelgen.GraphBuilder(1)
    tq, tk, h = 7, 9, 2
    d = h * hd
    g.const("sq", np.array([tq, h, hd], np.int64))
    g.const("sk", np.array([tk, h, hd], np.int64))
    g.const("so", np.array([tq, d], np.int64))
    g.const("scale", np.array(1.0 / np.sqrt(hd), np.float32))
    g.op("Transpose", [g.op("Reshape", ["Q", "sq"], "q3")], "qh", perm=[1, 0, 2])
    g.op("Transpose", [g.op("Reshape", ["K", "sk"], "k3")], "kt", perm=[1, 2, 0])
    g.op("Transpose", [g.op("Reshape", ["V", "sk"], "v3")], "vh", perm=[1, 0, 2])
    g.op("Softmax", [g.op("Mul", [g.op("MatMul", ["qh", "kt"], "scores"), "scale"], "scaled")], "attn", axis=-1)
    g.op("Reshape", [g.op("Transpose", [g.op("MatMul", ["attn", "vh"], "ctx")], "ctx_t", perm=[1, 0, 2]), "so"], "Y")
    data = g.finish([("Q", [tq, d]), ("K", [tk, d]), ("V", [tk, d])], [("Y", [tq, d])], opset=13)
    (tmp_path / "model.onnx").write_bytes(data)
    rng = np.random.default_rng(3)
    feeds = {n: rng.standard_normal(s).astype(np.float32) for n, s in (("Q", (tq, d)), ("K", (tk, d)), ("V", (tk, d)))}
    ins = [feeds["Q"], feeds["K"], feeds["V"]]
    outs, rep = node_runner.run_model(str(tmp_path), ins, "hip", strict=True, fake_native=True)
    assert rep["nodes"] == 5                       # 4 Reshapes + the attention node
    calls = rep["nativeCalls"]
    if one_launch:
        assert calls.get("attention") == 1 and "gemm" not in calls and "softmax" not in calls
    else:
        assert calls.get("attention") is None and calls["gemm"] == 2 and calls["softmax"] == 1
    assert rep["liveBuffers"] == rep["initializerCopies"]
    want = graph_ref.run_graph(modelgen.parse_model(data), feeds)["Y"]
    np.testing.assert_allclose(outs[0], want, rtol=0, atol=1e-6)
    plain, rep_p = node_runner.run_model(str(tmp_path), ins, "hip", strict=True, fuse=False, fake_native=True)
    assert rep_p["nodes"] == 12
    np.testing.assert_allclose(outs[0], plain[0], rtol=0, atol=1e-6)


def test_fused_matmul_keeps_the_broadcasting_of_the_nodes_it_absorbed(tmp_path):
    """Two shapes where the absorbed Mul / Add broadcast differently from the kernel's alpha and C term:
    a one-element constant of rank 4 (the Mul raises the result's rank: not absorbed) and a matrix-vector
    product, whose result [m] gets a bias [m] (absorbed; the node then runs the Add separately).  The fused
    graph gives the unfused graph's bits and shapes."""
    g = modelgen.GraphBuilder(8)
    m, k = 6, 10
    rng = g.rng()
    g.const("v", rng.standard_normal((k,)).astype(np.float32))
    g.const("bm", rng.standard_normal((m,)).astype(np.float32))
    g.const("W", rng.standard_normal((k, k)).astype(np.float32))
    g.const("s4", np.full((1, 1, 1, 1), 0.5, np.float32))
    g.const("s1", np.full((1,), 0.25, np.float32))
    g.op("Relu", [g.op("Add", [g.op("MatMul", ["X", "v"], "xv"), "bm"], "xvb")], "Y1")      # [m,k] x [k] -> [m], + [m]
    g.op("Mul", [g.op("MatMul", ["X", "W"], "xw"), "s4"], "Y2")                              # -> [1,1,m,k]
    g.op("Mul", [g.op("MatMul", ["X", "W"], "xw2"), "s1"], "Y3")                             # -> [m,k], absorbed
    data = g.finish([("X", [m, k])], [("Y1", [m]), ("Y2", [1, 1, m, k]), ("Y3", [m, k])], opset=13)
    (tmp_path / "model.onnx").write_bytes(data)
    X = np.random.default_rng(9).standard_normal((m, k)).astype(np.float32)
    outs, rep = node_runner.run_model(str(tmp_path), [X], "hip", strict=True, fake_native=True)
    plain, rep_p = node_runner.run_model(str(tmp_path), [X], "hip", strict=True, fuse=False, fake_native=True)
    assert rep["nodes"] < rep_p["nodes"]
    for a, b, shape in zip(outs, plain, ((m,), (1, 1, m, k), (m, k))):
        assert a.shape == b.shape == shape, (a.shape, b.shape)
        assert_bit_exact(a, b, "fused vs unfused %s" % (shape,))
    want = graph_ref.run_graph(modelgen.parse_model(data), {"X": X})
    for got, name in zip(outs, ("Y1", "Y2", "Y3")):
        np.testing.assert_allclose(got, want[name], rtol=0, atol=1e-5)


def test_neighbouring_linear_layers_run_as_one_group(tmp_path):
    """Projections of one input and rank-3 MatMuls next to rank-2 ones:
    grouped into one node; the rank-2 ones take one native call, a group with the rank-3 product in it
    runs product by product.  Bit-identical to the ungrouped graph."""
    g = modelgen.GraphBuilder(5)
    t, d = 5, 12
    rng = g.rng()
    for name, shape in (("Wq", (d, d)), ("Wk", (d, 8)), ("Wv", (d, d)), ("bq", (d,)), ("bk", (8,)), ("W3", (d, 4))):
        g.const(name, (rng.standard_normal(shape) * 0.3).astype(np.float32))
    g.const("s3", np.array([1, t, d], np.int64))
    g.op("Add", [g.op("MatMul", ["X", "Wq"], "q_mm"), "bq"], "q")
    g.op("Add", [g.op("MatMul", ["X", "Wk"], "k_mm"), "bk"], "k")
    g.op("MatMul", ["X", "Wv"], "v")
    g.op("Reshape", ["X", "s3"], "x3")
    g.op("MatMul", ["x3", "W3"], "p3")          # rank 3, alone in its run (the Reshape separates it)
    g.op("MatMul", ["q", "Wq"], "qq")
    g.op("MatMul", ["x3", "Wv"], "pv")          # rank 3 next to a rank-2 product: grouped, run one by one
    g.op("MatMul", [g.op("Add", ["qq", "v"], "qv"), "Wk"], "Y")
    data = g.finish([("X", [t, d])], [("Y", [t, 8]), ("k", [t, 8]), ("p3", [1, t, 4]), ("pv", [1, t, d])], opset=13)
    (tmp_path / "model.onnx").write_bytes(data)
    feeds = {"X": np.random.default_rng(6).standard_normal((t, d)).astype(np.float32)}
    outs, rep = node_runner.run_model(str(tmp_path), [feeds["X"]], "hip", strict=True, fake_native=True)
    calls = rep["nativeCalls"]
    # (q, k) as a group; (p3, qq, pv) grouped but rank 3 among them: one by one; X Wv + qq as a fused node; Y
    assert calls["linearGroup"] == 1 and calls["gemm"] == 5 and rep["nodes"] == 5
    plain, rep_p = node_runner.run_model(str(tmp_path), [feeds["X"]], "hip", strict=True, fuse=False, fake_native=True)
    assert rep_p["nodes"] > rep["nodes"]
    for a, b in zip(outs, plain):
        assert_bit_exact(a, b, "grouped linear layers")
    want = graph_ref.run_graph(modelgen.parse_model(data), feeds)
    for got, name in zip(outs, ("Y", "k", "p3", "pv")):
        np.testing.assert_allclose(got, want[name], rtol=0, atol=2e-5)


def test_layernorm_with_the_add_that_follows(tmp_path):
    """LayerNormalization -> Add(constant) becomes one two-output node: same-shape addends ride in the
    launch (layernormAdd), broadcasting ones are added by the Add kernel inside the node.  The
    normalised tensor keeps its other readers.  Bit-identical to the unfused graph."""
    g = modelgen.GraphBuilder(2)
    t, d = 6, 16
    rng = g.rng()
    g.const("gamma", rng.standard_normal(d).astype(np.float32))
    g.const("beta", rng.standard_normal(d).astype(np.float32))
    g.const("pos", rng.standard_normal((t, d)).astype(np.float32))
    g.const("row", rng.standard_normal((d,)).astype(np.float32))
    g.op("LayerNormalization", ["X", "gamma", "beta"], "n1", axis=-1, epsilon=1e-5)
    g.op("Add", ["n1", "pos"], "n1p")
    g.op("Mul", ["n1", "n1p"], "m")
    g.op("LayerNormalization", ["m", "gamma", "beta"], "n2", axis=-1, epsilon=1e-5)
    g.op("Add", ["row", "n2"], "n2r")
    g.op("Sub", ["n2r", "n2"], "Y")
    data = g.finish([("X", [t, d])], [("Y", [t, d])], opset=17)
    (tmp_path / "model.onnx").write_bytes(data)
    feeds = {"X": np.random.default_rng(9).standard_normal((t, d)).astype(np.float32)}
    outs, rep = node_runner.run_model(str(tmp_path), [feeds["X"]], "hip", strict=True, fake_native=True)
    assert rep["nodes"] == 4
    calls = rep["nativeCalls"]
    assert calls["layernormAdd"] == 1 and calls["layernorm"] == 1 and calls["binary"] == 3
    assert rep["liveBuffers"] == rep["initializerCopies"]
    plain, rep_p = node_runner.run_model(str(tmp_path), [feeds["X"]], "hip", strict=True, fuse=False, fake_native=True)
    assert rep_p["nodes"] == 6
    assert_bit_exact(outs[0], plain[0], "LayerNormalization+Add fused")
    want = graph_ref.run_graph(modelgen.parse_model(data), feeds)["Y"]
    np.testing.assert_allclose(outs[0], want, rtol=0, atol=5e-6)


def test_detr_style_graph_on_the_hip_host_path(tmp_path):
    """The config-5 graph at toy size: every operator and shape trick it uses (head split by
    Reshape+Transpose, K^T by Transpose, scalar Mul, Softmax, LayerNormalization, fused MatMul+bias,
    Sigmoid) through the hip host code."""
    data, g = modelgen.detr_model(image=(64, 96), d=32, heads=4, ffn=64, enc_layers=2, dec_layers=2, queries=10,
                                  classes=7, width=8, blocks=(1, 1, 1, 1))
    (tmp_path / "model.onnx").write_bytes(data)
    X = np.random.default_rng(8).standard_normal((1, 3, 64, 96)).astype(np.float32)
    outs, rep = node_runner.run_model(str(tmp_path), [X], "hip", strict=True, fake_native=True)
    assert list(rep["stats"]["nodesByBackend"]) == ["hip"] and rep["liveBuffers"] == rep["initializerCopies"]
    want = graph_ref.run_graph(modelgen.parse_model(data), {"input": X})
    np.testing.assert_allclose(outs[0], want["logits"], rtol=0, atol=1e-5)
    np.testing.assert_allclose(outs[1], want["boxes"], rtol=0, atol=1e-5)
    plain, rep_p = node_runner.run_model(str(tmp_path), [X], "hip", strict=True, fuse=False, fake_native=True)
    assert rep_p["nodes"] > rep["nodes"]
    assert_bit_exact(plain[0], outs[0], "fusion keeps the logits")


@pytest.mark.parametrize("opset", [11, 13])
def test_export_style_glue_graph(tmp_path, opset):
    """Shape -> Gather -> Unsqueeze -> Concat -> Reshape on the metadata side and Split / Concat /
    Slice / Cast / Squeeze / Unsqueeze on the data, with axes as attributes (opset 11) and as
    inputs (opset 13).  Shape and Constant are the only nodes placed on the cpu, as in the
    reference (operatorTable.ts:47-50; Constant exists for cpu only)."""
    data, _ = modelgen.glue_model(opset)
    X = np.random.default_rng(1).standard_normal((2, 6, 4, 5)).astype(np.float32)
    model, hip, cpu, rep = both_paths(tmp_path, data, {"X": X})
    assert rep["stats"]["nodesByBackend"] == {"cpu": 2, "hip": len(model["nodes"]) - 2}, rep["stats"]
    assert rep["stats"]["retriedOnCpu"] == []
    want = graph_ref.run_graph(model, {"X": X})
    for got_hip, got_cpu, (name, _) in zip(hip, cpu, model["outputs"]):
        assert_bit_exact(got_hip, got_cpu, name + ": hip host path vs cpu path")
        assert_bit_exact(got_hip, want[name], name + ": vs the python oracle")
    assert hip[1].dtype == np.int32
    assert rep["liveBuffers"] == rep["initializerCopies"]


def _graph_vs_eager(tmp_path, data, feeds_a, feeds_b, fake_native, flags=("--graph",), runs=(3, 4)):
    """Runs 1..4 with {graph: true}: eager warm-up, capture + launch, replay, replay; even runs use
    feeds_a, odd runs feeds_b.  Returns (outputs of run 3 (a), outputs of run 4 (b), eager a, eager b, report).
    `flags`: what the CLI passes on to runner.run (nothing = the runner's default); `runs`: an odd and an
    even session length to compare instead of 3 and 4."""
    (tmp_path / "model.onnx").write_bytes(data)
    model = modelgen.parse_model(data)
    a = [feeds_a[n] for n, _ in model["inputs"]]
    b = [feeds_b[n] for n, _ in model["inputs"]]
    alt = []
    for i, arr in enumerate(b):
        p = tmp_path / ("alt_%d.bin" % i)
        np.ascontiguousarray(arr).tofile(str(p))
        alt.append(str(p))
    kw = dict(strict=True, fake_native=fake_native)
    eager_a, _ = node_runner.run_model(str(tmp_path), a, "hip", **kw)
    eager_b, _ = node_runner.run_model(str(tmp_path), b, "hip", **kw)
    extra = list(flags) + ["--alt-inputs", ",".join(alt)]
    g3, rep3 = node_runner.run_model(str(tmp_path), a, "hip", runs=runs[0], extra=extra, **kw)
    g4, rep4 = node_runner.run_model(str(tmp_path), a, "hip", runs=runs[1], extra=extra, **kw)
    return g3, g4, eager_a, eager_b, rep4


def test_projection_shortcuts_become_side_branches(tmp_path):
    """modelTransform.hoistSideBranches: in a ResNet the projection shortcut of each stage's first block is moved
    up to the block's start and bracketed with branchBegin / branchEnd, its consumer preceded by branchJoin;
    results equal the cpu path bit for bit in the node loop, in a recorded run, and with the pass switched off."""
    data, _ = modelgen.resnet50_model(batch=2, image=32, width=8, blocks=(1, 2, 1, 1), classes=10)
    X = np.random.default_rng(2).standard_normal((2, 3, 32, 32)).astype(np.float32)
    (tmp_path / "model.onnx").write_bytes(data)
    want, _ = node_runner.run_model(str(tmp_path), [X], "cpu", oracle_cpu=True)
    kw = dict(strict=True, fake_native=True)
    eager, rep = node_runner.run_model(str(tmp_path), [X], "hip", extra=["--no-graph"], **kw)
    assert rep["nativeCalls"]["branchBegin"] == 4 and rep["nativeCalls"]["branchEnd"] == 4 and rep["nativeCalls"]["branchJoin"] == 4
    assert_bit_exact(eager[0], want[0], "node loop with the shortcuts moved up")
    replay, rep = node_runner.run_model(str(tmp_path), [X], "hip", runs=4, extra=["--graph"], **kw)
    assert rep["graph"]["captured"] and rep["nativeCalls"]["branchBegin"] == 2 * 4    # one eager run, one recording
    assert_bit_exact(replay[0], want[0], "replay with side branches")
    plain, rep = node_runner.run_model(str(tmp_path), [X], "hip", runs=3, extra=["--graph", "--no-side-branches"], **kw)
    assert "branchBegin" not in rep["nativeCalls"]
    assert_bit_exact(plain[0], want[0], "pass switched off")


def test_two_runs_in_flight_on_the_host_path(tmp_path):
    """runner.submit / runner.collect against the stand-in addon: whatever the session length, the last run's
    outputs equal the eager run of its input; the second lane is recorded once, every pipelined run brackets its
    work with lane switches, and nothing but the initializer copies outlives disposeGraph."""
    data, _ = modelgen.resnet50_model(batch=2, image=32, width=8, blocks=(1, 1, 1, 1), classes=10)
    Xa = np.random.default_rng(2).standard_normal((2, 3, 32, 32)).astype(np.float32)
    Xb = np.random.default_rng(3).standard_normal((2, 3, 32, 32)).astype(np.float32)
    g5, g8, ea, eb, rep = _graph_vs_eager(tmp_path, data, {"input": Xa}, {"input": Xb}, True,
                                          flags=("--in-flight",), runs=(5, 8))
    assert rep["graph"] == {"captured": True, "lanes": 2, "unsupported": None}
    assert_bit_exact(g5[0], ea[0], "fifth run (first one on the second lane)")
    assert_bit_exact(g8[0], eb[0], "eighth run")
    # 8 runs: 2 eager, run 3 records lane 0 and launches, runs 4, 6, 8 replay lane 0, run 5 records lane 1, 7 replays it
    assert rep["nativeCalls"]["graphBegin"] == 2 and rep["nativeCalls"]["graphLaunch"] == 6
    assert rep["nativeCalls"]["setLane"] >= 2 * 5
    assert rep["liveBuffers"] == rep["initializerCopies"]


def test_graph_replay_on_the_host_path(tmp_path):
    data, _ = modelgen.resnet50_model(batch=2, image=32, width=8, blocks=(1, 1, 1, 1), classes=10)
    Xa = np.random.default_rng(2).standard_normal((2, 3, 32, 32)).astype(np.float32)
    Xb = np.random.default_rng(3).standard_normal((2, 3, 32, 32)).astype(np.float32)
    g3, g4, ea, eb, rep = _graph_vs_eager(tmp_path, data, {"input": Xa}, {"input": Xb}, True)
    assert rep["graph"] == {"captured": True, "lanes": 1, "unsupported": None}
    assert rep["stats"]["graphReplay"] is True and list(rep["stats"]["nodesByBackend"]) == ["hip"]
    assert_bit_exact(g3[0], ea[0], "third run (replay, first input)")
    assert_bit_exact(g4[0], eb[0], "fourth run (replay, second input)")
    assert rep["nativeCalls"]["graphLaunch"] == 3
    assert rep["liveBuffers"] == rep["initializerCopies"]          # the graph's buffers are gone after disposeGraph


def test_a_caller_that_passes_no_option_gets_the_graph_after_two_runs(tmp_path):
    """runner.run(inputs) as the reference's callers write it: runs 1 and 2 walk the node loop, run 3 is
    recorded and launched, later runs replay -- with the bits of the eager runs of the same inputs.  Two
    runs never record anything; {graph: false} keeps every run in the node loop."""
    data, _ = modelgen.resnet50_model(batch=2, image=32, width=8, blocks=(1, 1, 1, 1), classes=10)
    Xa = np.random.default_rng(2).standard_normal((2, 3, 32, 32)).astype(np.float32)
    Xb = np.random.default_rng(3).standard_normal((2, 3, 32, 32)).astype(np.float32)
    g5, g6, ea, eb, rep = _graph_vs_eager(tmp_path, data, {"input": Xa}, {"input": Xb}, True, flags=(), runs=(5, 6))
    assert rep["graph"] == {"captured": True, "lanes": 1, "unsupported": None}
    assert rep["stats"]["graphReplay"] is True
    assert_bit_exact(g5[0], ea[0], "fifth run (replay, first input)")
    assert_bit_exact(g6[0], eb[0], "sixth run (replay, second input)")
    assert rep["nativeCalls"]["graphLaunch"] == 4 and rep["nativeCalls"]["graphBegin"] == 1
    assert rep["liveBuffers"] == rep["initializerCopies"]
    _, rep2 = node_runner.run_model(str(tmp_path), [Xa], "hip", runs=2, fake_native=True)
    assert rep2["graph"]["captured"] is False and "graphBegin" not in rep2["nativeCalls"]
    _, rep_off = node_runner.run_model(str(tmp_path), [Xa], "hip", runs=5, fake_native=True, extra=["--no-graph"])
    assert "graphBegin" not in rep_off["nativeCalls"] and "graphReplay" not in rep_off["stats"]


def test_exporter_shaped_model_bytes_decode_and_run(tmp_path):
    """A ModelProto laid out the way the PyTorch exporter writes one (the shape of the reference's
    example/minimum/model/model.onnx: ir_version, producer name and version, then the graph with its
    node before its name, value infos with TypeProto.Tensor shapes, opset_import last), assembled here
    byte by byte from the field numbers of onnx.proto rather than by this package's own encoder.  The
    decoder must skip the fields it has no use for and find the rest; the one Relu node then has to
    reproduce the reference's own vector (test/unit/cpuOperator.test.ts:15-18) on both backends."""
    def varint(v):
        out = bytearray()
        while True:
            out.append((v & 0x7F) | (0x80 if v > 0x7F else 0))
            v >>= 7
            if not v:
                return bytes(out)

    def field(number, payload):            # wire type 2: length-delimited
        return varint(number << 3 | 2) + varint(len(payload)) + payload

    def scalar(number, value):             # wire type 0: varint
        return varint(number << 3 | 0) + varint(value)

    def value_info(name, dims):            # ValueInfoProto{name=1, type=2{tensor_type=1{elem_type=1, shape=2{dim=1{dim_value=1}}}}}
        shape = b"".join(field(1, scalar(1, d)) for d in dims)
        return field(1, name) + field(2, field(1, scalar(1, 1) + field(2, shape)))

    node = field(1, b"in0") + field(2, b"out0") + field(3, b"Relu_0") + field(4, b"Relu")
    graph = field(1, node) + field(2, b"exported-graph") + field(11, value_info(b"in0", [2, 3])) + \
        field(12, value_info(b"out0", [2, 3]))
    model = scalar(1, 6) + field(2, b"pytorch") + field(3, b"1.7") + field(7, graph) + field(8, scalar(2, 9))
    assert len(model) == 112 and model[:2] == b"\x08\x06"      # ir_version = 6 comes first
    (tmp_path / "model.onnx").write_bytes(model)
    parsed = modelgen.parse_model(model)
    assert parsed["opset"] == 9 and [n["op_type"] for n in parsed["nodes"]] == ["Relu"]
    assert parsed["inputs"] == [("in0", [2, 3])] and parsed["outputs"] == [("out0", [2, 3])]
    x = np.array([[-2, -0.5, 0], [1, 3, -0.0]], np.float32)
    want = np.array([[0, 0, 0], [1, 3, 0]], np.float32)
    for backend, kw in (("cpu", dict(oracle_cpu=True)), ("hip", dict(fake_native=True))):
        out, rep = node_runner.run_model(str(tmp_path), [x], backend, **kw)
        assert rep["outputs"][0]["name"] == "out0" and rep["outputs"][0]["dims"] == [2, 3]
        assert_bit_exact(out[0], want, "Relu through %s" % backend)


def test_cli_reports_device_time_of_every_run(tmp_path):
    """--measure-all: one device time per timed run, eager (an event per node boundary) and replayed
    (one event pair around the graph launch)."""
    data, _ = modelgen.resnet50_model(batch=1, image=32, width=4, blocks=(1, 1, 1, 1), classes=5)
    (tmp_path / "model.onnx").write_bytes(data)
    X = np.random.default_rng(4).standard_normal((1, 3, 32, 32)).astype(np.float32)
    _, eager = node_runner.run_model(str(tmp_path), [X], "hip", fake_native=True, runs=3, extra=["--measure-all"])
    assert len(eager["deviceMsPerRun"]) == 3 and "performance" not in eager
    _, replay = node_runner.run_model(str(tmp_path), [X], "hip", fake_native=True, runs=4, warmup=2,
                                      extra=["--graph", "--measure-all"])
    assert replay["graph"]["captured"] and len(replay["deviceMsPerRun"]) == 4
    _, plain = node_runner.run_model(str(tmp_path), [X], "hip", fake_native=True, runs=2)
    assert "deviceMsPerRun" not in plain


def test_graph_mode_falls_back_when_the_run_needs_device_data_on_the_host(tmp_path):
    """The glue graph computes a Reshape shape on the device; reading it back cannot be recorded."""
    data, _ = modelgen.glue_model(11)
    X = np.random.default_rng(1).standard_normal((2, 6, 4, 5)).astype(np.float32)
    g3, g4, ea, eb, rep = _graph_vs_eager(tmp_path, data, {"X": X}, {"X": X * 2}, True)
    assert rep["graph"]["captured"] is False and "captur" in rep["graph"]["unsupported"]
    assert_bit_exact(g3[0], ea[0])
    assert_bit_exact(g4[0], eb[0])
    assert rep["liveBuffers"] == rep["initializerCopies"]
