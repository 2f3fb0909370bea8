"""The Node.js host on the hip backend: WebDNN.load() + runner.run() on a real MI355X, against the
same graph on the cpu path (the JavaScript oracle) and against the C oracle.

Every run is strict: the per-node CPU retry of the reference's runner is off, and the per-backend
node counter must show every node on `hip`, so that a fallback cannot fake a pass."""
import numpy as np
import pytest

import graph_ref
import node_runner
from util import assert_bit_exact, assert_close_max
from webdnn_amd import modelgen

pytestmark = pytest.mark.gpu


def run_both(tmp_path, model_bytes, feeds, fuse=True):
    (tmp_path / "model.onnx").write_bytes(model_bytes)
    model = modelgen.parse_model(model_bytes)
    ordered = [feeds[n] for n, _ in model["inputs"]]
    hip, report = node_runner.run_model(str(tmp_path), ordered, "hip", strict=True, fuse=fuse)
    assert report["backend"] == "hip"
    assert list(report["stats"]["nodesByBackend"]) == ["hip"], report["stats"]
    assert report["stats"]["retriedOnCpu"] == []
    return model, hip, report


def test_gemm_config1(tmp_path):
    data, _ = modelgen.gemm_model()
    A = np.random.default_rng(1).uniform(-1, 1, (256, 512)).astype(np.float32)
    model, hip, _ = run_both(tmp_path, data, {"A": A})
    want = graph_ref.run_graph(model, {"A": A})["Y"]
    assert_close_max(hip[0], want, 1e-4, "config 1 through the runner")


def test_ffn_config2_fused_and_unfused(tmp_path):
    data, _ = modelgen.ffn_model()
    X = np.random.default_rng(2).standard_normal((8, 512, 768)).astype(np.float32)
    model, fused, rep_f = run_both(tmp_path, data, {"X": X}, fuse=True)
    _, plain, rep_p = run_both(tmp_path, data, {"X": X}, fuse=False)
    assert rep_p["nodes"] == 5 and rep_f["nodes"] == 2          # MatMul+Add+Relu, MatMul+Add
    assert_bit_exact(fused[0], plain[0], "fusion does not change the result")
    rows = np.sort(np.random.default_rng(3).choice(8 * 512, 48, replace=False))
    sub = modelgen.parse_model(data)
    want = graph_ref.run_graph(sub, {"X": X.reshape(-1, 768)[rows]})["out"]
    assert_close_max(fused[0].reshape(-1, 768)[rows], want, 1e-4, "config 2 rows")


def test_conv_config3(tmp_path):
    data, _ = modelgen.conv_model()
    X = np.random.default_rng(4).uniform(0, 1, (32, 64, 56, 56)).astype(np.float32)
    model, hip, rep = run_both(tmp_path, data, {"X": X})
    assert rep["nodes"] == 1                                        # Conv+Relu fused
    want = graph_ref.run_graph(model, {"X": X})["Y"]
    assert_close_max(hip[0], want, 1e-4, "config 3 through the runner")


def test_resnet_tiny_matches_cpu_path(tmp_path):
    data, _ = modelgen.resnet50_model(batch=2, image=64, classes=10, width=16, blocks=(2, 1, 1, 1))
    X = np.random.default_rng(5).standard_normal((2, 3, 64, 64)).astype(np.float32)
    model, hip, rep = run_both(tmp_path, data, {"input": X})
    cpu, rep_cpu = node_runner.run_model(str(tmp_path), [X], "cpu", oracle_cpu=True)
    assert rep_cpu["stats"]["nodesByBackend"] == {"cpu": rep_cpu["nodes"]}
    assert np.abs(hip[0] - cpu[0]).max() <= 1e-3, "logits within 1e-3 of the cpu backend"
    _, plain, _ = run_both(tmp_path, data, {"input": X}, fuse=False)
    assert_bit_exact(hip[0], plain[0], "fusion does not change the logits")


def test_resnet50_batch32_logits(tmp_path):
    """Config 4 at full size: logits within 1e-3 (absolute) of the CPU oracle."""
    data, g = modelgen.resnet50_model()
    X = np.random.default_rng(6).standard_normal((32, 3, 224, 224)).astype(np.float32)
    model, hip, rep = run_both(tmp_path, data, {"input": X})
    assert hip[0].shape == (32, 1000) and np.isfinite(hip[0]).all()
    # the oracle follows 4 of the 32 images (every op of the graph is per-image)
    pick = [0, 7, 19, 31]
    want = graph_ref.run_graph(model, {"input": X[pick]})["logits"]
    err = np.abs(hip[0][pick] - want).max()
    assert err <= 1e-3, "max |logit diff| %.3e" % err


def test_non_strict_falls_back_per_node(tmp_path):
    """An operator the hip backend rejects at run time is retried once on the cpu operators
    (reference: core/runnerImpl.ts:511-520) when strict mode is off, and fails loudly when it is on."""
    g = modelgen.GraphBuilder(0)
    g.op("Softmax", ["X"], "s", axis=1)          # non-last axis: hip throws, and so does the cpu operator
    data = g.finish([("X", [2, 3, 4])], [("s", [2, 3, 4])])
    (tmp_path / "model.onnx").write_bytes(data)
    X = np.zeros((2, 3, 4), np.float32)
    with pytest.raises(RuntimeError, match="only reducing final axis"):
        node_runner.run_model(str(tmp_path), [X], "hip", strict=True)
    with pytest.raises(RuntimeError, match="only reducing final axis"):
        node_runner.run_model(str(tmp_path), [X], "hip", strict=False, oracle_cpu=True)
    # an operator whose hip implementation throws (tests/js/retry_entries.js) and whose cpu one works
    g = modelgen.GraphBuilder(0)
    g.op("Relu", ["X"], "r")
    g.op("TestFlaky", ["r"], "m")
    g.op("Relu", ["m"], "Y")
    data = g.finish([("X", [4, 6])], [("Y", [4, 6])])
    (tmp_path / "model.onnx").write_bytes(data)
    X = np.random.default_rng(7).standard_normal((4, 6)).astype(np.float32)
    retry = ["--cpu-entries", node_runner.RETRY_ENTRIES]
    outs, rep = node_runner.run_model(str(tmp_path), [X], "hip", strict=False, extra=retry)
    assert rep["stats"]["retriedOnCpu"] == ["TestFlaky_1"]
    assert rep["stats"]["nodesByBackend"] == {"hip": 2, "cpu": 1}
    assert_bit_exact(outs[0], 2 * np.maximum(X, 0), "retried node")
    with pytest.raises(RuntimeError, match="the hip implementation refuses"):
        node_runner.run_model(str(tmp_path), [X], "hip", strict=True, extra=retry)
    # ReduceMean over a leading axis runs on the device
    g = modelgen.GraphBuilder(0)
    g.op("ReduceMean", ["X"], "Y", axes=[0, 2], keepdims=0)
    data = g.finish([("X", [5, 6, 7])], [("Y", [6])])
    (tmp_path / "model.onnx").write_bytes(data)
    X3 = np.random.default_rng(8).standard_normal((5, 6, 7)).astype(np.float32)
    outs, rep = node_runner.run_model(str(tmp_path), [X3], "hip", strict=True)
    assert rep["stats"]["nodesByBackend"] == {"hip": 1}
    from oracle import ref
    assert np.abs(outs[0] - ref.reduce_mean(X3, [0, 2], 0)).max() <= 1e-7


def test_detr_style_small(tmp_path):
    data, g = modelgen.detr_model(image=(128, 160), d=64, heads=8, ffn=128, enc_layers=2, dec_layers=2, queries=20,
                                  classes=11, width=16, blocks=(1, 1, 1, 1))
    X = np.random.default_rng(9).standard_normal((1, 3, 128, 160)).astype(np.float32)
    model, hip, rep = run_both(tmp_path, data, {"input": X})
    want = graph_ref.run_graph(model, {"input": X})
    assert np.abs(hip[0] - want["logits"]).max() <= 1e-3 and np.abs(hip[1] - want["boxes"]).max() <= 1e-3


def test_detr_r50_config5(tmp_path):
    """Config 5 at full size (input [1,3,800,1088], 850 tokens, 6+6 layers): outputs within 1e-3 of the oracle."""
    data, g = modelgen.detr_model()
    X = np.random.default_rng(10).standard_normal((1, 3, 800, 1088)).astype(np.float32)
    model, hip, rep = run_both(tmp_path, data, {"input": X})
    assert hip[0].shape == (100, 92) and hip[1].shape == (100, 4)
    want = graph_ref.run_graph(model, {"input": X})
    assert np.abs(hip[0] - want["logits"]).max() <= 1e-3, np.abs(hip[0] - want["logits"]).max()
    assert np.abs(hip[1] - want["boxes"]).max() <= 1e-3


@pytest.mark.parametrize("opset", [11, 13])
def test_export_style_glue_graph(tmp_path, opset):
    """Layout glue (Split / Concat / Slice / Cast / Squeeze / Unsqueeze / Gather) on the device and the
    shape chain around Reshape; bit-exact, since nothing here does arithmetic except one Mul and Add."""
    data, _ = modelgen.glue_model(opset)
    X = np.random.default_rng(1).standard_normal((2, 6, 4, 5)).astype(np.float32)
    (tmp_path / "model.onnx").write_bytes(data)
    model = modelgen.parse_model(data)
    hip, rep = node_runner.run_model(str(tmp_path), [X], "hip", strict=True)
    assert rep["stats"]["nodesByBackend"] == {"cpu": 2, "hip": len(model["nodes"]) - 2}, rep["stats"]
    assert rep["stats"]["retriedOnCpu"] == []
    want = graph_ref.run_graph(model, {"X": X})
    assert_bit_exact(hip[0], want["Y"], "Y")
    assert_bit_exact(hip[1], want["ints"], "ints")


def test_optimized_model_directory(tmp_path):
    """model-hip.onnx + WDN2 weight files (raw and 8-bit coded) through WebDNN.load({optimized: true})."""
    from webdnn_amd import tensor_export
    data, _ = modelgen.resnet50_model(batch=4, image=64, width=16, blocks=(1, 1, 1, 1), classes=10)
    X = np.random.default_rng(2).standard_normal((4, 3, 64, 64)).astype(np.float32)
    model, want, _ = run_both(tmp_path, data, {"input": X})
    raw = tmp_path / "raw"
    tensor_export.export_model_directory(str(raw), data, split_size=100000)
    got, rep = node_runner.run_model(str(raw), [X], "hip", strict=True, extra=["--optimized"])
    assert_bit_exact(got[0], want[0], "raw weight files")
    assert list(rep["stats"]["nodesByBackend"]) == ["hip"]
    # 8-bit coded weights: the same graph with the weights the reader reconstructs
    coded = tmp_path / "coded"
    _, paths = tensor_export.export_model_directory(str(coded), data, split_size=0, compression_algorithm=1)
    got8, _ = node_runner.run_model(str(coded), [X], "hip", strict=True, extra=["--optimized"])
    decoded = tensor_export.load_tensors(paths)
    stripped, _ = modelgen.strip_initializers(data)
    m = modelgen.parse_model(stripped)
    m["initializers"] = decoded
    ref8 = graph_ref.run_graph(m, {"input": X})
    out_name = model["outputs"][0][0]
    assert_close_max(got8[0], ref8[out_name], 1e-3, "8-bit coded weights")


def _graph_runs(tmp_path, data, a, b, runs, resident=False, flags=("--graph",)):
    alt = []
    for i, arr in enumerate(b):
        p = tmp_path / ("alt_%d.bin" % i)
        np.ascontiguousarray(arr).tofile(str(p))
        alt.append(str(p))
    return node_runner.run_model(str(tmp_path), a, "hip", strict=True, runs=runs,
                                 extra=list(flags) + ["--alt-inputs", ",".join(alt)] + (["--resident-inputs"] if resident else []))


def test_graph_replay_equals_eager_runs(tmp_path):
    """runner.run(inputs, {graph: true}): eager warm-up, capture + launch, then replays with inputs that
    change from run to run; every compared run must equal the eager run of the same input bit for bit
    (same kernels, same order)."""
    data, _ = modelgen.resnet50_model(batch=8, image=64, width=16, blocks=(1, 2, 1, 1), classes=10)
    Xa = np.random.default_rng(2).standard_normal((8, 3, 64, 64)).astype(np.float32)
    Xb = np.random.default_rng(3).standard_normal((8, 3, 64, 64)).astype(np.float32)
    (tmp_path / "model.onnx").write_bytes(data)
    ea, _ = node_runner.run_model(str(tmp_path), [Xa], "hip", strict=True)
    eb, _ = node_runner.run_model(str(tmp_path), [Xb], "hip", strict=True)
    for runs, want in ((2, eb), (3, ea), (6, eb), (7, ea)):
        got, rep = _graph_runs(tmp_path, data, [Xa], [Xb], runs)
        assert rep["graph"] == {"captured": True, "lanes": 1, "unsupported": None}, rep["graph"]
        assert rep["stats"]["graphReplay"] is True
        assert_bit_exact(got[0], want[0], "run %d of a graph-mode session" % runs)


def test_two_runs_in_flight_equal_eager_runs(tmp_path):
    """runner.submit / runner.collect: run i+1 is enqueued on the library's other lane before the outputs of run
    i are fetched.  Inputs alternate from run to run; whatever the session length, the last run's outputs must
    equal the eager run of the input it was given bit for bit (each lane replays its own recording of the same
    node loop: same kernels in the same order, stream-scheduled launches included, which have a workspace
    per lane), and from the fifth run on (the fourth with {graph: true}) both lanes hold a captured run."""
    data, _ = modelgen.resnet50_model(batch=8, image=64, width=16, blocks=(1, 2, 1, 1), classes=10)
    Xa = np.random.default_rng(2).standard_normal((8, 3, 64, 64)).astype(np.float32)
    Xb = np.random.default_rng(3).standard_normal((8, 3, 64, 64)).astype(np.float32)
    (tmp_path / "model.onnx").write_bytes(data)
    ea, _ = node_runner.run_model(str(tmp_path), [Xa], "hip", strict=True, extra=["--no-graph"])
    eb, _ = node_runner.run_model(str(tmp_path), [Xb], "hip", strict=True, extra=["--no-graph"])
    for flags in (("--in-flight",), ("--in-flight", "--graph")):
        first_both = 5 if flags == ("--in-flight",) else 4   # (auto: two eager runs, then lane 0, lane 0 again, lane 1)
        for runs, want in ((2, eb), (3, ea), (4, eb), (5, ea), (6, eb), (9, ea), (12, eb)):
            for resident in (False, True):
                got, rep = _graph_runs(tmp_path, data, [Xa], [Xb], runs, resident=resident, flags=flags)
                assert rep["graph"]["unsupported"] is None, rep["graph"]
                assert rep["graph"]["lanes"] == (2 if runs >= first_both else (1 if runs >= first_both - 2 else 0)), (flags, runs, rep["graph"])
                assert list(rep["stats"]["nodesByBackend"]) == ["hip"]
                assert_bit_exact(got[0], want[0], "run %d of a session with two runs in flight %s" % (runs, flags))


def test_many_runs_in_flight_every_output_checked(tmp_path):
    """300 runs with alternating inputs, two and three in flight, from the host and resident: every collected
    output equals, byte for byte, the first output seen for its input (an eager run), so a hand-over between the
    lanes, a recycled block or a side branch that is wrong once in a hundred runs shows."""
    data, _ = modelgen.resnet50_model(batch=8, image=64, width=16, blocks=(1, 2, 1, 1), classes=10)
    Xa = np.random.default_rng(2).standard_normal((8, 3, 64, 64)).astype(np.float32)
    Xb = np.random.default_rng(3).standard_normal((8, 3, 64, 64)).astype(np.float32)
    (tmp_path / "model.onnx").write_bytes(data)
    eb, _ = node_runner.run_model(str(tmp_path), [Xb], "hip", strict=True, extra=["--no-graph"])
    for lanes in ("2", "3"):
        for resident in (False, True):
            got, rep = _graph_runs(tmp_path, data, [Xa], [Xb], 300, resident=resident, flags=("--in-flight", lanes, "--check-each"))
            assert rep["checkEach"] == {"checkedRuns": 298, "mismatchedRuns": 0}, (lanes, resident, rep["checkEach"])
            assert rep["graph"]["lanes"] == int(lanes)
            assert_bit_exact(got[0], eb[0], "the last of 300 runs")


def test_three_runs_in_flight_equal_eager_runs(tmp_path):
    """The same with three lanes (load option inFlight = 3): from the sixth run on all three hold a recording."""
    data, _ = modelgen.resnet50_model(batch=8, image=64, width=16, blocks=(1, 2, 1, 1), classes=10)
    Xa = np.random.default_rng(2).standard_normal((8, 3, 64, 64)).astype(np.float32)
    Xb = np.random.default_rng(3).standard_normal((8, 3, 64, 64)).astype(np.float32)
    (tmp_path / "model.onnx").write_bytes(data)
    ea, _ = node_runner.run_model(str(tmp_path), [Xa], "hip", strict=True, extra=["--no-graph"])
    eb, _ = node_runner.run_model(str(tmp_path), [Xb], "hip", strict=True, extra=["--no-graph"])
    for runs, want in ((5, ea), (6, eb), (7, ea), (10, eb), (13, ea)):
        got, rep = _graph_runs(tmp_path, data, [Xa], [Xb], runs, flags=("--in-flight", "3"))
        assert rep["graph"]["lanes"] == min(3, runs - 3) and rep["graph"]["unsupported"] is None, (runs, rep["graph"])
        assert_bit_exact(got[0], want[0], "run %d of a session with three runs in flight" % runs)


def test_runs_without_an_option_are_replayed_from_the_third_on(tmp_path):
    """runner.run([CPUTensor]) with no option (graph "auto"): two eager runs, the third recorded, the rest
    replayed; each compared run equals the eager run of the input it was given, bit for bit."""
    data, _ = modelgen.resnet50_model(batch=8, image=64, width=16, blocks=(1, 2, 1, 1), classes=10)
    Xa = np.random.default_rng(2).standard_normal((8, 3, 64, 64)).astype(np.float32)
    Xb = np.random.default_rng(3).standard_normal((8, 3, 64, 64)).astype(np.float32)
    (tmp_path / "model.onnx").write_bytes(data)
    ea, _ = node_runner.run_model(str(tmp_path), [Xa], "hip", strict=True, extra=["--no-graph"])
    eb, _ = node_runner.run_model(str(tmp_path), [Xb], "hip", strict=True, extra=["--no-graph"])
    for runs, want, captured in ((2, eb, False), (3, ea, True), (4, eb, True), (7, ea, True)):
        got, rep = _graph_runs(tmp_path, data, [Xa], [Xb], runs, flags=())
        assert rep["graph"]["captured"] is captured and rep["graph"]["unsupported"] is None, rep["graph"]
        assert rep["stats"].get("graphReplay", False) is captured
        assert_bit_exact(got[0], want[0], "run %d of a session without options" % runs)


def test_graph_replay_with_two_resident_device_inputs(tmp_path):
    """The caller hands over tensors that already live on the device and alternates between two of
    them: run(A) eager, run(B) captured, then A, B, A ... replayed.  The graph reads from buffers of
    its own, so every run must equal the eager run of the tensor it was given, and the caller's
    tensors must come through unchanged (the last run reads A or B again after several replays)."""
    data, _ = modelgen.resnet50_model(batch=4, image=64, width=16, blocks=(1, 1, 1, 1), classes=10)
    Xa = np.random.default_rng(12).standard_normal((4, 3, 64, 64)).astype(np.float32)
    Xb = np.random.default_rng(13).standard_normal((4, 3, 64, 64)).astype(np.float32)
    (tmp_path / "model.onnx").write_bytes(data)
    ea, _ = node_runner.run_model(str(tmp_path), [Xa], "hip", strict=True)
    eb, _ = node_runner.run_model(str(tmp_path), [Xb], "hip", strict=True)
    assert np.abs(ea[0] - eb[0]).max() > 0
    for runs, want in ((2, eb), (3, ea), (4, eb), (5, ea), (8, eb)):
        got, rep = _graph_runs(tmp_path, data, [Xa], [Xb], runs, resident=True)
        assert rep["graph"] == {"captured": True, "lanes": 1, "unsupported": None}, rep["graph"]
        assert_bit_exact(got[0], want[0], "run %d with resident inputs" % runs)


def test_graph_replay_detr_style(tmp_path):
    data, g = modelgen.detr_model(image=(128, 160), d=64, heads=8, ffn=128, enc_layers=2, dec_layers=2, queries=20,
                                  classes=11, width=16, blocks=(1, 1, 1, 1))
    Xa = np.random.default_rng(9).standard_normal((1, 3, 128, 160)).astype(np.float32)
    Xb = np.random.default_rng(10).standard_normal((1, 3, 128, 160)).astype(np.float32)
    (tmp_path / "model.onnx").write_bytes(data)
    eb, _ = node_runner.run_model(str(tmp_path), [Xb], "hip", strict=True)
    got, rep = _graph_runs(tmp_path, data, [Xa], [Xb], 4)
    assert rep["graph"]["captured"] is True
    for g_, w in zip(got, eb):
        assert_bit_exact(g_, w, "DETR-style graph, fourth run")
