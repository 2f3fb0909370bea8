"""Benchmark of the hip backend hot path on ONE MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline]

Prints one JSON line.

Workload of `value` (benchmark config 4): ResNet-50 v1, batch 32, fp32, random-initialised weights
(seeded), BatchNorm folded, run through the Node.js descriptor runner on the `hip` backend
(WebDNN.load + runner.run) in strict mode — no CPU fallback.  A step is one runner.run() over one
batch whose input tensor is already resident in HBM; the step ends when the logits are back on the
host (the run's only synchronisation).  Steps call runner.run(x, {graph: true}): the first warm-up
run is eager, the second records the run's kernels into a HIP graph, every timed step launches that
graph (same kernels, same order, one launch) and reads the logits.  `value` = 32 * steps / total time.

`roofline` is for the dominant kernels of that workload, the implicit-GEMM contraction kernels (the
1x1 convs read X in place, the 3x3 stride-1 convs stage input rows in LDS or, from 128 channels on,
run as F(2x2, 3x3) minimal filtering -- transforms around a batched product of the same kernel -- the
rest gather taps; all share one tile schedule and epilogue): their algorithmic FLOPs (2*M*N*K per
Conv/Gemm node as the direct sum needs them, summed over the node list) over the device time of
the timed steps, measured with one HIP event pair on the library's stream around each graph replay
(the step's other kernels are inside that bracket, which makes the figure a lower bound).  Minimal
filtering issues fewer multiplications than that numerator counts: `mfma_flops_issued_per_step` and
`frac_issued` give what the matrix cores really execute per step and its share of the peak.
Inside `roofline`, so that one record holds everything the metric names:
  kernels        Gemm 4096^3 and the config-3 Conv as single-kernel figures (ms, GFLOP/s, fraction of the
                 fp32 MFMA peak), each timed as replays of a HIP graph that holds the launches back to back,
                 with the one-by-one launch time beside it;
  end_to_end     the same ResNet-50 step with the batch handed over as a host tensor on every run
                 (runner.run([CPUTensor]) with no option: H2D inside the timed region; the runner's
                 default records the third run and replays it), the same through the node loop only
                 ({graph: false}), the throughput with two runs in flight (runner.submit / collect: batch
                 i+1 enqueued on a second stream before batch i's logits are fetched), and the network
                 at batch 128;
  other_configs  configs 2 and 5 with their device time;
  bandwidth_kernels_frac_of_8TBps  the HBM-bound kernels at the configs' shapes.
`python bench.py --only layers` prints the per-layer table of the step's 54 Conv / Gemm nodes,
`--only bandwidth` the bandwidth kernels in full, `--only kernels` the two single kernels (for profiler runs).
`cpu_baseline` times the JavaScript restatement of the reference's CPU operators (oracle/js) through
the same runner with backendOrder ["cpu"] in Node.js on one host core, on three images of the batch (one per run, about 20 s).
"""
import argparse
import json
import os
import subprocess
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402

METRIC = "fp32 Gemm/Conv GFLOP/s (% MFMA peak) + ResNet-50 b32 images/sec, 1 MI355X"
PEAK_FP32_MFMA_TFLOPS = 157.3
# HBM-side bytes of the ResNet-50 step per Conv / Gemm node (54 nodes; contraction kernels, reduce passes
# and the transforms of the minimal-filtering convs): rocprofv3 --pmc FETCH_SIZE (x2.000) + WRITE_SIZE
# (x1.000), factors from a 256 MiB device copy; recorded in profiles/contraction_kernel_resnet50_b32.txt
# (bench.py cannot read counters itself).  The transform-domain tensors of the 13 minimal-filtering convs
# (four times the conv's input and output, written once, read once or twice) and the partial sums of
# tiles cut along K are in it; both live between consecutive launches and are counted in front of the
# Infinity Cache.
TRAFFIC_BYTES_PER_LAUNCH = 110.6e6  # (110.56 in the latest profile)
CLI = os.path.join(ROOT, "webdnn_amd", "js", "cli", "run_model.js")
ORACLE_JS = os.path.join(ROOT, "oracle", "js", "cpuOperators.js")


def node_run(model_dir, input_path, backend, runs, warmup, extra, options=None):
    cmd = ["node", CLI, "--model", model_dir, "--backend", backend, "--inputs", input_path,
           "--runs", str(runs), "--warmup", str(warmup)] + extra
    env = dict(os.environ)
    if options:
        env["WDH_OPTIONS"] = options     # library options of the child process (wdh_set_option names)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, env=env)
    if proc.returncode != 0:
        raise RuntimeError("node runner failed: %s" % proc.stderr[-2000:])
    return json.loads(proc.stdout.strip().splitlines()[-1])


def bench_resnet(steps, warmup, workdir):
    from webdnn_amd import modelgen

    batch = 32
    data, g = modelgen.resnet50_model(batch=batch)
    with open(os.path.join(workdir, "model.onnx"), "wb") as f:
        f.write(data)
    x = np.random.default_rng(6).standard_normal((batch, 3, 224, 224)).astype(np.float32)
    inp = os.path.join(workdir, "input.bin")
    x.tofile(inp)
    # graph mode: warm-up run 1 is eager, run 2 records the HIP graph, every timed step replays it
    timed = node_run(workdir, inp, "hip", steps, max(warmup, 2),
                     ["--strict", "--resident-inputs", "--graph", "--measure-all"])
    assert timed["backend"] == "hip" and list(timed["stats"]["nodesByBackend"]) == ["hip"], timed["stats"]
    assert timed["graph"]["captured"], timed["graph"]
    total_ms = sum(timed["msPerRun"])
    eager = node_run(workdir, inp, "hip", max(3, steps // 2), max(warmup, 2), ["--strict", "--resident-inputs", "--no-graph"])
    # one more run with per-node HIP events for the kernel-level figure.  The run is enqueued behind
    # a few milliseconds of queued streaming kernels, so that all of its launches are in the queue
    # before the device reaches them: the events then time the device, not the host's enqueue rate.
    eager_ms = sum(eager["msPerRun"]) / len(eager["msPerRun"])
    prof = node_run(workdir, inp, "hip", 1, 2, ["--strict", "--resident-inputs", "--no-graph", "--measure",
                                                "--queue-ahead", "%.1f" % (2 * eager_ms + 2)])
    assert prof["queueAhead"]["deviceMs"] > prof["stats"]["enqueueMs"], (prof["queueAhead"], prof["stats"])
    contraction_ms = sum(p["deviceElapsed"] for p in prof["performance"]
                         if p["opType"] in ("Conv", "WebDNNHipFusedConv", "Gemm"))
    launches = sum(1 for p in prof["performance"] if p["opType"] in ("Conv", "WebDNNHipFusedConv", "Gemm"))
    all_ms = sum(p["deviceElapsed"] or 0.0 for p in prof["performance"])
    # PCIe-inclusive: the input is a host tensor (runner.run([CPUTensor]), as in the reference), uploaded
    # by every run: 19.3 MB through the pinned staging buffers, then the same graph replay / node loop
    host_in = node_run(workdir, inp, "hip", max(3, steps // 4), 2, ["--strict", "--no-graph"])
    # no option at all: what a caller written for the reference does (the runner records the third run)
    host_in_graph = node_run(workdir, inp, "hip", steps, max(warmup, 3), ["--strict"])
    assert host_in_graph["graph"]["captured"], host_in_graph["graph"]
    # two runs in flight (runner.submit / runner.collect: run i+1 is enqueued on the library's second lane
    # before the outputs of run i are fetched), input resident and input from the host; the first timed
    # runs record the second lane and are left out of the mean
    def in_flight(extra, lanes=2):
        rep = node_run(workdir, inp, "hip", 2 * steps + 8, max(warmup, 3), ["--strict", "--in-flight", str(lanes)] + extra)
        assert rep["graph"]["lanes"] == lanes, rep["graph"]
        tail = rep["msPerRun"][8:]
        return sum(tail) / len(tail)
    pipe_resident_ms = in_flight(["--resident-inputs"])
    pipe_host_ms = in_flight([])
    pipe3_resident_ms = in_flight(["--resident-inputs"], 3)
    # the opt-in F(4x4, 3x3) form of the 3x3 convs: faster, but its logits miss the 1e-3 bar (1.7e-3)
    f4 = node_run(workdir, inp, "hip", max(3, steps // 2), max(warmup, 2),
                  ["--strict", "--resident-inputs", "--graph", "--measure-all"], options="conv3x3_f4x4_channels=64")
    return {
        "f4x4_ms_per_step": sum(f4["msPerRun"]) / len(f4["msPerRun"]),
        "two_in_flight_ms_per_step": pipe_resident_ms, "two_in_flight_host_input_ms_per_step": pipe_host_ms,
        "three_in_flight_ms_per_step": pipe3_resident_ms,
        "f4x4_device_ms": sum(f4["deviceMsPerRun"]) / len(f4["deviceMsPerRun"]),
        "flops_saved": g.flops_saved,
        "batch": batch, "flops": g.flops, "nodes": timed["nodes"], "ms_per_step": total_ms / steps,
        "images_per_s": batch * steps / total_ms * 1e3, "contraction_ms": contraction_ms,
        "contraction_launches": launches, "device_ms": all_ms,
        "graph_device_ms": sum(timed["deviceMsPerRun"]) / len(timed["deviceMsPerRun"]),
        "ms_per_step_host_input_eager": sum(host_in["msPerRun"]) / len(host_in["msPerRun"]),
        "ms_per_step_host_input": sum(host_in_graph["msPerRun"]) / len(host_in_graph["msPerRun"]),
        "ms_per_step_eager": sum(eager["msPerRun"]) / len(eager["msPerRun"]),
        "device": timed.get("device"), "node_version": timed["node"],
    }


def bench_resnet_large_batch(steps, warmup, workdir, batch=128):
    """The same network at four times the batch (not the configured workload, reported in `extra` only):
    per-launch start-up and drain weigh a quarter as much, which separates what the kernels reach in steady
    state from what a batch of 32 lets them show."""
    from webdnn_amd import modelgen

    d = os.path.join(workdir, "resnet50_b%d" % batch)
    os.makedirs(d, exist_ok=True)
    data, g = modelgen.resnet50_model(batch=batch)
    with open(os.path.join(d, "model.onnx"), "wb") as f:
        f.write(data)
    inp = os.path.join(d, "input.bin")
    np.random.default_rng(6).standard_normal((batch, 3, 224, 224)).astype(np.float32).tofile(inp)
    rep = node_run(d, inp, "hip", steps, max(warmup, 2), ["--strict", "--resident-inputs", "--graph", "--measure-all"])
    assert list(rep["stats"]["nodesByBackend"]) == ["hip"] and rep["graph"]["captured"], rep["stats"]
    ms = sum(rep["msPerRun"]) / len(rep["msPerRun"])
    dev_ms = sum(rep["deviceMsPerRun"]) / len(rep["deviceMsPerRun"])
    return {"workload": "ResNet-50 v1 batch %d, same runner, graph replay, input resident" % batch,
            "ms_per_step": round(ms, 4), "images_per_s": round(batch / ms * 1e3, 1),
            "device_ms": round(dev_ms, 4), "device_tflops": round(g.flops / dev_ms / 1e9, 2),
            "device_frac_mfma_peak": round(g.flops / dev_ms / 1e9 / PEAK_FP32_MFMA_TFLOPS, 4)}


def bench_report_only(workdir, steps, warmup):
    """Configs 2 and 5, reported but not part of `value`: the FFN MatMul chain and the DETR-R50-style graph."""
    from webdnn_amd import modelgen

    out = {}
    for key, (data, g), shape, label in (
        ("ffn_c2", modelgen.ffn_model(), (8, 512, 768),
         "MatMul chain X[8,512,768] -> 3072 -> 768 + residual, fused to 2 nodes (config 2)"),
        ("detr_r50_b1", modelgen.detr_model(), (1, 3, 800, 1088),
         "DETR-R50-style graph, input [1,3,800,1088], 850 tokens, 6+6 layers (config 5)"),
    ):
        d = os.path.join(workdir, key)
        os.makedirs(d, exist_ok=True)
        with open(os.path.join(d, "model.onnx"), "wb") as f:
            f.write(data)
        inp = os.path.join(d, "input.bin")
        np.random.default_rng(11).standard_normal(shape).astype(np.float32).tofile(inp)
        rep = node_run(d, inp, "hip", steps, max(warmup, 2), ["--strict", "--resident-inputs", "--graph", "--measure-all"])
        assert list(rep["stats"]["nodesByBackend"]) == ["hip"], rep["stats"]
        ms = sum(rep["msPerRun"]) / len(rep["msPerRun"])
        dev_ms = sum(rep["deviceMsPerRun"]) / len(rep["deviceMsPerRun"])
        eager = node_run(d, inp, "hip", steps, max(warmup, 2), ["--strict", "--resident-inputs", "--no-graph"])
        # two runs in flight (runner.submit / runner.collect); the first timed runs record the second lane
        pipe = node_run(d, inp, "hip", 2 * steps + 8, 3, ["--strict", "--resident-inputs", "--in-flight", "2"])
        pipe_ms = sum(pipe["msPerRun"][8:]) / len(pipe["msPerRun"][8:])
        out[key] = {"workload": label, "nodes": rep["nodes"], "ms_per_run": round(ms, 4),
                    "two_in_flight_ms_per_run": round(pipe_ms, 4),
                    "graph_replay": bool(rep["graph"]["captured"]),
                    "ms_per_run_eager": round(sum(eager["msPerRun"]) / len(eager["msPerRun"]), 4),
                    "gflops": round(g.flops / ms / 1e6, 1),
                    "frac_mfma_peak": round(g.flops / ms / 1e9 / PEAK_FP32_MFMA_TFLOPS, 4),
                    # device time of a replay (HIP events around the graph launch): the kernels alone,
                    # without the input upload, the output download and the host's share of runner.run
                    "device_ms": round(dev_ms, 4),
                    "device_gflops": round(g.flops / dev_ms / 1e6, 1),
                    "device_frac_mfma_peak": round(g.flops / dev_ms / 1e9 / PEAK_FP32_MFMA_TFLOPS, 4)}
    return out


def cpu_baseline_resnet(workdir, images=3):
    """ResNet-50 on `images` images of the batch, one per run (one JIT warm-up run first), through the
    runner's cpu path with the JS oracle operators: about 20 s of work on one host core."""
    from webdnn_amd import modelgen

    d = os.path.join(workdir, "cpu1")
    os.makedirs(d, exist_ok=True)
    data, g = modelgen.resnet50_model(batch=1)
    with open(os.path.join(d, "model.onnx"), "wb") as f:
        f.write(data)
    x = np.random.default_rng(6).standard_normal((1, 3, 224, 224)).astype(np.float32)
    inp = os.path.join(d, "input.bin")
    x.tofile(inp)
    rep = node_run(d, inp, "cpu", images, 0, ["--cpu-entries", ORACLE_JS])
    sec = sum(rep["msPerRun"]) / 1e3
    return {"value": round(images / sec, 4), "unit": "images/s", "cores": 1, "kind": "port",
            "sample": "%d images of the 32, one per run (ResNet-50, %.1f GFLOP each) through runner.run with "
                      "backendOrder [\"cpu\"] and the JavaScript restatement of the reference CPU operators, "
                      "Node %s, %.1f s" % (images, g.flops / 1e9, rep["node"], sec),
            "gflops": round(images * g.flops / sec / 1e9, 3)}


def timed_steps(ctx, step, steps, warmup, replays=3):
    """Device time of one `step` in milliseconds.  The steps are recorded once into a HIP graph and
    the graph is replayed: back-to-back launches without the host's enqueue time between them, which
    is how the runner executes a model (runner.run(x, {graph: true})).  HIP events on the library's
    stream bracket the timed replays.  `eager_ms` of the result is the same loop launched call by
    call."""
    for _ in range(max(warmup, 1)):
        step()                      # also builds conv tap tables, which a capture cannot
    ctx.sync()
    ctx.event_record(2)
    for _ in range(steps):
        step()
    ctx.event_record(3)
    ctx.sync()
    eager = ctx.event_elapsed_ms(2, 3) / steps
    ctx.graph_begin()
    try:
        for _ in range(steps):
            step()
    finally:
        gid = ctx.graph_end()
    ctx.graph_launch(gid)           # first replay: untimed
    ctx.sync()
    ctx.event_record(0)
    for _ in range(replays):
        ctx.graph_launch(gid)
    ctx.event_record(1)
    ctx.sync()
    ms = ctx.event_elapsed_ms(0, 1) / (steps * replays)
    ctx.graph_destroy(gid)
    timed_steps.last_eager_ms = eager
    return ms


def bench_kernels(steps, warmup, calibrate_copy=False):
    """The two single-kernel figures the metric names, through the C ABI (ctypes)."""
    from webdnn_amd import capi
    from webdnn_amd import hostops as H

    ctx = H.HipContext(0).initialize()
    rng = np.random.default_rng(0)
    if calibrate_copy:
        # a plain copy of known size: reads 256 MiB, writes 256 MiB
        nbytes = 256 << 20
        src, dst = ctx.empty_tensor([nbytes // 4]), ctx.empty_tensor([nbytes // 4])
        for _ in range(3):
            capi.call("wdh_copy", dst.handle, 0, src.handle, 0, nbytes)
        ctx.sync()
    n = 4096
    A = ctx.move_tensor(rng.uniform(-1, 1, (n, n)).astype(np.float32))
    B = ctx.move_tensor(rng.uniform(-1, 1, (n, n)).astype(np.float32))
    C = ctx.move_tensor(rng.uniform(-1, 1, (n,)).astype(np.float32))
    gemm_ms = timed_steps(ctx, lambda: H.gemm(ctx, A, B, C).dispose(), steps, warmup)
    gemm_eager = timed_steps.last_eager_ms
    X = ctx.move_tensor(rng.uniform(0, 1, (32, 64, 56, 56)).astype(np.float32))
    W = ctx.move_tensor((rng.standard_normal((64, 64, 3, 3)) * np.sqrt(2 / 576)).astype(np.float32))
    Bv = ctx.move_tensor(np.zeros(64, np.float32))
    conv_ms = timed_steps(ctx, lambda: H.conv(ctx, X, W, Bv, pads=[1, 1, 1, 1], epilogue="relu").dispose(),
                          steps, warmup)
    conv_eager = timed_steps.last_eager_ms
    gemm_flops, conv_flops = 2.0 * n ** 3, 2.0 * 100352 * 64 * 576

    def entry(workload, flops, ms, eager):
        tf = flops / ms / 1e9
        return {"workload": workload, "ms": round(ms, 4), "gflops": round(tf * 1e3, 1),
                "frac_mfma_peak": round(tf / PEAK_FP32_MFMA_TFLOPS, 4),
                "timing": "HIP events around replays of a HIP graph holding the launches back to back",
                "ms_launched_one_by_one": round(eager, 4)}

    return {
        "gemm_4096": entry("Gemm M=N=K=4096 + bias[4096], alpha=beta=1, U[-1,1] (north_star NS-4096)", gemm_flops, gemm_ms,
                           gemm_eager),
        "conv_c3": entry("Conv 3x3 X[32,64,56,56] W[64,64,3,3] pad 1 + bias + Relu fused (config 3)", conv_flops, conv_ms,
                         conv_eager),
    }


def bench_resnet_layers(steps, warmup, batch=32, only=None):
    """Every distinct Conv / Gemm launch of the ResNet-50 step, through the C ABI with back-to-back
    launches (operands hot in the caches, unlike inside the graph): shape, how often the step runs
    it, microseconds, TFLOP/s, and how the launch was laid out (tile, whole / K-split tiles, form).
    `only`: run just the layers whose label contains this text (one layer under a profiler)."""
    from webdnn_amd import hostops as H
    from webdnn_amd import modelgen

    ctx = H.HipContext(0).initialize()
    rng = np.random.default_rng(0)
    data, _ = modelgen.resnet50_model(batch=batch)
    model = modelgen.parse_model(data)
    shapes = {name: list(dims) for name, dims in model["inputs"]}
    shapes.update({name: list(a.shape) for name, a in model["initializers"].items()})
    consumers = {}
    for nd in model["nodes"]:
        for i in nd["inputs"]:
            consumers.setdefault(i, []).append(nd)
    layers = {}
    for nd in model["nodes"]:
        ins, out = nd["inputs"], nd["outputs"][0]
        if nd["op_type"] == "Conv":
            x, w = shapes[ins[0]], shapes[ins[1]]
            a = nd["attrs"]
            s = H.conv_shape(x, w, a.get("dilations"), a.get("group", 1), a.get("kernel_shape"), a.get("pads"),
                             a.get("strides"))
            shapes[out] = [x[0], w[0], s["out_shape"][0], s["out_shape"][1]]
            nxt = consumers.get(out, [])
            residual = len(nxt) == 1 and nxt[0]["op_type"] == "Add"      # what the fusion pass absorbs
            key = (tuple(x), tuple(w), tuple(s["pads"]), tuple(s["strides"]), residual)
            layers.setdefault(key, {"count": 0, "kind": "Conv"})["count"] += 1
        elif nd["op_type"] == "Gemm":
            key = (tuple(shapes[ins[0]]), tuple(shapes[ins[1]]), (), (), False)
            layers.setdefault(key, {"count": 0, "kind": "Gemm"})["count"] += 1
            shapes[out] = [shapes[ins[0]][0], shapes[ins[1]][0]]
        elif nd["op_type"] in ("Relu", "Add"):
            shapes[out] = shapes[ins[0]]
        elif nd["op_type"] == "MaxPool":
            a = nd["attrs"]
            x = shapes[ins[0]]
            s = H.maxpool_shape(x, a["kernel_shape"], pads=a.get("pads"), strides=a.get("strides"))
            shapes[out] = [x[0], x[1], s["out_shape"][0], s["out_shape"][1]]
        elif nd["op_type"] == "GlobalAveragePool":
            shapes[out] = shapes[ins[0]][:2] + [1, 1]
        elif nd["op_type"] == "Flatten":
            shapes[out] = [shapes[ins[0]][0], int(np.prod(shapes[ins[0]][1:]))]
    rows = []
    for (x, w, pads, strides, residual), info in layers.items():
        if info["kind"] == "Conv":
            label = "Conv %dx%d s%d %d->%d @%dx%d%s" % (w[2], w[3], strides[0], x[1], w[0], x[2], x[3],
                                                         " +residual" if residual else "")
        else:
            label = "Gemm [%d,%d] x [%d,%d]^T" % (x[0], x[1], w[0], w[1])
        if only and only not in label:
            continue
        if info["kind"] == "Conv":
            X = ctx.move_tensor(rng.uniform(0, 1, x).astype(np.float32))
            W = ctx.move_tensor((rng.standard_normal(w) * np.sqrt(2.0 / (w[1] * w[2] * w[3]))).astype(np.float32))
            B = ctx.move_tensor(np.zeros(w[0], np.float32))
            # (constant_weights: what the runner passes for an initializer's device copy)
            probe = H.conv(ctx, X, W, B, pads=list(pads), strides=list(strides), epilogue="relu", constant_weights=True)
            plan, odims = ctx.last_plan(), probe.dims
            R = ctx.move_tensor(rng.uniform(0, 1, odims).astype(np.float32)) if residual else None
            probe.dispose()
            ms = timed_steps(ctx, lambda: H.conv(ctx, X, W, B, pads=list(pads), strides=list(strides), epilogue="relu",
                                                 residual=R, constant_weights=True).dispose(), steps, warmup)
            m, n, k = w[0], odims[0] * odims[2] * odims[3], w[1] * w[2] * w[3]
            out_elems = int(np.prod(odims))
            nbytes = 4 * (int(np.prod(x)) + int(np.prod(w)) + w[0] + out_elems * (2 if residual else 1))
            for t in (X, W, B) + ((R,) if R is not None else ()):
                t.dispose()
        else:
            A = ctx.move_tensor(rng.standard_normal(x).astype(np.float32))
            Wt = ctx.move_tensor((rng.standard_normal(w) * 0.01).astype(np.float32))
            Bv = ctx.move_tensor(np.zeros(w[0], np.float32))
            H.gemm(ctx, A, Wt, Bv, trans_b=1).dispose()
            plan = ctx.last_plan()
            ms = timed_steps(ctx, lambda: H.gemm(ctx, A, Wt, Bv, trans_b=1).dispose(), steps, warmup)
            m, n, k = x[0], w[0], x[1]
            nbytes = 4 * (x[0] * x[1] + w[0] * w[1] + w[0] + x[0] * w[0])
            for t in (A, Wt, Bv):
                t.dispose()
        flops = 2.0 * m * n * k
        # the layer's own roofline: the larger of its matrix-core time and its HBM time at the two peaks
        mfma_us = flops / PEAK_FP32_MFMA_TFLOPS / 1e6
        hbm_us = nbytes / 8000.0 / 1e3
        rows.append({"layer": label, "count": info["count"], "m": m, "n": n, "k": k, "us": round(ms * 1e3, 1),
                     "tflops": round(flops / ms / 1e9, 1),
                     "frac_mfma_peak": round(flops / ms / 1e9 / PEAK_FP32_MFMA_TFLOPS, 3),
                     "algorithmic_MB": round(nbytes / 1e6, 1),
                     "bound": "mfma" if mfma_us >= hbm_us else "hbm",
                     "frac_of_bound": round(max(mfma_us, hbm_us) / (ms * 1e3), 3), **plan})
    total_us = sum(r["us"] * r["count"] for r in rows)
    total_flops = sum(2.0 * r["m"] * r["n"] * r["k"] * r["count"] for r in rows)
    return {"note": "each distinct layer with its fused bias/residual/Relu epilogue and its K-split reduce pass, "
                    "launches recorded into a HIP graph and replayed back to back; us = HIP events / launches; "
                    "bound / frac_of_bound: max(FLOP / 157.3 TFLOP/s, algorithmic bytes / 8 TB/s) over the time",
            "launches": sum(r["count"] for r in rows), "sum_us": round(total_us, 1),
            "tflops": round(total_flops / total_us / 1e6, 1), "layers": rows}


def bench_bandwidth(steps, warmup):
    """GB/s of the HBM-bound kernels at the shapes the configs use: algorithmic bytes (every input and
    output element once) over the average launch time, against the 8 TB/s peak."""
    from webdnn_amd import hostops as H

    ctx = H.HipContext(0).initialize()
    rng = np.random.default_rng(0)
    f = lambda *shape: ctx.move_tensor(rng.standard_normal(shape).astype(np.float32))
    out = {}

    def run(name, workload, nbytes, fn):
        ms = timed_steps(ctx, fn, steps, warmup)
        gbs = nbytes / ms / 1e6
        out[name] = {"workload": workload, "ms": round(ms, 4), "GB/s": round(gbs, 1),
                     "frac_hbm_peak": round(gbs / 8000.0, 4)}

    x = f(32, 256, 56, 56)
    y = f(32, 256, 56, 56)
    n = x.length * 4
    run("add", "Add [32,256,56,56] + same shape (ResNet residual)", 3 * n, lambda: H.binary(ctx, "Add", x, y).dispose())
    b = f(256, 1, 1)
    run("add_bcast", "Add [32,256,56,56] + [256,1,1]", 2 * n, lambda: H.binary(ctx, "Add", x, b).dispose())
    run("relu", "Relu [32,256,56,56]", 2 * n, lambda: H.unary(ctx, "Relu", x).dispose())
    x.dispose(); y.dispose()
    s = f(8, 850, 850)
    run("softmax", "Softmax [8,850,850] (DETR encoder attention)", 2 * s.length * 4, lambda: H.softmax(ctx, s).dispose())
    s.dispose()
    ln, g, be = f(32 * 850, 256), f(256), f(256)
    run("layernorm", "LayerNormalization [27200,256]", 2 * ln.length * 4,
        lambda: H.layer_normalization(ctx, ln, g, be).dispose())
    ln.dispose()
    st = f(32, 64, 112, 112)
    run("maxpool", "MaxPool 3x3 s2 p1 [32,64,112,112] (ResNet stem)", st.length * 4 + 32 * 64 * 56 * 56 * 4,
        lambda: H.maxpool(ctx, st, kernel_shape=[3, 3], pads=[1, 1, 1, 1], strides=[2, 2]).dispose())
    st.dispose()
    gp = f(32, 2048, 7, 7)
    run("global_avgpool", "GlobalAveragePool [32,2048,7,7]", gp.length * 4 + 32 * 2048 * 4,
        lambda: H.global_average_pool(ctx, gp).dispose())
    gp.dispose()
    t = f(32, 850, 8, 32)
    run("transpose", "Transpose [32,850,8,32] perm (0,2,1,3) (attention heads)", 2 * t.length * 4,
        lambda: H.transpose(ctx, t, [0, 2, 1, 3]).dispose())
    run("transpose_last", "Transpose [32,850,8,32] perm (0,2,3,1) (K^T, through LDS tiles)", 2 * t.length * 4,
        lambda: H.transpose(ctx, t, [0, 2, 3, 1]).dispose())
    t.dispose()
    c1, c2 = f(32, 128, 56, 56), f(32, 128, 56, 56)
    run("concat", "Concat 2 x [32,128,56,56] on axis 1", 4 * c1.length * 4, lambda: H.concat(ctx, [c1, c2], 1).dispose())
    run("slice", "Slice [32,128,56,56] -> [32,128,48,50]", 2 * 32 * 128 * 48 * 50 * 4,
        lambda: H.slice_(ctx, c1, [4, 3], [52, 53], [2, 3]).dispose())
    c1.dispose(); c2.dispose()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--layer", default=None,
                    help="with --only layers: run just the layers whose label contains this text, e.g. "
                         "'1x1 s1 256->1024' (for per-layer profiler runs)")
    ap.add_argument("--only", choices=["all", "kernels", "bandwidth", "layers"], default="all",
                    help="kernels: only the in-process Gemm 4096 / Conv C3 launches plus one device-to-device "
                         "copy of known size (the unit for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (the path shards by batch with no "
                 "exchange; multi-GPU runs are not part of it). Use --gpus 1.")

    if args.only == "bandwidth":
        print(json.dumps({"bandwidth_kernels": bench_bandwidth(args.steps, args.warmup),
                          "unit": "GB/s of algorithmic bytes", "peak": 8000.0}))
        return
    if args.only == "layers":
        print(json.dumps({"resnet50_layers": bench_resnet_layers(args.steps, args.warmup, only=args.layer)}))
        return
    if args.only == "kernels":
        print(json.dumps({"kernels": bench_kernels(args.steps, args.warmup, calibrate_copy=True)}))
        return

    with tempfile.TemporaryDirectory(prefix="webdnn_bench_") as workdir:
        resnet = bench_resnet(args.steps, args.warmup, workdir)
        report_only = bench_report_only(workdir, max(3, args.steps // 2), min(args.warmup, 3))
        large_batch = bench_resnet_large_batch(max(3, args.steps // 3), 2, workdir)
        baseline = None if args.no_cpu_baseline else cpu_baseline_resnet(workdir)
    kernels = bench_kernels(args.steps, args.warmup)
    bandwidth = bench_bandwidth(args.steps, args.warmup)

    # The timed steps are graph replays: one HIP event pair brackets each replay on the library's
    # stream.  That device time covers the 54 Conv / Gemm nodes (contraction launches, reduce passes,
    # transforms) plus the step's three other kernels (MaxPool, GlobalAveragePool, one copy: about 1.5 %
    # of it), so FLOPs over it is a lower bound for the contraction kernels alone.
    achieved = resnet["flops"] / resnet["graph_device_ms"] / 1e9
    batch = resnet["batch"]
    pick = lambda d, *keys: {k: d[k] for k in keys}
    line = {
        "metric": METRIC,
        "value": round(resnet["images_per_s"], 1),
        "unit": "images/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(resnet["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "ResNet-50 v1 batch 32 [32,3,224,224] fp32, random init (seeded), BN folded, "
                               "%d nodes after Conv+Add+Relu fusion, Node.js runner on the hip backend, strict; "
                               "a step = runner.run(x) with x resident in HBM, ending with the logits on the host "
                               "(benchmark config 4); the same step fed a host tensor is in roofline.end_to_end"
                               % resnet["nodes"]},
        "roofline": {
            "bound": "mfma",
            "kernel": "contraction kernels (implicit-GEMM Conv: in-place 1x1, LDS-tile 3x3, F(2x2,3x3) minimal filtering "
                      "for 3x3 from 128 channels on, gathered forms, stem; Gemm head), %d Conv/Gemm nodes per step; device "
                      "time = HIP events around each timed graph replay (whole step: transforms, MaxPool and "
                      "GlobalAveragePool included); achieved = direct-sum FLOPs (2MNK per node) / that time"
                      % resnet["contraction_launches"],
            "achieved": round(achieved, 2),
            "peak": PEAK_FP32_MFMA_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4),
            "traffic": TRAFFIC_BYTES_PER_LAUNCH,
            "traffic_note": "bytes per Conv/Gemm node from rocprofv3 FETCH_SIZE+WRITE_SIZE, see profiles/; algorithmic "
                            "64.1e6; the excess is the transform-domain tensors of the 13 F(2x2,3x3) convs (36.6e6 per "
                            "node), which pass between consecutive launches through the Infinity Cache",
            "flops_per_step": resnet["flops"],
            # what the matrix cores execute: minimal filtering replaces 36 multiplications per 2x2 block by 16
            "mfma_flops_issued_per_step": resnet["flops"] - resnet["flops_saved"],
            "frac_issued": round((resnet["flops"] - resnet["flops_saved"]) / resnet["graph_device_ms"] / 1e9
                                 / PEAK_FP32_MFMA_TFLOPS, 4),
            "avg_launch_ms": round(resnet["graph_device_ms"] / resnet["contraction_launches"], 5),
            "step_device_ms": round(resnet["graph_device_ms"], 4),
            # the two single-kernel figures the metric names (graph replays of back-to-back launches)
            "kernels": {
                "gemm_4096": pick(kernels["gemm_4096"], "ms", "gflops", "frac_mfma_peak", "ms_launched_one_by_one"),
                "conv_c3": pick(kernels["conv_c3"], "ms", "gflops", "frac_mfma_peak", "ms_launched_one_by_one"),
            },
            # ResNet-50 b32 images/s by how the batch reaches the device and how runner.run is called
            "end_to_end": {
                "resident_input_images_per_s": round(resnet["images_per_s"], 1),
                "host_input_images_per_s": round(batch / resnet["ms_per_step_host_input"] * 1e3, 1),
                "host_input_ms_per_step": round(resnet["ms_per_step_host_input"], 4),
                "host_input_note": "runner.run([CPUTensor]) with no option, as the reference's callers write it: "
                                   "19.3 MB over PCIe inside every timed step; the runner records the third run "
                                   "and replays it (graph \"auto\")",
                "host_input_node_loop_images_per_s": round(batch / resnet["ms_per_step_host_input_eager"] * 1e3, 1),
                "resident_input_node_loop_ms_per_step": round(resnet["ms_per_step_eager"], 4),
                "two_in_flight_images_per_s": round(batch / resnet["two_in_flight_ms_per_step"] * 1e3, 1),
                "two_in_flight_host_input_images_per_s": round(batch / resnet["two_in_flight_host_input_ms_per_step"] * 1e3, 1),
                "two_in_flight_frac_mfma_peak": round(resnet["flops"] / resnet["two_in_flight_ms_per_step"] / 1e9
                                                      / PEAK_FP32_MFMA_TFLOPS, 4),
                "three_in_flight_images_per_s": round(batch / resnet["three_in_flight_ms_per_step"] * 1e3, 1),
                "two_in_flight_note": "runner.submit / runner.collect (an addition to the reference's API): batch i+1 is "
                                      "enqueued on a second HIP stream before the logits of batch i are fetched; wall "
                                      "clock per step in steady state, the fraction from that wall clock",
                "f4x4_option_images_per_s": round(batch / resnet["f4x4_ms_per_step"] * 1e3, 1),
                "f4x4_option_device_ms": round(resnet["f4x4_device_ms"], 4),
                "f4x4_option_note": "WDH_OPTIONS=conv3x3_f4x4_channels=64: 3x3 convs as F(4x4,3x3); not the default "
                                    "because its logits differ from the CPU path's by 1.7e-3 (bar 1e-3)",
                "batch128_device_frac_mfma_peak": large_batch["device_frac_mfma_peak"],
                "batch128_images_per_s": large_batch["images_per_s"],
            },
            "other_configs": {
                "ffn_c2_device_ms": report_only["ffn_c2"]["device_ms"],
                "ffn_c2_device_frac_mfma_peak": report_only["ffn_c2"]["device_frac_mfma_peak"],
                "detr_r50_b1_ms_per_run": report_only["detr_r50_b1"]["ms_per_run"],
                "detr_r50_b1_device_ms": report_only["detr_r50_b1"]["device_ms"],
                "detr_r50_b1_device_frac_mfma_peak": report_only["detr_r50_b1"]["device_frac_mfma_peak"],
                "detr_r50_b1_two_in_flight_ms_per_run": report_only["detr_r50_b1"]["two_in_flight_ms_per_run"],
            },
            "bandwidth_kernels_frac_of_8TBps": {k: v["frac_hbm_peak"] for k, v in bandwidth.items()},
        },
        # the same figures once more as plain scalars
        "gemm_4096_frac_mfma_peak": kernels["gemm_4096"]["frac_mfma_peak"],
        "conv_c3_frac_mfma_peak": kernels["conv_c3"]["frac_mfma_peak"],
        "host_input_images_per_s": round(batch / resnet["ms_per_step_host_input"] * 1e3, 1),
        "host_input_node_loop_images_per_s": round(batch / resnet["ms_per_step_host_input_eager"] * 1e3, 1),
        "two_in_flight_images_per_s": round(batch / resnet["two_in_flight_ms_per_step"] * 1e3, 1),
        "two_in_flight_host_input_images_per_s": round(batch / resnet["two_in_flight_host_input_ms_per_step"] * 1e3, 1),
        "device": resnet["device"],
    }
    if baseline is not None:
        line["cpu_baseline"] = baseline
    text = json.dumps(line)
    assert len(text) < 8000, "the bench line must stay under 8 KB (%d)" % len(text)
    print(text)


if __name__ == "__main__":
    main()
