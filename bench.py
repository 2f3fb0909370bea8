"""Benchmark of the hip backend hot path on ONE MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints one JSON line.  A step is one pass of the workload over synthetic, seeded inputs that are
already resident in HBM when the timed region starts.  `roofline` is measured live with HIP events
on the library's own stream around the same launches; `cpu_baseline` times the CPU oracle (a
restatement of the reference's CPU operators) on one host core over a bounded sample.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402

METRIC = "fp32 Gemm/Conv GFLOP/s (% MFMA peak) + ResNet-50 b32 images/sec, 1 MI355X"
PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0


def timed_steps(ctx, step, steps, warmup):
    """Wall clock over exactly `steps` calls bracketed by stream syncs, plus the HIP-event time of
    the same region on the library's stream."""
    for _ in range(warmup):
        step()
    ctx.sync()
    t0 = time.perf_counter()
    ctx.event_record(0)
    for _ in range(steps):
        step()
    ctx.event_record(1)
    ctx.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    dev_ms = ctx.event_elapsed_ms(0, 1) / steps
    return wall_ms, dev_ms


def bench_gemm(ctx, H, n, steps, warmup, rng):
    A = ctx.move_tensor(rng.uniform(-1, 1, (n, n)).astype(np.float32))
    B = ctx.move_tensor(rng.uniform(-1, 1, (n, n)).astype(np.float32))
    C = ctx.move_tensor(rng.uniform(-1, 1, (n,)).astype(np.float32))

    def step():
        H.gemm(ctx, A, B, C).dispose()

    wall_ms, dev_ms = timed_steps(ctx, step, steps, warmup)
    flops = 2.0 * n * n * n
    return {"wall_ms": wall_ms, "dev_ms": dev_ms, "flops": flops, "gflops": flops / dev_ms / 1e6}


def bench_conv3(ctx, H, steps, warmup, rng):
    X = ctx.move_tensor(rng.uniform(0, 1, (32, 64, 56, 56)).astype(np.float32))
    W = ctx.move_tensor((rng.standard_normal((64, 64, 3, 3)) * np.sqrt(2 / 576)).astype(np.float32))
    Bv = ctx.move_tensor(np.zeros(64, np.float32))

    def step():
        H.conv(ctx, X, W, Bv, pads=[1, 1, 1, 1], epilogue="relu").dispose()

    wall_ms, dev_ms = timed_steps(ctx, step, steps, warmup)
    flops = 2.0 * 100352 * 64 * 576
    return {"wall_ms": wall_ms, "dev_ms": dev_ms, "flops": flops, "gflops": flops / dev_ms / 1e6}


def cpu_baseline_gemm(n, rows, rng):
    """The oracle's Gemm (double accumulation, one thread) on `rows` rows of the n x n problem."""
    from oracle import ref

    ref.set_threads(1)
    A = rng.uniform(-1, 1, (rows, n)).astype(np.float32)
    B = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    C = rng.uniform(-1, 1, (n,)).astype(np.float32)
    t0 = time.perf_counter()
    ref.gemm(A, B, C)
    dt = time.perf_counter() - t0
    return 2.0 * rows * n * n / dt / 1e9, dt


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (the path shards by batch with no "
                 "exchange; multi-GPU runs are not part of it). Use --gpus 1.")

    from webdnn_amd import hostops as H

    ctx = H.HipContext(0).initialize()
    rng = np.random.default_rng(0)
    n = 4096
    gemm = bench_gemm(ctx, H, n, args.steps, args.warmup, rng)
    conv = bench_conv3(ctx, H, args.steps, args.warmup, rng)

    line = {
        "metric": METRIC,
        "value": round(gemm["flops"] / gemm["wall_ms"] / 1e6, 1),
        "unit": "GFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(gemm["wall_ms"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "Gemm M=N=K=4096, A,B U[-1,1] seed 0, C[4096] bias, alpha=beta=1 (north_star NS-4096)"},
        "roofline": {
            "bound": "mfma",
            "kernel": "contraction_kernel<A k-contiguous, B n-contiguous, 16-byte loads>",
            "achieved": round(gemm["gflops"] / 1e3, 2),
            "peak": PEAK_FP32_MFMA_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(gemm["gflops"] / 1e3 / PEAK_FP32_MFMA_TFLOPS, 4),
            "traffic": None,
        },
        "extra": {
            "conv_c3": {
                "workload": "Conv 3x3 X[32,64,56,56] W[64,64,3,3] pad 1 + bias + Relu fused (config 3)",
                "gflops": round(conv["gflops"], 1),
                "ms": round(conv["dev_ms"], 4),
                "frac_mfma_peak": round(conv["gflops"] / 1e3 / PEAK_FP32_MFMA_TFLOPS, 4),
            },
        },
    }
    if not args.no_cpu_baseline:
        rows = 128
        gf, dt = cpu_baseline_gemm(n, rows, rng)
        line["cpu_baseline"] = {
            "value": round(gf, 3),
            "unit": "GFLOP/s",
            "cores": 1,
            "kind": "port",
            "sample": "oracle Gemm on %d of the %d rows of A against the full B (%.1f s)" % (rows, n, dt),
        }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
