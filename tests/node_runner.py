"""Drives webdnn_amd/js/cli/run_model.js from the tests."""
import json
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLI = os.path.join(ROOT, "webdnn_amd", "js", "cli", "run_model.js")
ORACLE_ENTRIES = os.path.join(ROOT, "oracle", "js", "cpuOperators.js")
FAKE_NATIVE = os.path.join(ROOT, "tests", "js", "fake_native.js")
RETRY_ENTRIES = os.path.join(ROOT, "tests", "js", "retry_entries.js")


def run_model(model_dir, inputs, backend, strict=True, fuse=True, oracle_cpu=False, runs=1, warmup=0,
              measure=False, extra=(), timeout=600, fake_native=False):
    """inputs: list of numpy arrays in graph-input order.  Returns (outputs, report)."""
    files = []
    for i, a in enumerate(inputs):
        p = os.path.join(model_dir, "input_%d.bin" % i)
        np.ascontiguousarray(a).tofile(p)
        files.append(p)
    out_path = os.path.join(model_dir, "output_%s.bin" % backend)
    if fake_native:
        extra = list(extra) + ["--native", FAKE_NATIVE]
    cmd = ["node", CLI, "--model", model_dir, "--backend", backend, "--inputs", ",".join(files),
           "--output", out_path, "--runs", str(runs), "--warmup", str(warmup)]
    if strict:
        cmd.append("--strict")
    if not fuse:
        cmd.append("--no-fuse")
    if measure:
        cmd.append("--measure")
    if oracle_cpu:
        cmd += ["--cpu-entries", ORACLE_ENTRIES]
    cmd += list(extra)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=timeout)
    if proc.returncode != 0:
        raise RuntimeError("run_model failed (%d): %s" % (proc.returncode, proc.stderr[-2000:]))
    report = json.loads(proc.stdout.strip().splitlines()[-1])
    flat = np.fromfile(out_path, dtype=np.float32)
    outputs, pos = [], 0
    for o in report["outputs"]:
        n = int(np.prod(o["dims"], dtype=np.int64)) if o["dims"] else 1
        part = flat[pos:pos + n]
        if o.get("dataType") == "int32":
            part = part.view(np.int32)
        outputs.append(part.reshape(o["dims"]))
        pos += n
    return outputs, report
