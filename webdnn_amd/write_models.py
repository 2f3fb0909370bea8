"""Writes the benchmark graphs (benchmark configs 1-5) as model directories for the Node.js runner.

    python -m webdnn_amd.write_models OUT_DIR [gemm ffn conv resnet50 detr]

Each model goes to OUT_DIR/<name>/model.onnx with a seeded input batch in OUT_DIR/<name>/input.bin, so that
`node webdnn_amd/js/cli/run_model.js --model OUT_DIR/<name> --inputs OUT_DIR/<name>/input.bin ...` can run it
(for instance under rocprofv3).  Shapes and initialisation follow example/benchmark/make_models.py:142-162 of
the reference and the configs' descriptions; weights are random (seeded), there is nothing to download.
"""
import os
import sys

import numpy as np

from . import modelgen

MODELS = {
    "gemm": (lambda: modelgen.gemm_model(), (256, 512), "uniform"),
    "ffn": (lambda: modelgen.ffn_model(), (8, 512, 768), "normal"),
    "conv": (lambda: modelgen.conv_model(), (32, 64, 56, 56), "uniform01"),
    "resnet50": (lambda: modelgen.resnet50_model(batch=32), (32, 3, 224, 224), "normal"),
    "detr": (lambda: modelgen.detr_model(), (1, 3, 800, 1088), "normal"),
}


def write(out_dir, names):
    for name in names:
        build, shape, dist = MODELS[name]
        data, _ = build()
        d = os.path.join(out_dir, name)
        os.makedirs(d, exist_ok=True)
        with open(os.path.join(d, "model.onnx"), "wb") as f:
            f.write(data)
        rng = np.random.default_rng(11)
        if dist == "normal":
            x = rng.standard_normal(shape)
        elif dist == "uniform":
            x = rng.uniform(-1, 1, shape)
        else:
            x = rng.uniform(0, 1, shape)
        x.astype(np.float32).tofile(os.path.join(d, "input.bin"))
        print("%s: %s, input %s" % (name, os.path.join(d, "model.onnx"), list(shape)))


if __name__ == "__main__":
    if len(sys.argv) < 2:
        sys.exit(__doc__)
    write(sys.argv[1], sys.argv[2:] or list(MODELS))
