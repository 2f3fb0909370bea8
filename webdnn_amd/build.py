"""Builds the native pieces of the hip backend in-tree.

  libwebdnn_hip.so   HIP kernels + C ABI (include/webdnn_hip.h), gfx950 only
  webdnn_hip.node    N-API addon that exposes the C ABI to the Node.js host

Run as ``python -m webdnn_amd.build``.  hipcc cross-compiles for gfx950, so no
GPU is needed to build.
"""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "webdnn_amd", "csrc")
LIBDIR = os.path.join(ROOT, "webdnn_amd", "lib")
LIB = os.path.join(LIBDIR, "libwebdnn_hip.so")
ADDON_SRC = os.path.join(ROOT, "webdnn_amd", "napi", "addon.c")
ADDON = os.path.join(LIBDIR, "webdnn_hip.node")

HIP_SOURCES = ["runtime.hip", "gemm.hip", "contraction_gemm_akc.hip", "contraction_gemm_amc.hip", "contraction_conv_gather.hip",
               "contraction_conv_pixels.hip", "contraction_conv3x3.hip", "conv_patch.hip", "winograd.hip", "elementwise.hip", "reduce.hip", "attention.hip", "pool_layout.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # fp32 add/mul must not fuse: Add/Mul results are compared bit for bit
    "-ffp-contract=off",
    # packed fp32 instructions are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    if out.strip():
        print(out)


def build_library(verbose=True, only=None):
    """Compiles the HIP sources (side by side, one hipcc each) and links them.  `only`: recompile
    just these sources and reuse the other objects if they are still there (kernel work)."""
    from concurrent.futures import ThreadPoolExecutor

    os.makedirs(LIBDIR, exist_ok=True)
    objdir = os.path.join(LIBDIR, "obj")
    os.makedirs(objdir, exist_ok=True)

    def compile_one(src):
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        if only is not None and src not in only and os.path.exists(obj):
            return obj
        if verbose:
            print("[build] hipcc", src)
        _run(["hipcc", *HIPCC_FLAGS, "-I", os.path.join(ROOT, "include"), "-I", CSRC,
              "-c", os.path.join(CSRC, src), "-o", obj])
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(HIP_SOURCES))) as pool:
        objs = list(pool.map(compile_one, HIP_SOURCES))
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB])
    return LIB


def build_addon(verbose=True):
    if not os.path.exists(ADDON_SRC):
        return None
    if verbose:
        print("[build] gcc addon.c")
    # links against the library next to it ($ORIGIN), so the pair can be moved together
    _run(["gcc", "-O2", "-fPIC", "-shared", "-std=c11", "-Wall", "-DNODE_GYP_MODULE_NAME=webdnn_hip",
          "-I", "/usr/include/node", "-I", os.path.join(ROOT, "include"),
          ADDON_SRC, "-o", ADDON, "-L", LIBDIR, "-lwebdnn_hip", "-Wl,-rpath,$ORIGIN"])
    return ADDON


def build_all(verbose=True):
    lib = build_library(verbose)
    addon = build_addon(verbose)
    return lib, addon


if __name__ == "__main__":
    if len(sys.argv) > 1:      # python -m webdnn_amd.build gemm.hip ...: recompile these, relink
        build_library(only=sys.argv[1:])
        build_addon()
    else:
        build_all()
    print("built", LIB)
    sys.exit(0)
