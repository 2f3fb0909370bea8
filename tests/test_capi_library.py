"""The C-ABI shared library: it loads, and it exports exactly what include/webdnn_hip.h declares.
No compute call is made here (no GPU in this tier); calls that need the device must fail cleanly."""
import os
import re

import pytest

from webdnn_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "webdnn_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(wdh_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert declared_symbols() == sorted(capi.SIGNATURES)


def test_library_exports_every_declared_symbol():
    lib = capi.load()
    for name in declared_symbols():
        assert hasattr(lib, name), name


def test_argument_counts_match_header():
    text = open(os.path.join(ROOT, "include", "webdnn_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    for name, (_, argtypes) in capi.SIGNATURES.items():
        m = re.search(r"\b%s\s*\(([^;]*?)\)\s*;" % name, text, flags=re.S)
        assert m, name
        params = m.group(1).strip()
        n = 0 if params in ("", "void") else params.count(",") + 1
        assert n == len(argtypes), "%s: header has %d parameters, binding %d" % (name, n, len(argtypes))


def test_calls_before_init_fail_cleanly():
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is present; the uninitialised state is exercised in the CPU tier")
    lib = capi.load()
    assert lib.wdh_alloc(16) == 0
    assert "wdh_init" in capi.last_error()
    with pytest.raises(capi.HipError) as err:
        capi.call("wdh_sync")
    assert err.value.code == -5
    with pytest.raises(capi.HipError) as err:
        capi.call("wdh_init", 0)        # no device here: ENODEV, never a crash
    assert err.value.code == -1


def _init_with_options(text):
    """wdh_init(0) in a fresh process with WDH_OPTIONS set: (status, last error)."""
    import subprocess
    import sys

    code = ("import sys; sys.path.insert(0, %r)\n"
            "from webdnn_amd import capi\n"
            "lib = capi.load(); rc = lib.wdh_init(0)\n"
            "print(rc); print(capi.last_error())\n" % ROOT)
    env = dict(os.environ, WDH_OPTIONS=text)
    out = subprocess.run([sys.executable, "-c", code], env=env, stdout=subprocess.PIPE, text=True, check=True).stdout
    rc, _, msg = out.partition("\n")
    return int(rc), msg.strip()


@pytest.mark.parametrize("text, needle", [
    ("no_such_option=1", "unknown option"),
    ("split_k", "not name=value"),
    ("split_k=three", "not an integer"),
    ("split_k=0", "split_k"),                       # a known name with a value outside its range
    ("wide_stores=1," + "x" * 600, "longer than"),
])
def test_bad_environment_options_fail_before_the_device_is_touched(text, needle):
    """A malformed or unknown item of WDH_OPTIONS is WDH_EINVAL (-2) whether or not a GPU is there: the
    string is checked first, so the library is never left initialised with half of the options applied."""
    rc, msg = _init_with_options(text)
    assert rc == -2 and needle in msg, (rc, msg)


def test_good_environment_options_reach_the_device_step():
    import torch

    rc, msg = _init_with_options("split_k=2,wide_stores=0")
    if torch.cuda.is_available():
        assert rc == 0, msg
    else:
        assert rc == -1, (rc, msg)      # options accepted; the missing device is the first failure


def test_stem_kernel_steps_aside_for_images_beyond_its_32_bit_indexing():
    """wdh::conv_patch_applies (an internal predicate, called here by its C++ symbol): the stem conv's own
    kernel indexes an image with 32-bit offsets, so an image of 2 GiB or more must be left to the gathered
    form; the ordinary stem geometry qualifies."""
    import ctypes

    fn = getattr(capi.load(), "_ZN3wdh18conv_patch_appliesEiiiiiiiiiiiiiii")
    fn.restype = ctypes.c_bool
    fn.argtypes = [ctypes.c_int] * 15

    def applies(h, w, pt=3, pl=3):
        oh, ow = (h + 2 * pt - 7) // 2 + 1, (w + 2 * pl - 7) // 2 + 1
        return fn(3, 64, 7, 7, 2, 2, 1, 1, 1, h, w, pt, pl, oh, ow)

    assert applies(224, 224) and applies(800, 1088)
    assert not applies(14000, 14000)        # an image (and its results) beyond 2 GiB
    assert not fn(4, 64, 7, 7, 2, 2, 1, 1, 1, 224, 224, 3, 3, 112, 112)


def test_typed_surface_lists_every_addon_function_with_its_argument_count():
    """interface/backend/hip/hipNative.d.ts is written by hand: it must name exactly the functions the
    addon exports, each with as many parameters as the addon's ARGS() check demands."""
    addon = open(os.path.join(ROOT, "webdnn_amd", "napi", "addon.c")).read()
    exported = dict(re.findall(r'\{"(\w+)",\s*(js_\w+)\}', addon))
    argc = {}
    for js_name, c_name in exported.items():
        body = addon[addon.index("FN(%s)" % c_name):]
        m = re.search(r'ARGS\("\w+",\s*(\d+)\)', body[:body.index("\n}\n")])
        argc[js_name] = int(m.group(1)) if m else 0          # js_shutdown takes none and has no ARGS()
    text = open(os.path.join(ROOT, "webdnn_amd", "js", "interface", "backend", "hip", "hipNative.d.ts")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    iface = text[text.index("export interface HipNative {"):]
    declared = {}
    for name, params in re.findall(r"^\s{2}(\w+)\(([^)]*)\)\s*:", iface, flags=re.M | re.S):
        declared[name] = 0 if not params.strip() else params.count(",") + 1
    assert declared == argc
