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
