"""Helpers shared by the tests."""
import numpy as np


def bits(a):
    a = np.ascontiguousarray(a)
    return a.view(np.uint32) if a.dtype.itemsize == 4 else a


def assert_bit_exact(got, want, what=""):
    assert got.shape == want.shape, "%s: shape %s != %s" % (what, got.shape, want.shape)
    assert got.dtype == want.dtype, "%s: dtype %s != %s" % (what, got.dtype, want.dtype)
    if got.dtype == np.float32:
        # NaN payloads may differ; every NaN must sit where the reference has one
        gn, wn = np.isnan(got), np.isnan(want)
        assert np.array_equal(gn, wn), "%s: NaN positions differ" % what
        same = bits(np.where(gn, 0, got)) == bits(np.where(wn, 0, want))
    else:
        same = got == want
    if not np.all(same):
        bad = np.argwhere(~same)
        idx = tuple(bad[0])
        raise AssertionError("%s: %d of %d elements differ, first at %s: got %r want %r" % (
            what, len(bad), got.size, idx, got[idx], want[idx]))


def assert_close_max(got, want, rel, what=""):
    """max|got - want| <= rel * max|want|  (the Gemm/Conv criterion, rel = 1e-4)."""
    assert got.shape == want.shape, "%s: shape %s != %s" % (what, got.shape, want.shape)
    if want.size == 0:
        return
    err = float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64))))
    scale = float(np.max(np.abs(want)))
    assert err <= rel * scale + 1e-30, "%s: max|diff| %.3e > %.1e * max|ref| %.3e" % (what, err, rel, scale)


def ulp_diff(a, b):
    """Distance in fp32 units in the last place (finite inputs)."""
    a = np.ascontiguousarray(a, np.float32).view(np.int32).astype(np.int64)
    b = np.ascontiguousarray(b, np.float32).view(np.int32).astype(np.int64)
    a = np.where(a < 0, -(a & 0x7fffffff), a)
    b = np.where(b < 0, -(b & 0x7fffffff), b)
    return np.abs(a - b)


def load_kat():
    """tests/golden/kat.json with "inf"/"-inf" strings turned back into floats."""
    import json
    import os

    def restore(obj):
        if obj == "inf":
            return float("inf")
        if obj == "-inf":
            return float("-inf")
        if isinstance(obj, list):
            return [restore(o) for o in obj]
        if isinstance(obj, dict):
            return {k: restore(v) for k, v in obj.items()}
        return obj

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "kat.json")
    with open(path) as f:
        return restore(json.load(f))["cases"]


def arr(values, shape, dtype=np.float32):
    return np.asarray(values, dtype=dtype).reshape(shape)
