"""Host-side shape logic of the hip backend (webdnn_amd/hostops.py) against the oracle's own
shape computation (written separately, in C, from the same reference files) on random cases."""
import numpy as np
import pytest

from oracle import ref
from webdnn_amd import hostops as H

RNG = np.random.default_rng(7)


def test_matmul_shapes():
    for _ in range(300):
        ra, rb = RNG.integers(1, 4), RNG.integers(1, 4)
        k = int(RNG.integers(1, 5))
        a = [int(RNG.integers(1, 4)) for _ in range(ra - 1)] + [k]
        b = [int(RNG.integers(1, 4)) for _ in range(rb)]
        if rb == 1:
            b = [k]
        else:
            b[-2] = k
        # batch dims must broadcast
        if ra == 3 and rb == 3 and a[0] != b[0]:
            (a if RNG.integers(0, 2) else b)[0] = 1
        A, B = np.zeros(a, np.float32), np.zeros(b, np.float32)
        try:
            want = ref.matmul(A, B).shape
        except ref.RefThrows:
            with pytest.raises(H.OperatorError):
                res = H.matmul_shape(a, b)
                if len(res[0]) > 3:
                    raise H.OperatorError("rank")
            continue
        result, squeezed, sa, sb, inner = H.matmul_shape(a, b)
        assert tuple(squeezed) == want and inner == k


def test_conv_shapes():
    for _ in range(300):
        h, w = int(RNG.integers(5, 20)), int(RNG.integers(5, 20))
        k = [int(RNG.integers(1, 4)), int(RNG.integers(1, 4))]
        pads = [int(v) for v in RNG.integers(0, 3, 4)]
        strides = [int(v) for v in RNG.integers(1, 4, 2)]
        dil = [int(v) for v in RNG.integers(1, 3, 2)]
        X, W = np.zeros((1, 2, h, w), np.float32), np.zeros((3, 2, k[0], k[1]), np.float32)
        want = ref.conv(X, W, None, dil, 1, None, pads, strides).shape
        got = H.conv_shape(X.shape, W.shape, dil, 1, None, pads, strides)
        assert (1, 3, got["out_shape"][0], got["out_shape"][1]) == want


def test_maxpool_shapes():
    for _ in range(400):
        h, w = int(RNG.integers(6, 20)), int(RNG.integers(6, 20))
        k = [int(RNG.integers(1, 4)), int(RNG.integers(1, 4))]
        strides = [int(v) for v in RNG.integers(1, 4, 2)]
        dil = [int(v) for v in RNG.integers(1, 3, 2)]
        auto_pad = ["NOTSET", "SAME_UPPER", "SAME_LOWER", "VALID"][int(RNG.integers(0, 4))]
        pads = [int(v) for v in RNG.integers(0, 2, 4)] if auto_pad == "NOTSET" else None
        ceil_mode = int(RNG.integers(0, 2))
        X = np.zeros((1, 1, h, w), np.float32)
        Y, pads_want = ref.maxpool(X, k, auto_pad, ceil_mode, dil, pads, strides, return_pads=True)
        got = H.maxpool_shape(X.shape, k, auto_pad, ceil_mode, dil, pads, strides)
        assert tuple(got["out_shape"]) == Y.shape[2:]
        assert list(got["pads"]) == pads_want


def test_broadcast_and_reshape():
    assert H.broadcast_uni([4, 5], [5]) == [0, 1]
    assert H.broadcast_uni([4, 5], [4, 1]) == [1, 0]
    assert H.broadcast_uni([4, 5], []) == [0, 0]
    with pytest.raises(H.OperatorError):
        H.broadcast_uni([4, 5], [3])
    with pytest.raises(H.OperatorError):
        H.broadcast_uni([5], [1, 5])
    dims, (sl, sr) = H.broadcast_multi([[2, 3, 10, 12], [1, 3, 1, 12]])
    assert dims == [2, 3, 10, 12] and sl == [360, 120, 12, 1] and sr == [0, 12, 0, 1]
    with pytest.raises(H.OperatorError):
        H.broadcast_multi([[2, 3], [4]])
    for shape in ([0, -1], [8, 0, 5], [4, -1, 5], [120], [-1]):
        X = np.zeros((2, 3, 4, 5), np.float32)
        assert tuple(H.reshape_shape(list(X.shape), X.size, shape)) == ref.reshape(X, shape).shape
    with pytest.raises(H.OperatorError):
        H.reshape_shape([2, 3], 6, [-1, -1])
