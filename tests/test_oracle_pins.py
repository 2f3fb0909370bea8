"""Pins the CPU oracle (oracle/webdnn_cpu_ref.c) without running the reference.

Each oracle function is checked against something it was NOT written from:
  * an independent brute-force evaluation in pure Python floats (IEEE doubles, like JavaScript
    numbers) written from the operator's definition — e.g. DIRECT convolution for Conv, whereas
    the oracle goes through im2col -> matmul -> transpose -> bias;
  * a library routine in float64 (numpy / torch) within 1 fp32 ulp;
  * invariants of the mathematics (alpha = 0, beta = 0, transposes, 1x1 conv == Gemm, delta
    kernels, shift invariance, permutation inverses);
  * the error behaviour the reference documents (where it throws).
"""
import itertools
import math

import numpy as np
import pytest
import torch

from oracle import ref
from util import assert_bit_exact, assert_close_max, ulp_diff

RNG = np.random.default_rng(1234)


def rnd(*shape, lo=-1.0, hi=1.0):
    return RNG.uniform(lo, hi, shape).astype(np.float32)


def f32(x):
    return np.float32(x)


# ---------------------------------------------------------------- Gemm
def py_gemm(A, B, C, alpha, beta, ta, tb):
    """Definition: Y = alpha * op(A) op(B) + beta * C, double accumulation in k order, fp32 store
    after the alpha product and again after the C term."""
    A = A.T if ta else A
    B = B.T if tb else B
    m, k = A.shape
    n = B.shape[1]
    Y = np.zeros((m, n), np.float32)
    Cb = np.broadcast_to(C, (m, n)) if C is not None else None
    for i in range(m):
        for j in range(n):
            s = 0.0
            for x in range(k):
                s += float(A[i, x]) * float(B[x, j])
            y = f32(s * alpha)
            if Cb is not None:
                y = f32(float(y) + float(Cb[i, j]) * beta)
            Y[i, j] = y
    return Y


@pytest.mark.parametrize("ta,tb", list(itertools.product((0, 1), (0, 1))))
@pytest.mark.parametrize("cshape", [(5,), (7, 1), (7, 5), (1,), (), None])
def test_gemm_brute_force(ta, tb, cshape):
    m, n, k = 7, 5, 13
    A = rnd(k, m) if ta else rnd(m, k)
    B = rnd(n, k) if tb else rnd(k, n)
    C = rnd(*cshape) if cshape is not None else None
    alpha, beta = 0.75, -1.25
    assert_bit_exact(ref.gemm(A, B, C, alpha, beta, ta, tb), py_gemm(A, B, C, alpha, beta, ta, tb), "gemm")


def test_gemm_float64_closed_form_config1():
    # benchmark config 1: A[256,512] . B[1024,512]^T + C[1024]
    A, B, C = rnd(256, 512), rnd(1024, 512), rnd(1024)
    want = (A.astype(np.float64) @ B.astype(np.float64).T).astype(np.float32)
    want = (want.astype(np.float64) + C.astype(np.float64)).astype(np.float32)
    got = ref.gemm(A, B, C, 1.0, 1.0, 0, 1)
    assert ulp_diff(got, want).max() <= 1  # BLAS sums in another order: last double bit may differ


def test_gemm_invariants():
    A, B, C = rnd(6, 9), rnd(9, 4), rnd(4)
    assert_bit_exact(ref.gemm(A, B, C, 0.0, 2.0), np.broadcast_to(f32(2.0) * C, (6, 4)).astype(np.float32) + 0.0,
                     "alpha=0")
    assert_bit_exact(ref.gemm(A, B, C, 1.5, 0.0), ref.gemm(A, B, None, 1.5, 1.0), "beta=0")
    assert_bit_exact(ref.gemm(A.T.copy(), B, C, 1, 1, 1, 0), ref.gemm(A, B, C), "transA")
    assert_bit_exact(ref.gemm(A, B.T.copy(), C, 1, 1, 0, 1), ref.gemm(A, B, C), "transB")
    eye = np.eye(9, dtype=np.float32)
    assert_bit_exact(ref.gemm(A, eye), A, "identity B")


def test_gemm_throws():
    with pytest.raises(ref.RefThrows):
        ref.gemm(rnd(3, 4), rnd(5, 6))            # k mismatch, base/gemm.ts:56-58
    with pytest.raises(ref.RefThrows):
        ref.gemm(rnd(2, 3, 4), rnd(4, 6))         # rank != 2, base/gemm.ts:36-38
    with pytest.raises(ref.RefThrows):
        ref.gemm(rnd(3, 4), rnd(4, 6), rnd(5))    # C not broadcastable, operatorUtil.ts:201-203
    with pytest.raises(ref.RefThrows):
        ref.gemm(rnd(3, 4), rnd(4, 6), rnd(1, 3, 6))  # C rank > 2, operatorUtil.ts:187-189


# ---------------------------------------------------------------- MatMul
@pytest.mark.parametrize("sa,sb", [((3, 4), (4, 5)), ((2, 3, 4), (4, 5)), ((1, 3, 128), (4, 128, 1)),
                                   ((4, 3, 6), (4, 6, 2)), ((6,), (6, 3)), ((2, 3, 6), (6,)), ((6,), (6,)),
                                   ((4, 1, 6), (6, 2))])
def test_matmul_numpy_semantics(sa, sb):
    A, B = rnd(*sa), rnd(*sb)
    got = ref.matmul(A, B)
    want = np.matmul(A.astype(np.float64), B.astype(np.float64)).astype(np.float32)
    assert got.shape == want.shape
    assert ulp_diff(got, want).max() <= 1


def test_matmul_is_per_batch_gemm():
    A, B = rnd(3, 5, 7), rnd(3, 7, 4)
    got = ref.matmul(A, B)
    for b in range(3):
        assert_bit_exact(got[b], ref.gemm(A[b], B[b]), "batch %d" % b)


def test_matmul_throws():
    with pytest.raises(ref.RefThrows):
        ref.matmul(rnd(2, 2, 3, 4), rnd(4, 5))      # result rank 4, cpu matmul.ts:50-53
    with pytest.raises(ref.RefThrows):
        ref.matmul(rnd(3, 4), rnd(5, 6))            # inner mismatch, base/matmul.ts:56-58
    with pytest.raises(ref.RefThrows):
        ref.matmul(np.float32(2.0), rnd(5, 6))      # scalar, base/matmul.ts:33-35


# ---------------------------------------------------------------- Conv
def py_conv_direct(X, W, Bv, dil, group, pads, strides):
    """Direct convolution from the definition: double accumulation over (ci, ky, kx), fp32 store of
    the sum, then fp32 store of sum + bias."""
    n, c, h, w = X.shape
    cout, cg, kh, kw = W.shape
    og = cout // group
    oh = (h + pads[0] + pads[2] - dil[0] * (kh - 1) - 1) // strides[0] + 1
    ow = (w + pads[1] + pads[3] - dil[1] * (kw - 1) - 1) // strides[1] + 1
    Y = np.zeros((n, cout, oh, ow), np.float32)
    for b, co, oy, ox in itertools.product(range(n), range(cout), range(oh), range(ow)):
        g = co // og
        s = 0.0
        for ci, ky, kx in itertools.product(range(cg), range(kh), range(kw)):
            iy = oy * strides[0] - pads[0] + ky * dil[0]
            ix = ox * strides[1] - pads[1] + kx * dil[1]
            v = float(X[b, g * cg + ci, iy, ix]) if 0 <= iy < h and 0 <= ix < w else 0.0
            s += v * float(W[co, ci, ky, kx])
        y = f32(s)
        if Bv is not None:
            y = f32(float(y) + float(Bv[co]))
        Y[b, co, oy, ox] = y
    return Y


CONV_CASES = [
    # n, c, h, w, cout, k, pads, strides, dil, group, bias  (after test/model_test/make_models.py:623-643)
    (2, 3, 6, 7, 4, 3, [1, 1, 1, 1], [1, 1], [1, 1], 1, True),
    (1, 4, 7, 6, 6, 3, [1, 0, 2, 1], [2, 2], [1, 1], 2, True),
    (1, 2, 9, 9, 3, 3, [2, 2, 2, 2], [1, 1], [2, 2], 1, False),
    (2, 4, 5, 5, 4, 3, [1, 1, 1, 1], [1, 1], [1, 1], 4, True),
    (1, 3, 12, 11, 5, 7, [3, 3, 3, 3], [2, 2], [1, 1], 1, True),
    (2, 6, 4, 5, 3, 1, [0, 0, 0, 0], [2, 2], [1, 1], 1, False),
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_direct_brute_force(case):
    n, c, h, w, cout, k, pads, strides, dil, group, bias = case
    X, W = rnd(n, c, h, w, lo=0), rnd(cout, c // group, k, k)
    Bv = rnd(cout) if bias else None
    got = ref.conv(X, W, Bv, dil, group, None, pads, strides)
    assert_bit_exact(got, py_conv_direct(X, W, Bv, dil, group, pads, strides), "conv")
    lib = torch.nn.functional.conv2d(
        torch.nn.functional.pad(torch.from_numpy(X).double(), (pads[1], pads[3], pads[0], pads[2])),
        torch.from_numpy(W).double(), torch.from_numpy(Bv).double() if bias else None,
        stride=strides, dilation=dil, groups=group).numpy()
    assert got.shape == lib.shape
    assert_close_max(got, lib.astype(np.float32), 1e-6, "conv vs torch float64")


def test_conv_default_attributes_and_shape():
    X, W = rnd(1, 2, 5, 6), rnd(3, 2, 2, 3)
    got = ref.conv(X, W)                         # pads 0, strides 1, dilations 1, kernel from W
    assert got.shape == (1, 3, 4, 4)
    assert_bit_exact(got, py_conv_direct(X, W, None, [1, 1], 1, [0, 0, 0, 0], [1, 1]), "defaults")


def test_conv_1x1_is_gemm_and_delta_is_shift():
    X, W = rnd(2, 5, 4, 3), rnd(7, 5, 1, 1)
    got = ref.conv(X, W)
    for b in range(2):
        want = ref.gemm(W.reshape(7, 5), X[b].reshape(5, 12)).reshape(7, 4, 3)
        assert_bit_exact(got[b], want, "1x1")
    delta = np.zeros((1, 1, 3, 3), np.float32)
    delta[0, 0, 0, 2] = 1.0                      # picks x[iy-1, ix+1]
    X1 = rnd(1, 1, 6, 6)
    got = ref.conv(X1, delta, pads=[1, 1, 1, 1])
    want = np.zeros_like(X1)
    want[0, 0, 1:, :-1] = X1[0, 0, :-1, 1:]
    assert_bit_exact(got, want, "delta kernel")


def test_conv_throws_on_non_2d():
    with pytest.raises(ref.RefThrows):
        ref.conv(rnd(1, 2, 5), rnd(3, 2, 2, 2))   # cpu conv.ts:140-142


# ---------------------------------------------------------------- Binary / Unary
@pytest.mark.parametrize("op,fn", [("Add", np.add), ("Sub", np.subtract), ("Mul", np.multiply), ("Div", np.divide)])
@pytest.mark.parametrize("sl,sr", [((2, 3, 10, 12), ()), ((2, 3, 10, 12), (1, 3, 1, 12)), ((), ()),
                                   ((4, 1), (3,)), ((2, 1, 3, 1, 2, 1), (1, 2, 1, 2, 1, 3))])
def test_binary_is_ieee_fp32(op, fn, sl, sr):
    L, R = rnd(*sl, lo=-3, hi=3), rnd(*sr, lo=-3, hi=3)
    with np.errstate(all="ignore"):
        want = fn(L, R)                           # numpy fp32 op == double op rounded (IEEE)
    assert_bit_exact(ref.binary(op, L, R), np.asarray(want, np.float32), op)


def test_binary_special_values_and_int32():
    L = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, 3.4e38, 1.0], np.float32)
    R = np.array([-0.0, 0.0, -np.inf, 1.0, 1.0, 0.5, 3.4e38, 0.0], np.float32)
    with np.errstate(all="ignore"):
        for op, fn in (("Add", np.add), ("Sub", np.subtract), ("Mul", np.multiply), ("Div", np.divide)):
            assert_bit_exact(ref.binary(op, L, R), fn(L, R), op)
    a = np.array([2147483647, -2147483648, 7, -7, 100000], np.int32)
    b = np.array([1, -1, 2, 2, 100000], np.int32)
    assert ref.binary("Add", a, b).tolist() == [-2147483648, 2147483647, 9, -5, 200000]
    assert ref.binary("Div", a, b).tolist() == [2147483647, -2147483648, 3, -3, 1]   # truncation
    assert ref.binary("Mul", a, b).tolist()[:4] == [2147483647, -2147483648, 14, -14]
    assert ref.binary("Mul", a, b).tolist()[4] == (100000 * 100000) % 2 ** 32 - 2 ** 32 * ((100000 * 100000) % 2 ** 32 >= 2 ** 31)
    assert ref.binary("Div", np.array([5, 0], np.int32), np.array([0, 0], np.int32)).tolist() == [0, 0]


def test_binary_throws():
    with pytest.raises(ref.RefThrows):
        ref.binary("Add", rnd(2, 3), rnd(4))                           # operatorUtil.ts:237-239
    with pytest.raises(ref.RefThrows):
        ref.binary("Add", rnd(2), np.zeros(2, np.int32))                 # binary7.ts:20-24
    with pytest.raises(ref.RefThrows):
        ref.binary("Add", rnd(1, 1, 1, 1, 1, 1, 2), rnd(2))              # rank 7, binary7.ts:63-66


def test_unary():
    x = np.array([-2, -0.5, 0, 1, 3], np.float32)
    assert ref.unary("Relu", x).tolist() == [0, 0, 0, 1, 3]            # test/unit/cpuOperator.test.ts:15-18
    y = ref.unary("Relu", np.array([np.nan, -0.0, -np.inf, np.inf], np.float32))
    assert np.isnan(y[0]) and not np.signbit(y[1]) and y[2] == 0 and y[3] == np.inf
    assert ref.unary("Relu", np.array([-3, 0, 4], np.int32)).tolist() == [0, 0, 4]
    v = rnd(1000, lo=-20, hi=20)
    sig = 1.0 / (1.0 + np.exp(-v.astype(np.float64)))
    assert_close_max(ref.unary("Sigmoid", v), sig.astype(np.float32), 1e-6, "sigmoid")
    p = rnd(1000, lo=0, hi=50)
    assert_bit_exact(ref.unary("Sqrt", p), np.sqrt(p), "sqrt")          # correctly rounded either way
    assert_close_max(ref.unary("Exp", v), np.exp(v.astype(np.float64)).astype(np.float32), 1e-6, "exp")
    assert_close_max(ref.unary("Tanh", v), np.tanh(v.astype(np.float64)).astype(np.float32), 1e-6, "tanh")
    with pytest.raises(ref.RefThrows):
        ref.unary("Sigmoid", np.zeros(3, np.int32))                      # unary.ts:21-23


# ---------------------------------------------------------------- Softmax / LayerNorm / means
def test_softmax_closed_form_and_invariants():
    x = rnd(3, 4, 5, 6, lo=-5, hi=5)                                      # make_models.py:727
    got = ref.softmax(x)
    xd = x.astype(np.float64)
    e = np.exp(xd - xd.max(-1, keepdims=True))
    assert_close_max(got, (e / e.sum(-1, keepdims=True)).astype(np.float32), 1e-6, "softmax")
    assert np.abs(got.astype(np.float64).sum(-1) - 1).max() < 1e-6
    assert_close_max(ref.softmax(x + f32(3.0)), got, 1e-5, "shift invariance")
    assert_bit_exact(ref.softmax(np.full((2, 7), 0.3, np.float32)), np.full((2, 7), f32(1 / 7), np.float32), "uniform")
    hot = ref.softmax(np.array([[0, 1000, 0]], np.float32))
    assert hot.tolist() == [[0, 1, 0]]
    with pytest.raises(ref.RefThrows):
        ref.softmax(x, axis=1)                                            # softmax.ts:28-32
    assert_bit_exact(ref.softmax(x, axis=3), got, "axis=ndim-1")


def test_means():
    x = rnd(2, 5, 7, 7)
    want = x.astype(np.float64).mean((2, 3), keepdims=True).astype(np.float32)
    assert ulp_diff(ref.global_average_pool(x), want).max() <= 1
    seq = np.array([[[[sum_seq(x[b, c])] ] for c in range(5)] for b in range(2)], np.float32)
    assert_bit_exact(ref.global_average_pool(x), seq, "sequential double sum / (h*w)")
    assert_bit_exact(ref.reduce_mean_last(x.reshape(10, 49)).reshape(2, 5, 1, 1), seq, "ReduceMean")
    with pytest.raises(ref.RefThrows):
        ref.global_average_pool(rnd(2, 3, 4))                            # globalaveragepool.ts:16-18


def test_reduce_mean_over_any_axes():
    """The general form (one pass per axis, fp32 between passes).  Pinned by: exact rational
    arithmetic on integers small enough that every pass is exact; a brute-force pass-by-pass
    evaluation in Python floats; numpy float64 means within the ulps the passes can cost; the
    trailing-axis function it generalises; shapes with and without keepdims."""
    from fractions import Fraction

    rng = np.random.default_rng(21)
    xi = rng.integers(-500, 500, (3, 4, 5, 6)).astype(np.float32)
    for axes in ([0], [1, 3], [0, 1, 2, 3], [2], [-1, -3]):
        ax = sorted(a % 4 for a in axes)
        got = ref.reduce_mean(xi, axes, 1)
        cnt = int(np.prod([xi.shape[a] for a in ax]))
        exact = xi.astype(np.int64).sum(tuple(ax), keepdims=True)
        want = np.vectorize(lambda v: np.float32(Fraction(int(v), cnt)))(exact).astype(np.float32)
        assert_bit_exact(got, want, "integers: every pass exact, one rounding at the end %s" % (axes,))
    x = rnd(3, 4, 5, 6)
    # brute force, two axes: pass over axis 1 (fp32 store), then over axis 3 divided by 4*6
    first = np.zeros((3, 5, 6), np.float32)
    for o in range(3):
        for i in range(5):
            for j in range(6):
                acc = 0.0
                for r in range(4):
                    acc += float(x[o, r, i, j])
                first[o, i, j] = acc
    second = np.zeros((3, 5), np.float32)
    for o in range(3):
        for i in range(5):
            acc = 0.0
            for r in range(6):
                acc += float(first[o, i, r])
            second[o, i] = acc / 24
    assert_bit_exact(ref.reduce_mean(x, [1, 3], 0), second, "pass by pass")
    assert ref.reduce_mean(x, [3, 1], 1).shape == (3, 1, 5, 1)                 # order of the list is irrelevant
    assert_bit_exact(ref.reduce_mean(x, [3, 1], 0), second, "axes are sorted")
    for axes in ([0], [2], [0, 2], [1, 2, 3], []):
        ax = tuple(axes) if axes else (0, 1, 2, 3)
        want = x.astype(np.float64).mean(ax, keepdims=True).astype(np.float32)
        got = ref.reduce_mean(x, axes, 1)
        assert got.shape == want.shape
        # every pass rounds a partial sum once: half an ulp of a value no larger than the sum of
        # the magnitudes, which the divisions turn into half an ulp of max|x| per pass at most
        assert np.abs(got - want).max() <= len(ax) * 2.0 ** -24 * np.abs(x).max(), axes
    assert_bit_exact(ref.reduce_mean(x, [3], 1), ref.reduce_mean_last(x), "trailing axis")
    assert_bit_exact(ref.reduce_mean(x, [-1], 1), ref.reduce_mean_last(x), "negative axis")
    assert ref.reduce_mean(x, [], 0).shape == () and ref.reduce_mean(x, [0, 3], 0).shape == (4, 5)


def sum_seq(plane):
    s = 0.0
    for v in plane.reshape(-1):
        s += float(v)
    return f32(s / plane.size)


def test_layernorm_is_the_decomposed_subgraph():
    x, g, b = rnd(6, 256, lo=-3, hi=3), rnd(256), rnd(256)
    eps = f32(1e-5)
    mean = ref.reduce_mean_last(x)
    d = ref.binary("Sub", x, mean)
    var = ref.reduce_mean_last(ref.binary("Mul", d, d))
    s = ref.unary("Sqrt", ref.binary("Add", var, np.array(eps, np.float32)))
    want = ref.binary("Add", ref.binary("Mul", ref.binary("Div", d, s), g), b)
    assert_bit_exact(ref.layernorm_decomposed(x, g, b, 1e-5), want, "decomposed identity")
    xd = x.astype(np.float64)
    closed = (xd - xd.mean(-1, keepdims=True)) / np.sqrt(xd.var(-1, keepdims=True) + 1e-5) * g + b
    assert_close_max(want, closed.astype(np.float32), 1e-5, "ONNX-17 closed form")
    plain = ref.layernorm_decomposed(x, None, None, 1e-5).astype(np.float64)
    assert np.abs(plain.mean(-1)).max() < 1e-6 and np.abs(plain.var(-1) - 1).max() < 1e-4


# ---------------------------------------------------------------- MaxPool / Transpose / layout
def np_maxpool(X, k, pads, strides, dil, oh, ow):
    n, c, h, w = X.shape
    Y = np.full((n, c, oh, ow), -np.inf, np.float32)
    for oy, ox, ky, kx in itertools.product(range(oh), range(ow), range(k[0]), range(k[1])):
        iy, ix = oy * strides[0] - pads[0] + ky * dil[0], ox * strides[1] - pads[1] + kx * dil[1]
        if 0 <= iy < h and 0 <= ix < w:
            Y[:, :, oy, ox] = np.maximum(Y[:, :, oy, ox], X[:, :, iy, ix])
    return Y


@pytest.mark.parametrize("ceil_mode", [0, 1])
@pytest.mark.parametrize("pads", [[0, 0, 0, 0], [1, 1, 1, 1]])
def test_maxpool_against_torch(ceil_mode, pads):
    X = rnd(2, 3, 10, 12)                                                # make_models.py:650-653
    got = ref.maxpool(X, [3, 3], ceil_mode=ceil_mode, pads=pads, strides=[2, 2])
    lib = torch.nn.functional.max_pool2d(torch.from_numpy(X), 3, 2, pads[0], ceil_mode=bool(ceil_mode)).numpy()
    # torch drops a last window that starts in the right padding; the reference keeps it
    # (operators/base/maxpool.ts:43-58), so compare the common part and the brute force in full
    hh, ww = min(got.shape[2], lib.shape[2]), min(got.shape[3], lib.shape[3])
    assert_bit_exact(got[:, :, :hh, :ww], lib[:, :, :hh, :ww], "torch")
    assert_bit_exact(got, np_maxpool(X, [3, 3], pads, [2, 2], [1, 1], got.shape[2], got.shape[3]), "brute force")


def test_maxpool_auto_pad_and_errors():
    X = rnd(1, 2, 7, 8)
    up, pads_up = ref.maxpool(X, [3, 3], auto_pad="SAME_UPPER", strides=[2, 3], return_pads=True)
    lo, pads_lo = ref.maxpool(X, [3, 3], auto_pad="SAME_LOWER", strides=[2, 3], return_pads=True)
    assert up.shape == lo.shape == (1, 2, 4, 3)
    assert pads_up == [1, 0, 1, 1] and pads_lo == [1, 1, 1, 0]           # base/maxpool.ts:81-111
    assert_bit_exact(up, np_maxpool(X, [3, 3], pads_up, [2, 3], [1, 1], 4, 3), "SAME_UPPER")
    assert_bit_exact(lo, np_maxpool(X, [3, 3], pads_lo, [2, 3], [1, 1], 4, 3), "SAME_LOWER")
    va = ref.maxpool(X, [3, 3], auto_pad="VALID", strides=[2, 3])
    assert va.shape == (1, 2, 3, 2)
    assert_bit_exact(va, np_maxpool(X, [3, 3], [0, 0, 0, 0], [2, 3], [1, 1], 3, 2), "VALID")
    nanx = X.copy()
    nanx[0, 0, 0, 0] = np.nan
    assert not np.isnan(ref.maxpool(nanx, [3, 3])).any()                 # `v > mv` never picks NaN
    with pytest.raises(ref.RefThrows):
        ref.maxpool(X, [3, 3], n_outputs=2)                              # cpu maxpool.ts:19-22
    with pytest.raises(ref.RefThrows):
        ref.maxpool(rnd(2, 7, 8), [3, 3])                                # cpu maxpool.ts:24-26
    with pytest.raises(ref.RefThrows):
        ref.maxpool(X, [3, 3], auto_pad="SAME")                          # base/maxpool.ts:124-126


@pytest.mark.parametrize("ndim", [1, 2, 3, 4])
def test_transpose_all_permutations(ndim):
    shape = (3, 4, 2, 5)[:ndim]
    X = rnd(*shape)
    for perm in itertools.permutations(range(ndim)):
        got = ref.transpose(X, list(perm))
        assert_bit_exact(got, np.ascontiguousarray(np.transpose(X, perm)), "perm %s" % (perm,))
        inv = [perm.index(i) for i in range(ndim)]
        assert_bit_exact(ref.transpose(got, inv), X, "inverse")
    assert_bit_exact(ref.transpose(X), np.ascontiguousarray(X.T), "default perm = reversed")


def test_transpose_rank_limits_and_ints():
    X6 = RNG.integers(-9, 9, (2, 3, 2, 2, 3, 2)).astype(np.int32)
    perm = [5, 3, 0, 4, 1, 2]
    assert_bit_exact(ref.transpose(X6, perm), np.ascontiguousarray(np.transpose(X6, perm)), "rank 6 int32")
    with pytest.raises(ref.RefThrows):
        ref.transpose(rnd(1, 1, 1, 1, 1, 1, 2))                          # cpu transpose.ts:38-41
    with pytest.raises(ref.RefThrows):
        ref.transpose(rnd(2, 3), [0])                                    # base/transpose.ts:25-27


def test_layout_ops():
    X = rnd(2, 3, 4, 5)
    assert ref.flatten(X).shape == (2, 60)
    with pytest.raises(ref.RefThrows):
        ref.flatten(X, axis=2)                                           # base/flatten.ts:10-12
    assert ref.reshape(X, [0, -1]).shape == (2, 60)                      # base/reshape5.ts:45-73
    assert ref.reshape(X, [8, 0, 5]).shape == (8, 3, 5)                  # 0 copies input dim 1
    assert ref.reshape(X, [4, -1, 5]).shape == (4, 6, 5)
    with pytest.raises(ref.RefThrows):
        ref.reshape(X, [-1, -1])                                         # base/reshape5.ts:53-55
    assert ref.gather(np.array([5, 6, 7], np.int32), np.array(2, np.int32)).tolist() == 7
    with pytest.raises(ref.RefThrows):
        ref.gather(np.zeros((2, 2), np.int32), np.array(0, np.int32))    # cpu gather.ts:23-27


# ---- Squeeze / Unsqueeze / Concat / Split / Slice / Cast ----------------------------------
# Pinned against numpy's own routines on cases where the reference's rules and numpy's
# coincide, and against hand-derived answers where the reference deviates (Slice clamping,
# ToInt32 wrap-around).

def test_squeeze_unsqueeze():
    x = np.arange(2 * 1 * 3 * 1, dtype=np.float32).reshape(2, 1, 3, 1)
    assert ref.squeeze(x).shape == (2, 3)
    assert ref.squeeze(x, [1]).shape == (2, 3, 1)
    assert ref.squeeze(x, [-1, 1]).shape == (2, 3)
    assert np.array_equal(ref.squeeze(x, [3]), np.squeeze(x, 3))
    with pytest.raises(ref.RefThrows):
        ref.squeeze(x, [0])
    y = np.arange(6, dtype=np.float32).reshape(2, 3)
    assert ref.unsqueeze(y, [0]).shape == (1, 2, 3)
    assert ref.unsqueeze(y, [1, -1]).shape == (2, 1, 3, 1)
    assert np.array_equal(ref.unsqueeze(y, [0, 3]), np.expand_dims(y, (0, 3)))
    assert ref.unsqueeze(np.float32(3.0), [0]).shape == (1,)


@pytest.mark.parametrize("axis", [-4, -1, 0, 1, 2, 3])
def test_concat_is_numpy_concatenate(axis):
    rng = np.random.default_rng(axis + 10)
    shape = [2, 3, 4, 5]
    parts = []
    ax = axis % 4
    for n in (1, 3, 2):
        s = list(shape)
        s[ax] = n
        parts.append(rng.standard_normal(s).astype(np.float32))
    assert_bit_exact(ref.concat(parts, axis), np.concatenate(parts, axis))
    ints = [np.array([1, 2], np.int32), np.array([3], np.int32)]
    assert_bit_exact(ref.concat(ints, 0), np.array([1, 2, 3], np.int32))
    with pytest.raises(ref.RefThrows):
        ref.concat(parts, 4)


def test_split_is_numpy_split():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((4, 6, 5)).astype(np.float32)
    for axis, n in [(0, 2), (1, 3), (2, 5), (-1, 1), (-2, 2)]:
        for a, b in zip(ref.split(x, n, axis), np.split(x, n, axis)):
            assert_bit_exact(a, np.ascontiguousarray(b))
    a, b, c = ref.split(x, 3, 1, [1, 2, 3])
    assert_bit_exact(a, np.ascontiguousarray(x[:, :1]))
    assert_bit_exact(b, np.ascontiguousarray(x[:, 1:3]))
    assert_bit_exact(c, np.ascontiguousarray(x[:, 3:]))
    # an uneven axis without `split`: floor(len / n) each, the remainder is dropped (split.ts:26-30)
    parts = ref.split(x, 4, 1)
    assert [p.shape[1] for p in parts] == [1, 1, 1, 1]
    assert_bit_exact(parts[3], x[:, 3:4])
    with pytest.raises(ref.RefThrows):
        ref.split(x, 2, 3)


def test_slice_matches_numpy_where_rules_coincide_and_clamps_like_the_reference():
    rng = np.random.default_rng(4)
    x = rng.standard_normal((5, 6, 7)).astype(np.float32)
    assert_bit_exact(ref.slice_(x, [1, 2], [4, 6], [0, 2]), x[1:4, :, 2:6])
    assert_bit_exact(ref.slice_(x, [0, 0, 0], [5, 6, 7]), x)
    assert_bit_exact(ref.slice_(x, [1], [-1], [-1], [2]), x[:, :, 1:-1:2])
    assert_bit_exact(ref.slice_(x, [-3], [1000], [1]), x[:, -3:])
    assert_bit_exact(ref.slice_(x, [-1], [-1000], [2], [-1]), x[:, :, ::-1])
    assert_bit_exact(ref.slice_(x, [5], [0], [1], [-2]), x[:, 5:0:-2])
    assert ref.slice_(x, [3], [2], [0]).shape == (0, 6, 7)
    # the reference clamps start to size-1 even for a forward step: [5:5] on 5 elements
    # yields the last one (numpy would return none)
    assert_bit_exact(ref.slice_(x, [5], [5], [0]), x[4:5])
    assert_bit_exact(ref.slice_(x, [9], [100], [1]), x[:, 5:6])
    with pytest.raises(ref.RefThrows):
        ref.slice_(np.zeros((1,) * 7, np.float32), [0], [1])


def test_cast_and_toint32():
    v = np.array([0.0, -0.0, 1.9, -1.9, 2147483647.0, 2147483648.0, -2147483648.0, 4294967296.0,
                  4294967297.0, 3e9, -3e9, 1e20, np.nan, np.inf, -np.inf], np.float32)
    want = np.array([0, 0, 1, -1, -2147483648, -2147483648, -2147483648, 0,
                     0, -1294967296, 1294967296, 0, 0, 0, 0], np.int32)
    # 2147483647 is not a float32: it rounds to 2^31; 4294967297 rounds to 2^32;
    # 1e20f = 0x56bc76 * 2^44, a multiple of 2^32
    assert_bit_exact(ref.cast(v, 6), want)
    assert_bit_exact(ref.cast(v, 7), want)
    assert_bit_exact(ref.cast(np.array([3, -7, 2 ** 31 - 1], np.int32), 1),
                     np.array([3.0, -7.0, 2147483648.0], np.float32))
    assert ref.cast(np.array([1.5], np.float32), 1).dtype == np.float32
    with pytest.raises(ref.RefThrows):
        ref.cast(v, 10)
