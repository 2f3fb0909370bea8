"""Parity of the hip backend with the oracle, through the C ABI, on a real MI355X.

Criteria: bit-exact for indexing / layout / selection ops and for
fp32 Add/Sub/Mul/Div/Relu; max|diff| <= 1e-4 * max|ref| for Gemm / MatMul / Conv.  Softmax and
LayerNormalization, for which north_star names no figure, use 1e-6 and 1e-5 of max|ref| (the
oracle evaluates exp in double and rounds once; the kernel evaluates it in fp32).
"""
import ctypes
import itertools

import numpy as np
import pytest

import kat_runner
from oracle import ref
from util import assert_bit_exact, assert_close_max, load_kat
from webdnn_amd import capi
from webdnn_amd import hostops as H

pytestmark = pytest.mark.gpu

GEMM_TOL = 1e-4
RNG = np.random.default_rng(2024)


def uni(*shape, lo=-1.0, hi=1.0):
    return RNG.uniform(lo, hi, shape).astype(np.float32)


def nrm(*shape, std=1.0):
    return (RNG.standard_normal(shape) * std).astype(np.float32)


# ------------------------------------------------------------------ known answers
CASES = load_kat()


@pytest.mark.parametrize("case", CASES, ids=[kat_runner.case_id(c) for c in CASES])
def test_known_answers_bit_exact(ctx, case):
    assert_bit_exact(kat_runner.run_hip(ctx, case), kat_runner.expected(case), case["op"])


# ------------------------------------------------------------------ Gemm
def hip_gemm(ctx, A, B, C=None, alpha=1.0, beta=1.0, ta=0, tb=0, epilogue=None):
    tc = ctx.move_tensor(C) if C is not None else None
    return H.gemm(ctx, ctx.move_tensor(A), ctx.move_tensor(B), tc, alpha, beta, ta, tb, epilogue).get_data()


def test_gemm_config1(ctx):
    """benchmark config 1: A[256,512], B[1024,512] transB=1, C[1024], alpha=beta=1."""
    A, B, C = uni(256, 512), uni(1024, 512), uni(1024)
    assert_close_max(hip_gemm(ctx, A, B, C, 1.0, 1.0, 0, 1), ref.gemm(A, B, C, 1.0, 1.0, 0, 1), GEMM_TOL, "C1")


@pytest.mark.parametrize("ta,tb", list(itertools.product((0, 1), (0, 1))))
@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (7, 5, 3), (128, 128, 16), (129, 127, 17), (130, 250, 37),
                                   (64, 300, 1), (1, 513, 40), (257, 1, 33), (100, 92, 256), (32, 1000, 2048)])
def test_gemm_shapes_and_transposes(ctx, m, n, k, ta, tb):
    A = uni(k, m) if ta else uni(m, k)
    B = uni(n, k) if tb else uni(k, n)
    C = uni(n)
    got = hip_gemm(ctx, A, B, C, 0.75, -1.25, ta, tb)
    assert_close_max(got, ref.gemm(A, B, C, 0.75, -1.25, ta, tb), GEMM_TOL, "gemm")


@pytest.mark.parametrize("cshape", [(45,), (1, 45), (33, 1), (33, 45), (1,), (), (1, 1)])
def test_gemm_c_broadcast(ctx, cshape):
    A, B, C = uni(33, 20), uni(20, 45), uni(*cshape)
    assert_close_max(hip_gemm(ctx, A, B, C, 1.0, 0.5), ref.gemm(A, B, C, 1.0, 0.5), GEMM_TOL, "C%s" % (cshape,))


def test_gemm_invariants_and_edges(ctx):
    A, B, C = uni(40, 24), uni(24, 36), uni(36)
    # alpha = 0 -> beta * C exactly; beta = 0 == no C
    assert_bit_exact(hip_gemm(ctx, A, B, C, 0.0, 2.0), ref.gemm(A, B, C, 0.0, 2.0), "alpha=0")
    assert_bit_exact(hip_gemm(ctx, A, B, C, 1.5, 0.0), hip_gemm(ctx, A, B, None, 1.5, 1.0), "beta=0")
    # transposes are the same product
    assert_bit_exact(hip_gemm(ctx, np.ascontiguousarray(A.T), B, C, 1, 1, 1, 0), hip_gemm(ctx, A, B, C), "transA")
    # identity B returns A exactly (one nonzero term per sum)
    assert_bit_exact(hip_gemm(ctx, A, np.eye(24, dtype=np.float32)), A, "identity")
    # fused Relu epilogue == Relu(Gemm)
    y = hip_gemm(ctx, A, B, C)
    assert_bit_exact(hip_gemm(ctx, A, B, C, epilogue="relu"), np.maximum(y, 0) + 0.0, "relu epilogue")
    # empty inner dimension: the sum over nothing is 0, the C term remains
    Z0, Z1, C6 = np.zeros((5, 0), np.float32), np.zeros((0, 6), np.float32), uni(6)
    assert_bit_exact(hip_gemm(ctx, Z0, Z1, C6), ref.gemm(Z0, Z1, C6), "k=0")
    e = H.gemm(ctx, ctx.move_tensor(np.zeros((0, 8), np.float32)), ctx.move_tensor(uni(8, 4)))
    assert e.dims == [0, 4] and e.get_data().shape == (0, 4)
    with pytest.raises(H.OperatorError):
        H.gemm(ctx, ctx.move_tensor(uni(3, 4)), ctx.move_tensor(uni(5, 6)))
    with pytest.raises(H.OperatorError):
        H.gemm(ctx, ctx.move_tensor(uni(3, 4)), ctx.move_tensor(uni(4, 6)), ctx.move_tensor(uni(5)))


def test_gemm_4096_sampled_rows_and_linearity(ctx):
    """The north-star size.  The oracle checks 48 sampled rows; linearity in A covers the rest:
    (A1 + A2) B == A1 B + A2 B within fp32 accumulation error."""
    n = 4096
    A, B, C = uni(n, n), uni(n, n), uni(n)
    tb, tc = ctx.move_tensor(B), ctx.move_tensor(C)
    got = H.gemm(ctx, ctx.move_tensor(A), tb, tc).get_data()
    rows = RNG.choice(n, 48, replace=False)
    assert_close_max(got[rows], ref.gemm(A[rows], B, C), GEMM_TOL, "NS-4096 rows")
    A2 = uni(n, n)
    got2 = H.gemm(ctx, ctx.move_tensor(A2), tb, None).get_data()
    both = H.gemm(ctx, ctx.move_tensor(A + A2), tb, tc).get_data()
    assert_close_max(both, got + got2, GEMM_TOL, "linearity")


# ------------------------------------------------------------------ MatMul
@pytest.mark.parametrize("sa,sb", [((3, 4), (4, 5)), ((2, 3, 4), (4, 5)), ((1, 3, 128), (4, 128, 1)),
                                   ((4, 3, 6), (4, 6, 2)), ((6,), (6, 3)), ((2, 3, 6), (6,)), ((6,), (6,)),
                                   ((8, 850, 32), (8, 32, 850)), ((8, 850, 850), (8, 850, 32)),
                                   ((850, 1, 256), (256, 2048)), ((850, 1, 2048), (2048, 256)),
                                   ((8, 100, 32), (8, 32, 850)), ((1, 77, 33), (5, 33, 9))])
def test_matmul_shapes(ctx, sa, sb):
    A, B = nrm(*sa), nrm(*sb)
    got = H.matmul(ctx, ctx.move_tensor(A), ctx.move_tensor(B))
    want = ref.matmul(A, B)
    assert tuple(got.dims) == want.shape
    assert_close_max(got.get_data(), want, GEMM_TOL, "matmul %s x %s" % (sa, sb))


def test_matmul_rejects_what_the_reference_rejects(ctx):
    with pytest.raises(H.OperatorError):
        H.matmul(ctx, ctx.move_tensor(nrm(2, 2, 3, 4)), ctx.move_tensor(nrm(4, 5)))
    with pytest.raises(H.OperatorError):
        H.matmul(ctx, ctx.move_tensor(nrm(3, 4)), ctx.move_tensor(nrm(5, 6)))


def test_ffn_chain_config2(ctx):
    """benchmark config 2: X[8,512,768] -> MatMul W1 -> Add b1 -> Relu -> MatMul W2 -> Add X.
    Full size on the GPU; the oracle follows 64 sampled token rows (the chain is row-wise)."""
    X, W1, b1, W2 = nrm(8, 512, 768), nrm(768, 3072, std=0.02), np.zeros(3072, np.float32), nrm(3072, 768, std=0.02)
    tX, tW1, tb1, tW2 = (ctx.move_tensor(t) for t in (X, W1, b1, W2))
    h = H.matmul(ctx, tX, tW1)
    hb = H.binary(ctx, "Add", h, tb1)
    hr = H.unary(ctx, "Relu", hb)
    y = H.matmul(ctx, hr, tW2)
    out = H.binary(ctx, "Add", y, tX).get_data()
    rows = np.sort(RNG.choice(8 * 512, 64, replace=False))
    xs = X.reshape(-1, 768)[rows]
    o_h = ref.matmul(xs, W1)
    o_hr = ref.unary("Relu", ref.binary("Add", o_h, b1))
    o_out = ref.binary("Add", ref.matmul(o_hr, W2), xs)
    assert_close_max(h.get_data().reshape(-1, 3072)[rows], o_h, GEMM_TOL, "MatMul 1")
    assert_close_max(out.reshape(-1, 768)[rows], o_out, GEMM_TOL, "FFN output")
    # the fused forms compute the same chain
    hf = H.matmul(ctx, tX, tW1, bias=tb1, epilogue="relu")
    assert_bit_exact(hf.get_data(), hr.get_data(), "fused MatMul+Add+Relu")
    of = H.matmul(ctx, hf, tW2, residual=tX)
    assert_bit_exact(of.get_data(), out, "fused MatMul+Add(residual)")


# ------------------------------------------------------------------ Conv
def hip_conv(ctx, X, W, B=None, dil=None, group=1, pads=None, strides=None, epilogue=None, R=None):
    return H.conv(ctx, ctx.move_tensor(X), ctx.move_tensor(W), ctx.move_tensor(B) if B is not None else None,
                  dil, group, None, pads, strides, epilogue, ctx.move_tensor(R) if R is not None else None).get_data()


def he(cout, cin, k):
    return nrm(cout, cin, k, k, std=float(np.sqrt(2.0 / (cin * k * k))))


def test_conv_config3_full(ctx):
    """benchmark config 3: X[32,64,56,56] U[0,1], W[64,64,3,3] He-normal, bias zeros, pad 1, then Relu."""
    X, W, B = uni(32, 64, 56, 56, lo=0), he(64, 64, 3), np.zeros(64, np.float32)
    want = ref.conv(X, W, B, pads=[1, 1, 1, 1])
    got = hip_conv(ctx, X, W, B, pads=[1, 1, 1, 1])
    assert_close_max(got, want, GEMM_TOL, "C3 conv")
    fused = hip_conv(ctx, X, W, B, pads=[1, 1, 1, 1], epilogue="relu")
    assert_bit_exact(fused, np.maximum(got, 0) + 0.0, "C3 fused Relu")
    assert_close_max(fused, ref.unary("Relu", want), GEMM_TOL, "C3 conv+relu")


CONV_SHAPES = [
    # n, cin, h, w, cout, k, pads, strides, dil, group  — ResNet-50 layer forms and the reference's
    # conv1..conv11 attribute mix (test/model_test/make_models.py:623-643)
    (2, 3, 224, 224, 64, 7, [3, 3, 3, 3], [2, 2], [1, 1], 1),     # stem
    (2, 64, 56, 56, 256, 1, [0, 0, 0, 0], [1, 1], [1, 1], 1),
    (2, 256, 56, 56, 128, 1, [0, 0, 0, 0], [2, 2], [1, 1], 1),    # strided 1x1 (v1 bottleneck)
    (2, 256, 56, 56, 512, 1, [0, 0, 0, 0], [2, 2], [1, 1], 1),    # downsample branch
    (2, 128, 28, 28, 128, 3, [1, 1, 1, 1], [1, 1], [1, 1], 1),
    (2, 256, 14, 14, 256, 3, [1, 1, 1, 1], [1, 1], [1, 1], 1),
    (3, 512, 7, 7, 512, 3, [1, 1, 1, 1], [1, 1], [1, 1], 1),
    (3, 512, 7, 7, 2048, 1, [0, 0, 0, 0], [1, 1], [1, 1], 1),
    (2, 128, 57, 57, 128, 3, [1, 1, 1, 1], [2, 2], [1, 1], 1),    # odd size, stride 2
    (2, 8, 14, 15, 12, 3, [1, 0, 2, 1], [2, 1], [1, 1], 2),       # groups, asymmetric pads
    (1, 6, 20, 20, 6, 3, [2, 2, 2, 2], [1, 1], [2, 2], 1),        # dilation 2
    (2, 16, 9, 9, 16, 3, [1, 1, 1, 1], [1, 1], [1, 1], 16),       # depthwise
    (1, 5, 6, 7, 3, 2, [0, 0, 0, 0], [1, 1], [1, 1], 1),          # even kernel, no pad
    (1, 2048, 25, 34, 256, 1, [0, 0, 0, 0], [1, 1], [1, 1], 1),   # DETR input projection
    # 1x1 stride 1 with whole tiles: X is read in place as the B matrix
    (16, 32, 14, 14, 80, 1, [0, 0, 0, 0], [1, 1], [1, 1], 1),     # 64-pixel tiles straddle images (196 each)
    (4, 64, 8, 8, 48, 1, [0, 0, 0, 0], [1, 1], [1, 1], 2),        # groups
    (16, 1024, 14, 14, 256, 1, [0, 0, 0, 0], [1, 1], [1, 1], 1),  # deep K: tiles cut along K, reduce pass
    (2, 256, 56, 56, 64, 1, [0, 0, 0, 0], [1, 1], [1, 1], 1),
    (2, 48, 12, 12, 24, 1, [0, 0, 0, 0], [1, 1], [1, 1], 1),      # 288 pixels: not whole tiles, gathers instead
]


@pytest.mark.parametrize("shape", CONV_SHAPES)
def test_conv_shapes(ctx, shape):
    n, cin, h, w, cout, k, pads, strides, dil, group = shape
    X, W, B = uni(n, cin, h, w, lo=0), he(cout, cin // group, k), nrm(cout)
    want = ref.conv(X, W, B, dil, group, None, pads, strides)
    got = hip_conv(ctx, X, W, B, dil, group, pads, strides)
    assert got.shape == want.shape
    assert_close_max(got, want, GEMM_TOL, "conv %s" % (shape,))


def test_conv_residual_epilogue_and_no_bias(ctx):
    X, W = uni(2, 32, 14, 14, lo=0), he(48, 32, 3)
    R = nrm(2, 48, 14, 14)
    plain = hip_conv(ctx, X, W, pads=[1, 1, 1, 1])
    assert_close_max(plain, ref.conv(X, W, pads=[1, 1, 1, 1]), GEMM_TOL, "no bias")
    fused = hip_conv(ctx, X, W, pads=[1, 1, 1, 1], epilogue="relu", R=R)
    assert_bit_exact(fused, np.maximum(plain + R, 0) + 0.0, "conv + residual + relu")
    with pytest.raises(H.OperatorError):
        H.conv(ctx, ctx.move_tensor(uni(2, 3, 8)), ctx.move_tensor(uni(4, 3, 3, 3)))


def test_conv_1x1_equals_gemm(ctx):
    X, W = uni(2, 40, 6, 5), uni(24, 40, 1, 1)
    got = hip_conv(ctx, X, W)
    for b in range(2):
        g = hip_gemm(ctx, W.reshape(24, 40), X[b].reshape(40, 30))
        assert_close_max(got[b].reshape(24, 30), g, 1e-6, "1x1 == gemm")
    # whole tiles (256 pixels, 32 channels): the in-place path, with residual and Relu fused
    X, W, R = uni(4, 32, 8, 8), uni(24, 32, 1, 1), nrm(4, 24, 8, 8)
    got = hip_conv(ctx, X, W)
    for b in range(4):
        g = hip_gemm(ctx, W.reshape(24, 32), X[b].reshape(32, 64))
        assert_close_max(got[b].reshape(24, 64), g, 1e-6, "1x1 == gemm, in place")
    fused = hip_conv(ctx, X, W, epilogue="relu", R=R)
    assert_bit_exact(fused, np.maximum(got + R, 0) + 0.0, "1x1 conv + residual + relu")


# ------------------------------------------------------------------ elementwise
@pytest.mark.parametrize("op", ["Add", "Sub", "Mul", "Div"])
@pytest.mark.parametrize("sl,sr", [((2, 3, 10, 12), ()), ((2, 3, 10, 12), (1, 3, 1, 12)), ((), ()),
                                   ((2, 3, 10, 12), (2, 3, 10, 12)), ((4, 1), (3,)), ((8, 512, 3072), (3072,)),
                                   ((2, 1, 3, 1, 2, 1), (1, 2, 1, 2, 1, 3)), ((5, 7), (5, 1)), ((1, 3, 1, 12), (2, 3, 10, 12)),
                                   ((3, 1031), (3, 1031)), ((2, 64, 7, 7), (1, 64, 1, 1)), ((850, 1, 256), (850, 1, 1)),
                                   ((3, 5000), (3, 1)), ((2, 5, 4101), (5, 1)), ((4, 16, 28, 28), (16, 1, 1)),
                                   ((16, 1, 1), (4, 16, 28, 28)), ((7, 300), (300,)), ((4100,), (1,)),
                                   # rows that fill power-of-two tiles badly: the flat walk, 16-byte and 4-byte units
                                   ((3, 64, 56, 56), (64, 1, 1)), ((64, 1, 1), (3, 64, 56, 56)), ((2, 3, 37, 50), (3, 1, 50)),
                                   ((2, 2, 3, 70, 50), (2, 1, 70, 1)), ((300, 50), (50,)), ((2, 40, 2500), (1, 40, 1))])
def test_binary_bit_exact(ctx, op, sl, sr):
    L, R = uni(*sl, lo=-3, hi=3), uni(*sr, lo=-3, hi=3)
    got = H.binary(ctx, op, ctx.move_tensor(L), ctx.move_tensor(R))
    want = ref.binary(op, L, R)
    assert tuple(got.dims) == want.shape
    assert_bit_exact(got.get_data(), want, "%s %s %s" % (op, sl, sr))


def test_binary_special_values_int32_pow_and_errors(ctx):
    L = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, 3.4e38, 1.0, 1e-39, -1e-39, 2e-38], np.float32)
    R = np.array([-0.0, 0.0, -np.inf, 1.0, 1.0, 0.5, 3.4e38, 0.0, 1e-39, 3.0, 0.25], np.float32)
    for op in ("Add", "Sub", "Mul", "Div"):
        got = H.binary(ctx, op, ctx.move_tensor(L), ctx.move_tensor(R)).get_data()
        assert_bit_exact(got, ref.binary(op, L, R), op + " specials (incl. denormals)")
    a = np.array([2147483647, -2147483648, 7, -7, 100000, 5, 0], np.int32)
    b = np.array([1, -1, 2, 2, 100000, 0, 0], np.int32)
    for op in ("Add", "Sub", "Mul", "Div"):
        got = H.binary(ctx, op, ctx.move_tensor(a), ctx.move_tensor(b)).get_data()
        assert_bit_exact(got, ref.binary(op, a, b), op + " int32")
    ia = RNG.integers(-2 ** 31, 2 ** 31 - 1, (3, 37, 50)).astype(np.int32)    # int32 through the flat walk
    ib = RNG.integers(-50000, 50000, (37, 1)).astype(np.int32)
    for op in ("Add", "Mul"):
        got = H.binary(ctx, op, ctx.move_tensor(ia), ctx.move_tensor(ib)).get_data()
        assert_bit_exact(got, ref.binary(op, ia, ib), op + " int32, broadcast rows")
    base, ex = uni(4, 50, lo=0.1, hi=4), uni(50, lo=-3, hi=3)
    got = H.binary(ctx, "Pow", ctx.move_tensor(base), ctx.move_tensor(ex)).get_data()
    assert_close_max(got, ref.binary("Pow", base, ex), 1e-6, "Pow")
    with pytest.raises(H.OperatorError):
        H.binary(ctx, "Add", ctx.move_tensor(uni(2, 3)), ctx.move_tensor(uni(4)))
    with pytest.raises(H.OperatorError):
        H.binary(ctx, "Add", ctx.move_tensor(uni(2)), ctx.move_tensor(np.zeros(2, np.int32)))


def test_unary(ctx):
    x = np.array([-2, -0.5, 0, 1, 3, np.nan, -0.0, -np.inf, np.inf, 1e-40, -1e-40], np.float32)
    assert_bit_exact(H.unary(ctx, "Relu", ctx.move_tensor(x)).get_data(), ref.unary("Relu", x), "Relu specials")
    big = nrm(8, 512, 3073)
    assert_bit_exact(H.unary(ctx, "Relu", ctx.move_tensor(big)).get_data(), ref.unary("Relu", big), "Relu big")
    xi = np.array([-3, 0, 4, -2147483648], np.int32)
    assert_bit_exact(H.unary(ctx, "Relu", ctx.move_tensor(xi)).get_data(), ref.unary("Relu", xi), "Relu int32")
    v = uni(1, 100, 4, lo=-20, hi=20)
    for op, tol in (("Sigmoid", 1e-6), ("Exp", 1e-6), ("Tanh", 1e-6), ("Reciprocal", 1e-7)):
        assert_close_max(H.unary(ctx, op, ctx.move_tensor(v)).get_data(), ref.unary(op, v), tol, op)
    p = uni(1000, lo=0, hi=50)
    assert_bit_exact(H.unary(ctx, "Sqrt", ctx.move_tensor(p)).get_data(), ref.unary("Sqrt", p), "Sqrt")
    for op in ("Abs", "Neg"):
        assert_bit_exact(H.unary(ctx, op, ctx.move_tensor(v)).get_data(), ref.unary(op, v), op)
    with pytest.raises(H.OperatorError):
        H.unary(ctx, "Sigmoid", ctx.move_tensor(xi))


# ------------------------------------------------------------------ row reductions
@pytest.mark.parametrize("shape", [(8, 850, 850), (8, 100, 850), (8, 100, 100), (3, 4, 5, 6), (7, 1), (5, 64), (3, 129),
                                   (4, 1025), (2, 2049), (3, 5000), (1, 1), (5, 256), (3, 1024), (2, 2048), (4, 852), (9, 132),
                                   (9001, 100), (8195, 260), (8193, 513), (8200, 1024)])   # more rows than resident wavefronts
def test_softmax(ctx, shape):
    x = nrm(*shape, std=3.0)
    got = H.softmax(ctx, ctx.move_tensor(x)).get_data()
    assert_close_max(got, ref.softmax(x), 1e-6, "softmax %s" % (shape,))
    assert np.abs(got.astype(np.float64).sum(-1) - 1).max() < 1e-5


def test_softmax_edges(ctx):
    x = np.array([[0, 1000, 0], [-np.inf, 0, -np.inf], [5, 5, 5]], np.float32)
    assert_bit_exact(H.softmax(ctx, ctx.move_tensor(x)).get_data(), ref.softmax(x), "one-hot / uniform")
    with pytest.raises(H.OperatorError):
        H.softmax(ctx, ctx.move_tensor(nrm(2, 3, 4)), axis=1)


@pytest.mark.parametrize("shape", [(850, 1, 256), (100, 1, 256), (6, 2048), (3, 5000), (4, 7), (2, 3, 1), (9, 1000),
                                   (5, 250), (7, 1024), (3, 132), (17, 64), (1, 4), (13, 200), (8191, 256), (66, 8),
                                   (27200, 256), (8195, 250), (8193, 1000), (8194, 1028)])       # more rows than resident wavefronts
def test_layernorm(ctx, shape):
    x, g, b = nrm(*shape, std=2.0), nrm(shape[-1]), nrm(shape[-1])
    got = H.layer_normalization(ctx, ctx.move_tensor(x), ctx.move_tensor(g), ctx.move_tensor(b)).get_data()
    assert_close_max(got, ref.layernorm_decomposed(x, g, b, 1e-5), 1e-5, "layernorm %s" % (shape,))
    plain = H.layer_normalization(ctx, ctx.move_tensor(x)).get_data()
    assert_close_max(plain, ref.layernorm_decomposed(x, None, None, 1e-5), 1e-5, "layernorm no affine")


@pytest.mark.parametrize("shape", [(32, 2048, 7, 7), (4, 16, 56, 56), (1, 3, 1, 1), (2, 5, 3, 300), (3, 1400, 5, 5),
                                   (70, 64, 8, 8), (5, 1000, 1, 2)])
def test_global_average_pool_and_reduce_mean(ctx, shape):
    x = nrm(*shape)
    got = H.global_average_pool(ctx, ctx.move_tensor(x))
    want = ref.global_average_pool(x)
    assert tuple(got.dims) == want.shape
    # double sums in another order may differ in the last double bit -> at most 1 fp32 ulp
    from util import ulp_diff
    assert ulp_diff(got.get_data(), want).max() <= 1
    flat = x.reshape(-1, shape[2] * shape[3])
    rm = H.reduce_mean_last(ctx, ctx.move_tensor(flat)).get_data()
    assert ulp_diff(rm, ref.reduce_mean_last(flat)).max() <= 1


@pytest.mark.parametrize("shape,axes,keep", [
    ((6, 7, 8), [0], 1), ((6, 7, 8), [1], 0), ((6, 7, 8), [2], 1), ((6, 7, 8), [0, 2], 0), ((6, 7, 8), [], 1),
    ((3, 4, 5, 6), [1, 2], 1), ((3, 4, 5, 6), [-1, 0], 0), ((2, 850, 256), [1], 1), ((32, 64, 56, 56), [0], 0),
    ((4, 2048, 7, 7), [2, 3], 1), ((1, 100, 1, 256), [3, 1], 0), ((5,), [0], 0), ((300, 1000), [0], 1)])
def test_reduce_mean_over_any_axes(ctx, shape, axes, keep):
    """reduce.ts:40-131, 369-405: one pass per axis.  A pass over an inner axis adds in the
    reference's order (bit-exact); a pass over the last axis adds across a wavefront, which may
    cost the last bit of the double sum, at most 1 fp32 ulp per such pass."""
    from util import ulp_diff

    x = nrm(*shape)
    got = H.reduce_mean(ctx, ctx.move_tensor(x), axes, keep)
    want = ref.reduce_mean(x, axes, keep)
    assert tuple(got.dims) == want.shape
    ax = sorted(a % len(shape) for a in axes) if axes else list(range(len(shape)))
    if ax[-1] != len(shape) - 1:
        assert_bit_exact(got.get_data(), want, "ReduceMean %s over %s" % (shape, axes))
    else:
        assert ulp_diff(got.get_data(), want).max() <= 1
    with pytest.raises(H.OperatorError):
        H.reduce_mean(ctx, ctx.move_tensor(x), [len(shape)], keep)


# ------------------------------------------------------------------ MaxPool
def test_maxpool_resnet_stem_full(ctx):
    x = nrm(32, 64, 112, 112)
    got = H.maxpool(ctx, ctx.move_tensor(x), [3, 3], pads=[1, 1, 1, 1], strides=[2, 2]).get_data()
    assert_bit_exact(got, ref.maxpool(x, [3, 3], pads=[1, 1, 1, 1], strides=[2, 2]), "stem maxpool")


@pytest.mark.parametrize("attrs", [
    dict(kernel_shape=[3, 3], strides=[2, 2]),
    dict(kernel_shape=[3, 3], strides=[2, 2], ceil_mode=1),
    dict(kernel_shape=[3, 3], strides=[2, 3], auto_pad="SAME_UPPER"),
    dict(kernel_shape=[3, 3], strides=[2, 3], auto_pad="SAME_LOWER"),
    dict(kernel_shape=[3, 3], strides=[2, 3], auto_pad="VALID"),
    dict(kernel_shape=[2, 2], strides=[2, 2], dilations=[2, 2], pads=[1, 1, 1, 1]),
    dict(kernel_shape=[2, 2], strides=[3, 3], pads=[1, 1, 1, 1], ceil_mode=1),
    dict(kernel_shape=[1, 1]),
    dict(kernel_shape=[5, 5], strides=[2, 2], pads=[2, 2, 2, 2]),
    dict(kernel_shape=[3, 2], strides=[1, 2], pads=[1, 0, 1, 1]),
    dict(kernel_shape=[3, 3], strides=[4, 4], pads=[1, 1, 1, 1]),
])
def test_maxpool_attributes(ctx, attrs):
    # small planes take the thread-per-cell kernel, the larger ones the LDS band kernel
    # (with and without 16-byte loads)
    for shape in ((2, 3, 10, 13), (2, 3, 40, 46), (1, 2, 36, 48), (1, 1, 70, 130)):
        x = nrm(*shape)
        x[0, 0, 0, 0] = np.nan
        x[0, 0, 5, 7] = np.nan
        x[0, 0, -1, -1] = -np.inf
        got = H.maxpool(ctx, ctx.move_tensor(x), **attrs)
        want = ref.maxpool(x, **attrs)
        assert tuple(got.dims) == want.shape
        assert_bit_exact(got.get_data(), want, "maxpool %s on %s" % (attrs, shape))


@pytest.mark.parametrize("pads", [[1, 1, 1, 1], [1, 1, 0, 0], [1, 1, 0, 1], [1, 1, 1, 0]])
@pytest.mark.parametrize("shape", [(2, 3, 8, 8), (1, 2, 7, 12), (3, 1, 33, 64), (1, 1, 400, 544), (2, 2, 5, 4)])
def test_maxpool_3x3_stride2_pairs(ctx, shape, pads):
    """The stem's pooling geometry on rows that are a multiple of four wide takes a kernel of its own
    (two cells per thread); other pads of the same window fall back to the general kernels.  Even and
    odd heights, NaN and -inf cells, a plane of NaN only."""
    x = nrm(*shape)
    x[0, 0, 0, 0] = np.nan
    x[0, 0, 3, 2] = np.nan
    x[0, 0, -1, -1] = -np.inf
    x[-1, -1, :2, :4] = np.nan
    for ceil_mode in (0, 1):
        got = H.maxpool(ctx, ctx.move_tensor(x), [3, 3], pads=pads, strides=[2, 2], ceil_mode=ceil_mode)
        want = ref.maxpool(x, [3, 3], pads=pads, strides=[2, 2], ceil_mode=ceil_mode)
        assert tuple(got.dims) == want.shape
        assert_bit_exact(got.get_data(), want, "maxpool 3x3/2 pads %s ceil %d on %s" % (pads, ceil_mode, shape))


def test_maxpool_errors(ctx):
    t = ctx.move_tensor(nrm(1, 1, 6, 6))
    with pytest.raises(H.OperatorError):
        H.maxpool(ctx, t, [3, 3], n_outputs=2)
    with pytest.raises(H.OperatorError):
        H.maxpool(ctx, t, [3, 3], storage_order=1)
    with pytest.raises(H.OperatorError):
        H.maxpool(ctx, t, [3, 3], auto_pad="SAME")
    with pytest.raises(H.OperatorError):
        H.maxpool(ctx, ctx.move_tensor(nrm(2, 6, 6)), [3, 3])


# ------------------------------------------------------------------ layout
@pytest.mark.parametrize("ndim", [1, 2, 3, 4])
def test_transpose_all_permutations(ctx, ndim):
    shape = (19, 70, 3, 33)[:ndim]
    x = nrm(*shape)
    t = ctx.move_tensor(x)
    for perm in itertools.permutations(range(ndim)):
        got = H.transpose(ctx, t, list(perm)).get_data()
        assert_bit_exact(got, ref.transpose(x, list(perm)), "perm %s" % (perm,))
    assert_bit_exact(H.transpose(ctx, t).get_data(), ref.transpose(x), "default perm")


@pytest.mark.parametrize("shape,perm", [((1, 256, 850), (2, 0, 1)), ((850, 8, 32), (1, 0, 2)), ((8, 850, 32), (0, 2, 1)),
                                         ((8, 850, 32), (1, 0, 2)), ((2, 3, 2, 2, 3), (4, 0, 3, 1, 2)),
                                         ((2, 3, 2, 2, 3, 2), (5, 3, 0, 4, 1, 2)), ((64, 64, 3, 3), (2, 3, 1, 0)),
                                         ((1000, 2048), (1, 0)), ((3, 1, 5), (2, 1, 0)), ((4, 300, 16), (0, 2, 1)),
                                         ((2, 40, 3000), (1, 0, 2)), ((5, 6, 7, 4100), (2, 0, 1, 3)),
                                         # the tiled exchange with 16-byte reads / 8-byte writes: odd and even row
                                         # lengths of the result, every tile width, rows that start off 8-byte boundaries
                                         ((2, 850, 8, 32), (0, 2, 3, 1)), ((3, 851, 16), (0, 2, 1)), ((2, 77, 32), (2, 0, 1)),
                                         ((1, 333, 260), (0, 2, 1)), ((3, 1001, 20), (0, 2, 1)), ((3, 64, 64), (0, 2, 1))])
def test_transpose_model_shapes(ctx, shape, perm):
    x = nrm(*shape)
    got = H.transpose(ctx, ctx.move_tensor(x), list(perm)).get_data()
    assert_bit_exact(got, ref.transpose(x, list(perm)), "%s %s" % (shape, perm))
    xi = RNG.integers(-2 ** 31, 2 ** 31 - 1, shape).astype(np.int32)
    assert_bit_exact(H.transpose(ctx, ctx.move_tensor(xi), list(perm)).get_data(), ref.transpose(xi, list(perm)), "int32")


def test_flatten_reshape_alias_and_gather(ctx):
    x = nrm(2, 3, 4, 5)
    t = ctx.move_tensor(x)
    f = H.flatten(ctx, t)
    assert f.dims == [2, 60] and f.handle == t.handle            # shares the buffer (cpu flatten.ts:11-20)
    assert_bit_exact(f.get_data(), ref.flatten(x), "flatten")
    r = H.reshape(ctx, t, [0, -1, 5])
    assert_bit_exact(r.get_data(), ref.reshape(x, [0, -1, 5]), "reshape")
    t.dispose()                                                   # aliases keep the buffer alive
    assert_bit_exact(r.get_data(), ref.reshape(x, [0, -1, 5]), "alias outlives source")
    f.dispose()
    r.dispose()
    with pytest.raises(H.OperatorError):
        H.flatten(ctx, ctx.move_tensor(x), axis=2)
    data = np.array([5, 6, 7], np.int32)
    got = H.gather(ctx, ctx.move_tensor(data), ctx.move_tensor(np.array(2, np.int32)))
    assert got.dims == [] and got.get_data().tolist() == ref.gather(data, np.array(2, np.int32)).tolist()
    table = nrm(10, 4, 6)
    idx = np.array([[3, -1], [0, 9]], np.int32)
    got = H.gather(ctx, ctx.move_tensor(table), ctx.move_tensor(idx), axis=0).get_data()
    assert_bit_exact(got, table[idx], "gather axis 0")
    got = H.gather(ctx, ctx.move_tensor(table), ctx.move_tensor(np.array([2, 0, -2], np.int32)), axis=1).get_data()
    assert_bit_exact(got, np.take(table, [2, 0, -2], axis=1), "gather axis 1")


def test_squeeze_unsqueeze_alias(ctx):
    x = nrm(2, 1, 3, 1)
    t = ctx.move_tensor(x)
    for axes in ([], [1], [-1, 1], [3]):
        y = H.squeeze(ctx, t, axes)
        assert y.handle == t.handle                               # zero-copy (cpu squeeze.ts:12-37)
        assert_bit_exact(y.get_data(), ref.squeeze(x, axes), "squeeze %s" % axes)
    with pytest.raises(H.OperatorError):
        H.squeeze(ctx, t, [0])
    for axes in ([0], [1, -1], [0, 5]):
        y = H.unsqueeze(ctx, t, axes)
        assert y.handle == t.handle
        assert_bit_exact(y.get_data(), ref.unsqueeze(x, axes), "unsqueeze %s" % axes)


@pytest.mark.parametrize("axis", [-4, -1, 0, 1, 2, 3])
def test_concat(ctx, axis):
    shape = [3, 5, 4, 6]
    ax = axis % 4
    parts = []
    for n in (1, 7, 0, 2):
        sh = list(shape)
        sh[ax] = n
        parts.append(nrm(*sh))
    got = H.concat(ctx, [ctx.move_tensor(p) for p in parts], axis).get_data()
    assert_bit_exact(got, ref.concat(parts, axis), "concat axis %d" % axis)


def test_concat_model_shapes_ints_and_errors(ctx):
    # DETR-style: positional halves [1,128,25,34] x2 on axis 1; shape pieces (int32) on axis 0
    a, b = nrm(1, 128, 25, 34), nrm(1, 128, 25, 34)
    assert_bit_exact(H.concat(ctx, [ctx.move_tensor(a), ctx.move_tensor(b)], 1).get_data(), ref.concat([a, b], 1))
    big = [nrm(850, 8, 32) for _ in range(3)]
    assert_bit_exact(H.concat(ctx, [ctx.move_tensor(t) for t in big], -1).get_data(), ref.concat(big, -1))
    ints = [np.array([1, 2], np.int32), np.array([3], np.int32)]
    got = H.concat(ctx, [ctx.move_tensor(t) for t in ints], 0).get_data()
    assert_bit_exact(got, ref.concat(ints, 0))
    with pytest.raises(H.OperatorError):
        H.concat(ctx, [ctx.move_tensor(a)], 4)
    with pytest.raises(H.OperatorError):
        H.concat(ctx, [ctx.move_tensor(a), ctx.move_tensor(nrm(1, 128, 25, 33))], 1)


@pytest.mark.parametrize("axis,n,parts", [(0, 2, ()), (1, 3, ()), (2, 5, ()), (-1, 1, ()), (1, 3, (1, 2, 3)),
                                           (1, 4, ()), (2, 3, (0, 4, 1))])
def test_split(ctx, axis, n, parts):
    x = nrm(4, 6, 5)
    got = H.split(ctx, ctx.move_tensor(x), n, axis, parts)
    want = ref.split(x, n, axis, parts)
    assert len(got) == len(want)
    for g, w in zip(got, want):
        assert_bit_exact(g.get_data(), w, "split axis %d" % axis)


def test_split_qkv_and_errors(ctx):
    x = nrm(850, 768)                                             # packed q,k,v projections
    got = H.split(ctx, ctx.move_tensor(x), 3, 1)
    for g, w in zip(got, ref.split(x, 3, 1)):
        assert_bit_exact(g.get_data(), w)
    with pytest.raises(H.OperatorError):
        H.split(ctx, ctx.move_tensor(x), 2, 2)
    with pytest.raises(H.OperatorError):
        H.split(ctx, ctx.move_tensor(x), 2, 1, (500, 500))


@pytest.mark.parametrize("args", [
    dict(starts=[1, 2], ends=[4, 6], axes=[0, 2]),
    dict(starts=[0, 0, 0], ends=[5, 6, 7]),
    dict(starts=[1], ends=[-1], axes=[-1], steps=[2]),
    dict(starts=[-3], ends=[1000], axes=[1]),
    dict(starts=[-1], ends=[-1000], axes=[2], steps=[-1]),
    dict(starts=[5, 4], ends=[0, -100], axes=[1, 0], steps=[-2, -3]),
    dict(starts=[3], ends=[2], axes=[0]),
    dict(starts=[5], ends=[5], axes=[0]),                        # reference quirk: start clamps to size-1
    dict(starts=[9], ends=[100], axes=[1]),
])
def test_slice(ctx, args):
    x = nrm(5, 6, 7)
    got = H.slice_(ctx, ctx.move_tensor(x), **args).get_data()
    assert_bit_exact(got, ref.slice_(x, **args), "slice %s" % args)


def test_slice_ranks_ints_and_errors(ctx):
    x6 = nrm(2, 3, 2, 3, 2, 5)
    args = dict(starts=[1, 0, 1], ends=[3, 2, 5], axes=[1, 3, 5], steps=[1, 1, 2])
    assert_bit_exact(H.slice_(ctx, ctx.move_tensor(x6), **args).get_data(), ref.slice_(x6, **args))
    v = np.arange(10, dtype=np.int32)
    assert_bit_exact(H.slice_(ctx, ctx.move_tensor(v), [2], [9], [0], [3]).get_data(), ref.slice_(v, [2], [9], [0], [3]))
    big = nrm(32, 256, 56, 56)                                     # crop of a feature map, 100 MB in
    args = dict(starts=[4, 3], ends=[52, 53], axes=[2, 3])
    assert_bit_exact(H.slice_(ctx, ctx.move_tensor(big), **args).get_data(), ref.slice_(big, **args))
    rows = nrm(2, 3, 200, 300)                                     # short odd rows gathered into a dense plane
    tr = ctx.move_tensor(rows)
    for args in (dict(starts=[5, 1], ends=[190, 52], axes=[2, 3]),                 # plane of 9435: several workgroups
                 dict(starts=[199, 3], ends=[-500, 10], axes=[2, 3], steps=[-1, 1]),  # rows taken backwards
                 dict(starts=[0, 250], ends=[200, 299], axes=[2, 3], steps=[3, 1]),   # every third row
                 dict(starts=[1, 0, 17], ends=[3, 37, 50], axes=[1, 2, 3])):
        assert_bit_exact(H.slice_(ctx, tr, **args).get_data(), ref.slice_(rows, **args), "slice %s" % args)
    r5 = nrm(2, 3, 2, 40, 45)
    args = dict(starts=[1, 2, 1], ends=[3, 40, 44], axes=[1, 3, 4])
    assert_bit_exact(H.slice_(ctx, ctx.move_tensor(r5), **args).get_data(), ref.slice_(r5, **args))
    wide = nrm(6, 8, 4400)                                         # long rows: 16-byte pieces where alignment allows
    tw = ctx.move_tensor(wide)
    for args in (dict(starts=[7], ends=[-100], axes=[1], steps=[-1]), dict(starts=[4], ends=[4300], axes=[2]),
                 dict(starts=[1], ends=[4399], axes=[2]), dict(starts=[5, 8], ends=[0, 4104], axes=[0, 2], steps=[-2, 1]),
                 dict(starts=[4399], ends=[-5000], axes=[2], steps=[-1])):
        assert_bit_exact(H.slice_(ctx, tw, **args).get_data(), ref.slice_(wide, **args), "slice %s" % args)
    with pytest.raises(H.OperatorError):
        H.slice_(ctx, ctx.move_tensor(nrm(*([1] * 7))), [0], [1])
    with pytest.raises(H.OperatorError):
        H.slice_(ctx, ctx.move_tensor(v), [0], [1], [0], [0])


def test_cast(ctx):
    v = np.array([0.0, -0.0, 1.9, -1.9, 2147483648.0, -2147483648.0, 4294967296.0, 3e9, -3e9, 1e20,
                  np.nan, np.inf, -np.inf, 123456.7], np.float32)
    for to in (6, 7, 2):
        assert_bit_exact(H.cast(ctx, ctx.move_tensor(v), to).get_data(), ref.cast(v, to), "f32 -> int32")
    assert_bit_exact(H.cast(ctx, ctx.move_tensor(v), 1).get_data(), ref.cast(v, 1), "f32 -> f32")
    i = np.array([3, -7, 2 ** 31 - 1, -2 ** 31, 16777217], np.int32)
    assert_bit_exact(H.cast(ctx, ctx.move_tensor(i), 1).get_data(), ref.cast(i, 1), "int32 -> f32")
    assert_bit_exact(H.cast(ctx, ctx.move_tensor(i), 7).get_data(), ref.cast(i, 7), "int32 -> int32")
    big = uni(1000, 1001, lo=-5e9, hi=5e9)
    assert_bit_exact(H.cast(ctx, ctx.move_tensor(big), 6).get_data(), ref.cast(big, 6), "f32 -> int32, 1M values")
    with pytest.raises(H.OperatorError):
        H.cast(ctx, ctx.move_tensor(v), 10)


def test_strided_copy_rejects_views_outside_the_buffers(ctx):
    t = ctx.move_tensor(nrm(4, 4))
    y = ctx.empty_tensor([4, 4], "float32")
    i32, i64 = ctypes.c_int32 * 2, ctypes.c_int64 * 2
    ok = (t.handle, 0, y.handle, 0, 2, i32(4, 4), i64(4, 1), i64(4, 1))
    capi.call("wdh_strided_copy", *ok)
    for bad in [(t.handle, 1, y.handle, 0, 2, i32(4, 4), i64(4, 1), i64(4, 1)),      # X overruns
                (t.handle, 0, y.handle, 0, 2, i32(4, 4), i64(4, 1), i64(5, 1)),      # Y overruns
                (t.handle, 0, y.handle, 0, 2, i32(4, 4), i64(-4, 1), i64(4, 1)),     # X before its start
                (t.handle, -1, y.handle, 0, 2, i32(4, 4), i64(4, 1), i64(4, 1)),
                (t.handle, 0, y.handle, 0, 7, i32(4, 4), i64(4, 1), i64(4, 1))]:
        with pytest.raises(capi.HipError) as err:
            capi.call("wdh_strided_copy", *bad)
        assert err.value.code == -2
    # reversed rows through a negative X stride
    capi.call("wdh_strided_copy", t.handle, 12, y.handle, 0, 2, i32(4, 4), i64(-4, 1), i64(4, 1))
    assert_bit_exact(y.get_data(), t.get_data()[::-1].copy())


# ------------------------------------------------------------------ runtime
def test_buffers_offsets_large_copies_and_pool(ctx):
    n = 20 * 1024 * 1024 + 13                 # 80 MiB: several staging chunks each way
    x = RNG.integers(-2 ** 31, 2 ** 31 - 1, n).astype(np.int32)
    t = ctx.move_tensor(x)
    assert_bit_exact(t.get_data(), x, "large round trip")
    part = np.empty(1000, np.int32)
    capi.call("wdh_read", t.handle, 4 * 12345, part.ctypes.data_as(ctypes.c_void_p), part.nbytes)
    assert_bit_exact(part, x[12345:13345], "offset read")
    patch = np.arange(50, dtype=np.int32)
    capi.call("wdh_write", t.handle, 4 * 777, patch.ctypes.data_as(ctypes.c_void_p), patch.nbytes)
    x[777:827] = patch
    u = ctx.empty_tensor([n], "int32")
    capi.call("wdh_copy", u.handle, 0, t.handle, 0, 4 * n)
    assert_bit_exact(u.get_data(), x, "device copy after patch")
    before = ctx.mem_stats()
    t.dispose()
    u.dispose()
    after = ctx.mem_stats()
    assert after["in_use"] < before["in_use"] and after["cached"] > before["cached"]
    v = ctx.empty_tensor([n], "int32")        # served from the pool: no new reservation
    assert ctx.mem_stats()["peak"] == after["peak"]
    v.dispose()
    z = ctx.empty_tensor([0])
    assert z.get_data().shape == (0,)
    z.dispose()


def _small_net(ctx, x, w1, b1, w2, b2, wf, bf):
    """conv+relu -> maxpool -> conv+residual+relu -> global pool -> flatten -> gemm; every tensor but the
    result is disposed on the way, as the runner does."""
    a = H.conv(ctx, x, w1, b1, pads=[1, 1, 1, 1], epilogue="relu")
    p = H.maxpool(ctx, a, kernel_shape=[3, 3], pads=[1, 1, 1, 1], strides=[2, 2])
    a.dispose()
    c = H.conv(ctx, p, w2, b2, pads=[1, 1, 1, 1], epilogue="relu", residual=p)
    p.dispose()
    g = H.global_average_pool(ctx, c)
    c.dispose()
    f = H.flatten(ctx, g)
    g.dispose()
    y = H.gemm(ctx, f, wf, bf, trans_b=1)
    f.dispose()
    return y


def test_captured_graph_replays_like_eager_runs(ctx):
    """One run recorded into a HIP graph, then replayed with new input contents; every replay is
    compared with an eager run of the same input, with eager work, syncs and pool traffic in between."""
    x_np = [uni(4, 16, 28, 28, lo=0) for _ in range(4)]
    w1, b1 = ctx.move_tensor(he(32, 16, 3)), ctx.move_tensor(nrm(32))
    w2, b2 = ctx.move_tensor(he(32, 32, 3)), ctx.move_tensor(nrm(32))
    wf, bf = ctx.move_tensor(nrm(10, 32)), ctx.move_tensor(nrm(10))
    x = ctx.move_tensor(x_np[0])
    eager = []
    for xn in x_np:                                   # also warms the pool and the conv tap tables
        x.set_data(xn)
        y = _small_net(ctx, x, w1, b1, w2, b2, wf, bf)
        eager.append(y.get_data())
        y.dispose()
    before = ctx.mem_stats()
    x.set_data(x_np[0])
    ctx.graph_begin()
    y = _small_net(ctx, x, w1, b1, w2, b2, wf, bf)    # recorded, not executed
    gid = ctx.graph_end()
    for i in (0, 1, 2, 3, 1):
        x.set_data(x_np[i])
        ctx.graph_launch(gid)
        assert_bit_exact(y.get_data(), eager[i], "replay with input %d" % i)
        # unrelated eager work between replays must neither disturb nor be disturbed
        other = H.conv(ctx, x, w1, b1, pads=[1, 1, 1, 1])
        junk = [ctx.move_tensor(nrm(64, 1024)) for _ in range(3)]
        want_other = other.get_data()
        ctx.graph_launch(gid)
        assert_bit_exact(other.get_data(), want_other, "an eager tensor survives a replay")
        assert_bit_exact(y.get_data(), eager[i], "second replay with input %d" % i)
        other.dispose()
        for j in junk:
            j.dispose()
    held = ctx.mem_stats()["in_use"]
    ctx.graph_destroy(gid)
    assert ctx.mem_stats()["in_use"] < held                        # the graph's blocks went back to the pool
    assert_bit_exact(y.get_data(), eager[1], "the output handle outlives the graph")
    y.dispose()
    assert ctx.mem_stats()["in_use"] == before["in_use"]
    with pytest.raises(capi.HipError):
        ctx.graph_launch(gid)


def test_capture_refuses_what_cannot_be_recorded(ctx):
    x = ctx.move_tensor(uni(1, 4, 9, 9))
    ctx.graph_begin()
    with pytest.raises(capi.HipError) as err:
        x.get_data()                                               # a read needs the stream drained
    assert err.value.code == -5
    with pytest.raises(capi.HipError) as err:
        ctx.graph_end()
    assert "abandoned" in str(err.value)
    # a conv geometry never run before needs its tap table built, which cannot happen while capturing
    w = ctx.move_tensor(he(5, 4, 3))
    ctx.graph_begin()
    with pytest.raises(capi.HipError) as err:
        H.conv(ctx, x, w, None, pads=[2, 2, 2, 2], dilations=[2, 2])
    assert "once before capturing" in str(err.value)
    with pytest.raises(capi.HipError):
        ctx.graph_end()
    with pytest.raises(capi.HipError):
        ctx.graph_end()                                            # no capture open any more
    # the library is usable afterwards
    y = H.conv(ctx, x, w, None, pads=[2, 2, 2, 2], dilations=[2, 2])
    assert y.get_data().shape == (1, 5, 9, 9)


def test_errors_are_reported_not_fatal(ctx):
    with pytest.raises(capi.HipError) as err:
        capi.call("wdh_free", 123456789)
    assert "unknown buffer handle" in str(err.value)
    small = ctx.empty_tensor([4])
    with pytest.raises(capi.HipError) as err:
        capi.call("wdh_unary", 0, 0, small.handle, small.handle, 1000)
    assert "needs" in str(err.value)
    with pytest.raises(capi.HipError):
        capi.call("wdh_unary", 99, 0, small.handle, small.handle, 4)
    with pytest.raises(capi.HipError):
        capi.call("wdh_gemm", small.handle, small.handle, 0, small.handle, 1, 64, 64, 64, 0, 64, 1, 0, 64, 1, 0, 0,
                  1.0, 1.0, 0, 0)
    with pytest.raises(capi.HipError):
        capi.call("wdh_conv2d", small.handle, small.handle, 0, small.handle, 1, 3, 8, 8, 4, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1,
                  2, 0, 0)     # channels not divisible by group
    # the context still works afterwards
    x = uni(4)
    small.set_data(x)
    assert_bit_exact(small.get_data(), x, "still alive")
    small.dispose()
    with pytest.raises(H.OperatorError):
        _ = small.handle
    ctx.event_record(10)
    ctx.event_record(11)
    assert ctx.event_elapsed_ms(10, 11) >= 0.0
    info = ctx.device_info()
    assert info["name"].startswith("gfx950") and info["compute_units"] > 0


# ------------------------------------------------------------------ tile shapes
@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4])
def test_every_tile_shape_computes_the_same(ctx, tile):
    """wdh_gemm / wdh_conv2d pick a workgroup tile per problem; every shape must agree."""
    A, B, C = uni(150, 70), uni(70, 300), uni(300)
    X, W, Bv = uni(2, 24, 17, 19, lo=0), he(40, 24, 3), nrm(40)
    At, Bt = uni(70, 150), uni(300, 70)
    try:
        ctx.set_option("contraction_tile", tile)
        g = hip_gemm(ctx, A, B, C)
        gt = hip_gemm(ctx, At, Bt, C, 1.0, 1.0, 1, 1)
        c = hip_conv(ctx, X, W, Bv, pads=[1, 1, 1, 1], strides=[2, 1])
    finally:
        ctx.set_option("contraction_tile", -1)
    assert_close_max(g, ref.gemm(A, B, C), GEMM_TOL, "gemm tile %d" % tile)
    assert_close_max(gt, ref.gemm(At, Bt, C, 1.0, 1.0, 1, 1), GEMM_TOL, "gemm TT tile %d" % tile)
    assert_close_max(c, ref.conv(X, W, Bv, pads=[1, 1, 1, 1], strides=[2, 1]), GEMM_TOL, "conv tile %d" % tile)
    with pytest.raises(capi.HipError):
        ctx.set_option("contraction_tile", 9)
    with pytest.raises(capi.HipError):
        ctx.set_option("no_such_option", 1)


@pytest.mark.parametrize("split", [1, 2, 5, 64])
def test_split_k_is_the_same_sum(ctx, split):
    """Split-K cuts the K loop into chunks whose sums a second kernel adds in chunk order."""
    A, B, C = uni(70, 333), uni(333, 90), uni(90)
    X, W, Bv, R = uni(2, 40, 7, 7, lo=0), he(24, 40, 3), nrm(24), nrm(2, 24, 7, 7)
    A3, B3 = nrm(3, 50, 200), nrm(3, 200, 30)
    try:
        ctx.set_option("split_k", split)
        g = hip_gemm(ctx, A, B, C, 0.5, 2.0, epilogue="relu")
        c = hip_conv(ctx, X, W, Bv, pads=[1, 1, 1, 1], epilogue="relu", R=R)
        m3 = H.matmul(ctx, ctx.move_tensor(A3), ctx.move_tensor(B3)).get_data()
        cg = hip_conv(ctx, uni(1, 8, 9, 9), he(6, 4, 3), nrm(6), group=2)
    finally:
        ctx.set_option("split_k", -1)
    assert_close_max(g, ref.unary("Relu", ref.gemm(A, B, C, 0.5, 2.0)), GEMM_TOL, "gemm split %d" % split)
    want = ref.unary("Relu", ref.binary("Add", ref.conv(X, W, Bv, pads=[1, 1, 1, 1]), R))
    assert_close_max(c, want, GEMM_TOL, "conv split %d" % split)
    assert_close_max(m3, ref.matmul(A3, B3), GEMM_TOL, "batched matmul split %d" % split)
    assert cg.shape == (1, 6, 7, 7)


def test_planned_splits_are_deterministic_and_match_forced_ones(ctx):
    """Tail tiles beyond full rounds (ResNet stage 1/2 forms) and all-tile splits (stage 3/4 forms):
    chunks are added in index order, so repeated runs agree bit for bit."""
    cases = [(uni(8, 128, 28, 28, lo=0), he(128, 128, 3), nrm(128), [1, 1, 1, 1]),
             (uni(32, 64, 56, 56, lo=0), he(64, 64, 3), nrm(64), [1, 1, 1, 1]),
             (uni(4, 512, 7, 7, lo=0), he(512, 512, 3), nrm(512), [1, 1, 1, 1]),
             (uni(8, 1024, 14, 14, lo=0), he(256, 1024, 1), nrm(256), [0, 0, 0, 0])]
    for X, W, Bv, pads in cases:
        outs = [hip_conv(ctx, X, W, Bv, pads=pads, epilogue="relu") for _ in range(3)]
        for o in outs[1:]:
            assert_bit_exact(o, outs[0], "conv %s" % (X.shape,))
        assert_close_max(outs[0], ref.unary("Relu", ref.conv(X, W, Bv, pads=pads)), GEMM_TOL)


def test_split_k_auto_on_deep_small_layers(ctx):
    """ResNet stage-4 forms (few pixels, long K) take the split path by themselves."""
    X, W, Bv = uni(4, 512, 7, 7, lo=0), he(512, 512, 3), nrm(512)
    assert_close_max(hip_conv(ctx, X, W, Bv, pads=[1, 1, 1, 1]), ref.conv(X, W, Bv, pads=[1, 1, 1, 1]), GEMM_TOL,
                     "3x3 512 @7x7")
    A, B = uni(64, 4096), uni(4096, 48)
    assert_close_max(hip_gemm(ctx, A, B), ref.gemm(A, B), GEMM_TOL, "skinny gemm")


# ------------------------------------------------------------------ every contraction path
BIG_KERNEL_CONVS = [
    # n, cin, h, w, cout, kh, kw, pads, strides, dil, group: more than 63 taps -> the flat-load gather
    (2, 6, 30, 31, 10, 9, 9, [4, 4, 4, 4], [1, 1], [1, 1], 1),
    (1, 8, 40, 37, 12, 11, 11, [5, 3, 2, 5], [2, 3], [1, 1], 2),
    (2, 4, 45, 45, 6, 9, 9, [8, 8, 8, 8], [2, 2], [2, 2], 1),
    (1, 3, 64, 50, 5, 11, 9, [0, 0, 0, 0], [1, 2], [1, 1], 1),
    (1, 16, 26, 26, 16, 9, 9, [4, 4, 4, 4], [1, 1], [1, 1], 16),   # depthwise
    (3, 5, 23, 29, 70, 8, 9, [3, 4, 4, 4], [1, 1], [1, 1], 1),     # two row tiles, ragged K (360)
]


@pytest.mark.parametrize("shape", BIG_KERNEL_CONVS)
def test_conv_kernels_of_more_than_63_taps(ctx, shape):
    n, cin, h, w, cout, kh, kw, pads, strides, dil, group = shape
    X, B = uni(n, cin, h, w, lo=0), nrm(cout)
    W = nrm(cout, cin // group, kh, kw, std=float(np.sqrt(2.0 / (cin // group * kh * kw))))
    want = ref.conv(X, W, B, dil, group, None, pads, strides)
    got = hip_conv(ctx, X, W, B, dil, group, pads, strides)
    assert_close_max(got, want, GEMM_TOL, "conv %s" % (shape,))
    R = nrm(*want.shape)
    fused = hip_conv(ctx, X, W, B, dil, group, pads, strides, epilogue="relu", R=R)
    assert_bit_exact(fused, np.maximum(got + R, 0) + 0.0, "big-kernel conv + residual + relu")


def test_conv_reference_large_im2col_case(ctx):
    """The reference's conv11 (test/model_test/make_models.py:641-643): Conv2d(1, 1, 4, 1, 1) on
    (32, 1, 1027, 1027), the case that makes its CPU backend split the im2col buffer."""
    X, W, B = uni(32, 1, 1027, 1027), nrm(1, 1, 4, 4, std=0.25), nrm(1)
    got = hip_conv(ctx, X, W, B, pads=[1, 1, 1, 1])
    assert got.shape == (32, 1, 1026, 1026)
    for img in (0, 17, 31):
        want = ref.conv(X[img:img + 1], W, B, pads=[1, 1, 1, 1])
        assert_close_max(got[img:img + 1], want, GEMM_TOL, "conv11 image %d" % img)


@pytest.mark.parametrize("ta,tb", list(itertools.product([0, 1], [0, 1])))
def test_flat_load_loop_and_checked_epilogue_on_ordinary_sizes(ctx, ta, tb):
    """descriptor_loads = 0 sends ordinary operands down the paths that 2 GiB operands take: flat
    loads in the general loop, the bounds-checked epilogue, the flat-load conv gather."""
    m, n, k = 150, 203, 77
    A, B, C = (uni(k, m) if ta else uni(m, k)), (uni(n, k) if tb else uni(k, n)), uni(n)
    A2, B2 = (uni(64, 256) if ta else uni(256, 64)), (uni(128, 64) if tb else uni(64, 128))
    X, W, Bv, R = uni(3, 16, 19, 21, lo=0), he(40, 16, 3), nrm(40), nrm(3, 40, 19, 21)
    X1, W1 = uni(4, 32, 8, 8), uni(24, 32, 1, 1)
    want = {}
    for mode in (1, 0):
        try:
            ctx.set_option("descriptor_loads", mode)
            got = {
                "gemm": hip_gemm(ctx, A, B, C, 0.5, 2.0, ta, tb, epilogue="relu"),
                "gemm whole tiles": hip_gemm(ctx, A2, B2, None, 1.0, 1.0, ta, tb),
                "conv 3x3": hip_conv(ctx, X, W, Bv, pads=[1, 1, 1, 1], epilogue="relu", R=R),
                "conv 3x3 s2": hip_conv(ctx, X, W, Bv, pads=[1, 0, 1, 2], strides=[2, 1]),
                "conv 1x1": hip_conv(ctx, X1, W1),
            }
        finally:
            ctx.set_option("descriptor_loads", 1)
        if mode == 1:
            want = got
            continue
        assert_close_max(got["gemm"], ref.unary("Relu", ref.gemm(A, B, C, 0.5, 2.0, ta, tb)), GEMM_TOL, "flat gemm")
        assert_close_max(got["gemm whole tiles"], ref.gemm(A2, B2, None, 1.0, 1.0, ta, tb), GEMM_TOL, "flat gemm 2")
        assert_close_max(got["conv 3x3"], ref.unary("Relu", ref.binary("Add", ref.conv(X, W, Bv, pads=[1, 1, 1, 1]), R)),
                         GEMM_TOL, "flat conv")
        assert_close_max(got["conv 3x3 s2"], ref.conv(X, W, Bv, pads=[1, 0, 1, 2], strides=[2, 1]), GEMM_TOL, "flat conv s2")
        assert_close_max(got["conv 1x1"], ref.conv(X1, W1), GEMM_TOL, "flat conv 1x1")
        for key in got:
            # the two forms add the same products; only the order inside a K slab may differ
            assert_close_max(got[key], want[key], 1e-5, "descriptor vs flat: " + key)
    with pytest.raises(capi.HipError):
        ctx.set_option("descriptor_loads", 2)


def test_gemm_with_strides_dense_in_neither_index(ctx):
    """wdh_gemm called directly with operands that are contiguous in neither index (a view with a
    step along both axes): the scalar kernel that follows the reference's loop order."""
    m, n, k, batch = 37, 29, 53, 3
    Abig, Bbig = uni(batch, m, 2 * k), uni(batch, k, 3 * n)   # A[b, i, 2x], B[b, x, 3j]
    C, R = uni(m, 1), nrm(batch, m, n)
    A, B = Abig[:, :, ::2], Bbig[:, :, ::3]
    ta, tb, tc, tr = (ctx.move_tensor(v) for v in (Abig, Bbig, C, R))
    y = ctx.empty_tensor([batch, m, n])
    capi.call("wdh_gemm", ta.handle, tb.handle, tc.handle, y.handle, batch, m, n, k,
              m * 2 * k, 2 * k, 2, k * 3 * n, 3 * n, 3, 1, 0, 0.75, 1.5, 1, tr.handle)
    want = np.stack([ref.gemm(A[b], B[b], C, 0.75, 1.5) for b in range(batch)])
    want = ref.unary("Relu", ref.binary("Add", want, R))
    assert_close_max(y.get_data(), want, GEMM_TOL, "strided gemm")
    # both operands transposed views with a step
    At = np.ascontiguousarray(np.swapaxes(Abig, 1, 2))        # [b, 2k, m]
    ta2 = ctx.move_tensor(At)
    y2 = ctx.empty_tensor([batch, m, n])
    capi.call("wdh_gemm", ta2.handle, tb.handle, 0, y2.handle, batch, m, n, k,
              2 * k * m, 1, 2 * m, k * 3 * n, 3 * n, 3, 0, 0, 1.0, 1.0, 0, 0)
    want2 = np.stack([ref.gemm(A[b], B[b]) for b in range(batch)])
    assert_close_max(y2.get_data(), want2, GEMM_TOL, "strided gemm, A transposed")


def test_gemm_operand_of_more_than_2_gib(ctx):
    """A [528384, 1024] spans 2.16 GB: 32-bit byte offsets cannot address it, so the kernel takes
    the flat-load loop.  The oracle runs on sampled rows."""
    m, k, n = 528384, 1024, 64
    rng = np.random.default_rng(7)
    A = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    B = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    C = rng.uniform(-1, 1, (n,)).astype(np.float32)
    ta, tb, tc = ctx.move_tensor(A), ctx.move_tensor(B), ctx.move_tensor(C)
    y = H.gemm(ctx, ta, tb, tc)
    got = y.get_data()
    rows = np.concatenate([np.arange(0, 64), rng.integers(0, m, 192), np.arange(m - 64, m),
                           np.arange(524288 - 8, 524288 + 8)])   # around the 2 GiB line of A
    want = ref.gemm(A[rows], B, C)
    assert_close_max(got[rows], want, GEMM_TOL, "2 GiB gemm, sampled rows")
    # every row, against the BLAS product in double
    full = (A.astype(np.float64) @ B.astype(np.float64) + C).astype(np.float32)
    assert_close_max(got, full, GEMM_TOL, "2 GiB gemm, all rows vs float64 BLAS")
    for t in (ta, tb, tc, y):
        t.dispose()
    capi.call("wdh_trim", 0)   # hand the 2 GiB block back to the driver


HALO_CONVS = [
    # n, cin, h, w, cout, pads, group: 3x3 stride 1, channels in blocks of 8 -> the LDS-tile kernel
    (2, 8, 56, 56, 16, [1, 1, 1, 1], 1),       # 16-byte row pieces
    (3, 16, 28, 28, 70, [1, 1, 1, 1], 1),      # 64-pixel tiles straddle images (784 each); two row tiles
    (5, 24, 14, 14, 40, [1, 1, 1, 1], 1),      # 8-byte pieces
    (7, 32, 7, 7, 33, [1, 1, 1, 1], 1),        # 4-byte pieces, a tile spans three images
    (2, 8, 12, 20, 9, [0, 0, 0, 0], 1),        # no padding
    (2, 16, 9, 12, 12, [2, 1, 0, 2], 1),       # unequal pads, wider than the kernel's reach
    (1, 8, 5, 8, 8, [1, 1, 1, 1], 1),          # 40 pixels: a single partial tile
    (2, 32, 10, 16, 24, [1, 1, 1, 1], 4),      # groups
    (1, 64, 3, 3, 64, [1, 1, 1, 1], 1),        # plane smaller than the kernel's halo
    (2, 8, 6, 120, 8, [1, 1, 1, 1], 1),        # rows too wide for the LDS tile: falls back to the gather
    (33, 8, 2, 2, 8, [1, 1, 1, 1], 1),         # 4-pixel images: too many rows per tile, falls back
]


@pytest.mark.parametrize("shape", HALO_CONVS)
def test_conv3x3_lds_tile_kernel(ctx, shape):
    n, cin, h, w, cout, pads, group = shape
    X, W, B = uni(n, cin, h, w, lo=0), he(cout, cin // group, 3), nrm(cout)
    want = ref.conv(X, W, B, None, group, None, pads, None)
    R = nrm(*want.shape)
    got = {}
    for halo in (1, 0):
        try:
            ctx.set_option("conv3x3_halo", halo)
            got[halo] = hip_conv(ctx, X, W, B, None, group, pads)
            fused = hip_conv(ctx, X, W, B, None, group, pads, epilogue="relu", R=R)
            for split in (2, 64):
                ctx.set_option("split_k", split)
                cut = hip_conv(ctx, X, W, B, None, group, pads)
                ctx.set_option("split_k", -1)
                assert_close_max(cut, want, GEMM_TOL, "halo %d split %d %s" % (halo, split, shape))
        finally:
            ctx.set_option("conv3x3_halo", 1)
            ctx.set_option("split_k", -1)
        assert_close_max(got[halo], want, GEMM_TOL, "halo %d %s" % (halo, shape))
        assert_bit_exact(fused, np.maximum(got[halo] + R, 0) + 0.0, "halo %d + residual + relu" % halo)
    assert_close_max(got[1], got[0], 1e-5, "LDS-tile form vs gathered form")


STEM_CONVS = [
    # n, h, w, pads: 7x7 stride 2, 3 -> 64 channels -> the kernel with weights and patch in LDS
    (2, 224, 224, [3, 3, 3, 3]),     # the ResNet stem: 14 x 7 whole tiles per image
    (1, 64, 96, [3, 3, 3, 3]),
    (3, 37, 53, [3, 3, 3, 3]),       # odd sizes: ragged tiles on both axes
    (2, 40, 70, [2, 3, 3, 1]),       # unequal pads
    (2, 45, 33, [0, 0, 0, 0]),       # no padding
    (5, 7, 7, [0, 0, 0, 0]),         # one output pixel per image
    (1, 9, 200, [5, 6, 4, 7]),       # pads wider than half the kernel
]


@pytest.mark.parametrize("shape", STEM_CONVS)
def test_conv7x7_stem_kernel(ctx, shape):
    n, h, w, pads = shape
    X, W, B = uni(n, 3, h, w, lo=-1), he(64, 3, 7), nrm(64)
    want = ref.conv(X, W, B, None, 1, None, pads, [2, 2])
    R = nrm(*want.shape)
    got = {}
    for stem in (1, 0):
        try:
            ctx.set_option("conv_stem", stem)
            got[stem] = hip_conv(ctx, X, W, B, None, 1, pads, [2, 2])
            form = ctx.last_plan()["form"]
            nobias = hip_conv(ctx, X, W, None, None, 1, pads, [2, 2])
            fused = hip_conv(ctx, X, W, B, None, 1, pads, [2, 2], epilogue="relu", R=R)
        finally:
            ctx.set_option("conv_stem", 1)
        assert ("stem" in form) == bool(stem), form
        assert_close_max(got[stem], want, GEMM_TOL, "stem %d %s" % (stem, shape))
        assert_close_max(nobias, want - B.reshape(1, 64, 1, 1), GEMM_TOL, "stem %d, no bias %s" % (stem, shape))
        assert_bit_exact(fused, np.maximum(got[stem] + R, 0) + 0.0, "stem %d + residual + relu" % stem)
    assert_close_max(got[1], got[0], 1e-5, "stem kernel vs gathered form")


def test_conv7x7_stem_geometry_without_descriptors_takes_the_flat_gather(ctx):
    """descriptor_loads = 0 stands for operands of 2 GiB and more: the stem's kernel addresses a whole
    image's results through one descriptor, so it must step aside."""
    X, W, B = uni(2, 3, 40, 56, lo=-1), he(64, 3, 7), nrm(64)
    want = ref.conv(X, W, B, None, 1, None, [3, 3, 3, 3], [2, 2])
    try:
        ctx.set_option("descriptor_loads", 0)
        got = hip_conv(ctx, X, W, B, None, 1, [3, 3, 3, 3], [2, 2])
        form = ctx.last_plan()["form"]
    finally:
        ctx.set_option("descriptor_loads", 1)
    assert form == "conv, gathered taps (flat loads)", form
    assert_close_max(got, want, GEMM_TOL, "stem geometry, flat loads")


def test_conv7x7_stem_kernel_keeps_nan_and_inf_inside_their_receptive_fields(ctx):
    """One step of the stem kernel's K order has no partner tap: what the idle half of the wavefront
    multiplies must be a true zero, or an Inf elsewhere in the tile's patch would leak into every pixel."""
    X, W = uni(1, 3, 40, 40, lo=-1), he(64, 3, 7)
    X[0, 1, 20, 21] = np.inf
    X[0, 2, 5, 30] = np.nan
    got = {}
    for stem in (1, 0):
        try:
            ctx.set_option("conv_stem", stem)
            got[stem] = hip_conv(ctx, X, W, None, None, 1, [3, 3, 3, 3], [2, 2])
        finally:
            ctx.set_option("conv_stem", 1)
    assert np.array_equal(np.isfinite(got[1]), np.isfinite(got[0]))
    assert 0 < np.count_nonzero(~np.isfinite(got[1])) < got[1].size // 4
    fin = np.isfinite(got[0])
    assert_close_max(got[1][fin], got[0][fin], 1e-5, "finite outputs")


@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4])
def test_conv3x3_lds_tile_kernel_every_tile_shape(ctx, tile):
    """The LDS-tile kernel exists for the same five workgroup tiles as the gathered form."""
    cases = [(3, 16, 28, 28, 70, [1, 1, 1, 1], 1), (5, 24, 14, 14, 200, [1, 1, 1, 1], 1),
             (9, 32, 7, 7, 33, [1, 0, 1, 2], 1), (2, 32, 20, 56, 24, [1, 1, 1, 1], 2)]
    for n, cin, h, w, cout, pads, group in cases:
        X, W, B = uni(n, cin, h, w, lo=0), he(cout, cin // group, 3), nrm(cout)
        want = ref.conv(X, W, B, None, group, None, pads, None)
        try:
            ctx.set_option("contraction_tile", tile)
            got = hip_conv(ctx, X, W, B, None, group, pads)
            ctx.set_option("split_k", 3)
            cut = hip_conv(ctx, X, W, B, None, group, pads, epilogue="relu")
        finally:
            ctx.set_option("contraction_tile", -1)
            ctx.set_option("split_k", -1)
        assert_close_max(got, want, GEMM_TOL, "tile %d %s" % (tile, (n, cin, h, w, cout)))
        assert_close_max(cut, ref.unary("Relu", want), GEMM_TOL, "tile %d split 3" % tile)


@pytest.mark.parametrize("batch,m,n,k", [(8, 850, 32, 850), (8, 100, 32, 100), (3, 70, 50, 33), (2, 64, 64, 256)])
def test_gemm_ex_writes_the_result_where_a_transpose_would_put_it(ctx, batch, m, n, k):
    """wdh_gemm_ex with sYb = n, sY0 = batch*n stores [batch, m, n] as [m, batch, n] (attention heads
    merged back); operands read through the strides an absorbed Transpose leaves behind."""
    rng = np.random.default_rng(batch * 1000 + m)
    # A as [m, batch, k] (tokens, heads, d) read as [batch, m, k]; B as [k_tokens.., ] read transposed
    A_store = rng.uniform(-1, 1, (m, batch, k)).astype(np.float32)
    B_store = rng.uniform(-1, 1, (n, batch, k)).astype(np.float32)      # B[b, x, j] = B_store[j, b, x]
    A = np.ascontiguousarray(A_store.transpose(1, 0, 2))
    B = np.ascontiguousarray(B_store.transpose(1, 2, 0))
    ta, tb = ctx.move_tensor(A_store), ctx.move_tensor(B_store)
    want = np.stack([ref.gemm(A[b], B[b], None, 0.25, 1.0) for b in range(batch)])
    for split in (-1, 3):
        y = ctx.empty_tensor([m, batch, n])
        y.set_data(np.full((m, batch, n), np.nan, np.float32))
        try:
            ctx.set_option("split_k", split)
            capi.call("wdh_gemm_ex", ta.handle, tb.handle, 0, y.handle, batch, m, n, k,
                      k, batch * k, 1, k, 1, batch * k, 0, 0, 0.25, 1.0, 0, 0, n, batch * n)
        finally:
            ctx.set_option("split_k", -1)
        got = y.get_data()
        assert_close_max(got.transpose(1, 0, 2), want, GEMM_TOL, "interleaved result, split %d" % split)
        # the same product stored batch-major must hold the same bits
        d = ctx.empty_tensor([batch, m, n])
        try:
            ctx.set_option("split_k", split)
            capi.call("wdh_gemm", ta.handle, tb.handle, 0, d.handle, batch, m, n, k,
                      k, batch * k, 1, k, 1, batch * k, 0, 0, 0.25, 1.0, 0, 0)
        finally:
            ctx.set_option("split_k", -1)
        assert_bit_exact(got.transpose(1, 0, 2), d.get_data(), "same sums, other addresses")
        y.dispose(); d.dispose()
    y = ctx.empty_tensor([m, batch, n])
    with pytest.raises(capi.HipError):      # rows would overlap
        capi.call("wdh_gemm_ex", ta.handle, tb.handle, 0, y.handle, batch, m, n, k,
                  k, batch * k, 1, k, 1, batch * k, 0, 0, 1.0, 1.0, 0, 0, n, n)
    with pytest.raises(capi.HipError):      # row stride below the row length
        capi.call("wdh_gemm_ex", ta.handle, tb.handle, 0, y.handle, batch, m, n, k,
                  k, batch * k, 1, k, 1, batch * k, 0, 0, 1.0, 1.0, 0, 0, m * n, n - 1)


@pytest.mark.parametrize("n,cin,h,w,cout,group", [(3, 32, 10, 10, 40, 1), (1, 64, 50, 68, 70, 1), (5, 32, 6, 6, 24, 2),
                                                  (2, 16, 2, 2, 8, 1)])
def test_conv_1x1_in_place_with_a_ragged_last_tile(ctx, n, cin, h, w, cout, group):
    """1x1 stride-1 convs read X as the B matrix also when the pixel count is no multiple of the tile
    (DETR's 13600-, 3400- and 850-pixel stages): the last tile hangs over the end of the pixels."""
    X, W, B = uni(n, cin, h, w, lo=0), he(cout, cin // group, 1), nrm(cout)
    R = nrm(n, cout, h, w)
    got = hip_conv(ctx, X, W, B, None, group)
    assert ctx.last_plan()["form"] == "conv 1x1, X in place"
    assert_close_max(got, ref.conv(X, W, B, None, group), GEMM_TOL, "ragged in-place 1x1")
    fused = hip_conv(ctx, X, W, B, None, group, epilogue="relu", R=R)
    assert_bit_exact(fused, np.maximum(got + R, 0) + 0.0, "ragged in-place 1x1 + residual + relu")


WINOGRAD_CONVS = [
    # n, cin, h, w, cout, pads
    (32, 256, 14, 14, 256, [1, 1, 1, 1]),     # ResNet-50 stage 3
    (8, 512, 7, 7, 512, [1, 1, 1, 1]),        # odd output planes: the last 2x2 block of a row and column is half empty
    (4, 128, 28, 28, 128, [1, 1, 1, 1]),
    (1, 128, 25, 34, 160, [1, 1, 1, 1]),      # a DETR plane
    (2, 32, 9, 11, 48, [1, 1, 1, 1]),         # below the channel count the plan picks by itself
    (2, 16, 8, 8, 16, [0, 0, 0, 0]),          # no padding
    (3, 48, 10, 7, 16, [2, 0, 1, 2]),         # unequal pads, wider than the filter's reach on one side
    (1, 16, 3, 3, 32, [1, 1, 1, 1]),
    (2, 64, 21, 18, 64, [1, 1, 1, 1]),        # neither side a multiple of the block of either form
]


WINOGRAD_FORMS = {2: "conv 3x3, F(2x2,3x3)", 3: "conv 3x3, F(4x4,3x3)"}


@pytest.mark.parametrize("mode", [2, 3])
@pytest.mark.parametrize("shape", WINOGRAD_CONVS)
def test_conv3x3_by_minimal_filtering(ctx, shape, mode):
    """3x3 stride-1 convs as F(2x2, 3x3) / F(4x4, 3x3): transformed filters and input patches, 16 / 36 batched
    products, results transformed back under bias + residual + Relu.  Not the direct form's sums, so the bar is
    the Gemm/Conv tolerance against the oracle -- for the forced form, for what the plan picks, and with the
    filters kept from a first call (WDH_CONV_CONSTANT_WEIGHTS).  Inputs of both signs as well as the
    non-negative ones a Relu leaves: the transforms of F(4x4, 3x3) cancel more with mixed signs."""
    n, cin, h, w, cout, pads = shape
    X, W, B = uni(n, cin, h, w, lo=0), he(cout, cin, 3), nrm(cout)
    want0 = ref.conv(X, W, B, pads=pads)
    R = nrm(*want0.shape)
    want = ref.unary("Relu", ref.binary("Add", want0, R))
    form = WINOGRAD_FORMS[mode]
    try:
        ctx.set_option("conv3x3_winograd", mode)
        got = hip_conv(ctx, X, W, B, pads=pads, epilogue="relu", R=R)
        assert ctx.last_plan()["form"].startswith(form), ctx.last_plan()
        assert_close_max(got, want, GEMM_TOL, "%s %s" % (form, shape))
        assert_close_max(hip_conv(ctx, X, W, None, pads=pads), ref.conv(X, W, None, pads=pads), GEMM_TOL, "no bias")
        Xs = nrm(n, cin, h, w)
        assert_close_max(hip_conv(ctx, Xs, W, B, pads=pads), ref.conv(Xs, W, B, pads=pads), GEMM_TOL, "signed input")
        # filters kept across calls: same bits as computing them every time; other weights in the same
        # buffer (wdh_write) or in a new buffer are seen
        tx, tw, tb, tr = (ctx.move_tensor(v) for v in (X, W, B, R))
        kept = [H.conv(ctx, tx, tw, tb, pads=pads, epilogue="relu", residual=tr, constant_weights=True).get_data()
                for _ in range(3)]
        for k in kept:
            assert_bit_exact(k, got, "kept filters")
        W2 = he(cout, cin, 3)
        capi.call("wdh_write", tw.handle, 0, W2.ctypes.data, W2.nbytes)
        want2 = ref.unary("Relu", ref.binary("Add", ref.conv(X, W2, B, pads=pads), R))
        again = H.conv(ctx, tx, tw, tb, pads=pads, epilogue="relu", residual=tr, constant_weights=True).get_data()
        assert_close_max(again, want2, GEMM_TOL, "weights rewritten in place")
        if mode == 3:
            # filters kept for one form are not taken for the other
            ctx.set_option("conv3x3_winograd", 2)
            other = H.conv(ctx, tx, tw, tb, pads=pads, epilogue="relu", residual=tr, constant_weights=True).get_data()
            assert ctx.last_plan()["form"].startswith(WINOGRAD_FORMS[2])
            assert_close_max(other, want2, GEMM_TOL, "the other form after kept filters")
        for t in (tx, tw, tb, tr):
            t.dispose()
    finally:
        ctx.set_option("conv3x3_winograd", 1)
    if mode == 3:
        auto = hip_conv(ctx, X, W, B, pads=pads, epilogue="relu", R=R)
        assert_close_max(auto, want, GEMM_TOL, "the plan's own choice %s" % (ctx.last_plan()["form"],))
        picked = ctx.last_plan()["form"].startswith(WINOGRAD_FORMS[2])
        assert picked == (cin >= 128 and cout >= 128), ctx.last_plan()
        try:
            ctx.set_option("conv3x3_f4x4_channels", 64)     # F(4x4, 3x3) on request, from that many channels on
            fast = hip_conv(ctx, X, W, B, pads=pads, epilogue="relu", R=R)
            assert_bit_exact(fast, got if cin >= 64 and cout >= 64 else auto, "conv3x3_f4x4_channels")
        finally:
            ctx.set_option("conv3x3_f4x4_channels", 0)
        try:
            ctx.set_option("conv3x3_winograd", 0)
            direct = hip_conv(ctx, X, W, B, pads=pads, epilogue="relu", R=R)
            assert not ctx.last_plan()["form"].startswith("conv 3x3, F("), ctx.last_plan()
            assert_close_max(direct, want, GEMM_TOL, "direct form")
        finally:
            ctx.set_option("conv3x3_winograd", 1)


@pytest.mark.parametrize("mode", [2, 3])
def test_conv3x3_minimal_filtering_keeps_special_values_local_and_replays(ctx, mode):
    """An Inf in the input reaches only the outputs whose receptive field holds it... in the transform domain
    it meets finite values of its input patch, so the output blocks whose patches hold it may turn NaN, never a
    block further away; and the form replays from a captured graph with kept filters."""
    X, W, B = uni(2, 128, 12, 12, lo=0), he(128, 128, 3), nrm(128)
    X[1, 5, 6, 6] = np.inf
    try:
        ctx.set_option("conv3x3_winograd", mode)
        got = hip_conv(ctx, X, W, B, pads=[1, 1, 1, 1])
        assert ctx.last_plan()["form"].startswith(WINOGRAD_FORMS[mode])
        bad = ~np.isfinite(got)
        assert not bad[0].any(), "the other image is untouched"
        # with one row and column of padding, input (6, 6) lies in the patches of the 2x2 blocks 2 and 3 of its
        # row and column and in the patch of 4x4 block 1: output rows and columns 4..7 either way
        ys, xs = np.nonzero(bad[1].any(axis=0))
        assert ys.min() >= 4 and ys.max() <= 7 and xs.min() >= 4 and xs.max() <= 7, (ys, xs)
        Xc = np.where(np.isfinite(X), X, 0).astype(np.float32)
        tx, tw, tb = (ctx.move_tensor(v) for v in (Xc, W, B))
        eager = H.conv(ctx, tx, tw, tb, pads=[1, 1, 1, 1], constant_weights=True)
        want = eager.get_data()
        eager.dispose()
        ctx.sync()
        ctx.graph_begin()
        try:
            out = H.conv(ctx, tx, tw, tb, pads=[1, 1, 1, 1], constant_weights=True)
        finally:
            gid = ctx.graph_end()
        for rep in range(3):
            ctx.graph_launch(gid)
            ctx.sync()
            assert_bit_exact(out.get_data(), want, "replay %d" % rep)
        out.dispose()
        ctx.graph_destroy(gid)
        for t in (tx, tw, tb):
            t.dispose()
    finally:
        ctx.set_option("conv3x3_winograd", 1)


def test_memory_limit_and_the_direct_form_as_fallback(ctx):
    """memory_limit_mib caps what the pool asks of the driver: an allocation beyond it fails with WDH_ENOMEM
    (after cached blocks went back), one inside it works, and a 3x3 conv that cannot get the transform-domain
    tensors of its minimal-filtering form (here 2 x 16 x 256 x 3136 floats = 98 MiB) takes a direct form
    instead of failing -- also when the caller vouches for the weights, and without leaving half-made kept
    filters behind for the call after the limit is lifted."""
    X, W, B = uni(16, 256, 28, 28, lo=0), he(256, 256, 3), nrm(256)
    want = ref.conv(X, W, B, pads=[1, 1, 1, 1])
    tx, tw, tb = (ctx.move_tensor(v) for v in (X, W, B))
    ctx.sync()
    capi.call("wdh_trim", 0)
    stats = ctx.mem_stats()
    reserved = stats["in_use"] + stats["cached"]
    try:
        ctx.set_option("memory_limit_mib", (reserved >> 20) + 64)
        assert capi.load().wdh_alloc(128 << 20) == 0
        assert "memory_limit_mib" in capi.last_error()
        small = capi.load().wdh_alloc(8 << 20)
        assert small > 0
        capi.call("wdh_free", small)
        for flag in (False, True):
            y = H.conv(ctx, tx, tw, tb, pads=[1, 1, 1, 1], constant_weights=flag)
            assert ctx.last_plan()["form"] == "conv 3x3, LDS tile", ctx.last_plan()
            assert_close_max(y.get_data(), want, GEMM_TOL, "direct form under the limit")
            y.dispose()
    finally:
        ctx.set_option("memory_limit_mib", 0)
    y = H.conv(ctx, tx, tw, tb, pads=[1, 1, 1, 1], constant_weights=True)
    assert ctx.last_plan()["form"].startswith(WINOGRAD_FORMS[2]), ctx.last_plan()
    assert_close_max(y.get_data(), want, GEMM_TOL, "minimal filtering once the limit is lifted")
    for t in (y, tx, tw, tb):
        t.dispose()


@pytest.mark.parametrize("n,cin,h,w,cout,sh,group", [
    (4, 256, 56, 56, 128, 2, 1),       # the stride-2 1x1 convs that open ResNet-50's stages 2 and 3
    (4, 512, 28, 28, 1024, 2, 1),
    (3, 32, 10, 24, 40, 2, 1),         # ragged last tile, rows of 12 output pixels
    (3, 32, 12, 20, 40, 2, 1),         # rows of 10 output pixels: a thread's two pixel pairs lie in different rows
    (2, 32, 9, 16, 24, 1, 1),          # column stride only
    (2, 32, 13, 8, 24, 3, 2),          # row stride 3, two groups
    (1, 16, 4, 8, 8, 2, 1),            # fewer pixels than a tile
])
def test_conv_1x1_column_stride_2_in_place(ctx, n, cin, h, w, cout, sh, group):
    """An unpadded 1x1 conv with column stride 2 whose output rows hold an even number of pixels reads X
    in place (two 16-byte pieces per four output pixels, every other element kept).  Against the oracle, and
    bit for bit against the gathered form of the same geometry (the same products added in the same order)."""
    X, W, B = uni(n, cin, h, w, lo=0), he(cout, cin // group, 1), nrm(cout)
    oh, ow = (h - 1) // sh + 1, (w - 1) // 2 + 1
    R = nrm(n, cout, oh, ow)
    got = hip_conv(ctx, X, W, B, None, group, None, [sh, 2], epilogue="relu", R=R)
    assert ctx.last_plan()["form"] == "conv 1x1 stride 2, X in place", ctx.last_plan()
    want = ref.unary("Relu", ref.binary("Add", ref.conv(X, W, B, None, group, None, None, [sh, 2]), R))
    assert_close_max(got, want, GEMM_TOL, "1x1 column stride 2 in place")
    try:
        ctx.set_option("conv1x1_stride2_in_place", 0)
        gathered = hip_conv(ctx, X, W, B, None, group, None, [sh, 2], epilogue="relu", R=R)
        assert ctx.last_plan()["form"] == "conv, gathered taps"
    finally:
        ctx.set_option("conv1x1_stride2_in_place", 1)
    assert_close_max(gathered, want, GEMM_TOL, "gathered")


def test_conv_1x1_column_stride_2_falls_back_where_rows_do_not_fit(ctx):
    """Output rows with an odd number of pixels (7 of 14), padding, or a column stride of 3: gathered."""
    for shape, strides, pads in (((2, 64, 14, 14), [2, 2], None), ((2, 32, 16, 16), [2, 2], [1, 1, 1, 1]),
                                 ((2, 32, 16, 24), [2, 3], None)):
        X, W = uni(*shape, lo=0), he(24, shape[1], 1)
        got = hip_conv(ctx, X, W, None, None, 1, pads, strides)
        assert ctx.last_plan()["form"] == "conv, gathered taps", (shape, ctx.last_plan())
        assert_close_max(got, ref.conv(X, W, None, None, 1, None, pads, strides), GEMM_TOL, "fallback %s" % (shape,))


@pytest.mark.parametrize("batch,m,n,k,tb", [(1, 850, 256, 256, 0), (1, 850, 256, 2048, 0), (8, 850, 32, 850, 0),
                                            (1, 200, 1000, 256, 1), (3, 70, 45, 333, 1), (1, 100, 92, 256, 0),
                                            (8, 100, 100, 128, 1), (2, 33, 31, 500, 0)])
def test_small_products_cut_k_across_the_wavefronts_of_a_workgroup(ctx, batch, m, n, k, tb):
    """Few result tiles, K >= 128: one launch of 32x32 blocks (gemm_wavesplit_kernel).  Against the
    oracle, and against the ordinary tiles with a reduce pass (same products, another order)."""
    rng = np.random.default_rng(m * 7 + k)
    A = rng.uniform(-1, 1, (batch, m, k)).astype(np.float32)
    B = rng.uniform(-1, 1, (batch, n, k) if tb else (batch, k, n)).astype(np.float32)
    C = rng.uniform(-1, 1, (n,)).astype(np.float32)
    R = rng.standard_normal((batch, m, n)).astype(np.float32)
    ta, tb_, tc, tr = (ctx.move_tensor(v) for v in (A, B, C, R))
    sb = (k * n, 1, k) if tb else (k * n, n, 1)
    out = {}
    for mode in (1, 0):
        y = ctx.empty_tensor([batch, m, n])
        try:
            ctx.set_option("gemm_wavesplit", mode)
            capi.call("wdh_gemm", ta.handle, tb_.handle, tc.handle, y.handle, batch, m, n, k,
                      m * k, k, 1, sb[0], sb[1], sb[2], 0, 1, 0.5, 2.0, 1, tr.handle)
        finally:
            ctx.set_option("gemm_wavesplit", 1)
        out[mode] = (y.get_data(), ctx.last_plan())
        y.dispose()
    assert out[1][1]["tile"] == "32x32" and out[0][1]["tile"] != "32x32", (out[1][1], out[0][1])
    want = np.stack([ref.gemm(A[b], B[b], C, 0.5, 2.0, 0, tb) for b in range(batch)])
    want = ref.unary("Relu", ref.binary("Add", want, R))
    assert_close_max(out[1][0], want, GEMM_TOL, "wave-split product")
    assert_close_max(out[1][0], out[0][0], 1e-5, "wave-split vs tiles + reduce pass")
    again = ctx.empty_tensor([batch, m, n])
    capi.call("wdh_gemm", ta.handle, tb_.handle, tc.handle, again.handle, batch, m, n, k,
              m * k, k, 1, sb[0], sb[1], sb[2], 0, 1, 0.5, 2.0, 1, tr.handle)
    assert_bit_exact(again.get_data(), out[1][0], "same order every time")


def test_few_blocks_with_a_long_k_keep_the_ordinary_tiles(ctx):
    """The ResNet classifier head, [32,2048] x [1000,2048]^T: 32 blocks of 32x32 would leave the 8 MB of
    weights to 32 workgroups; it stays with 64x64 tiles whose K is shared out (as a stream of K slabs,
    or in chunks with a reduce pass when that schedule is switched off)."""
    A, B, C = uni(32, 2048), uni(1000, 2048), uni(1000)
    got = hip_gemm(ctx, A, B, C, 1.0, 1.0, 0, 1)
    assert ctx.last_plan()["tile"] == "64x64" and ctx.last_plan()["split"] != 1
    assert_close_max(got, ref.gemm(A, B, C, 1.0, 1.0, 0, 1), GEMM_TOL, "classifier head")


@pytest.mark.parametrize("tile", [-1, 0, 1, 2, 3, 4])
def test_sixteen_byte_stores_hold_the_bits_of_four_byte_stores(ctx, tile):
    """Whole tiles leave through LDS in 16-byte stores when the result's rows allow it
    (wide_stores, on by default).  Same arithmetic, so the same bits as the per-element
    stores: Gemm with a bias along n, along m, a full C, MatMul-style residual + Relu, and
    Conv in all three forms with bias + residual + Relu.  Repeated, since a store that races
    with the registers it reads shows only now and then."""
    def both(run):
        out = []
        for wide in (0, 1):
            try:
                ctx.set_option("wide_stores", wide)
                ctx.set_option("contraction_tile", tile)
                out.append(run())
            finally:
                ctx.set_option("wide_stores", 1)
                ctx.set_option("contraction_tile", -1)
        return out

    m, n, k = 1024, 1536, 96
    A, B = uni(m, k), uni(k, n)
    tA, tB = ctx.move_tensor(A), ctx.move_tensor(B)
    for what, C in (("bias along n", uni(n)), ("bias along m", uni(m, 1)), ("full C", uni(m, n)), ("no C", None)):
        tC = ctx.move_tensor(C) if C is not None else None
        for rep in range(3):
            narrow, wide = both(lambda: H.gemm(ctx, tA, tB, tC, 0.5, 2.0, epilogue="relu").get_data())
            assert_bit_exact(wide, narrow, "gemm, %s, tile %d" % (what, tile))
        assert_close_max(wide, ref.unary("Relu", ref.gemm(A, B, C, 0.5, 2.0)), GEMM_TOL, "gemm, " + what)
    convs = [(4, 64, 56, 56, 64, 3, [1, 1, 1, 1], [1, 1]),    # LDS-tile form
             (4, 64, 28, 28, 256, 1, [0, 0, 0, 0], [1, 1]),   # X in place
             (4, 24, 30, 30, 80, 3, [1, 1, 1, 1], [2, 2]),    # gathered: 15x15 outputs, rows not 16-byte multiples
             (4, 24, 32, 32, 80, 5, [2, 2, 2, 2], [2, 2])]    # gathered: 16x16 outputs
    for n_, cin, h, w, cout, kk, pads, strides in convs:
        X, W, Bv = uni(n_, cin, h, w, lo=0), he(cout, cin, kk), nrm(cout)
        want = ref.conv(X, W, Bv, None, 1, None, pads, strides)
        R = nrm(*want.shape)
        narrow, wide = both(lambda: hip_conv(ctx, X, W, Bv, None, 1, pads, strides, "relu", R))
        assert_bit_exact(wide, narrow, "conv %s tile %d" % ((cin, h, cout, kk), tile))
        assert_close_max(wide, np.maximum(want + R, 0), GEMM_TOL, "conv %s" % ((cin, h, cout, kk),))


def attention_chain_ref(q, k, v, heads, alpha):
    """The oracle's MatMul -> Mul -> Softmax -> MatMul per head."""
    tq, width = q.shape
    d = width // heads
    out = np.empty((tq, width), np.float32)
    for h in range(heads):
        sl = slice(h * d, (h + 1) * d)
        s = ref.matmul(np.ascontiguousarray(q[:, sl]), np.ascontiguousarray(k[:, sl].T))
        s = ref.binary("Mul", s, np.float32(alpha).reshape(()))
        out[:, sl] = ref.matmul(ref.softmax(s), np.ascontiguousarray(v[:, sl]))
    return out


@pytest.mark.parametrize("tq,tk,heads,d", [(850, 850, 8, 32), (100, 850, 8, 32), (100, 100, 8, 32), (1, 1, 1, 32),
                                           (33, 1024, 2, 64), (70, 257, 3, 128), (32, 31, 4, 32), (5, 1000, 1, 64)])
def test_attention_one_launch_equals_the_four_node_chain(ctx, tq, tk, heads, d):
    """wdh_attention against the oracle's chain, and against the library's own unfused chain
    (MatMul with strided heads, scale as alpha, Softmax, MatMul) within 1e-5."""
    rng = np.random.default_rng(tq * 7 + tk)
    q = rng.standard_normal((tq, heads * d)).astype(np.float32)
    k = rng.standard_normal((tk, heads * d)).astype(np.float32)
    v = rng.standard_normal((tk, heads * d)).astype(np.float32)
    alpha = 1.0 / np.sqrt(d)
    tq_, tk_, tv_ = ctx.move_tensor(q), ctx.move_tensor(k), ctx.move_tensor(v)
    got = H.attention(ctx, tq_, tk_, tv_, heads, alpha).get_data()
    want = attention_chain_ref(q, k, v, heads, alpha)
    assert_close_max(got, want, GEMM_TOL, "attention vs oracle chain")
    # the unfused chain on the device, heads addressed through strides
    w = heads * d
    scores = ctx.empty_tensor([heads, tq, tk])
    capi.call("wdh_gemm_ex", tq_.handle, tk_.handle, 0, scores.handle, heads, tq, tk, d,
              d, w, 1, d, 1, w, 0, 0, float(alpha), 1.0, 0, 0, tq * tk, tk)
    probs = H.softmax(ctx, scores)
    chain = ctx.empty_tensor([tq, w])
    capi.call("wdh_gemm_ex", probs.handle, tv_.handle, 0, chain.handle, heads, tq, d, tk,
              tq * tk, tk, 1, d, w, 1, 0, 0, 1.0, 1.0, 0, 0, d, w)
    assert_close_max(got, chain.get_data(), 1e-5, "attention vs unfused chain")


def test_attention_special_values_and_limits(ctx):
    """A +inf in V beside masked keys, a NaN score, and the shapes the entry point turns down."""
    rng = np.random.default_rng(5)
    q = rng.standard_normal((40, 32)).astype(np.float32)
    k = rng.standard_normal((50, 32)).astype(np.float32)
    v = rng.standard_normal((50, 32)).astype(np.float32)
    v[49, 3] = np.inf
    q[7, 0] = np.nan
    got = H.attention(ctx, ctx.move_tensor(q), ctx.move_tensor(k), ctx.move_tensor(v), 1, 0.25).get_data()
    want = attention_chain_ref(q, k, v, 1, 0.25)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(np.isinf(got), np.isinf(want))
    fin = np.isfinite(want)
    assert_close_max(got[fin], want[fin], GEMM_TOL, "finite cells")
    t = lambda *s: ctx.move_tensor(rng.standard_normal(s).astype(np.float32))
    with pytest.raises(capi.HipError):
        H.attention(ctx, t(4, 48), t(4, 48), t(4, 48), 1, 1.0)            # head dimension 48
    with pytest.raises(capi.HipError):
        H.attention(ctx, t(4, 32), t(1025, 32), t(1025, 32), 1, 1.0)      # more keys than LDS holds
    with pytest.raises(H.OperatorError):
        H.attention(ctx, t(4, 64), t(6, 64), t(5, 64), 2, 1.0)            # k and v disagree
    assert H.attention(ctx, t(0, 64), t(6, 64), t(6, 64), 2, 1.0).dims == [0, 64]


@pytest.mark.parametrize("shape", [(850, 256), (100, 1, 256), (27200, 256), (9, 1000), (5, 250), (3, 5000), (4100, 64)])
def test_layernorm_add_holds_what_the_two_nodes_store(ctx, shape):
    """wdh_layernorm_add: first result = wdh_layernorm's bits, second = the Add kernel's bits on it."""
    x, p = nrm(*shape), nrm(*shape)
    g, b = nrm(shape[-1]), nrm(shape[-1])
    tx, tg, tb, tp = (ctx.move_tensor(t) for t in (x, g, b, p))
    y, y2 = H.layer_normalization_add(ctx, tx, tg, tb, tp)
    alone = H.layer_normalization(ctx, tx, tg, tb)
    assert_bit_exact(y.get_data(), alone.get_data(), "normalised rows %s" % (shape,))
    assert_bit_exact(y2.get_data(), H.binary(ctx, "Add", alone, tp).get_data(), "rows + addend %s" % (shape,))
    assert_close_max(y.get_data(), ref.layernorm_decomposed(x, g, b, 1e-5), 1e-5, "against the oracle")
    with pytest.raises(H.OperatorError):
        H.layer_normalization_add(ctx, tx, tg, tb, ctx.move_tensor(nrm(shape[-1])))


def test_linear_group_holds_the_bits_of_separate_gemms(ctx):
    """wdh_linear_group: the projections of an attention block (and a mix of shapes, one of them too
    large for the one-launch form, one without bias, one with a ragged K) against wdh_gemm one by one."""
    rng = np.random.default_rng(11)
    t = lambda *s: ctx.move_tensor(rng.standard_normal(s).astype(np.float32))
    groups = [
        [(850, 256, 256, True)] * 3,
        [(100, 256, 256, True), (850, 256, 256, True), (850, 256, 256, True)],
        [(100, 256, 256, True), (850, 2048, 256, True), (37, 130, 200, False), (64, 64, 1000, True),
         (5, 7, 3, True), (100, 92, 256, True), (100, 256, 256, False), (33, 257, 129, True)],
    ]
    for shapes in groups:
        for epi in (None, "relu"):
            problems = [(t(m, k), t(k, n), t(n) if bias else None) for m, n, k, bias in shapes]
            got = H.linear_group(ctx, problems, epi)
            for (a, w, b), y in zip(problems, got):
                want = H.gemm(ctx, a, w, b, epilogue=epi).get_data()
                assert_bit_exact(y.get_data(), want, "group member %s" % (a.dims,))
                assert_close_max(want, ref.unary("Relu", ref.gemm(a.get_data(), w.get_data(), None if b is None else b.get_data()))
                                 if epi else ref.gemm(a.get_data(), w.get_data(), None if b is None else b.get_data()),
                                 GEMM_TOL, "against the oracle")
    assert H.linear_group(ctx, []) == []
    a, w = t(4, 8), t(8, 4)
    y = ctx.empty_tensor([4, 4])
    arr = lambda *v: (ctypes.c_int64 * len(v))(*v)
    i32 = lambda *v: (ctypes.c_int32 * len(v))(*v)
    with pytest.raises(capi.HipError):   # one buffer as two results
        capi.call("wdh_linear_group", 2, arr(a.handle, a.handle), arr(w.handle, w.handle), arr(0, 0),
                  arr(y.handle, y.handle), i32(4, 4), i32(4, 4), i32(8, 8), 0)
