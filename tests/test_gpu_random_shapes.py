"""Seeded random shapes through the C ABI against the oracle.

The fixed cases of test_gpu_parity.py aim at the shapes of the configs; these walk the index
arithmetic of the kernels with shapes nobody chose: broadcast patterns, permutations, slices with
negative steps, pooling geometries, Gemm edges in every layout, 1x1 convs on both sides of the
conditions for the in-place path.  Same criteria as there: bit-exact for layout / selection ops and
fp32 Add/Sub/Mul/Div, 1e-4 * max|ref| for Gemm / MatMul / Conv, 1e-6 / 1e-5 for Softmax / LayerNorm.
Every case prints nothing and is small (the oracle is the slow side); seeds are fixed.
"""
import numpy as np
import pytest

from oracle import ref
from util import assert_bit_exact, assert_close_max
from webdnn_amd import hostops as H

pytestmark = pytest.mark.gpu


def rng_for(name, i):
    return np.random.default_rng([sum(map(ord, name)), i])


def f32(r, shape, lo=-2.0, hi=2.0):
    return r.uniform(lo, hi, shape).astype(np.float32)


@pytest.mark.parametrize("i", range(40))
def test_binary_broadcast_patterns(ctx, i):
    r = rng_for("binary", i)
    rank = int(r.integers(1, 6))
    out = [int(r.choice([1, 2, 3, 4, 5, 7, 8, 16, 33, 64, 100])) for _ in range(rank)]
    if i % 5 == 0:
        out[-1] = int(r.choice([256, 784, 1024, 1100, 4100]))      # long innermost axis
    sides = []
    for _ in range(2):
        keep = int(r.integers(0, rank + 1))                         # drop leading axes
        shape = [d if r.random() < 0.6 else 1 for d in out[rank - keep:]]
        sides.append(shape)
    op = ["Add", "Sub", "Mul", "Div"][i % 4]
    if i % 7 == 3:
        L = r.integers(-1000, 1000, sides[0]).astype(np.int32)
        R = r.integers(1, 50, sides[1]).astype(np.int32)
    else:
        L, R = f32(r, sides[0]), f32(r, sides[1], 0.5, 3.0)
    got = H.binary(ctx, op, ctx.move_tensor(L), ctx.move_tensor(R))
    want = ref.binary(op, L, R)
    assert tuple(got.dims) == want.shape
    assert_bit_exact(got.get_data(), want, "%s %s %s" % (op, sides[0], sides[1]))


@pytest.mark.parametrize("i", range(30))
def test_transpose_random_permutations(ctx, i):
    r = rng_for("transpose", i)
    rank = int(r.integers(2, 6))
    shape = [int(r.choice([1, 2, 3, 5, 8, 16, 17, 32, 40, 64, 130])) for _ in range(rank)]
    while np.prod(shape) > 400_000:
        shape[int(np.argmax(shape))] //= 2
    perm = [int(p) for p in r.permutation(rank)]
    x = f32(r, shape)
    got = H.transpose(ctx, ctx.move_tensor(x), perm).get_data()
    assert_bit_exact(got, ref.transpose(x, perm), "%s perm %s" % (shape, perm))


@pytest.mark.parametrize("i", range(30))
def test_slice_and_concat_random(ctx, i):
    r = rng_for("slice", i)
    rank = int(r.integers(1, 5))
    shape = [int(r.choice([1, 3, 4, 7, 8, 12, 20, 33, 64, 260])) for _ in range(rank)]
    shape[-1] = int(r.choice([4, 8, 50, 64, 260, 1028]))
    while np.prod(shape) > 300_000:
        shape[int(np.argmax(shape[:-1] + [0]))] = max(1, shape[int(np.argmax(shape[:-1] + [0]))] // 2)
    x = f32(r, shape)
    axes = sorted(int(a) for a in r.choice(rank, size=int(r.integers(1, rank + 1)), replace=False))
    starts, ends, steps = [], [], []
    for a in axes:
        n = shape[a]
        step = int(r.choice([1, 1, 1, 2, 3, -1, -2]))
        lo, hi = sorted(int(v) for v in r.integers(-n - 2, n + 3, 2))
        if step < 0:
            lo, hi = hi, lo
        starts.append(lo); ends.append(hi); steps.append(step)
    want = ref.slice_(x, starts, ends, axes, steps)
    got = H.slice_(ctx, ctx.move_tensor(x), starts, ends, axes, steps)
    assert tuple(got.dims) == want.shape
    assert_bit_exact(got.get_data(), want, "slice %s %s %s %s of %s" % (starts, ends, axes, steps, shape))
    # concat of the tensor with a differently sized sibling along a random axis
    ax = int(r.integers(0, rank))
    other = list(shape)
    other[ax] = int(r.choice([1, 2, 5, 8]))
    y = f32(r, other)
    got = H.concat(ctx, [ctx.move_tensor(x), ctx.move_tensor(y), ctx.move_tensor(x)], ax).get_data()
    assert_bit_exact(got, ref.concat([x, y, x], ax), "concat axis %d of %s + %s" % (ax, shape, other))


@pytest.mark.parametrize("i", range(30))
def test_maxpool_random_geometry(ctx, i):
    r = rng_for("maxpool", i)
    h, w = int(r.integers(5, 70)), int(r.choice([6, 8, 13, 16, 24, 31, 48, 56, 100]))
    kh, kw = int(r.integers(1, 5)), int(r.integers(1, 5))
    sh, sw = int(r.integers(1, 4)), int(r.integers(1, 4))
    dh, dw = int(r.integers(1, 3)), int(r.integers(1, 3))
    if dh * (kh - 1) + 1 > h or dw * (kw - 1) + 1 > w:
        dh = dw = 1
        kh, kw = min(kh, h), min(kw, w)
    pads = [int(r.integers(0, (dh * (kh - 1)) // 2 + 1)), int(r.integers(0, (dw * (kw - 1)) // 2 + 1)),
            int(r.integers(0, (dh * (kh - 1)) // 2 + 1)), int(r.integers(0, (dw * (kw - 1)) // 2 + 1))]
    x = f32(r, (int(r.integers(1, 3)), int(r.integers(1, 5)), h, w))
    x[0, 0, 0, 0] = np.nan
    attrs = dict(kernel_shape=[kh, kw], strides=[sh, sw], dilations=[dh, dw], pads=pads, ceil_mode=int(i % 3 == 0))
    want = ref.maxpool(x, **attrs)
    got = H.maxpool(ctx, ctx.move_tensor(x), **attrs)
    assert tuple(got.dims) == want.shape
    assert_bit_exact(got.get_data(), want, "maxpool %s on %s" % (attrs, x.shape))


@pytest.mark.parametrize("i", range(40))
def test_gemm_random_edges_and_layouts(ctx, i):
    r = rng_for("gemm", i)
    m, n = int(r.choice([1, 5, 31, 32, 64, 65, 100, 130, 200, 257])), int(r.choice([1, 4, 32, 33, 64, 92, 129, 256, 300]))
    k = int(r.choice([1, 3, 16, 17, 32, 48, 100, 256, 850, 1030]))
    ta, tb = int(r.integers(0, 2)), int(r.integers(0, 2))
    A = f32(r, (k, m) if ta else (m, k), -1, 1)
    B = f32(r, (n, k) if tb else (k, n), -1, 1)
    cshape = [None, (n,), (1, n), (m, 1), (m, n), (1,), ()][i % 7]
    C = f32(r, cshape) if cshape is not None else None
    alpha, beta = (1.0, 1.0) if i % 3 else (float(r.uniform(-2, 2)), float(r.uniform(-2, 2)))
    want = ref.gemm(A, B, C, alpha, beta, ta, tb)
    tc = ctx.move_tensor(C) if C is not None else None
    got = H.gemm(ctx, ctx.move_tensor(A), ctx.move_tensor(B), tc, alpha, beta, ta, tb).get_data()
    assert_close_max(got, want, 1e-4, "gemm m%d n%d k%d ta%d tb%d C%s" % (m, n, k, ta, tb, cshape))


@pytest.mark.parametrize("i", range(24))
def test_matmul_random_batches(ctx, i):
    r = rng_for("matmul", i)
    b, m, n, k = int(r.choice([1, 2, 3, 8])), int(r.choice([1, 7, 64, 100, 130])), int(r.choice([1, 32, 33, 64, 100])), \
        int(r.choice([1, 16, 32, 40, 100, 260]))
    form = i % 4
    if form == 0:
        A, B = f32(r, (b, m, k), -1, 1), f32(r, (b, k, n), -1, 1)
    elif form == 1:
        A, B = f32(r, (b, m, k), -1, 1), f32(r, (k, n), -1, 1)       # broadcast B
    elif form == 2:
        A, B = f32(r, (m, k), -1, 1), f32(r, (b, k, n), -1, 1)       # broadcast A
    else:
        A, B = f32(r, (k,), -1, 1), f32(r, (k, n), -1, 1)            # 1-D promotion
    want = ref.matmul(A, B)
    got = H.matmul(ctx, ctx.move_tensor(A), ctx.move_tensor(B))
    assert tuple(got.dims) == want.shape
    assert_close_max(got.get_data(), want, 1e-4, "matmul %s x %s" % (A.shape, B.shape))


@pytest.mark.parametrize("i", range(30))
def test_conv_random_geometry(ctx, i):
    r = rng_for("conv", i)
    if i % 2 == 0:
        # 1x1: channel counts, plane sizes and batches on both sides of the in-place path's conditions
        k, pads, strides, dil = 1, [0, 0, 0, 0], [[1, 1], [1, 1], [2, 2]][i % 3], [1, 1]
        group = int(r.choice([1, 1, 2]))
        cin = int(r.choice([8, 16, 24, 32, 64])) * group
        cout = int(r.choice([8, 24, 64, 72])) * group
        h, w = int(r.choice([4, 7, 8, 14, 16])), int(r.choice([4, 7, 8, 14, 16]))
        n = int(r.choice([1, 2, 4, 8, 16]))
    else:
        k = int(r.choice([2, 3, 3, 5]))
        dil = [int(r.integers(1, 3)), int(r.integers(1, 3))]
        strides = [int(r.integers(1, 3)), int(r.integers(1, 3))]
        pads = [int(r.integers(0, k)) for _ in range(4)]
        group = int(r.choice([1, 1, 2, 4]))
        cin, cout = int(r.choice([1, 2, 3, 5])) * group, int(r.choice([1, 2, 4, 7])) * group
        h, w = int(r.integers(dil[0] * (k - 1) + 1, 24)), int(r.integers(dil[1] * (k - 1) + 1, 24))
        n = int(r.integers(1, 4))
    X = f32(r, (n, cin, h, w), 0, 1)
    W = f32(r, (cout, cin // group, k, k), -0.5, 0.5)
    Bs = f32(r, (cout,)) if i % 4 else None
    want = ref.conv(X, W, Bs, dil, group, None, pads, strides)
    tb = ctx.move_tensor(Bs) if Bs is not None else None
    got = H.conv(ctx, ctx.move_tensor(X), ctx.move_tensor(W), tb, dil, group, None, pads, strides)
    assert tuple(got.dims) == want.shape
    assert_close_max(got.get_data(), want, 1e-4, "conv n%d cin%d %dx%d cout%d k%d pads%s s%s d%s g%d"
                     % (n, cin, h, w, cout, k, pads, strides, dil, group))


@pytest.mark.parametrize("i", range(24))
def test_conv3x3_minimal_filtering_random_geometry(ctx, i):
    """3x3 stride-1 convs through both minimal-filtering forms (and, every third case, through whatever the
    plan picks) on random planes, pads 0..2 per side, channel counts in multiples of 16, with and without
    bias, residual and Relu."""
    r = rng_for("wino", i)
    mode = [2, 3, 1][i % 3]
    cin = 16 * int(r.integers(1, 13 if mode != 1 else 17))
    cout = 16 * int(r.integers(1, 13 if mode != 1 else 17)) if i % 4 else int(r.integers(1, 40))
    pads = [int(r.integers(0, 3)) for _ in range(4)]
    h, w = int(r.integers(3, 30)), int(r.integers(3, 30))
    n = int(r.integers(1, 6))
    X = f32(r, (n, cin, h, w), -1 if i % 2 else 0, 1)
    W = (f32(r, (cout, cin, 3, 3), -1, 1) * np.float32(np.sqrt(2.0 / (cin * 9)))).astype(np.float32)
    Bs = f32(r, (cout,)) if i % 5 else None
    want = ref.conv(X, W, Bs, None, 1, None, pads, None)
    R = f32(r, want.shape) if i % 2 else None
    if R is not None:
        want = ref.binary("Add", want, R)
    if i % 3 == 0:
        want = ref.unary("Relu", want)
    try:
        ctx.set_option("conv3x3_winograd", mode)
        got = H.conv(ctx, ctx.move_tensor(X), ctx.move_tensor(W), ctx.move_tensor(Bs) if Bs is not None else None,
                     None, 1, None, pads, None, "relu" if i % 3 == 0 else None,
                     ctx.move_tensor(R) if R is not None else None)
        form = ctx.last_plan()["form"]
    finally:
        ctx.set_option("conv3x3_winograd", 1)
    if mode != 1:
        assert form.startswith("conv 3x3, F(%dx%d,3x3)" % ((2, 2) if mode == 2 else (4, 4))), form
    assert tuple(got.dims) == want.shape
    assert_close_max(got.get_data(), want, 1e-4, "3x3 n%d cin%d %dx%d cout%d pads%s mode %d (%s)"
                     % (n, cin, h, w, cout, pads, mode, form))


@pytest.mark.parametrize("i", range(40))
def test_conv_random_network_sized_geometry(ctx, i):
    """1x1 and 3x3 convs with the channel counts, planes and batches of real networks (16 .. 512 channels, planes up
    to 59 x 59, stride 1 or 2, ragged output channels, with and without bias, residual and Relu): whichever form
    the plan picks -- in place, in place with stride 2, LDS tile, minimal filtering, gathered; whole tiles, tiles
    cut along K, small products -- against the oracle."""
    r = rng_for("netconv", i)
    k = int(r.choice([1, 1, 3, 3, 3]))
    s = int(r.choice([1, 1, 2]))
    n = int(r.choice([1, 2, 4, 8, 16, 32]))
    cin = 16 * int(r.integers(1, 33))
    cout = int(r.choice([16 * int(r.integers(1, 33)), int(r.integers(1, 600))]))
    h, w = int(r.integers(max(k, 4), 60)), int(r.integers(max(k, 4), 60))
    pads = [int(r.integers(0, k)) for _ in range(4)] if k == 3 else [0] * 4
    macs = n * cin * cout * (h // s) * (w // s) * k * k
    if macs > 6e8:
        n = max(1, int(n * 6e8 / macs))          # (keeps the oracle's share of a case under a second)
    X = f32(r, (n, cin, h, w), -1 if i % 2 else 0, 1)
    W = (f32(r, (cout, cin, k, k), -1, 1) * np.float32(np.sqrt(2.0 / (cin * k * k)))).astype(np.float32)
    Bs = f32(r, (cout,)) if i % 3 else None
    want = ref.conv(X, W, Bs, None, 1, None, pads, [s, s])
    R = f32(r, want.shape) if i % 2 else None
    if R is not None:
        want = ref.binary("Add", want, R)
    relu = i % 5 < 3
    if relu:
        want = ref.unary("Relu", want)
    got = H.conv(ctx, ctx.move_tensor(X), ctx.move_tensor(W), ctx.move_tensor(Bs) if Bs is not None else None, None, 1, None,
                 pads, [s, s], "relu" if relu else None, ctx.move_tensor(R) if R is not None else None)
    plan = ctx.last_plan()
    assert tuple(got.dims) == want.shape
    assert_close_max(got.get_data(), want, 1e-4, "conv n%d cin%d %dx%d cout%d k%d s%d pads%s (%s, %s, split %d)"
                     % (n, cin, h, w, cout, k, s, pads, plan["form"], plan["tile"], plan["split"]))


@pytest.mark.parametrize("i", range(20))
def test_row_reductions_random_lengths(ctx, i):
    r = rng_for("rows", i)
    rows = int(r.choice([1, 3, 64, 65, 200]))
    length = int(r.choice([1, 2, 7, 49, 64, 100, 128, 132, 256, 850, 1024, 1500, 2048, 2100, 4096]))
    x = f32(r, (rows, length), -4, 4)
    assert_close_max(H.softmax(ctx, ctx.move_tensor(x)).get_data(), ref.softmax(x), 1e-6, "softmax %s" % (x.shape,))
    g, b = f32(r, (length,)), f32(r, (length,))
    got = H.layer_normalization(ctx, ctx.move_tensor(x), ctx.move_tensor(g), ctx.move_tensor(b)).get_data()
    assert_close_max(got, ref.layernorm_decomposed(x, g, b, 1e-5), 1e-5, "layernorm %s" % (x.shape,))
    from util import ulp_diff
    rm = H.reduce_mean_last(ctx, ctx.move_tensor(x)).get_data()
    assert ulp_diff(rm, ref.reduce_mean_last(x)).max() <= 1
