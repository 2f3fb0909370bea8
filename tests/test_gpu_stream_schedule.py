"""Contraction launches scheduled as streams of K slabs (wdh_set_option "stream_k"): a fixed grid of
resident workgroups, each multiplying an equal contiguous share of all K slabs of the launch; a tile
shared by neighbouring workgroups is added up, in K order, by the workgroup that holds its last slabs.
Same criteria as every Gemm / Conv test (max|diff| <= 1e-4 * max|ref| against the oracle); the order
of a tile's partial sums is fixed, so repeated launches give identical bits."""
import itertools

import numpy as np
import pytest

from oracle import ref
from util import assert_bit_exact, assert_close_max
from webdnn_amd import hostops as H

pytestmark = pytest.mark.gpu

TOL = 1e-4
RNG = np.random.default_rng(31)


def uni(*shape, lo=-1.0, hi=1.0):
    return RNG.uniform(lo, hi, shape).astype(np.float32)


def he(cout, cin, k):
    return (RNG.standard_normal((cout, cin, k, k)) * np.sqrt(2.0 / (cin * k * k))).astype(np.float32)


@pytest.fixture
def stream_always(ctx):
    """Every launch that has a stream form takes it, whatever the plan would choose."""
    ctx.set_option("stream_k", 2)
    ctx.set_option("conv3x3_winograd", 0)       # the direct forms are what is scheduled here
    yield ctx
    for name, value in (("stream_k", 1), ("stream_wgs", 4), ("contraction_tile", -1), ("conv3x3_winograd", 1)):
        ctx.set_option(name, value)


def gemm(ctx, A, B, C=None, alpha=1.0, beta=1.0, ta=0, tb=0, epilogue=None):
    tc = ctx.move_tensor(C) if C is not None else None
    return H.gemm(ctx, ctx.move_tensor(A), ctx.move_tensor(B), tc, alpha, beta, ta, tb, epilogue).get_data()


def conv(ctx, X, W, B=None, pads=None, strides=None, group=1, dil=None, epilogue=None, R=None):
    tb = ctx.move_tensor(B) if B is not None else None
    tr = ctx.move_tensor(R) if R is not None else None
    return H.conv(ctx, ctx.move_tensor(X), ctx.move_tensor(W), tb, dilations=dil, group=group, pads=pads,
                  strides=strides, epilogue=epilogue, residual=tr).get_data()


GEMM_SHAPES = [(256, 1024, 512), (300, 500, 1024), (64, 64, 4096), (1000, 32, 2048), (130, 250, 1000),
               (129, 127, 77), (8, 8, 16), (2048, 2048, 576), (512, 96, 3000)]


@pytest.mark.parametrize("tile", [-1, 0, 2, 3, 4])
@pytest.mark.parametrize("m,n,k", GEMM_SHAPES)
def test_gemm_as_a_stream(stream_always, m, n, k, tile):
    ctx = stream_always
    ctx.set_option("gemm_wavesplit", 0)
    try:
        ctx.set_option("contraction_tile", tile)
        A, B, C = uni(m, k), uni(n, k), uni(n)
        got = gemm(ctx, A, B, C, 0.75, -1.25, 0, 1, "relu")
        plan = ctx.last_plan()
        want = ref.unary("Relu", ref.gemm(A, B, C, 0.75, -1.25, 0, 1))
        assert_close_max(got, want, TOL, "stream gemm %s tile %d (%s)" % ((m, n, k), tile, plan))
        # the stream schedule did run (operand rows that are not 16-byte aligned have no stream form)
        assert plan["split"] == (0 if k % 4 == 0 else 1), plan
        again = gemm(ctx, A, B, C, 0.75, -1.25, 0, 1, "relu")
        assert_bit_exact(again, got, "the same launch twice")
    finally:
        ctx.set_option("gemm_wavesplit", 1)


@pytest.mark.parametrize("ta,tb", list(itertools.product((0, 1), (0, 1))))
def test_gemm_layouts_and_batches_as_a_stream(stream_always, ta, tb):
    ctx = stream_always
    ctx.set_option("gemm_wavesplit", 0)
    try:
        m, n, k = 200, 264, 1536
        A = uni(k, m) if ta else uni(m, k)
        B = uni(n, k) if tb else uni(k, n)
        C = uni(m, n)
        got = gemm(ctx, A, B, C, 1.0, 0.5, ta, tb)
        assert ctx.last_plan()["split"] == 0
        assert_close_max(got, ref.gemm(A, B, C, 1.0, 0.5, ta, tb), TOL, "layout %d%d" % (ta, tb))
    finally:
        ctx.set_option("gemm_wavesplit", 1)
    # batched MatMul (z > 1): [5, 70, 640] x [5, 640, 90]
    a, b = uni(5, 70, 640), uni(5, 640, 90)
    got = H.matmul(ctx, ctx.move_tensor(a), ctx.move_tensor(b)).get_data()
    want = np.stack([ref.gemm(a[i], b[i]) for i in range(5)])
    assert_close_max(got, want, TOL, "batched matmul")


CONVS = [
    # n, cin, h, w, cout, k, stride, pad, group
    (8, 256, 14, 14, 256, 3, 1, 1, 1),      # LDS-tile 3x3, few tiles, deep K
    (4, 512, 7, 7, 512, 3, 1, 1, 1),
    (2, 64, 56, 56, 64, 3, 1, 1, 1),
    (3, 32, 20, 24, 48, 3, 1, 1, 2),        # groups
    (8, 1024, 14, 14, 256, 1, 1, 0, 1),     # 1x1 in place
    (8, 256, 14, 14, 1024, 1, 1, 0, 1),
    (4, 2048, 7, 7, 512, 1, 1, 0, 1),       # 7x7 planes
    (4, 512, 28, 28, 256, 1, 2, 0, 1),      # stride-2 1x1: in place, every other pixel
    (4, 512, 14, 14, 256, 1, 2, 0, 1),      # stride-2 1x1 onto 7x7 planes: gathered
    (2, 24, 17, 19, 40, 5, 2, 2, 1),        # gathered, 25 taps, ragged K
    (1, 16, 30, 30, 8, 7, 1, 3, 1),         # 49 taps
]


@pytest.mark.parametrize("tile", [-1, 0, 2, 3, 4])
@pytest.mark.parametrize("shape", CONVS)
def test_conv_as_a_stream(stream_always, shape, tile):
    ctx = stream_always
    n, cin, h, w, cout, k, s, p, g = shape
    ctx.set_option("contraction_tile", tile)
    X, W, B = uni(n, cin, h, w, lo=0.0), he(cout, cin // g, k), uni(cout)
    oh, ow = (h + 2 * p - k) // s + 1, (w + 2 * p - k) // s + 1
    R = uni(n, cout, oh, ow)
    got = conv(ctx, X, W, B, pads=[p] * 4, strides=[s, s], group=g, epilogue="relu", R=R)
    plan = ctx.last_plan()
    want = ref.unary("Relu", ref.binary("Add", ref.conv(X, W, B, pads=[p] * 4, strides=[s, s], group=g), R))
    assert_close_max(got, want, TOL, "stream conv %s tile %d (%s)" % (shape, tile, plan))
    assert plan["split"] == (0 if (cin // g * k * k) % 4 == 0 else 1), plan
    again = conv(ctx, X, W, B, pads=[p] * 4, strides=[s, s], group=g, epilogue="relu", R=R)
    assert_bit_exact(again, got, "the same launch twice")


@pytest.mark.parametrize("wgs", [1, 2, 3, 8])
def test_any_number_of_resident_workgroups(stream_always, wgs):
    ctx = stream_always
    ctx.set_option("stream_wgs", wgs)
    X, W, B = uni(8, 256, 14, 14, lo=0.0), he(256, 256, 3), uni(256)
    got = conv(ctx, X, W, B, pads=[1] * 4)
    assert ctx.last_plan()["split"] == 0
    assert_close_max(got, ref.conv(X, W, B, pads=[1] * 4), TOL, "3x3 with %d workgroups per CU" % wgs)
    A, Bm = uni(333, 2000), uni(2000, 222)
    got = gemm(ctx, A, Bm)
    assert_close_max(got, ref.gemm(A, Bm), TOL, "gemm with %d workgroups per CU" % wgs)


def test_stream_and_tile_per_workgroup_schedules_agree(ctx):
    """The default plan picks the stream schedule for deep 1x1 convs on small planes (ResNet-50's
    1024 -> 256 on 14x14); switched off, the same layer is cut into chunks with a reduce pass.  Two
    summation orders of the same products."""
    X, W, B = uni(32, 1024, 14, 14, lo=0.0), he(256, 1024, 1), uni(256)     # 392 tiles: more than one per CU
    want = ref.conv(X, W, B)
    try:
        outs = {}
        for mode in (0, 1, 2):
            ctx.set_option("stream_k", mode)
            outs[mode] = conv(ctx, X, W, B)
            split = ctx.last_plan()["split"]
            assert (split == 0) == (mode != 0), (mode, ctx.last_plan())
            assert_close_max(outs[mode], want, TOL, "stream_k=%d" % mode)
        assert_bit_exact(outs[1], outs[2], "chosen or forced, the same schedule")
    finally:
        ctx.set_option("stream_k", 1)


def test_launches_back_to_back_leave_the_flags_clear(stream_always):
    """Six stream launches of different shapes without a synchronisation between them, three times over:
    every launch finds the flags of the partial tiles at zero, as the launch before it left them."""
    ctx = stream_always
    jobs = []
    for (n, cin, hw, cout, k) in ((8, 256, 14, 256, 3), (4, 512, 7, 512, 3), (8, 1024, 14, 256, 1), (4, 2048, 7, 512, 1),
                                  (2, 128, 28, 128, 3), (8, 256, 14, 1024, 1)):
        X, W, B = uni(n, cin, hw, hw, lo=0.0), he(cout, cin, k), uni(cout)
        jobs.append((ctx.move_tensor(X), ctx.move_tensor(W), ctx.move_tensor(B), [k // 2] * 4,
                     ref.conv(X, W, B, pads=[k // 2] * 4)))
    for rep in range(3):
        outs = [H.conv(ctx, x, w, b, pads=pads) for x, w, b, pads, _ in jobs]
        for i, (out, job) in enumerate(zip(outs, jobs)):
            assert_close_max(out.get_data(), job[4], TOL, "round %d launch %d" % (rep, i))
            out.dispose()


def test_stream_launches_replay_from_a_captured_graph(stream_always):
    ctx = stream_always
    X, W, B = uni(8, 256, 14, 14, lo=0.0), he(256, 256, 3), uni(256)
    W2 = he(512, 256, 1)
    tx, tw, tb, tw2 = (ctx.move_tensor(v) for v in (X, W, B, W2))

    def net():
        a = H.conv(ctx, tx, tw, tb, pads=[1] * 4, epilogue="relu")
        b = H.conv(ctx, a, tw2, None)
        a.dispose()
        return b

    eager = net()
    want = eager.get_data()
    eager.dispose()
    ctx.sync()
    ctx.graph_begin()
    try:
        out = net()
    finally:
        gid = ctx.graph_end()
    for rep in range(4):
        ctx.graph_launch(gid)
        ctx.sync()
        assert_bit_exact(out.get_data(), want, "replay %d" % rep)
        H.unary(ctx, "Relu", tx).dispose()      # eager work between the replays
    out.dispose()
    ctx.graph_destroy(gid)


def test_a_wait_that_gives_up_is_reported_and_the_library_goes_on(stream_always):
    """stream_spin = 0: a finishing workgroup polls a neighbour's flag once.  Whether that one poll already
    finds the flag raised depends on timing, so the launch either succeeds or the next synchronisation
    reports the wait that gave up; either way every kernel ends, and the launch after it is correct."""
    from webdnn_amd import capi

    ctx = stream_always
    X, W, B = uni(8, 256, 14, 14, lo=0.0), he(256, 256, 3), uni(256)
    want = ref.conv(X, W, B, pads=[1] * 4)
    ctx.set_option("stream_spin", 0)
    try:
        try:
            got = conv(ctx, X, W, B, pads=[1] * 4)
            assert_close_max(got, want, TOL, "no wait had to give up")
        except capi.HipError as err:
            assert err.code == -4 and "partial tile" in str(err), err
    finally:
        ctx.set_option("stream_spin", 1 << 22)
    ctx.sync()
    assert_close_max(conv(ctx, X, W, B, pads=[1] * 4), want, TOL, "the launch after")
