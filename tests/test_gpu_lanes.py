"""Lanes (wdh_set_lane): a second HIP stream for captured runs and their transfers, so that two runs can be
in flight.  Through the C ABI: what a side lane accepts and refuses, that a run recorded there computes bit
for bit what lane 0 computes (launches scheduled as streams of K slabs included: each lane has its own
workspace), that replays on the two lanes may overlap, and that the buffer pool stays safe when blocks are
freed while a side lane is busy."""
import numpy as np
import pytest

from oracle import ref
from util import assert_bit_exact, assert_close_max
from webdnn_amd import capi
from webdnn_amd import hostops as H

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = H.HipContext(0).initialize()
    yield c
    c.set_lane(0)


def _rng(seed):
    return np.random.default_rng(seed)


def _chain(ctx, x, weights):
    """1x1 conv (stream-scheduled at this size when the plan picks it) -> 3x3 conv (minimal filtering) -> 1x1."""
    (w1, b1), (w2, b2), (w3, b3) = weights
    t1 = H.conv(ctx, x, w1, b1, epilogue="relu", constant_weights=True)
    t2 = H.conv(ctx, t1, w2, b2, pads=[1, 1, 1, 1], epilogue="relu", constant_weights=True)
    t1.dispose()
    y = H.conv(ctx, t2, w3, b3, epilogue="relu", residual=x, constant_weights=True)
    t2.dispose()
    return y


def test_a_side_lane_takes_recorded_work_and_transfers_only(ctx):
    A = ctx.move_tensor(_rng(1).standard_normal((64, 128)).astype(np.float32))
    B = ctx.move_tensor(_rng(2).standard_normal((128, 64)).astype(np.float32))
    want = H.matmul(ctx, A, B).get_data()
    with pytest.raises(capi.HipError):
        ctx.set_lane(4)                                                    # lanes 0..3
    with pytest.raises(capi.HipError):
        ctx.set_lane(-1)
    ctx.set_lane(1)
    try:
        with pytest.raises(capi.HipError) as e:
            H.matmul(ctx, A, B)
        assert "recorded work only" in str(e.value)
        # transfers work, and see what lane 0 wrote once lane 0 has been waited for (get_data did)
        assert_bit_exact(A.get_data(), _rng(1).standard_normal((64, 128)).astype(np.float32), "read on lane 1")
        fresh = ctx.move_tensor(np.arange(12, dtype=np.float32))          # alloc + upload on lane 1
        assert_bit_exact(fresh.get_data(), np.arange(12, dtype=np.float32), "upload and read on lane 1")
        fresh.dispose()
        ctx.graph_begin()
        try:
            out = H.matmul(ctx, A, B)
            with pytest.raises(capi.HipError) as e:
                capi.call("wdh_gemm_static", A.handle, B.handle, 0, out.handle, 1, 64, 64, 128, 0, 128, 1, 0, 64, 1, 0, 0,
                          1.0, 1.0, 0, 0)
            assert "lane 0" in str(e.value)
        finally:
            gid = ctx.graph_end()
        ctx.graph_begin()
        with pytest.raises(capi.HipError):
            ctx.set_lane(0)                                                # no lane switch while capturing ...
        with pytest.raises(capi.HipError) as e:
            ctx.graph_end()                                                # ... and the capture is abandoned
        assert "abandoned" in str(e.value)
        ctx.graph_launch(gid)
        assert_bit_exact(out.get_data(), want, "recorded on lane 1, replayed on lane 1")
        ctx.set_lane(0)
        ctx.graph_launch(gid)                                              # a graph is not tied to the lane it was recorded on
        assert_bit_exact(out.get_data(), want, "recorded on lane 1, replayed on lane 0")
        ctx.graph_destroy(gid)
        out.dispose()
    finally:
        ctx.set_lane(0)
    for t in (A, B):
        t.dispose()


def test_runs_recorded_on_both_lanes_agree_and_overlap(ctx):
    """A bottleneck block at ResNet-50's stage-3 size (its 1024 -> 256 conv is one the plan schedules as a
    stream of K slabs) recorded on lane 0 and on lane 1: equal to the eager result bit for bit, also when
    the two graphs are launched back to back without a wait in between, ten times over with fresh inputs."""
    r = _rng(7)
    def wb(co, ci, k):
        return (ctx.move_tensor((r.standard_normal((co, ci, k, k)) * np.sqrt(2.0 / (ci * k * k))).astype(np.float32)),
                ctx.move_tensor(r.standard_normal(co).astype(np.float32)))
    weights = [wb(256, 1024, 1), wb(256, 256, 3), wb(1024, 256, 1)]
    X = [r.uniform(0, 1, (32, 1024, 14, 14)).astype(np.float32) for _ in range(2)]
    xs = [ctx.move_tensor(x) for x in X]
    eager = []
    for x in xs:
        y = _chain(ctx, x, weights)
        eager.append(y.get_data())
        y.dispose()
    H.conv(ctx, xs[0], weights[0][0], weights[0][1], epilogue="relu").dispose()
    assert ctx.last_plan()["split"] == 0, ctx.last_plan()                  # (the stream schedule)
    ctx.sync()
    graphs = []
    for lane in (0, 1):
        ctx.set_lane(lane)
        ctx.graph_begin()
        try:
            y = _chain(ctx, xs[lane], weights)
        finally:
            gid = ctx.graph_end()
        graphs.append((gid, y))
        ctx.set_lane(0)
    for rep in range(10):
        fresh = [r.uniform(0, 1, (32, 1024, 14, 14)).astype(np.float32) if rep else X[i] for i in range(2)]
        want = eager
        if rep:
            want = []
            for i in range(2):
                capi.call("wdh_write", xs[i].handle, 0, fresh[i].ctypes.data, fresh[i].nbytes)
            ctx.sync()
        for lane in (0, 1):
            ctx.set_lane(lane)
            ctx.graph_launch(graphs[lane][0])
        got = []
        for lane in (0, 1):
            ctx.set_lane(lane)
            got.append(graphs[lane][1].get_data())
        ctx.set_lane(0)
        if rep:
            for i in range(2):
                y = _chain(ctx, xs[i], weights)
                want.append(y.get_data())
                y.dispose()
        for i in range(2):
            assert_bit_exact(got[i], want[i], "lane %d, repetition %d" % (i, rep))
    w = weights[1][0].get_data()
    assert_close_max(eager[0][:2], ref.unary("Relu", ref.binary("Add", ref.conv(
        ref.unary("Relu", ref.conv(ref.unary("Relu", ref.conv(X[0][:2], weights[0][0].get_data(), weights[0][1].get_data())),
                                   w, weights[1][1].get_data(), pads=[1, 1, 1, 1])),
        weights[2][0].get_data(), weights[2][1].get_data()), X[0][:2])), 1e-4, "the block against the oracle")
    # freeing while the side lane is busy: the block may not reach lane 0 before lane 1 has finished with it
    ctx.set_lane(1)
    ctx.graph_launch(graphs[1][0])
    ctx.set_lane(0)
    graphs[1][1].dispose()
    ctx.graph_destroy(graphs[1][0])
    filler = [ctx.move_tensor(np.zeros((32, 1024, 14, 14), np.float32)) for _ in range(3)]   # takes the freed blocks
    ctx.sync()
    graphs[0][1].dispose()
    ctx.graph_destroy(graphs[0][0])
    for t in filler + xs + [t for pair in weights for t in pair]:
        t.dispose()


def test_side_branch_of_a_recorded_run(ctx):
    """wdh_branch_begin / _end / _join: a projection shortcut recorded as a side branch of a residual block.
    Outside a recording the calls do nothing; a replay of the recording with the branch equals the eager result
    bit for bit, ten replays with fresh inputs; a branch left open is joined by wdh_graph_end; opening two at
    once or joining nothing abandons the recording."""
    r = _rng(11)
    def wb(co, ci, k):
        return (ctx.move_tensor((r.standard_normal((co, ci, k, k)) * np.sqrt(2.0 / (ci * k * k))).astype(np.float32)),
                ctx.move_tensor(r.standard_normal(co).astype(np.float32)))
    (w1, b1), (w2, b2), (w3, b3), (wd, bd) = wb(128, 256, 1), wb(128, 128, 3), wb(512, 128, 1), wb(512, 256, 1)
    X = r.uniform(0, 1, (8, 256, 28, 28)).astype(np.float32)
    x = ctx.move_tensor(X)

    def block(branch, join=True):
        if branch:
            capi.call("wdh_branch_begin")
        sc = H.conv(ctx, x, wd, bd, strides=[2, 2], constant_weights=True)
        if branch:
            capi.call("wdh_branch_end")
        t1 = H.conv(ctx, x, w1, b1, strides=[2, 2], epilogue="relu", constant_weights=True)
        t2 = H.conv(ctx, t1, w2, b2, pads=[1, 1, 1, 1], epilogue="relu", constant_weights=True)
        t1.dispose()
        if branch and join:
            capi.call("wdh_branch_join")
        y = H.conv(ctx, t2, w3, b3, epilogue="relu", residual=sc, constant_weights=True)
        t2.dispose()
        sc.dispose()
        return y

    def eager():
        y = block(False)
        out = y.get_data()
        y.dispose()
        return out

    want = eager()
    y = block(True)                                        # executing: the three calls are no-ops
    assert_bit_exact(y.get_data(), want, "eager with the branch calls")
    y.dispose()
    sc_ref = ref.conv(X[:1], wd.get_data(), bd.get_data(), strides=[2, 2])
    main = ref.unary("Relu", ref.conv(ref.unary("Relu", ref.conv(X[:1], w1.get_data(), b1.get_data(), strides=[2, 2])),
                                      w2.get_data(), b2.get_data(), pads=[1, 1, 1, 1]))
    assert_close_max(want[:1], ref.unary("Relu", ref.binary("Add", ref.conv(main, w3.get_data(), b3.get_data()), sc_ref)),
                     1e-4, "the block against the oracle")
    ctx.sync()
    for join in (True, False):                             # False: wdh_graph_end joins the branch itself
        ctx.graph_begin()
        try:
            out = block(True, join=join)
        finally:
            gid = ctx.graph_end()
        for rep in range(10):
            if rep:
                Xn = r.uniform(0, 1, X.shape).astype(np.float32)
                capi.call("wdh_write", x.handle, 0, Xn.ctypes.data, Xn.nbytes)
            ctx.graph_launch(gid)
            got = out.get_data()
            if not join:
                continue   # (its last conv is not ordered behind the shortcut: only the recording's end is)
            assert_bit_exact(got, eager(), "replay %d with a side branch" % rep)
        out.dispose()
        ctx.graph_destroy(gid)
        capi.call("wdh_write", x.handle, 0, X.ctypes.data, X.nbytes)
    for misuse in ("twice", "join"):
        ctx.graph_begin()
        with pytest.raises(capi.HipError):
            if misuse == "twice":
                capi.call("wdh_branch_begin")
                capi.call("wdh_branch_begin")
            else:
                capi.call("wdh_branch_join")
        with pytest.raises(capi.HipError) as e:
            ctx.graph_end()
        assert "abandoned" in str(e.value)
    y = block(True)
    assert_bit_exact(y.get_data(), want, "the library works on after an abandoned recording")
    y.dispose()
    for t in (x, w1, b1, w2, b2, w3, b3, wd, bd):
        t.dispose()
