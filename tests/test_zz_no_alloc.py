"""wdh_gemm_static, the entry point that allocates nothing: through the C ABI, against wdh_gemm
(the existing entry point it is a variant of), bit for bit, on two calls in a row of which the second
is the smaller, so that the static workspace still holds the first call's partial sums."""
import ctypes

import numpy as np
import pytest

from oracle import ref
from util import assert_bit_exact, assert_close_max
from webdnn_amd import capi

pytestmark = pytest.mark.gpu


def mem_stats():
    a, b, c = ctypes.c_uint64(), ctypes.c_uint64(), ctypes.c_uint64()
    capi.call("wdh_mem_stats", ctypes.byref(a), ctypes.byref(b), ctypes.byref(c))
    return a.value, b.value, c.value


def gemm_both(ctx, A, B, C, R, alpha, beta, epi):
    """Runs wdh_gemm and wdh_gemm_static on the same device buffers; returns (pooled, static)."""
    batch, m, k = A.shape
    n = B.shape[2]
    ta, tb, tc, tr = (ctx.move_tensor(v) for v in (A, B, C, R))
    y0, y1 = ctx.empty_tensor([batch, m, n]), ctx.empty_tensor([batch, m, n])
    args = lambda y: (ta.handle, tb.handle, tc.handle, y.handle, batch, m, n, k, m * k, k, 1, k * n, n, 1,
                      0, 1, alpha, beta, epi, tr.handle)
    capi.call("wdh_gemm", *args(y0))
    ctx.sync()
    # wdh_gemm left its partial-sum block in the pool's cache; with the cache emptied, a static call
    # that took a block from the pool and gave it back would show up as cached bytes (or a new peak)
    capi.call("wdh_trim", 0)
    before = mem_stats()
    assert before[1] == 0, before
    capi.call("wdh_gemm_static", *args(y1))
    after = mem_stats()
    assert after == before, "the call took memory from the pool or the driver: %s -> %s" % (before, after)
    # the callers it is for: a stream in capture mode (an allocation would fail the capture)
    ctx.sync()
    ctx.graph_begin()
    try:
        capi.call("wdh_gemm_static", *args(y1))
    finally:
        gid = ctx.graph_end()
    assert mem_stats() == before
    ctx.graph_launch(gid)
    ctx.sync()
    ctx.graph_destroy(gid)
    out = y0.get_data(), y1.get_data()
    for t in (ta, tb, tc, tr, y0, y1):
        t.dispose()
    return out


def test_static_workspace_gemm_equals_pooled_gemm_twice(ctx):
    rng = np.random.default_rng(77)
    # deep and skinny: the planner cuts every tile along K (partial sums + reduce pass)
    shapes = [(2, 100, 4096, 70), (1, 40, 1536, 33)]
    for batch, m, k, n in shapes:
        A = rng.uniform(-1, 1, (batch, m, k)).astype(np.float32)
        B = rng.uniform(-1, 1, (batch, k, n)).astype(np.float32)
        C = rng.uniform(-1, 1, (n,)).astype(np.float32)
        R = rng.standard_normal((batch, m, n)).astype(np.float32)
        pooled, static = gemm_both(ctx, A, B, C, R, 0.5, 2.0, 1)
        assert_bit_exact(static, pooled, "wdh_gemm_static vs wdh_gemm %s" % ((batch, m, k, n),))
        want = np.stack([ref.gemm(A[b], B[b], C, 0.5, 2.0) for b in range(batch)])
        want = ref.unary("Relu", ref.binary("Add", want, R))
        assert_close_max(static, want, 1e-4, "wdh_gemm_static vs the oracle")
    # forced splits: every tile leaves partial sums in the workspace, large call first
    try:
        for split, (batch, m, k, n) in ((8, (1, 300, 1024, 500)), (3, (1, 64, 256, 64))):
            ctx.set_option("split_k", split)
            A = rng.uniform(-1, 1, (batch, m, k)).astype(np.float32)
            B = rng.uniform(-1, 1, (batch, k, n)).astype(np.float32)
            C = rng.uniform(-1, 1, (n,)).astype(np.float32)
            R = np.zeros((batch, m, n), np.float32)
            pooled, static = gemm_both(ctx, A, B, C, R, 1.0, 1.0, 0)
            assert_bit_exact(static, pooled, "split %d" % split)
            assert_close_max(static, np.stack([ref.gemm(A[0], B[0], C)]), 1e-4, "split %d vs the oracle" % split)
    finally:
        ctx.set_option("split_k", -1)


def test_static_workspace_rejects_what_does_not_fit(ctx):
    m = n = 1024
    k = 2048
    ta, tb = ctx.empty_tensor([m, k]), ctx.empty_tensor([k, n])
    y = ctx.empty_tensor([m, n])
    args = (ta.handle, tb.handle, 0, y.handle, 1, m, n, k, 0, k, 1, 0, n, 1, 0, 0, 1.0, 1.0, 0, 0)
    try:
        ctx.set_option("split_k", 16)     # 256 tiles x 16 chunks x 16 KiB = 64 MiB of partial sums
        with pytest.raises(capi.HipError) as err:
            capi.call("wdh_gemm_static", *args)
        assert err.value.code == -2 and "static workspace" in str(err.value)
        capi.call("wdh_gemm", *args)      # the pooled form takes it
        ctx.set_option("split_k", 1)      # unsplit: no workspace at all
        capi.call("wdh_gemm_static", *args)
    finally:
        ctx.set_option("split_k", -1)
    ctx.sync()
    for t in (ta, tb, y):
        t.dispose()
