"""nnvhip_estimate_ranges_static: Star.estimateRanges through the entry point that allocates nothing
(its partial sums go to a fixed workspace in device memory), against nnvhip_estimate_ranges on the same
sets.  Two calls in a row share the workspace; the second set is smaller than the first, so anything
the first call left behind there would show."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _both(nnv, V, plb, pub):
    from nnv_amd import _lib
    from tests.gpu_util import DeviceDoubles
    ctx = nnv.default_context()
    N, n = V.shape[0], V.shape[1] - 1
    S = nnv.Star(V, np.zeros((1, n)), np.zeros(1), plb, pub)
    lb_d, ub_d = DeviceDoubles(N), DeviceDoubles(N)      # the caller's own output buffers (NaN-filled)
    used0, cached0 = ctx.pool_stats()
    _lib.check(ctx.lib.nnvhip_estimate_ranges_static(ctx.handle, S._h.h, lb_d.ptr, ub_d.ptr))
    ctx.synchronize()
    assert ctx.pool_stats() == (used0, cached0), "the call took memory from the pool"
    got = lb_d.get(), ub_d.get()
    exp = S.estimateRanges()          # the existing entry point (workspace from the context's pool)
    return got, exp


def test_static_workspace_ranges_equal_the_pooled_entry_point():
    import nnv_amd as nnv
    from oracle import nnv_oracle as o
    from tests.gpu_util import assert_close
    rs = np.random.RandomState(5)
    # first call: many column chunks (the workspace holds 9 x 4 x 2000 partial sums afterwards);
    # second call: a smaller set with fewer rows, fewer chunks; third: a single chunk (no reduction pass)
    for (N, n) in ((2000, 600), (333, 150), (70, 9)):
        V = rs.randn(N, n + 1)
        plb = -rs.rand(n) - 0.1
        pub = rs.rand(n) + 0.1
        (lb, ub), (elb, eub) = _both(nnv, V, plb, pub)
        # same kernels, same chunking: the values are the same bits; the bar of the fp64 path is 1e-9
        assert np.array_equal(lb, elb) and np.array_equal(ub, eub), "N=%d n=%d" % (N, n)
        olb, oub = o.estimate_ranges(o.OStar(V, np.zeros((1, n)), np.zeros(1), plb, pub))
        assert_close(lb, olb, "lb vs oracle")
        assert_close(ub, oub, "ub vs oracle")


def test_static_workspace_limits_are_errors():
    import nnv_amd as nnv
    from nnv_amd import _lib
    from tests.gpu_util import DeviceDoubles
    ctx = nnv.default_context()
    cfg_lb, cfg_ub = -np.ones(40), np.ones(40)
    net_in = nnv.Star(cfg_lb, cfg_ub)
    L = nnv.FullyConnectedLayer(np.random.RandomState(1).randn(64, 40), np.zeros(64))
    R = nnv.ReluLayer().reach(L.reach(net_in, "relax-star-area"), "relax-star-area", [], 1)
    buf = DeviceDoubles(64)
    # a ReLU output whose row reset / appended columns are not in memory yet would need a buffer: refused
    st = ctx.lib.nnvhip_estimate_ranges_static(ctx.handle, R._h.h, buf.ptr, None)
    assert st == _lib.ERR_ARG and b"not in memory" in ctx.lib.nnvhip_last_error()
    R.V                                    # a read writes them ...
    _lib.check(ctx.lib.nnvhip_estimate_ranges_static(ctx.handle, R._h.h, buf.ptr, None))
    ctx.synchronize()
    assert np.array_equal(buf.get(), R.estimateRanges()[0])
    assert ctx.lib.nnvhip_estimate_ranges_static(ctx.handle, R._h.h, None, None) == _lib.ERR_ARG


def test_two_contexts_share_the_workspace_in_turn_and_cached_ranges_need_none():
    """Two contexts (two streams) on the one GPU call the entry point alternately without synchronising in
    between: every result must be the context's own.  A handle that already caches its ranges is served from
    the cache."""
    import nnv_amd as nnv
    from nnv_amd import _lib
    from tests.gpu_util import DeviceDoubles
    a, b = _lib.Context(0), _lib.Context(0)
    rs = np.random.RandomState(9)
    sets, outs = [], []
    for i in range(6):
        ctx = a if i % 2 == 0 else b
        N, n = 1500 - 100 * i, 500 + 30 * i
        V = rs.randn(N, n + 1)
        S = nnv.Star(V, np.zeros((1, n)), np.zeros(1), -np.ones(n), np.ones(n), ctx=ctx)
        lb_d, ub_d = DeviceDoubles(N), DeviceDoubles(N)
        _lib.check(ctx.lib.nnvhip_estimate_ranges_static(ctx.handle, S._h.h, lb_d.ptr, ub_d.ptr))
        sets.append((ctx, S))
        outs.append((lb_d, ub_d))
    a.synchronize()
    b.synchronize()
    for (ctx, S), (lb_d, ub_d) in zip(sets, outs):
        elb, eub = S.estimateRanges()
        assert np.array_equal(lb_d.get(), elb) and np.array_equal(ub_d.get(), eub)
        # the handle now caches its ranges: the same call copies them and leaves the workspace alone
        lb2 = DeviceDoubles(S.dim)
        _lib.check(ctx.lib.nnvhip_estimate_ranges_static(ctx.handle, S._h.h, lb2.ptr, None))
        ctx.synchronize()
        assert np.array_equal(lb2.get(), elb)
    del sets, outs, S
