"""The per-context weight cache: a layer whose arrays are already on the device is not uploaded again
(repeated NN.reach, NN objects rebuilt around the same arrays, Star.affineMap(W, b) called again), whatever
object the caller wraps them in; any change of the arrays or the geometry is a different layer."""
import os

import numpy as np
import pytest

from tests.gpu_util import assert_close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def nnv():
    import nnv_amd
    nnv_amd.default_context()
    return nnv_amd


def test_second_reach_and_rebuilt_network_upload_nothing(nnv):
    from nnv_amd.configs import make_config
    ctx = nnv.default_context()
    cfg = make_config(1)
    opts = {"reachMethod": "relax-star-area", "relaxFactor": 1}
    S = nnv.Star(cfg["lb"], cfg["ub"])
    net = nnv.NN.from_config(cfg["layers"], cfg["name"])
    n_fc = sum(1 for L in cfg["layers"] if L["type"] == "fc")
    u0 = ctx.upload_stats()
    out1 = net.reach(S, opts)
    u1 = ctx.upload_stats()
    assert u1[0] - u0[0] <= n_fc            # (fewer if an earlier test left the same arrays resident)
    out2 = net.reach(S, opts)
    u2 = ctx.upload_stats()
    assert u2 == u1, "a second reach of a resident set copied %d bytes to the device" % (u2[2] - u1[2])
    net2 = nnv.NN.from_config(cfg["layers"], cfg["name"])     # new layer objects, same arrays
    out3 = net2.reach(S, opts)
    u3 = ctx.upload_stats()
    assert u3[:2] == u1[:2]
    assert np.array_equal(np.asarray(out1.V), np.asarray(out3.V)) and np.array_equal(np.asarray(out1.V), np.asarray(out2.V))


def test_affine_map_with_the_same_arrays_uploads_once(nnv):
    ctx = nnv.default_context()
    rs = np.random.RandomState(123)
    W, b = rs.randn(40, 12), rs.randn(40)
    S = nnv.Star(-np.ones(12), np.ones(12))
    u0 = ctx.upload_stats()
    A = S.affineMap(W, b)
    u1 = ctx.upload_stats()
    assert u1[0] - u0[0] == 1 and u1[1] - u0[1] == 8 * (40 * 12 + 40)
    B = S.affineMap(W.copy(), b.copy())      # other objects, same values
    u2 = ctx.upload_stats()
    assert u2[:2] == u1[:2]
    assert np.array_equal(np.asarray(A.V), np.asarray(B.V))
    exp = np.hstack([(W @ np.zeros(12) + b)[:, None], W])
    assert_close(np.asarray(A.V), exp, "affineMap")
    # anything that differs is another layer
    W2 = W.copy()
    W2[39, 11] = np.nextafter(W2[39, 11], 1.0)
    for Wx, bx in ((W2, b), (W, b + 1e-9), (W, None), (W.T.copy().reshape(40, 12), b)):
        before = ctx.upload_stats()[0]
        R = S.affineMap(Wx, bx)
        assert ctx.upload_stats()[0] == before + 1
        bb = np.zeros(40) if bx is None else bx
        assert_close(np.asarray(R.V), np.hstack([bb[:, None], Wx]), "affineMap of a changed layer", 1e-15)
    # the same values with another shape
    before = ctx.upload_stats()[0]
    S24 = nnv.Star(-np.ones(24), np.ones(24))
    S24.affineMap(W.reshape(20, 24, order="F"), b[:20])
    assert ctx.upload_stats()[0] == before + 1


def test_conv_layers_are_cached_by_arrays_and_geometry(nnv):
    ctx = nnv.default_context()
    rs = np.random.RandomState(7)
    W, b = rs.randn(3, 3, 2, 4), rs.randn(4)
    I = nnv.ImageStar(np.zeros((6, 6, 2)), np.ones((6, 6, 2)) * 0.1)
    u0 = ctx.upload_stats()[0]
    A = nnv.Conv2DLayer(W, b, [1, 1, 1, 1], [1, 1], [1, 1]).reach(I, "approx-star")
    assert ctx.upload_stats()[0] == u0 + 1
    B = nnv.Conv2DLayer(W.copy(), b.copy(), [1, 1, 1, 1], [1, 1], [1, 1]).reach(I, "approx-star")
    assert ctx.upload_stats()[0] == u0 + 1
    assert np.array_equal(np.asarray(A.V), np.asarray(B.V))
    C2 = nnv.Conv2DLayer(W, b, [0, 0, 0, 0], [1, 1], [1, 1]).reach(I, "approx-star")   # other padding: other layer
    assert ctx.upload_stats()[0] == u0 + 2
    assert np.asarray(C2.V).shape[0] == 4


def test_entries_nobody_holds_are_dropped_beyond_the_budget(nnv):
    """A context with a 1 MB budget: three 0.5 MB layers, created and let go one after the other."""
    from nnv_amd import _lib
    old = os.environ.get("NNVHIP_WEIGHT_CACHE_MB")
    os.environ["NNVHIP_WEIGHT_CACHE_MB"] = "1"
    try:
        ctx = _lib.Context(0)
    finally:
        if old is None:
            del os.environ["NNVHIP_WEIGHT_CACHE_MB"]
        else:
            os.environ["NNVHIP_WEIGHT_CACHE_MB"] = old
    rs = np.random.RandomState(1)
    Ws = [rs.randn(256, 256) for _ in range(3)]
    S = nnv.Star(-np.ones(256), np.ones(256), ctx=ctx)
    outs = [np.asarray(S.affineMap(W).V) for W in Ws]        # each layer is released when affineMap returns
    assert ctx.upload_stats()[0] == 3
    np.asarray(S.affineMap(Ws[2]).V)                         # most recent: still resident
    assert ctx.upload_stats()[0] == 3
    again = np.asarray(S.affineMap(Ws[0]).V)                 # least recent: was dropped, uploaded again
    assert ctx.upload_stats()[0] == 4
    assert np.array_equal(again, outs[0])
    del S


def test_equal_hashes_are_not_a_hit(nnv):
    """With every array hashing alike only the byte comparison can tell layers apart: two matrices of one shape
    must give two layers and two different results, and each must be found again by its own values."""
    from nnv_amd import _lib
    lib = _lib.load()
    ctx = _lib.Context(0)
    rs = np.random.RandomState(11)
    Wa, Wb = rs.randn(24, 16), rs.randn(24, 16)
    b = rs.randn(24)
    S = nnv.Star(-np.ones(16), np.ones(16), ctx=ctx)
    _lib.check(lib.nnvhip_debug_weak_weight_hash(1))
    try:
        A = np.asarray(S.affineMap(Wa, b).V)
        B = np.asarray(S.affineMap(Wb, b).V)
        assert ctx.upload_stats()[0] == 2
        assert_close(A, np.hstack([b[:, None], Wa]), "first layer", 1e-15)
        assert_close(B, np.hstack([b[:, None], Wb]), "second layer (same hash, other values)", 1e-15)
        A2 = np.asarray(S.affineMap(Wa.copy(), b.copy()).V)
        B2 = np.asarray(S.affineMap(Wb.copy(), b.copy()).V)
        assert ctx.upload_stats()[0] == 2, "layers with equal hashes were not found again by their values"
        assert np.array_equal(A, A2) and np.array_equal(B, B2)
        Bb = np.asarray(S.affineMap(Wb, b + 1.0).V)          # same matrix, other bias, same (weak) hash
        assert ctx.upload_stats()[0] == 3
        assert_close(Bb[:, 0], b + 1.0, "bias of the third layer", 1e-15)
    finally:
        _lib.check(lib.nnvhip_debug_weak_weight_hash(0))
    del S


def test_block_of_hash_constants_does_not_hide_what_came_before(nnv):
    """Two matrices that differ only in front of a 32-byte block equal to the hash's own mixing constants (a product
    that forgets its past would hash them alike) are different layers."""
    ctx = nnv.default_context()
    consts = np.array([0xa0761d6478bd642f, 0xe7037ed1a0b428db, 0x589965cc75374cc3, 0x8ebc6af09c88c6e3], dtype=np.uint64)
    flat = np.zeros(16)
    flat[:4] = [1.0, 2.0, 3.0, 4.0]
    flat[4:8] = consts.view(np.float64)
    flat[8:] = 0.5
    Wa = flat.reshape(8, 2, order="F")
    Wb = Wa.copy()
    Wb[0, 0] = -7.0
    assert np.all(np.isfinite(Wa))
    S = nnv.Star(-np.ones(2), np.ones(2))
    u0 = ctx.upload_stats()[0]
    A = np.asarray(S.affineMap(Wa).V)
    B = np.asarray(S.affineMap(Wb).V)
    assert ctx.upload_stats()[0] == u0 + 2
    assert A[0, 1] == 1.0 and B[0, 1] == -7.0


def test_unreferenced_layers_are_reported_and_released(nnv):
    from nnv_amd import _lib
    ctx = _lib.Context(0)
    rs = np.random.RandomState(5)
    S = nnv.Star(-np.ones(64), np.ones(64), ctx=ctx)
    W = rs.randn(64, 64)
    layer = nnv.FullyConnectedLayer(W, np.zeros(64))
    out = layer.reach(S, "approx-star")
    np.asarray(S.affineMap(rs.randn(64, 64)).V)              # its layer object is gone when affineMap returns
    n, dev, unref = ctx.weight_cache_stats()
    assert n == 2 and dev > 0 and 0 < unref < dev
    assert ctx.weight_cache_release() == 1
    n2, dev2, unref2 = ctx.weight_cache_stats()
    assert n2 == 1 and unref2 == 0 and dev2 == dev - unref
    again = layer.reach(S, "approx-star")                     # the layer somebody holds still works
    assert np.array_equal(np.asarray(out.V), np.asarray(again.V))
    del S, out, again, layer
