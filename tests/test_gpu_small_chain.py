"""NN.reach of small fully connected networks as ONE launch (nnvhip_reach_layers, chain.hip) against the
oracle and against the layer-by-layer path of the same library: every layer's set, the crossing lists in
new-predicate order, the constraint rows, for single sets and arrays, in all three crossing orders."""
import os

import numpy as np
import pytest

from tests.gpu_util import assert_close, compare_sets

pytestmark = pytest.mark.gpu

METHODS = ["relax-star-area", "relax-star-range", "relax-star-random"]


@pytest.fixture(scope="module")
def nnv():
    import nnv_amd
    nnv_amd.default_context()
    return nnv_amd


@pytest.fixture(scope="module")
def oracle():
    from oracle import nnv_oracle
    return nnv_oracle


def _fc(rs, out, inp, scale=1.0):
    return {"type": "fc", "W": rs.randn(out, inp) * scale / np.sqrt(inp), "b": rs.randn(out) * 0.2}


def _net(rs, widths, scale=1.5):
    layers = []
    for i in range(len(widths) - 1):
        layers.append(_fc(rs, widths[i + 1], widths[i], scale))
        if i < len(widths) - 2:
            layers.append({"type": "relu"})
    return layers


def _chain_launches(ctx, fn):
    """Runs fn with per-kernel timing on and returns (result, launches of the whole-reach kernel)."""
    ctx.kernel_time(8)
    ctx.set_timing(2)
    try:
        res = fn()
    finally:
        ctx.set_timing(0)
    return res, ctx.kernel_time(8)[1]


def _check_against_oracle(nnv, oracle, layers, dev_in, ora_in, method, expect_chain=True):
    ctx = nnv.default_context()
    net = nnv.NN.from_config(layers)
    out, launches = _chain_launches(ctx, lambda: net.reach(dev_in, {"reachMethod": method, "relaxFactor": 1}))
    if ctx.switch_is_on("no_small_chain", "dense_affine"):
        assert launches in (0, 1)     # a run under the switches that keep networks on the layer-by-layer path
    else:
        assert launches == (1 if expect_chain else 0)
    exp, exp_sets = oracle.nn_reach(layers, ora_in, method, 1.0, keep=True)
    many = isinstance(ora_in, list)
    prev = ora_in
    for li, (L, dset, oset) in enumerate(zip(layers, net.reachSet, exp_sets)):
        dl = list(dset) if many else [dset]
        ol = oset if many else [oset]
        pl = prev if many else [prev]
        assert len(dl) == len(ol)
        for si, (ds, os_, ps) in enumerate(zip(dl, ol, pl)):
            tag = "layer %d (%s) set %d" % (li + 1, L["type"], si)
            if L["type"] == "relu":
                lb, ub = oracle.estimate_ranges(ps)
                m1, m2 = oracle.relax_classify(lb, ub, method)
                ni, idx, clb, cub = ds.relu_info()
                assert ni == m1.size, tag
                assert np.array_equal(idx, m2), tag + ": crossing list / order"
                assert_close(clb, lb[m2], tag + ".lb")
                assert_close(cub, ub[m2], tag + ".ub")
            compare_sets(ds, os_, tag, L["type"] == "relu")
            if L["type"] == "fc":   # the kernel leaves the ranges of every FC output on the handle
                dlb, dub = ds.estimateRanges()
                elb, eub = oracle.estimate_ranges(os_)
                assert_close(dlb, elb, tag + ".lb", 1e-12)
                assert_close(dub, eub, tag + ".ub", 1e-12)
        prev = oset
    return net


@pytest.mark.parametrize("method", METHODS)
@pytest.mark.parametrize("widths,eps", [((5, 50, 50, 50, 5), 0.05), ((3, 17, 1), 0.4), ((8, 130, 70, 6), 0.02),
                                        ((40, 33, 64, 16, 16, 9), 0.1)])
def test_single_set(nnv, oracle, method, widths, eps):
    rs = np.random.RandomState(sum(widths) * 7 + METHODS.index(method))
    layers = _net(rs, widths)
    c = rs.rand(widths[0]) - 0.5
    lb, ub = c - eps, c + eps
    _check_against_oracle(nnv, oracle, layers, nnv.Star(lb, ub), oracle.star_from_box(lb, ub), method)


@pytest.mark.parametrize("method", ["relax-star-area", "relax-star-random"])
def test_array_of_boxes_with_different_predicate_counts(nnv, oracle, method):
    rs = np.random.RandomState(77)
    layers = _net(rs, (6, 40, 40, 4))
    n_boxes = 37
    lbs = rs.rand(6, n_boxes) - 0.6
    ubs = lbs + rs.rand(6, n_boxes) * 0.3
    ubs[2, ::3] = lbs[2, ::3]          # degenerate dimensions: those boxes have one generator less
    ubs[0, 5] = lbs[0, 5]
    dev = nnv.Star.from_boxes(lbs, ubs)
    ora = [oracle.star_from_box(lbs[:, i], ubs[:, i]) for i in range(n_boxes)]
    _check_against_oracle(nnv, oracle, layers, dev, ora, method)


def test_odd_sequences(nnv, oracle):
    """ReLU first, ReLU after ReLU, FC after FC, ReLU last; a general (non-box) input star."""
    rs = np.random.RandomState(5)
    V = rs.randn(12, 8)
    plb, pub = -rs.rand(7), rs.rand(7)
    dev = nnv.Star(V, np.zeros((1, 7)), np.zeros(1), plb, pub)
    ora = oracle.OStar(V, np.zeros((1, 7)), np.zeros(1), plb, pub)
    layers = [{"type": "relu"}, {"type": "relu"}, _fc(rs, 20, 12), _fc(rs, 9, 20), {"type": "relu"}, _fc(rs, 30, 9),
              {"type": "relu"}]
    _check_against_oracle(nnv, oracle, layers, dev, ora, "relax-star-range")


def test_same_sets_as_layer_by_layer(nnv, oracle):
    """Both paths of the library on the same network: identical structure, values to rounding."""
    ctx = nnv.default_context()
    rs = np.random.RandomState(11)
    layers = _net(rs, (5, 50, 50, 50, 50, 5))
    c = rs.rand(5) - 0.5
    S = nnv.Star(c - 0.03, c + 0.03)
    net_a, net_b = nnv.NN.from_config(layers), nnv.NN.from_config(layers)
    opts = {"reachMethod": "relax-star-area", "relaxFactor": 1}
    net_a.reach(S, opts)
    ctx.set_small_chain(False)
    try:
        _, launches = _chain_launches(ctx, lambda: net_b.reach(S, opts))
    finally:
        ctx.set_small_chain(True)
    assert launches == 0
    for i, (A, B) in enumerate(zip(net_a.reachSet, net_b.reachSet)):
        VA, VB = np.asarray(A.V), np.asarray(B.V)
        assert VA.shape == VB.shape
        assert_close(VA, VB, "layer %d V" % (i + 1), 1e-12)
        assert np.array_equal(VA == 0, VB == 0)
        assert_close(A.predicate_ub, B.predicate_ub, "layer %d predicate_ub" % (i + 1), 1e-12)
        if layers[i]["type"] == "relu":
            ia, ib = A.relu_info(), B.relu_info()
            assert ia[0] == ib[0] and np.array_equal(ia[1], ib[1])
            assert_close(A.C, B.C, "layer %d C" % (i + 1), 1e-12)
            assert_close(A.d, B.d, "layer %d d" % (i + 1), 1e-12)


def test_sets_of_a_chain_reach_feed_the_layer_kernels(nnv, oracle):
    """An intermediate set of the one-launch reach handed to the ordinary layer calls (its structure hints are
    those a ReLU step leaves) gives what the oracle gives."""
    rs = np.random.RandomState(3)
    layers = _net(rs, (4, 60, 60, 3))
    c = rs.rand(4) - 0.5
    lb, ub = c - 0.1, c + 0.1
    net = nnv.NN.from_config(layers)
    net.reach(nnv.Star(lb, ub), {"reachMethod": "relax-star-area", "relaxFactor": 1})
    _, exp_sets = oracle.nn_reach(layers, oracle.star_from_box(lb, ub), "relax-star-area", 1.0, keep=True)
    mid = net.reachSet[1]                      # output of the first ReLU
    big = _fc(rs, 300, 60)                     # too wide for nothing, but called directly: the layer kernels
    out = nnv.FullyConnectedLayer(big["W"], big["b"]).reach(mid, "relax-star-area")
    exp = oracle.nn_reach([big], exp_sets[1], "relax-star-area", 1.0)
    assert_close(np.asarray(out.V), exp.V, "FC of a chain set")
    r2 = nnv.ReluLayer().reach(out, "relax-star-area", [], 1)
    e2 = oracle.nn_reach([{"type": "relu"}], exp, "relax-star-area", 1.0)
    compare_sets(r2, e2, "ReLU after it")


def test_networks_beyond_the_limits_take_the_layer_loop(nnv, oracle):
    rs = np.random.RandomState(9)
    layers = _net(rs, (20, 1100, 10))          # more than 1024 neurons in a ReLU layer
    c = rs.rand(20) - 0.5
    _check_against_oracle(nnv, oracle, layers, nnv.Star(c - 0.01, c + 0.01), oracle.star_from_box(c - 0.01, c + 0.01),
                          "relax-star-area", expect_chain=False)
