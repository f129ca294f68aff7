"""relaxFactor < 1 on the GPU: the step with explicit lists against the oracle, the host LPs fed from
the resident set, and the six heuristics end to end."""
import numpy as np
import pytest

from tests.gpu_util import assert_close

pytestmark = pytest.mark.gpu

@pytest.fixture(scope="module")
def nnv():
    import nnv_amd
    nnv_amd.default_context()
    return nnv_amd


@pytest.fixture(scope="module")
def oracle():
    from oracle import nnv_oracle
    return nnv_oracle


METHODS = ["relax-star-range", "relax-star-area", "relax-star-bound", "relax-star-ub", "relax-star-random",
           "relax-star-static"]


def _star_pair(nnv, oracle, seed, N, n, hidden=None):
    """A star with triangle constraints (FC -> ReLU -> FC of a box star) on both sides."""
    rs = np.random.RandomState(seed)
    hidden = hidden or N
    lb, ub = -rs.rand(n) - 0.2, rs.rand(n) + 0.2
    W0, b0 = rs.randn(hidden, n), rs.randn(hidden) * 0.3
    W1, b1 = rs.randn(N, hidden) * 0.6, rs.randn(N) * 0.3
    D = nnv.Star(lb, ub).affineMap(W0, b0)
    D = nnv.PosLin.reach(D, "relax-star-area", [], 1).affineMap(W1, b1)
    O = oracle.affine_map(oracle.reach_relaxed_star(oracle.affine_map(oracle.star_from_box(lb, ub), W0, b0),
                                                    "relax-star-area", 1.0), W1, b1)
    return D, O


def _same_set(R, E, tol=1e-9, what=""):
    assert R.nVar == E.nVar and R.dim == E.dim, what
    assert_close(R.V, E.V, what + " V", tol)
    assert np.array_equal(np.asarray(R.V) == 0, E.V == 0), what
    assert_close(R.C, E.C, what + " C", tol)
    assert_close(R.d, E.d, what + " d", tol)
    assert_close(R.predicate_lb, E.predicate_lb, what + " pred_lb", tol)
    assert_close(R.predicate_ub, E.predicate_ub, what + " pred_ub", tol)


def test_lp_ranges_known_answer(nnv, golden):
    # Star.getRanges of the reference's stored S1 (eleven general constraint rows, no predicate bounds)
    g = golden["star_intersect_halfSpace"]
    S1 = nnv.Star(g["S1_V"], g["S1_C"], g["S1_d"].reshape(-1))
    lo, hi = S1.getRanges()
    np.testing.assert_allclose(lo, g["S1_lb"].reshape(-1), rtol=0, atol=1e-8)
    np.testing.assert_allclose(hi, g["S1_ub"].reshape(-1), rtol=0, atol=1e-8)
    assert abs(S1.getMin(1) - g["S1_lb"][1, 0]) < 1e-8 and abs(S1.getMax(0) - g["S1_ub"][0, 0]) < 1e-8
    xmin, xmax = S1.getRange(0)
    assert abs(xmin - 1.0) < 1e-8 and abs(xmax - g["S1_ub"][0, 0]) < 1e-8
    with pytest.raises(ValueError, match="Invalid index"):
        S1.getMin(2)


@pytest.mark.parametrize("N,n", [(12, 5), (300, 40), (1500, 30), (9000, 6)])
def test_fetch_rows(nnv, oracle, N, n):
    D, O = _star_pair(nnv, oracle, 3 + N, N, n, hidden=min(N, 64))
    rs = np.random.RandomState(N)
    rows = rs.permutation(N)[:min(N, 37)]
    got = D._h.fetch_rows(rows)
    assert got.shape == (rows.size, D.nVar + 1)
    assert np.array_equal(got, np.asarray(D.V)[rows, :])
    assert D._h.fetch_rows([]).shape == (0, D.nVar + 1)
    with pytest.raises(nnv.NNVHipError, match="Invalid index"):
        D._h.fetch_rows([N])


@pytest.mark.parametrize("N,n", [(7, 3), (64, 10), (1000, 20), (2500, 12), (9000, 5)])
def test_step_with_explicit_lists(nnv, oracle, N, n):
    # PosLin.multipleStepReachStarApprox_at_one(I.resetRow(reset), index, lb, ub) with lists that no
    # classification would produce: arbitrary order, bounds unrelated to the estimates
    D, O = _star_pair(nnv, oracle, N, N, n, hidden=min(N, 48))
    rs = np.random.RandomState(N + 1)
    perm = rs.permutation(N)
    n_reset, m = N // 3, N // 4
    reset, index = perm[:n_reset], perm[n_reset:n_reset + m]
    lb, ub = -rs.rand(m) - 0.01, rs.rand(m) + 0.01
    R = nnv.PosLin.multipleStepReachStarApprox_at_one(D, index, lb, ub, reset=reset)
    E = oracle.multiple_step_reach_star_approx_at_one(oracle.reset_row(O, reset), index, lb, ub)
    _same_set(R, E, what="explicit lists")
    assert np.array_equal(np.asarray(R.predicate_ub)[O.nVar:], ub)       # in list order, untouched
    ni, idx, rlb, rub = R.relu_info()
    assert ni == n_reset and np.array_equal(idx, index) and np.array_equal(rlb, lb) and np.array_equal(rub, ub)
    # the output feeds the next layer like any other ReLU output
    W = rs.randn(9, N)
    assert_close(R.affineMap(W, None).V, oracle.affine_map(E, W, None).V, "fc after explicit lists")
    # empty lists: the set itself
    R0 = nnv.PosLin.multipleStepReachStarApprox_at_one(D, [], [], [])
    assert R0.nVar == D.nVar and np.array_equal(R0.V, D.V)


def test_explicit_lists_are_validated(nnv, oracle):
    D, _ = _star_pair(nnv, oracle, 5, 20, 4)
    f = nnv.PosLin.multipleStepReachStarApprox_at_one
    with pytest.raises(nnv.NNVHipError, match="Invalid index"):
        f(D, [20], [-1.0], [1.0])
    with pytest.raises(nnv.NNVHipError, match="listed twice"):
        f(D, [3, 3], [-1.0, -1.0], [1.0, 1.0])
    with pytest.raises(nnv.NNVHipError, match="listed twice"):
        f(D, [3], [-1.0], [1.0], reset=[3])
    with pytest.raises(nnv.NNVHipError, match="lb < 0 < ub"):
        f(D, [3], [0.0], [1.0])
    with pytest.raises(ValueError, match="same length"):
        f(D, [3, 4], [-1.0], [1.0])


@pytest.mark.parametrize("method", METHODS)
@pytest.mark.parametrize("rf", [0.0, 0.5, 0.75])
def test_relaxed_step_with_lps(nnv, oracle, method, rf):
    # both sides hand the same LPs to the same solver, so the tightened bounds agree far below the
    # solver's own tolerance; everything else is the device against the restatement
    D, O = _star_pair(nnv, oracle, 21, 60, 6, hidden=40)
    R = nnv.PosLin.reach_relaxed_star_lp(D, method, rf, rng=np.random.RandomState(9))
    E = oracle.reach_relaxed_star_lp(O, method, rf, np.random.RandomState(9))
    _same_set(R, E, tol=1e-7, what="%s rf=%g" % (method, rf))
    _, idx, _, _ = R.relu_info()
    onehot = E.V[:, 1 + O.nVar:]
    assert np.array_equal(idx, [np.flatnonzero(onehot[:, j])[0] for j in range(onehot.shape[1])])
    if method != "relax-star-random":
        R2 = nnv.PosLin.reach(D, method, [], rf)
        assert np.array_equal(R2.V, R.V)
    lo1, hi1 = R.estimateRanges()
    lo0, hi0 = nnv.PosLin.reach(D, method, [], 1).estimateRanges()
    assert np.all(lo1 >= lo0 - 1e-7) and np.all(hi1 <= hi0 + 1e-7)


def test_layer_default_relax_factor_is_zero(nnv, oracle):
    # ReluLayer.reach(I, 'relax-star-range') without a factor optimises every crossing neuron
    # (nn/layers/ActivationFunctionLayer.m:108-172; the call of tests/soundness/test_soundness_relax_star.m:19)
    rs = np.random.RandomState(42)
    V = np.c_[rs.randn(5), rs.randn(5, 2) * 0.5]
    Cm, d = np.r_[np.eye(2), -np.eye(2)], np.ones(4)
    args = (V, Cm, d, -np.ones(2), np.ones(2))
    R = nnv.ReluLayer().reach(nnv.Star(*args), "relax-star-range")
    E = oracle.relu_reach(oracle.OStar(*args), "relax-star-range", 0.0)
    _same_set(R, E, tol=1e-8, what="default factor")


@pytest.mark.parametrize("method,rf", [("relax-star-area", 0.5), ("relax-star-range", 0.0), ("relax-star-bound", 0.25)])
def test_network_reach_with_relax_factor(nnv, oracle, method, rf):
    from nnv_amd.configs import make_config
    cfg = make_config(1)
    net = nnv.NN.from_config(cfg["layers"])
    out = net.reach(nnv.Star(cfg["lb"], cfg["ub"]), {"reachMethod": method, "relaxFactor": rf})
    E = oracle.nn_reach(cfg["layers"], oracle.star_from_box(cfg["lb"], cfg["ub"]), method, rf)
    assert out.nVar == E.nVar
    assert_close(out.V, E.V, "network V", 1e-6)
    lb, ub = out.estimateRanges()
    elb, eub = oracle.estimate_ranges(E)
    assert_close(lb, elb, "network lb", 1e-6)
    assert_close(ub, eub, "network ub", 1e-6)
    full = net.reach(nnv.Star(cfg["lb"], cfg["ub"]), {"reachMethod": method, "relaxFactor": 1})
    l1, u1 = full.estimateRanges()
    assert np.all(lb >= l1 - 1e-7) and np.all(ub <= u1 + 1e-7)
    assert out.nVar <= full.nVar


def test_lp_box_and_interval_box_known_answers(nnv, oracle, golden):
    # the reference's stored Star.getBox (LP) and Star.getBoxFast (interval arithmetic over the predicates'
    # bounding box) of one star: host LPs fed from the device, and the device's estimateRanges
    g = golden["star_getBoxFast"]
    d = g["I1_d"].reshape(-1)
    I1 = nnv.Star(g["I1_V"], g["I1_C"], d)
    lo, hi = I1.getRanges()
    np.testing.assert_allclose(lo, g["B1_lb"].reshape(-1), rtol=0, atol=1e-8)
    np.testing.assert_allclose(hi, g["B1_ub"].reshape(-1), rtol=0, atol=1e-8)
    n = g["I1_C"].shape[1]
    plb = np.array([oracle.lpsolver(np.eye(n)[j], g["I1_C"], d, None, None) for j in range(n)])
    pub = np.array([-oracle.lpsolver(-np.eye(n)[j], g["I1_C"], d, None, None) for j in range(n)])
    lb, ub = nnv.Star(g["I1_V"], g["I1_C"], d, plb, pub).estimateRanges()
    np.testing.assert_allclose(lb, g["B2_lb"].reshape(-1), rtol=0, atol=1e-8)
    np.testing.assert_allclose(ub, g["B2_ub"].reshape(-1), rtol=0, atol=1e-8)


def test_relu_layer_on_an_image_star_with_relax_factor(nnv, oracle):
    # ReluLayer.reach of an ImageStar goes toStar -> PosLin.reach -> toImageStar (nn/layers/ReluLayer.m:72-150),
    # also below relaxFactor 1
    rs = np.random.RandomState(6)
    lb = rs.rand(5, 4, 2) - 0.7
    ub = lb + 0.3 * rs.rand(5, 4, 2)
    Wt, b = rs.randn(3, 3, 2, 3) * 0.5, rs.randn(3) * 0.1
    conv = nnv.Conv2DLayer(Wt, b, [1, 1, 1, 1], [1, 1], [1, 1])
    D = nnv.ReluLayer().reach(conv.reach(nnv.ImageStar(lb, ub), "approx-star"), "relax-star-area", [], 1)
    W2, b2 = rs.randn(3, 3, 3, 2) * 0.5, rs.randn(2) * 0.1       # a second convolution: genuine constraints
    D = nnv.Conv2DLayer(W2, b2, [1, 1, 1, 1], [1, 1], [1, 1]).reach(D, "approx-star")
    O = oracle.relu_reach(oracle.conv2d_reach(oracle.image_star_from_bounds(lb, ub), Wt, b, [1, 1, 1, 1], [1, 1], [1, 1]),
                          "relax-star-area", 1.0)
    O = oracle.conv2d_reach(O, W2, b2, [1, 1, 1, 1], [1, 1], [1, 1])
    for method, rf in (("relax-star-range", 0.0), ("relax-star-area", 0.5)):
        R = nnv.ReluLayer().reach(D, method, [], rf)
        E = oracle.relu_reach(O, method, rf)
        assert isinstance(R, nnv.ImageStar) and (R.height, R.width, R.numChannel) == (E.height, E.width, E.numChannel)
        assert R.numPred == E.numPred
        assert_close(R.V.reshape(-1, R.numPred + 1, order="F"), E.V.reshape(-1, E.numPred + 1, order="F"), "V", 1e-7)
        assert_close(R.C, E.C, "C", 1e-7)
        assert_close(R.pred_ub, E.pred_ub, "pred_ub", 1e-7)


# ---- the six heuristics' bookkeeping on the hand-built star (expectations derived on paper from the reference's
# statements: tests/relax_lp_hand_case.py), device path against those lists, not against the oracle's twin of the
# same bookkeeping
@pytest.mark.parametrize("method,rf", [("relax-star-range", 0.5), ("relax-star-area", 0.5), ("relax-star-static", 0.5),
                                       ("relax-star-random", 0.5), ("relax-star-bound", 0.5), ("relax-star-bound", 0.25),
                                       ("relax-star-ub", 0.5), ("relax-star-ub", 0.25)])
def test_hand_case_bookkeeping(nnv, oracle, method, rf):
    from tests import relax_lp_hand_case as h
    S = nnv.Star(h.V, h.C, h.d, h.PRED_LB, h.PRED_UB)
    reset, index, lbs, ubs = h.EXPECTED[(method, rf)]
    R = nnv.PosLin.reach_relaxed_star_lp(S, method, rf, rng=h.FixedPermutation(h.RANDPERM[3]))
    ni, idx, clb, cub = R.relu_info()
    assert ni == len(reset)
    assert np.array_equal(idx, np.array(index) - 1), "new-predicate order"
    np.testing.assert_allclose(clb, lbs, rtol=0, atol=1e-8)
    np.testing.assert_allclose(cub, ubs, rtol=0, atol=1e-8)
    # the set itself: what the reference's one-shot step gives for exactly these lists
    O = oracle.OStar(h.V, h.C, h.d, h.PRED_LB, h.PRED_UB)
    E = oracle.multiple_step_reach_star_approx_at_one(oracle.reset_row(O, np.array(reset) - 1), np.array(index) - 1,
                                                      np.array(lbs), np.array(ubs))
    _same_set(R, E, 1e-8, "%s rf=%g" % (method, rf))
    zero_rows = np.flatnonzero(~np.asarray(R.V)[:, :3].any(axis=1))
    assert sorted(zero_rows + 1) == sorted(reset + index)
