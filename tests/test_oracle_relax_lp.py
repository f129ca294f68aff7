"""relaxFactor < 1: LP-tightened bounds (Star.getMins/getMaxs) and the six heuristics' bookkeeping.

The LP values come from MATLAB's linprog in the reference and from HiGHS here, so they are pinned to
solver tolerance only; the bookkeeping around them (which neurons are optimised, reset, kept, and in
which order the new predicates come) is pinned by the cases where the LP has a closed form."""
import itertools

import numpy as np
import pytest

from oracle import nnv_oracle as o

METHODS = ["relax-star-range", "relax-star-area", "relax-star-bound", "relax-star-ub", "relax-star-random",
           "relax-star-static"]


def test_lp_ranges_known_answer(golden):
    # the reference's stored Star.getRanges of S1 = S.intersectHalfSpace(H, g): eleven general
    # constraint rows, no predicate bounds -> every value comes out of the LP solver
    g = golden["star_intersect_halfSpace"]
    S1 = o.OStar(g["S1_V"], g["S1_C"], g["S1_d"])
    lo = o.get_mins(S1, [0, 1])
    hi = o.get_maxs(S1, [0, 1])
    np.testing.assert_allclose(lo, g["S1_lb"].reshape(-1), rtol=0, atol=1e-8)
    np.testing.assert_allclose(hi, g["S1_ub"].reshape(-1), rtol=0, atol=1e-8)
    # the last constraint row is the half-space itself: C1 = H*V(:,2:end), d1 = g - H*c
    H, gg = g["H"], g["g"].reshape(-1)
    assert np.array_equal(g["S1_C"][-1], (H @ g["S_V"][:, 1:]).reshape(-1))
    assert g["S1_d"].reshape(-1)[-1] == gg[0] - (H @ g["S_V"][:, 0])[0]


def test_box_only_lp_is_the_corner_minimum():
    # utils/lpsolver.m:36-50: all-zero A over a finite box -> sum(min(f.*lb, f.*ub))
    rs = np.random.RandomState(1)
    f = rs.randn(5)
    lb, ub = -rs.rand(5) - 0.2, rs.rand(5) + 0.1
    brute = min(float(f @ np.array(c)) for c in itertools.product(*zip(lb, ub)))
    assert abs(o.lpsolver(f, np.zeros((1, 5)), np.zeros(1), lb, ub) - brute) < 1e-13
    assert abs(o.lpsolver(f, np.zeros((0, 5)), np.zeros(0), lb, ub) - brute) < 1e-13
    # a negative right-hand side on the all-zero row is infeasible and must not take the shortcut
    with pytest.raises(RuntimeError):
        o.lpsolver(f, np.zeros((1, 5)), -np.ones(1), lb, ub)
    # one active constraint: a_0 <= 0 halves the box in the first coordinate
    A = np.zeros((1, 5))
    A[0, 0] = 1.0
    ub2 = ub.copy()
    ub2[0] = 0.0
    want = min(float(f @ np.array(c)) for c in itertools.product(*zip(lb, ub2)))
    assert abs(o.lpsolver(f, A, np.zeros(1), lb, ub) - want) < 1e-9


def test_zero_generator_row_returns_the_centre():
    V = np.array([[2.5, 0.0, 0.0], [1.0, 1.0, -1.0]])
    S = o.OStar(V, np.zeros((1, 2)), np.zeros(1), [-1, -1], [1, 1])
    assert o.get_min(S, 0) == 2.5 and o.get_max(S, 0) == 2.5
    assert o.get_min(S, 1) == -1.0 and o.get_max(S, 1) == 3.0
    with pytest.raises(ValueError, match="Invalid index"):
        o.get_min(S, 2)


def _two_layer_star(seed=0, N=12, n=5, sampler=False):
    """ReLU output of an FC-mapped box star, mapped again: a star with genuine triangle constraints.
    With sampler=True also returns a function drawing feasible predicate vectors (input predicates
    uniform in the box, the new ones set to their neurons' ReLU outputs)."""
    rs = np.random.RandomState(seed)
    I = o.star_from_box(-rs.rand(n) - 0.2, rs.rand(n) + 0.2)
    S = o.affine_map(I, rs.randn(N, n), rs.randn(N) * 0.3)
    R = o.reach_relaxed_star(S, "relax-star-area", 1.0)
    out = o.affine_map(R, rs.randn(N, N) * 0.6, rs.randn(N) * 0.3)
    if not sampler:
        return out
    _, idx = _crossing_triples(R, n)

    def draw(r):
        a = r.uniform(-1, 1, n)
        y = np.maximum(S.V[:, 0] + S.V[:, 1:] @ a, 0)
        return np.r_[a, y[idx]]
    return out, draw


def test_lp_bounds_are_never_looser_than_the_estimates():
    S = _two_layer_star()
    assert np.any(S.C)
    lb, ub = o.estimate_ranges(S)
    idx = np.arange(S.dim)
    lo, hi = o.get_mins(S, idx), o.get_maxs(S, idx)
    assert np.all(lo >= lb - 1e-8) and np.all(hi <= ub + 1e-8) and np.all(lo <= hi + 1e-9)
    assert np.any(lo > lb + 1e-6) or np.any(hi < ub - 1e-6)      # the constraints do bite somewhere


@pytest.mark.parametrize("method", METHODS)
def test_relax_factor_one_solves_no_lp(method, monkeypatch):
    S = _two_layer_star(1)
    monkeypatch.setattr(o, "lpsolver", lambda *a, **k: (_ for _ in ()).throw(AssertionError("LP solved")))
    A = o.reach_relaxed_star_lp(S, method, 1.0, np.random.RandomState(0))
    B = o.reach_relaxed_star(S, method, 1.0)
    for x, y in ((A.V, B.V), (A.C, B.C), (A.d, B.d), (A.predicate_lb, B.predicate_lb), (A.predicate_ub, B.predicate_ub)):
        assert np.array_equal(x, y)


def _crossing_triples(R, n_in):
    """{neuron: (ub of its predicate, its C2 row offset d2)} of a ReLU output set."""
    onehot = R.V[:, 1 + n_in:]
    idx = [int(np.flatnonzero(onehot[:, j])[0]) for j in range(onehot.shape[1])]
    assert all(np.count_nonzero(onehot[:, j]) == 1 for j in range(onehot.shape[1]))
    return {i: R.predicate_ub[n_in + j] for j, i in enumerate(idx)}, idx


@pytest.mark.parametrize("method", METHODS)
@pytest.mark.parametrize("rf", [0.0, 0.5])
def test_box_star_lp_equals_interval_bounds(method, rf):
    # an FC-mapped box star has no constraint but its predicate box, so every LP is the interval
    # closed form: the LP-tightened step must give the relaxFactor = 1 set, up to the order in which
    # the variant lists the new predicates
    rs = np.random.RandomState(7)
    n, N = 6, 40
    I = o.star_from_box(-rs.rand(n) - 0.2, rs.rand(n) + 0.2)
    S = o.affine_map(I, rs.randn(N, n), rs.randn(N) * 0.5)
    ref = o.reach_relaxed_star(S, "relax-star-static", 1.0)
    got = o.reach_relaxed_star_lp(S, method, rf, np.random.RandomState(3))
    assert got.nVar == ref.nVar and got.C.shape == ref.C.shape
    ref_ub, ref_idx = _crossing_triples(ref, n)
    got_ub, got_idx = _crossing_triples(got, n)
    assert sorted(ref_idx) == sorted(got_idx)
    for i in ref_idx:
        assert abs(ref_ub[i] - got_ub[i]) <= 1e-12
    m = len(ref_idx)
    perm = np.array([ref_idx.index(i) for i in got_idx])          # got column j <-> ref column perm[j]
    cols = np.r_[np.arange(n + 1), n + 1 + perm]
    assert np.array_equal(got.V, ref.V[:, cols])
    p0 = S.C.shape[0]
    rows = np.r_[np.arange(p0), p0 + perm, p0 + m + perm, p0 + 2 * m + perm]
    np.testing.assert_allclose(got.C, ref.C[np.ix_(rows, cols[1:] - 1)], rtol=0, atol=1e-12)
    np.testing.assert_allclose(got.d, ref.d[rows], rtol=0, atol=1e-12)
    # documented order: range/area/random/static list the untouched neurons first, then the optimised
    # ones that still cross; bound/ub keep ascending index order
    if method in ("relax-star-bound", "relax-star-ub"):
        assert got_idx == sorted(got_idx)
    if method == "relax-star-static":
        lb, ub = o.estimate_ranges(S)
        map2 = np.flatnonzero((lb < 0) & (ub > 0))
        n1 = int(np.floor((1 - rf) * map2.size + 0.5))
        assert got_idx == list(map2[n1:]) + list(map2[:n1])


@pytest.mark.parametrize("method", METHODS)
def test_lp_step_tightens_and_stays_sound(method):
    S, draw = _two_layer_star(2, N=14, n=5, sampler=True)
    loose = o.reach_relaxed_star(S, method, 1.0)
    tight = o.reach_relaxed_star_lp(S, method, 0.0, np.random.RandomState(5))
    assert tight.nVar <= loose.nVar                       # LP bounds can only take neurons off the crossing list
    # soundness: sampled points of S, pushed through ReLU, lie in the output set with the new predicates
    # set to the ReLU outputs of their neurons
    rs = np.random.RandomState(11)
    n_in = S.nVar
    _, idx = _crossing_triples(tight, n_in)
    for _ in range(200):
        a = draw(rs)
        assert np.all(S.C @ a <= S.d + 1e-9) and np.all(a >= S.predicate_lb - 1e-12) and np.all(a <= S.predicate_ub + 1e-12)
        y = np.maximum(S.V[:, 0] + S.V[:, 1:] @ a, 0)
        alpha = np.r_[a, y[idx]]
        assert np.all(tight.C @ alpha <= tight.d + 1e-7)
        assert np.all(alpha >= tight.predicate_lb - 1e-7) and np.all(alpha <= tight.predicate_ub + 1e-7)
        np.testing.assert_allclose(tight.V[:, 0] + tight.V[:, 1:] @ alpha, y, atol=1e-7)
    # and its interval bounds are inside the LP-free ones
    l0, u0 = o.estimate_ranges(loose)
    l1, u1 = o.estimate_ranges(tight)
    assert np.all(l1 >= l0 - 1e-7) and np.all(u1 <= u0 + 1e-7)


def test_round_is_matlabs():
    # n1 = round((1-rf)*numel(map2)): halves go up (numpy's round would send 2.5 to 2)
    assert o._round_half_away(2.5) == 3 and o._round_half_away(3.5) == 4 and o._round_half_away(2.4999) == 2


def test_lp_box_and_interval_box_known_answers(golden):
    # Star.getBox (one LP pair per state, set/Star.m:597-650) and Star.getBoxFast (interval arithmetic over
    # the bounding box of the predicate polytope, :658-677) of the reference's stored star I1
    g = golden["star_getBoxFast"]
    I1 = o.OStar(g["I1_V"], g["I1_C"], g["I1_d"])
    idx = np.arange(I1.dim)
    np.testing.assert_allclose(o.get_mins(I1, idx), g["B1_lb"].reshape(-1), rtol=0, atol=1e-8)
    np.testing.assert_allclose(o.get_maxs(I1, idx), g["B1_ub"].reshape(-1), rtol=0, atol=1e-8)
    # predicate bounding box by LP (what getPredicateBounds asks the polytope library for), then the same
    # interval formula estimateRanges uses
    n = I1.nVar
    plb = np.array([o.lpsolver(np.eye(n)[j], I1.C, I1.d, None, None) for j in range(n)])
    pub = np.array([-o.lpsolver(-np.eye(n)[j], I1.C, I1.d, None, None) for j in range(n)])
    lb, ub = o.estimate_ranges(o.OStar(I1.V, I1.C, I1.d, plb, pub))
    np.testing.assert_allclose(lb, g["B2_lb"].reshape(-1), rtol=0, atol=1e-8)
    np.testing.assert_allclose(ub, g["B2_ub"].reshape(-1), rtol=0, atol=1e-8)


# ---- the six heuristics' bookkeeping on a star whose LPs can be done by hand -------------------------------
def test_hand_case_lp_values():
    from tests import relax_lp_hand_case as h
    S = o.OStar(h.V, h.C, h.d, h.PRED_LB, h.PRED_UB)
    lb, ub = o.estimate_ranges(S)
    assert np.array_equal(lb, [-1, -4.5, -1.5, -2.5, 1.5, -1.75, -1.125, -0.75])
    assert np.array_equal(ub, [3, 3.5, 6.5, -1.5, 2.5, 2.25, 0.875, 1.25])
    np.testing.assert_allclose(o.get_maxs(S, np.arange(8)), [1, -0.5, 6.5, -1.5, 2.5, 2.25, 0.875, 0.25], rtol=0, atol=1e-9)
    np.testing.assert_allclose(o.get_mins(S, np.arange(8)), [-1, -4.5, 2.5, -2.5, 1.5, -1.75, -1.125, -0.75], rtol=0, atol=1e-9)


@pytest.mark.parametrize("method,rf", [("relax-star-range", 0.5), ("relax-star-area", 0.5), ("relax-star-static", 0.5),
                                       ("relax-star-random", 0.5), ("relax-star-bound", 0.5), ("relax-star-bound", 0.25),
                                       ("relax-star-ub", 0.5), ("relax-star-ub", 0.25)])
def test_hand_case_bookkeeping(method, rf):
    from tests import relax_lp_hand_case as h
    S = o.OStar(h.V, h.C, h.d, h.PRED_LB, h.PRED_UB)
    reset, index, lbs, ubs = h.EXPECTED[(method, rf)]
    R = o.reach_relaxed_star_lp(S, method, rf, rng=h.FixedPermutation(h.RANDPERM[3]))
    E = o.multiple_step_reach_star_approx_at_one(o.reset_row(S, np.array(reset) - 1), np.array(index) - 1,
                                                 np.array(lbs), np.array(ubs))
    assert R.V.shape == E.V.shape and R.C.shape == E.C.shape
    assert np.array_equal(R.V, E.V)                      # rows reset, unit vectors in the expected order
    np.testing.assert_allclose(R.C, E.C, rtol=0, atol=1e-8)
    np.testing.assert_allclose(R.d, E.d, rtol=0, atol=1e-8)
    np.testing.assert_allclose(R.predicate_ub, E.predicate_ub, rtol=0, atol=1e-8)
    assert np.array_equal(R.predicate_lb, E.predicate_lb)
