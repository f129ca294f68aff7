"""Pins the oracle's specification-check functions (the consumer of the reach set) against the
reference's known answers and against what the mathematics fixes."""
import itertools

import numpy as np
import pytest

from oracle import nnv_oracle as o


def test_halfspace_contains_known_answers():
    # tests/set/halfspace/test_half_space_contain.m: -x1 <= 5, x2 <= 0
    U = o.OHalfSpace([[-1, 0], [0, 1]], [5, 0])
    assert o.halfspace_contains(U, [2, -1]) is True
    assert o.halfspace_contains(U, [-2, 1]) is False
    # tests/soundness/test_soundness_HalfSpace.m tests 3-6
    H = o.OHalfSpace([[1, 0], [0, 1], [-1, 0], [0, -1]], [1, 1, 0, 0])
    assert H.dim == 2
    assert o.halfspace_contains(H, [0.5, 0.5]) and not o.halfspace_contains(H, [2, 0.5])
    assert o.halfspace_contains(H, [1, 0.5])  # boundary counts as inside
    H6 = o.OHalfSpace([1, 1], [1])
    assert o.halfspace_contains(H6, [0, 0]) and not o.halfspace_contains(H6, [1, 1])
    assert o.OHalfSpace([[1, 0, 0], [0, 1, 0]], [1, 1]).dim == 3
    with pytest.raises(ValueError):
        o.OHalfSpace([[1, 0]], [1, 2])


def test_is_empty_set_known_answers():
    # tests/set/star/test_star_isEmptySet.m:17-23: alpha <= 1 and alpha >= 2 is infeasible
    S1 = o.OStar([[1.0, 1.0]], [[1.0], [-1.0]], [1.0, -2.0])
    assert o.is_empty_set(S1) is True
    # a box star is never empty (lpsolver.m:36-50 answers it without a solver)
    assert o.is_empty_set(o.star_from_box([-1.0, -1.0], [1.0, 1.0])) is False
    # feasible strip with explicit predicate bounds
    S2 = o.OStar([[0.0, 1.0]], [[1.0], [-1.0]], [0.5, 0.25], [-1.0], [1.0])
    assert o.is_empty_set(S2) is False
    # the same strip pushed outside the predicate box
    S3 = o.OStar([[0.0, 1.0]], [[-1.0]], [-2.0], [-1.0], [1.0])
    assert o.is_empty_set(S3) is True


def test_is_empty_set_stored_verdicts(golden):
    # the two stars of tests/set/star/test_star_isEmptySet.m with the verdicts the reference stored for them
    g = golden["star_isEmptySet"]
    S = o.OStar(g["S_V"], g["S_C"], g["S_d"])
    S1 = o.OStar(g["S1_V"], g["S1_C"], g["S1_d"])
    assert o.is_empty_set(S) is bool(g["b_nonempty"].reshape(-1)[0])
    assert o.is_empty_set(S1) is bool(g["b_empty"].reshape(-1)[0])
    assert bool(g["b_empty"].reshape(-1)[0]) and not bool(g["b_nonempty"].reshape(-1)[0])


def test_intersect_half_space_rows_and_known_answer():
    # tests/soundness/test_set_conversion.m:60-68: box [-1,1]^2 meets x1 <= 0.5
    S = o.star_from_box([-1.0, -1.0], [1.0, 1.0])
    S2 = o.intersect_half_space(S, [[1, 0]], [0.5])
    assert S2 is not None
    # set/Star.m:577-581: appended row is H*V(:,2:end), rhs g - H*c; V and bounds untouched
    assert np.array_equal(S2.V, S.V) and S2.C.shape == (2, 2)
    assert np.array_equal(S2.C[-1], [1.0, 0.0]) and S2.d[-1] == 0.5
    # a half-space the box cannot reach gives the empty answer; the boundary case is non-empty
    assert o.intersect_half_space(S, [[1, 0]], [-1.5]) is None
    assert o.intersect_half_space(S, [[1, 0]], [-1.0]) is not None
    with pytest.raises(ValueError):
        o.intersect_half_space(S, [[1, 0, 0]], [0.0])
    with pytest.raises(ValueError):
        o.intersect_half_space(S, [[1, 0]], [0.0, 1.0])


def test_intersection_matches_brute_force_on_affine_image_of_box():
    # a star without extra constraints is the affine image of its predicate box: the intersection
    # with {Gx <= g} is empty iff min over the box of every... (single row) exceeds g; with one row
    # the minimum is attained at a corner, so corner enumeration decides it exactly.
    rs = np.random.RandomState(7)
    for trial in range(40):
        S = o.affine_map(o.star_from_box(rs.uniform(-1, 0, 3), rs.uniform(0, 1, 3)), rs.randn(3, 3), rs.randn(3))
        Gm = rs.randn(1, 3)
        corners = np.array(list(itertools.product([-1.0, 1.0], repeat=3))).T
        vals = Gm @ (S.V[:, :1] + S.V[:, 1:] @ corners)
        for gval in (vals.min() - 0.1, vals.min() + 0.1, vals.max() + 0.1):
            want_empty = vals.min() > gval
            assert (o.intersect_half_space(S, Gm, [gval]) is None) == want_empty


def test_robustness_set_rows():
    # nn/NN.m:1351-1360 for 4 classes, target 1 (0-based): rows e_t - e_j for j != t
    hs = o.robustness_set(4, 1, "max")
    assert len(hs) == 3 and all(h.G.shape == (1, 4) and h.g.tolist() == [0.0] for h in hs)
    assert np.array_equal(np.vstack([h.G for h in hs]), [[-1, 1, 0, 0], [0, 1, -1, 0], [0, 1, 0, -1]])
    hs = o.robustness_set(3, 0, "min")
    assert np.array_equal(np.vstack([h.G for h in hs]), [[-1, 1, 0], [-1, 0, 1]])
    with pytest.raises(ValueError):
        o.robustness_set(3, 3)


def test_verify_specification_semantics():
    # one set, one half-space
    S = o.star_from_box([0.0, 0.0], [1.0, 1.0])
    assert o.verify_specification(S, o.OHalfSpace([[1, 0]], [-0.5])) == 1     # x1 <= -0.5 unreachable
    assert o.verify_specification(S, o.OHalfSpace([[1, 0]], [0.5])) == 2      # meets it
    # OR of half-spaces: one reachable disjunct is enough for "unknown"
    far = o.OHalfSpace([[0, 1]], [-3.0])
    near = o.OHalfSpace([[-1, 0]], [-0.9])
    assert o.verify_specification(S, [far, far]) == 1
    assert o.verify_specification(S, [far, near]) == 2
    # array of sets: every set must miss every half-space
    T = o.star_from_box([5.0, 5.0], [6.0, 6.0])
    assert o.verify_specification([S, T], o.OHalfSpace([[1, 0]], [-0.5])) == 1
    assert o.verify_specification([S, T], o.OHalfSpace([[-1, 0]], [-5.5])) == 2
    # two rows in one half-space are an AND: x1 <= 0.5 and x1 >= 0.75 cannot both hold
    assert o.verify_specification(S, o.OHalfSpace([[1, 0], [-1, 0]], [0.5, -0.75])) == 1


def test_verdict_agrees_with_sampled_outputs():
    # point-wise meaning: if some concrete output of the network lies in the unsafe region the
    # verdict must be 2; if the verdict is 1 no sampled output may lie in it
    from nnv_amd.configs import make_config
    cfg = make_config(1)
    rs = np.random.RandomState(3)
    out = o.nn_reach(cfg["layers"], o.star_from_box(cfg["lb"], cfg["ub"]), "relax-star-area", 1.0)
    xs = cfg["lb"][:, None] + (cfg["ub"] - cfg["lb"])[:, None] * rs.rand(cfg["lb"].size, 200)
    ys = np.stack([o.evaluate(cfg["layers"], xs[:, i]) for i in range(xs.shape[1])], axis=1)
    for t in range(5):
        hs = o.robustness_set(5, t, "max")
        r = o.verify_specification(out, hs)
        hit = any(o.halfspace_contains(h, ys[:, i]) for h in hs for i in range(ys.shape[1]))
        assert r in (1, 2) and (r == 2 or not hit)
    assert o.verify_robustness(cfg["layers"], o.star_from_box(cfg["lb"], cfg["ub"]), "relax-star-area",
                               int(np.argmax(ys[:, 0]))) in (1, 2)
