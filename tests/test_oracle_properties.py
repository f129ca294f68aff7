"""Pin what no reference fixture covers (the relax-star ReLU step, conv, partition) by what the
mathematics fixes: hand-computed cases, brute force, library cross-checks and invariants."""
import itertools

import numpy as np
import pytest
import torch

from nnv_amd.configs import make_config
from oracle import nnv_oracle as o


def _rand_star(rs, N, n, p=2):
    V = rs.randn(N, n + 1)
    C = rs.randn(p, n)
    d = np.abs(rs.randn(p)) + 5.0
    lb = -np.abs(rs.rand(n)) - 0.1
    ub = np.abs(rs.rand(n)) + 0.1
    return o.OStar(V, C, d, lb, ub)


def test_estimate_ranges_is_corner_enumeration():
    rs = np.random.RandomState(0)
    S = _rand_star(rs, 7, 4)
    lb, ub = o.estimate_ranges(S)
    corners = [S.V[:, 0] + S.V[:, 1:] @ np.array(c)
               for c in itertools.product(*zip(S.predicate_lb, S.predicate_ub))]
    corners = np.array(corners)
    np.testing.assert_allclose(lb, corners.min(0), rtol=1e-13)
    np.testing.assert_allclose(ub, corners.max(0), rtol=1e-13)


def test_estimate_ranges_default_predicate_bounds():
    S = o.OStar(np.array([[1.0, 2.0, -3.0]]), np.zeros((1, 2)), np.zeros(1))
    lb, ub = o.estimate_ranges(S)
    assert lb[0] == 1 - 5 and ub[0] == 1 + 5


def test_scalar_triangle_by_hand():
    # x = 0.5 + 1.5*a, a in [-1,1]: lb=-1, ub=2 -> crossing; slope a = 2/3
    S = o.OStar(np.array([[0.5, 1.5]]), np.zeros((1, 1)), np.zeros(1), [-1.0], [1.0])
    R = o.reach_relaxed_star(S, "relax-star-area", 1.0)
    assert np.array_equal(R.V, np.array([[0.0, 0.0, 1.0]]))
    a = 2.0 / 3.0
    expC = np.array([[0.0, 0.0],          # old constraint, zero padded
                     [0.0, -1.0],         # y >= 0
                     [1.5, -1.0],         # y >= x
                     [-a * 1.5, 1.0]])    # y <= a (x - lb)
    expd = np.array([0.0, 0.0, -0.5, a * 0.5 - a * (-1.0)])
    np.testing.assert_allclose(R.C, expC, rtol=1e-15)
    np.testing.assert_allclose(R.d, expd, rtol=1e-15)
    assert np.array_equal(R.predicate_lb, [-1.0, 0.0]) and np.array_equal(R.predicate_ub, [1.0, 2.0])


def test_relu_all_positive_identity_all_negative_zero():
    # tests/soundness/test_soundness_ReluLayer.m:46-78
    rs = np.random.RandomState(1)
    G = 0.1 * rs.randn(6, 3)
    pos = o.OStar(np.c_[np.full(6, 5.0), G], np.zeros((1, 3)), np.zeros(1), -np.ones(3), np.ones(3))
    R = o.reach_relaxed_star(pos, "relax-star-range", 1.0)
    assert np.array_equal(R.V, pos.V) and R.nVar == 3 and R.C.shape == (1, 3)
    neg = o.OStar(np.c_[np.full(6, -5.0), G], np.zeros((1, 3)), np.zeros(1), -np.ones(3), np.ones(3))
    R = o.reach_relaxed_star(neg, "relax-star-range", 1.0)
    assert not R.V.any() and R.nVar == 3


def test_classification_ties():
    # ub == 0 is inactive (ub <= 0); lb == 0 with ub > 0 is active (not lb < 0)
    lb = np.array([-1.0, -1.0, 0.0, -2.0, 0.0])
    ub = np.array([0.0, 1.0, 1.0, -1.0, 0.0])
    m1, m2 = o.relax_classify(lb, ub, "relax-star-static")
    assert m1.tolist() == [0, 3, 4] and m2.tolist() == [1]


def test_sort_orders_and_stability():
    lb = np.array([-1.0, -2.0, -1.0, -4.0, -2.0, 1.0])
    ub = np.array([2.0, 1.0, 2.0, 0.5, 1.0, 3.0])
    _, idx = o.relax_classify(lb, ub, "relax-star-static")
    assert idx.tolist() == [0, 1, 2, 3, 4]
    _, rng = o.relax_classify(lb, ub, "relax-star-range")   # ub-lb = 3,3,3,4.5,3 -> stable
    assert rng.tolist() == [3, 0, 1, 2, 4]
    _, area = o.relax_classify(lb, ub, "relax-star-area")   # 0.5*|ub||lb| = 1,1,1,1,1 -> all tie
    assert area.tolist() == [0, 1, 2, 3, 4]
    with pytest.raises(ValueError, match="does not exist"):
        o.relax_classify(lb, ub, "relax-star")


def test_structure_invariants_and_permutation_equivalence():
    rs = np.random.RandomState(2)
    S = _rand_star(rs, 40, 6)
    lb, ub = o.estimate_ranges(S)
    outs = {m: o.reach_relaxed_star(S, m, 1.0) for m in o.RELAX_METHODS}
    ref = outs["relax-star-static"]
    m1, m2 = o.relax_classify(lb, ub, "relax-star-static")
    m = m2.size
    assert 0 < m < 40 and ref.nVar == 6 + m and ref.C.shape == (2 + 3 * m, 6 + m)
    assert not ref.V[m1].any() and not ref.V[m2, :7].any()
    assert np.array_equal(ref.V[:, 7:].sum(0), np.ones(m)) and np.array_equal(ref.V[m2, 7 + np.arange(m)], np.ones(m))
    act = np.setdiff1d(np.arange(40), np.r_[m1, m2])
    assert np.array_equal(ref.V[act, :7], S.V[act])
    assert np.array_equal(ref.predicate_lb[6:], np.zeros(m)) and np.array_equal(ref.predicate_ub[6:], ub[m2])
    assert ref.Z is None and ref.state_lb is None
    for name, R in outs.items():
        _, order = o.relax_classify(lb, ub, name)
        perm = np.array([np.flatnonzero(m2 == i)[0] for i in order])   # new column j <-> static column perm[j]
        cols = np.r_[np.arange(7), 7 + perm]
        assert np.array_equal(R.V, ref.V[:, cols]), name
        rows = np.r_[np.arange(2), 2 + perm, 2 + m + perm, 2 + 2 * m + perm]
        assert np.array_equal(R.C, ref.C[np.ix_(rows, cols[1:] - 1)]), name
        assert np.array_equal(R.d, ref.d[rows]), name
        assert np.array_equal(R.predicate_ub, ref.predicate_ub[cols[1:] - 1]), name


def _contained(S, y, alpha, tol=1e-9):
    """Containment check the reference's soundness tests do by LP
    (tests/soundness/soundness_test_utils.m:228-322), done constructively: the new predicate of a
    crossing neuron takes the value of its ReLU output."""
    ok = np.all(S.C @ alpha <= S.d + tol) and np.all(alpha >= S.predicate_lb - tol) and np.all(alpha <= S.predicate_ub + tol)
    return ok and np.allclose(S.V[:, 0] + S.V[:, 1:] @ alpha, y, atol=1e-9)


@pytest.mark.parametrize("method", ["relax-star-area", "relax-star-random"])
def test_containment_through_fc_net(method):
    cfg = make_config(1)
    I = o.star_from_box(cfg["lb"], cfg["ub"])
    out, rs_sets = o.nn_reach(cfg["layers"], I, method, 1.0, keep=True)
    rs = np.random.RandomState(3)
    n0 = I.nVar
    samples = [np.array(c, dtype=float) for c in itertools.islice(itertools.product([-1, 1], repeat=n0), 16)]
    samples += [rs.uniform(-1, 1, n0) for _ in range(16)]
    for a0 in samples:
        x = I.V[:, 0] + I.V[:, 1:] @ a0
        alpha = a0.copy()
        for L, S in zip(cfg["layers"], rs_sets):
            if L["type"] == "fc":
                x = L["W"] @ x + L["b"]
            else:
                y = np.maximum(x, 0)
                new = S.nVar - alpha.size
                onehot = S.V[:, 1 + alpha.size:]
                idx = np.array([np.flatnonzero(onehot[:, j])[0] for j in range(new)], dtype=int)
                alpha = np.r_[alpha, y[idx]]
                x = y
            assert _contained(S, x, alpha), L["type"]
        assert np.allclose(x, o.evaluate(cfg["layers"], I.V[:, 0] + I.V[:, 1:] @ a0))
        lb, ub = o.output_ranges(out)
        assert np.all(x >= lb - 1e-9) and np.all(x <= ub + 1e-9)


def test_conv_matches_torch_fp64():
    rs = np.random.RandomState(4)
    for (H, W, Cin, Cout, FH, FW, s, p, dil) in [(7, 6, 3, 4, 3, 3, 1, 1, 1), (9, 9, 2, 5, 3, 3, 2, 0, 1),
                                                 (8, 10, 1, 2, 3, 2, 2, 1, 1), (11, 9, 2, 3, 3, 3, 1, 2, 2)]:
        X = rs.randn(H, W, Cin, 5)
        Wt = rs.randn(FH, FW, Cin, Cout)
        b = rs.randn(Cout)
        got = o.conv2d_tensor(X, Wt, b, [p, p, p, p], [s, s], [dil, dil])
        ref = torch.nn.functional.conv2d(torch.from_numpy(X.transpose(3, 2, 0, 1).copy()),
                                         torch.from_numpy(Wt.transpose(3, 2, 0, 1).copy()),
                                         torch.from_numpy(b), stride=s, padding=p, dilation=dil)
        np.testing.assert_allclose(got, ref.numpy().transpose(2, 3, 1, 0), rtol=1e-12, atol=1e-12)
        # single-channel slices agree with the in-tree pure definition
        fm = sum(o.conv2d_feature_map(X[:, :, c, 0], Wt[:, :, c, 1], [p, p, p, p], [s, s], [dil, dil])
                 for c in range(Cin)) + b[1]
        np.testing.assert_allclose(got[:, :, 1, 0], fm, rtol=1e-12, atol=1e-12)


def test_conv_asymmetric_padding():
    X = np.arange(12, dtype=float).reshape(3, 4)[:, :, None, None]
    Wt = np.ones((2, 2, 1, 1))
    got = o.conv2d_tensor(X, Wt, None, [1, 0, 0, 2], [1, 1], [1, 1])[:, :, 0, 0]
    Xp = np.zeros((4, 6))
    Xp[1:, :4] = X[:, :, 0, 0]
    exp = np.array([[Xp[i:i + 2, j:j + 2].sum() for j in range(5)] for i in range(3)])
    assert np.array_equal(got, exp)


def test_conv_reach_and_fc_on_imagestar_layout():
    cfg = make_config(3, shrink=4)
    sh = cfg["image_shape"]
    I = o.image_star_from_bounds(cfg["lb"].reshape(sh, order="F"), cfg["ub"].reshape(sh, order="F"))
    assert I.numPred == sh[0] * sh[1] and I.im_lb is not None
    R = o.conv2d_reach(I, cfg["layers"][0]["W"], cfg["layers"][0]["b"], cfg["layers"][0]["padding"],
                       cfg["layers"][0]["stride"], cfg["layers"][0]["dilation"])
    assert R.im_lb is None and R.V.shape[3] == I.numPred + 1
    # linearity: a sampled image maps to centre + generators * alpha
    a = np.random.RandomState(5).uniform(-1, 1, I.numPred)
    x = I.V[:, :, :, 0] + I.V[:, :, :, 1:] @ a
    y = o.evaluate(cfg["layers"][:1], x)
    np.testing.assert_allclose(R.V[:, :, :, 0] + R.V[:, :, :, 1:] @ a, y, rtol=1e-12, atol=1e-12)
    out = o.nn_reach(cfg["layers"], I, "relax-star-area", 1.0)
    assert out.V.shape[:3] == (1, 1, 10)
    yfull = o.evaluate(cfg["layers"], x)
    lb, ub = o.output_ranges(out)
    assert np.all(yfull >= lb - 1e-9) and np.all(yfull <= ub + 1e-9)


def test_box_partition_order_and_arithmetic():
    lb = np.array([0.0, 10.0, -1.0])
    ub = np.array([1.0, 14.0, 1.0])
    boxes = o.box_partition(lb, ub, [0, 1], [2, 2])
    assert len(boxes) == 4
    got = [(b[0][0], b[1][0], b[0][1], b[1][1]) for b in boxes]
    assert got == [(0.0, 0.5, 10.0, 12.0), (0.0, 0.5, 12.0, 14.0), (0.5, 1.0, 10.0, 12.0), (0.5, 1.0, 12.0, 14.0)]
    assert all(b[0][2] == -1.0 and b[1][2] == 1.0 for b in boxes)
    # new_ub = new_lb + del (Box.m:84-85), not lb + i*del
    l, u = np.array([0.1]), np.array([0.4])
    parts = o.box_single_partition(l, u, 0, 3)
    d = (u[0] - l[0]) / 3
    assert parts[2][1][0] == (l[0] + 2 * d) + d


def test_batched_reach_is_per_set_reach():
    cfg = make_config(5, shrink=16)
    boxes = o.box_partition(cfg["lb"], cfg["ub"], cfg["partition"]["indexes"], cfg["partition"]["numbers"])
    stars = [o.star_from_box(l, u) for (l, u) in boxes]
    outs = o.nn_reach(cfg["layers"], stars, "relax-star-area", 1.0)
    one = o.nn_reach(cfg["layers"], stars[1], "relax-star-area", 1.0)
    assert len(outs) == len(boxes) and np.array_equal(outs[1].V, one.V) and np.array_equal(outs[1].C, one.C)
