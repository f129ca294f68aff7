"""GPU parity of the specification check (utils/verify_specification.m) through the C ABI:
LP-free bounds of G*x, the three-way verdict, the rows handed to the host LP, and the final
verify_specification / verify_robustness answers against the oracle."""
import numpy as np
import pytest

from oracle import nnv_oracle as o
from nnv_amd.configs import make_config
from tests.gpu_util import RTOL, assert_close, input_sets

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def nnv():
    import nnv_amd
    return nnv_amd


def reach_both(nnv, cfg, method="relax-star-area"):
    dev_in, ora_in = input_sets(cfg)
    net = nnv.NN.from_config(cfg["layers"], cfg["name"])
    dev = net.reach(dev_in, {"reachMethod": method, "relaxFactor": 1})
    ora = o.nn_reach(cfg["layers"], ora_in, method, 1.0)
    return net, dev, ora


def shrink_box(cfg, factor):
    c = 0.5 * (cfg["lb"] + cfg["ub"])
    r = 0.5 * (cfg["ub"] - cfg["lb"]) * factor
    cfg = dict(cfg)
    cfg["lb"], cfg["ub"] = c - r, c + r
    return cfg


def oracle_bounds(S, G):
    S = S.to_star() if isinstance(S, o.OImageStar) else S
    return o.estimate_ranges(o.affine_map(S, G, None))


@pytest.mark.parametrize("k,shrink", [(1, 1), (2, 1), (3, 1), (4, 8)])
def test_halfspace_bounds_and_rows_match_oracle(nnv, k, shrink):
    from nnv_amd import verify
    cfg = make_config(k, shrink)
    net, dev, ora = reach_both(nnv, cfg)
    N = dev.dim if hasattr(dev, "dim") else dev.toStar().dim
    rs = np.random.RandomState(40 + k)
    hs = [nnv.HalfSpace(rs.randn(r, N), rs.randn(r)) for r in (1, 3, 2)]
    verdict, lo, hi = verify.halfspace_check(dev, hs)
    G = np.vstack([h.G for h in hs])
    olo, ohi = oracle_bounds(ora, G)
    assert_close(lo[:, 0], olo, "lo")
    assert_close(hi[:, 0], ohi, "hi")
    # verdicts follow from the bounds (set/Star.m:577-578 rows, estimateRanges bounds)
    r0 = 0
    for h, H in enumerate(hs):
        r1 = r0 + H.G.shape[0]
        want = 1 if np.any(olo[r0:r1] > H.g) else 3 if np.all(ohi[r0:r1] <= H.g) else 2
        assert verdict[0, h] == want
        r0 = r1
    # the LP rows of Star.intersectHalfSpace
    S = dev if isinstance(dev, nnv.Star) else dev.toStar()
    So = ora.to_star() if isinstance(ora, o.OImageStar) else ora
    import ctypes as C
    from nnv_amd._lib import check, f64, ptr
    H = hs[1]
    C1 = np.empty((3, S.nVar), order="F")
    d1 = np.empty(3)
    check(S.ctx.lib.nnvhip_halfspace_rows(S.ctx.handle, S._h.h, 3, ptr(f64(H.G)), ptr(f64(H.g)), N, ptr(C1), ptr(d1)))
    assert_close(C1, H.G @ So.V[:, 1:], "C1")
    assert_close(d1, H.g - H.G @ So.V[:, 0], "d1")


def test_forced_verdicts_cover_all_three_codes(nnv):
    from nnv_amd import verify
    cfg = make_config(2)
    net, dev, ora = reach_both(nnv, cfg)
    lb, ub = o.estimate_ranges(ora)
    e0 = np.zeros((1, 10))
    e0[0, 0] = 1.0
    hs = [nnv.HalfSpace(e0, [lb[0] - 1.0]),            # x0 <= below its lower bound: disjoint
          nnv.HalfSpace(e0, [ub[0] + 1.0]),            # x0 <= above its upper bound: inside
          nnv.HalfSpace(e0, [0.5 * (lb[0] + ub[0])]),  # cuts the range: undecided
          nnv.HalfSpace(np.vstack([e0, -e0]), [ub[0] + 1.0, -(lb[0] - 1.0) - 1e300])]  # second row impossible
    verdict, lo, hi = verify.halfspace_check(dev, hs)
    assert verdict[0].tolist() == [1, 3, 2, 1]
    assert_close(lo[0, 0], lb[0], "lo")
    assert_close(hi[0, 0], ub[0], "hi")


@pytest.mark.parametrize("k,shrink,factor", [(1, 1, 1.0), (1, 1, 0.02), (2, 16, 1.0), (2, 16, 0.01), (3, 4, 1.0)])
def test_verify_robustness_matches_oracle(nnv, k, shrink, factor):
    from nnv_amd import verify
    cfg = shrink_box(make_config(k, shrink), factor)
    net, dev, ora = reach_both(nnv, cfg)
    n_out = cfg["layers"][-1]["W"].shape[0]
    got, want = [], []
    lp = 0
    for t in range(n_out):
        got.append(net.checkRobust(dev, t))
        lp += verify.last_stats.lp_solved
        want.append(o.verify_specification(ora, o.robustness_set(n_out, t, "max")))
    assert got == want
    centre = 0.5 * (cfg["lb"] + cfg["ub"])
    if cfg["kind"] == "image":
        centre = centre.reshape(cfg["image_shape"], order="F")
    centre_class = int(np.argmax(o.evaluate(cfg["layers"], centre)))
    assert want[centre_class] in (1, 2)
    if factor < 0.1:
        # a tiny box is certified for its own class, and every other target is refuted by a disjunct
        # that contains the whole set: all decided on the device, no LP
        assert want[centre_class] == 1 and lp == 0
    # end-to-end entry point
    dev_in, _ = input_sets(cfg)
    assert net.verify_robustness(dev_in, {"reachMethod": "relax-star-area", "relaxFactor": 1}, centre_class) == want[centre_class]


def test_lp_path_is_exercised_and_agrees(nnv):
    from nnv_amd import verify
    cfg = make_config(1)
    net, dev, ora = reach_both(nnv, cfg)
    lb, ub = o.estimate_ranges(ora)
    # half-spaces cutting through the estimated range of a coordinate: the device cannot decide.
    # Thresholds inside [lb, ub] but possibly outside the exact range exercise both LP answers.
    answers = set()
    for j in range(5):
        for frac in (0.001, 0.05, 0.5, 0.95):
            e = np.zeros((1, 5))
            e[0, j] = 1.0
            gval = lb[j] + frac * (ub[j] - lb[j])
            got = nnv.verify_specification(dev, nnv.HalfSpace(e, [gval]))
            assert verify.last_stats.undecided == 1 and verify.last_stats.lp_solved == 1
            want = o.verify_specification(ora, o.OHalfSpace(e, [gval]))
            assert got == want
            answers.add(got)
    assert answers == {1, 2}, "both LP outcomes should occur: %r" % answers


def test_array_of_sets_and_multiple_halfspaces(nnv):
    from nnv_amd import verify
    cfg = make_config(5, 64)
    net, dev, ora = reach_both(nnv, cfg)
    assert isinstance(dev, (list, nnv.SetArray)) and len(dev) == len(ora) > 1
    n_out = cfg["layers"][-1]["W"].shape[0]
    rs = np.random.RandomState(5)
    hs = [nnv.HalfSpace(rs.randn(2, n_out), rs.randn(2)) for _ in range(4)]
    verdict, lo, hi = verify.halfspace_check(dev, hs)
    G = np.vstack([h.G for h in hs])
    for i, S in enumerate(ora):
        olo, ohi = oracle_bounds(S, G)
        assert_close(lo[:, i], olo, "lo set %d" % i)
        assert_close(hi[:, i], ohi, "hi set %d" % i)
    for t in range(n_out):
        assert net.checkRobust(dev, t) == o.verify_specification(ora, o.robustness_set(n_out, t, "max"))


def test_hand_built_empty_set_and_errors(nnv):
    # an infeasible predicate (alpha <= -2 within [-1, 1]): the reference's LP reports every
    # intersection empty, so the answer is 1 even for a half-space that contains the whole image
    S = nnv.Star(np.array([[0.0, 1.0], [0.0, 0.5]]), np.array([[1.0]]), np.array([-2.0]), [-1.0], [1.0])
    H = nnv.HalfSpace([[1.0, 0.0]], [10.0])
    assert nnv.verify_specification(S, H, assume_nonempty=False) == 1
    assert nnv.verify_specification(S, H) == 1            # default: a set with the caller's own constraints gets its LP
    assert nnv.verify_specification(S, H, assume_nonempty=True) == 2
    # ... also after it went through layers: the emptiness travels with the constraints
    mapped = nnv.PosLin.reach(S.affineMap(np.array([[1.0, -1.0], [0.5, 2.0]]), np.array([0.1, -0.2])), "relax-star-area", [], 1)
    assert nnv.verify_specification(mapped, nnv.HalfSpace([[1.0, 0.0]], [100.0])) == 1
    So = o.OStar(np.array([[0.0, 1.0], [0.0, 0.5]]), np.array([[1.0]]), np.array([-2.0]), [-1.0], [1.0])
    assert o.verify_specification(So, o.OHalfSpace([[1.0, 0.0]], [10.0])) == 1
    with pytest.raises(ValueError, match="Inconsistent dimension between halfspace and star set"):
        nnv.verify_specification(S, nnv.HalfSpace([[1.0, 0.0, 0.0]], [0.0]))
    with pytest.raises(ValueError, match="Inconsistent dimension between half-space matrix and half-space vector"):
        nnv.HalfSpace([[1.0, 0.0]], [0.0, 1.0])


def test_disjoint_needs_a_margin(nnv):
    """A set that touches the half-space to within rounding is not called disjoint by the device pass: the pair
    goes to the LP like every pair does in the reference."""
    from nnv_amd import verify
    S = nnv.Star(np.array([1.0, 0.0]), np.array([2.0, 1.0]))        # x1 in [1, 2]
    near = nnv.HalfSpace([[1.0, 0.0]], [1.0 - 1e-13])                # x1 <= 1 - 1e-13: lo - g = 1e-13, inside the margin
    far = nnv.HalfSpace([[1.0, 0.0]], [1.0 - 1e-6])
    v, lo, hi = verify.halfspace_check(S, [near, far])
    assert v[0, 0] == verify.HS_UNDECIDED and v[0, 1] == verify.HS_DISJOINT
    # the LP settles it as the reference's does: feasible within the solver's tolerance -> "unknown", not "robust"
    So = o.star_from_box(np.array([1.0, 0.0]), np.array([2.0, 1.0]))
    assert nnv.verify_specification(S, near) == o.verify_specification(So, o.OHalfSpace([[1.0, 0.0]], [1.0 - 1e-13])) == 2
    assert nnv.verify_specification(S, far) == o.verify_specification(So, o.OHalfSpace([[1.0, 0.0]], [1.0 - 1e-6])) == 1
