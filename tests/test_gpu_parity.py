"""GPU parity tests: the HIP path (through the C ABI) against the CPU oracle on the same seeded inputs."""
import contextlib

import numpy as np
import pytest

from tests.gpu_util import RTOL, assert_close, assert_close_elementwise, compare_sets, flat_V, input_sets, run_both, run_cfg

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


def _rand_star_arrays(rs, N, n, p=3):
    V = rs.randn(N, n + 1)
    C = rs.randn(p, n)
    d = np.abs(rs.randn(p)) + 5.0
    lb = -np.abs(rs.rand(n)) - 0.1
    ub = np.abs(rs.rand(n)) + 0.1
    return V, C, d, lb, ub


def test_golden_affine_map_and_ranges(nnv, oracle, golden):
    g = golden["star_affineMap"]
    S = nnv.Star(g["S_V"], g["S_C"], g["S_d"])
    S1 = S.affineMap(g["W"], g["b"])
    assert np.array_equal(S1.V, g["S1_V"])
    assert np.array_equal(S1.C, g["S1_C"]) and np.array_equal(S1.d, g["S1_d"].reshape(-1))
    S3 = nnv.Star(g["box_lb"].reshape(-1), g["box_ub"].reshape(-1))
    assert np.array_equal(S3.V, oracle.star_from_box(g["box_lb"].reshape(-1), g["box_ub"].reshape(-1)).V)
    assert np.array_equal(S3.C, np.zeros((1, 3))) and np.array_equal(S3.d, np.zeros(1))
    lb, ub = S3.affineMap(g["W2"], None).estimateRanges()
    np.testing.assert_allclose(lb, g["S4_lb"].reshape(-1), rtol=0, atol=1e-14)
    np.testing.assert_allclose(ub, g["S4_ub"].reshape(-1), rtol=0, atol=1e-14)
    gi = golden["imagestar_getRange_issue"]
    I = nnv.ImageStar(gi["V"], np.zeros((1, 2)), np.zeros(1), gi["pred_lb"], gi["pred_ub"])
    l, u = I.estimateRanges()
    assert l.reshape(-1)[0] == -2.0 and u.reshape(-1)[0] == 2.0


def test_golden_conv_known_answer(nnv, golden):
    g = golden["conv2d_featureMap"]
    I = nnv.ImageStar(g["I"][:, :, None, None].repeat(2, axis=3) * np.array([1.0, 0.0]), np.zeros((1, 1)),
                      np.zeros(1), [-1.0], [1.0])
    L = nnv.Conv2DLayer(g["W"][:, :, None, None], np.zeros(1), g["padding"], g["stride"], g["dilation"])
    R = L.reach(I, "relax-star-area")
    assert np.array_equal(R.V[:, :, 0, 0], g["expected"])
    assert not R.V[:, :, 0, 1].any()


@pytest.mark.parametrize("N,n", [(1, 1), (5, 3), (16, 16), (50, 7), (129, 300), (1024, 2500), (3000, 65), (10, 4000)])
def test_star_roundtrip_and_ranges(nnv, oracle, N, n):
    rs = np.random.RandomState(N * 7 + n)
    V, C, d, lb, ub = _rand_star_arrays(rs, N, n)
    S = nnv.Star(V, C, d, lb, ub)
    assert (S.dim, S.nVar) == (N, n)
    assert np.array_equal(S.V, V) and np.array_equal(S.C, C) and np.array_equal(S.d, d)
    assert np.array_equal(S.predicate_lb, lb) and np.array_equal(S.predicate_ub, ub)
    glb, gub = S.estimateRanges()
    elb, eub = oracle.estimate_ranges(oracle.OStar(V, C, d, lb, ub))
    assert_close(glb, elb, "lb", 1e-12)
    assert_close(gub, eub, "ub", 1e-12)
    # default predicate bounds (-1/+1) when none are given
    S2 = nnv.Star(V, C, d)
    g2l, g2u = S2.estimateRanges()
    e2l, e2u = oracle.estimate_ranges(oracle.OStar(V, C, d))
    assert_close(g2l, e2l, "lb default", 1e-12)
    assert_close(g2u, e2u, "ub default", 1e-12)


@pytest.mark.parametrize("M,K,n", [(1, 1, 1), (5, 5, 5), (50, 5, 5), (10, 100, 1045), (64, 64, 63), (100, 784, 20),
                                   (130, 70, 257), (256, 300, 1000), (1024, 784, 785), (33, 1000, 129)])
def test_affine_fc(nnv, oracle, M, K, n):
    rs = np.random.RandomState(M + 3 * K + n)
    V, C, d, lb, ub = _rand_star_arrays(rs, K, n)
    W = rs.randn(M, K)
    b = rs.randn(M)
    S = nnv.Star(V, C, d, lb, ub)
    R = S.affineMap(W, b)
    E = oracle.affine_map(oracle.OStar(V, C, d, lb, ub), W, b)
    compare_sets(R, E, "affineMap %dx%dx%d" % (M, K, n))
    R2 = S.affineMap(W, None)
    assert_close(R2.V[:, 0], (W @ V)[:, 0], "no-bias centre")
    L = nnv.FullyConnectedLayer(W, b)
    R3 = L.reach(S, "relax-star-area", [], 1, None, "linprog")
    assert np.array_equal(R3.V, R.V)
    with pytest.raises(ValueError, match="affine mapping matrix"):
        S.affineMap(rs.randn(3, K + 1), None)
    with pytest.raises(ValueError, match="Unknown reachability method"):
        L.reach(S, "bogus")


@pytest.mark.parametrize("H,W,Cin,Cout,FH,FW,s,p,dil,n", [
    (5, 5, 1, 1, 3, 3, 1, 0, 1, 1), (7, 6, 3, 4, 3, 3, 1, 1, 1, 9), (9, 9, 2, 5, 3, 3, 2, 0, 1, 30),
    (8, 10, 1, 2, 3, 2, 2, 1, 1, 17), (11, 9, 2, 3, 3, 3, 1, 2, 2, 5), (28, 28, 1, 16, 3, 3, 1, 1, 1, 40),
    (14, 14, 16, 32, 3, 3, 2, 1, 1, 33), (15, 15, 32, 64, 3, 3, 1, 1, 1, 20), (12, 12, 40, 70, 5, 5, 2, 2, 1, 7),
    (13, 12, 2, 5, 6, 6, 1, 2, 1, 4), (20, 20, 3, 40, 7, 5, 2, 3, 2, 6)])   # more than 32 spatial taps: the general kernel
def test_affine_conv2d(nnv, oracle, H, W, Cin, Cout, FH, FW, s, p, dil, n):
    rs = np.random.RandomState(H * 31 + Cout)
    V = rs.randn(H, W, Cin, n + 1)
    C = rs.randn(2, n)
    d = np.ones(2)
    lb, ub = -np.ones(n), np.ones(n)
    Wt = rs.randn(FH, FW, Cin, Cout)
    b = rs.randn(Cout)
    I = nnv.ImageStar(V, C, d, lb, ub)
    L = nnv.Conv2DLayer(Wt, b, [p, p, p, p], [s, s], [dil, dil])
    R = L.reach(I, "relax-star-area", "single")
    E = oracle.conv2d_reach(oracle.OImageStar(V, C, d, lb, ub), Wt, b, [p, p, p, p], [s, s], [dil, dil])
    assert R.V.shape == E.V.shape
    compare_sets(R, E, "conv")
    with pytest.raises(ValueError, match="channels"):
        nnv.Conv2DLayer(rs.randn(3, 3, Cin + 1, 2), np.zeros(2)).reach(I, "relax-star-area")


def test_conv_asymmetric_padding(nnv, oracle):
    rs = np.random.RandomState(11)
    V = rs.randn(6, 7, 2, 4)
    Wt = rs.randn(2, 3, 2, 3)
    b = rs.randn(3)
    I = nnv.ImageStar(V, np.zeros((1, 3)), np.zeros(1), -np.ones(3), np.ones(3))
    R = nnv.Conv2DLayer(Wt, b, [1, 0, 2, 1], [1, 2], [1, 1]).reach(I, "relax-star-area")
    E = oracle.conv2d_reach(oracle.OImageStar(V, np.zeros((1, 3)), np.zeros(1), -np.ones(3), np.ones(3)), Wt, b,
                            [1, 0, 2, 1], [1, 2], [1, 1])
    compare_sets(R, E, "conv asym")


@pytest.mark.parametrize("method", ["relax-star-area", "relax-star-range", "relax-star-random", "relax-star-static",
                                    "relax-star-bound", "relax-star-ub"])
@pytest.mark.parametrize("N,n", [(7, 3), (64, 10), (1000, 50), (2500, 300)])
def test_relu_step(nnv, oracle, method, N, n):
    rs = np.random.RandomState(N + n)
    V, C, d, lb, ub = _rand_star_arrays(rs, N, n)
    V[:, 0] *= 3.0
    S = nnv.Star(V, C, d, lb, ub)
    R = nnv.PosLin.reach(S, method, [], 1, None, "linprog")
    O = oracle.OStar(V, C, d, lb, ub)
    E = oracle.reach_relaxed_star(O, method, 1.0)
    elb, eub = oracle.estimate_ranges(O)
    m1, m2 = oracle.relax_classify(elb, eub, method)
    ni, idx, clb, cub = R.relu_info()
    assert ni == m1.size and np.array_equal(idx, m2)           # classification + new-predicate order: exact
    assert np.array_equal(R.V, E.V)                            # zeroing / one-hot columns: exact
    compare_sets(R, E, "relu " + method)
    assert np.array_equal(R.C[:3 + 2 * m2.size], E.C[:3 + 2 * m2.size])   # C0, C1, C2 rows are copies: exact
    assert R.C.shape == (3 + 3 * m2.size, n + m2.size)


@pytest.mark.parametrize("method", ["relax-star-area", "relax-star-range"])
@pytest.mark.parametrize("N", [2, 3, 33, 64, 65, 127, 128, 129, 255, 257, 511, 513, 777, 1023, 1024, 1025, 2047, 4100, 8192, 9000])
def test_crossing_order_all_list_lengths_with_ties(nnv, oracle, method, N):
    # every neuron crosses; keys come from a handful of values so that most of them tie and the stable
    # rule (equal keys keep ascending neuron order) decides the order.  Bounds are exact in fp64:
    # one generator, centre 0, |V| in {1/8, 1/4, 1/2, 1}  ->  lb = -|v|, ub = |v|.
    rs = np.random.RandomState(N)
    mag = rs.choice([0.125, 0.25, 0.5, 1.0], size=N) * rs.choice([-1.0, 1.0], size=N)
    V = np.c_[np.zeros(N), mag]
    if N > 3:
        V[rs.choice(N, size=N // 7, replace=False), 0] = 4.0      # some active neurons in between
        V[rs.choice(N, size=N // 9, replace=False), 0] = -4.0     # and some inactive ones
    args = (V, np.zeros((1, 1)), np.zeros(1), [-1.0], [1.0])
    R = nnv.PosLin.reach(nnv.Star(*args), method, [], 1)
    O = oracle.OStar(*args)
    elb, eub = oracle.estimate_ranges(O)
    m1, m2 = oracle.relax_classify(elb, eub, method)
    ni, idx, clb, cub = R.relu_info()
    assert ni == m1.size
    assert np.array_equal(idx, m2)
    assert np.array_equal(clb, elb[m2]) and np.array_equal(cub, eub[m2])


def test_relu_ties_and_degenerate(nnv, oracle):
    # hand-built bounds: ub == 0 -> inactive, lb == 0 -> active; equal sort keys keep index order
    V = np.array([[-0.5, 0.5], [0.5, 0.5], [1.0, -3.0], [-1.0, 2.0], [2.0, 0.0], [-1.0, 0.0], [1.0, 3.0], [-1.0, -2.0]])
    S = nnv.Star(V, np.zeros((1, 1)), np.zeros(1), [-1.0], [1.0])
    for method in ("relax-star-area", "relax-star-range", "relax-star-static"):
        R = nnv.PosLin.reach(S, method, [], 1)
        E = oracle.reach_relaxed_star(oracle.OStar(V, np.zeros((1, 1)), np.zeros(1), [-1.0], [1.0]), method, 1.0)
        ni, idx, _, _ = R.relu_info()
        assert ni == 2
        assert np.array_equal(R.V, E.V) and np.array_equal(R.C, E.C) and np.array_equal(R.d, E.d), method
    # all active: identity, no new predicate; all inactive: zero set
    G = 0.1 * np.random.RandomState(1).randn(20, 4)
    for c, chk in ((5.0, lambda R, V: np.array_equal(R.V, V)), (-5.0, lambda R, V: not R.V.any())):
        Vc = np.c_[np.full(20, c), G]
        R = nnv.PosLin.reach(nnv.Star(Vc, np.zeros((1, 4)), np.zeros(1), -np.ones(4), np.ones(4)), "relax-star-area", [], 1)
        assert R.nVar == 4 and R.C.shape == (1, 4) and chk(R, Vc)
    with pytest.raises(ValueError, match="Invalid relax factor"):
        nnv.PosLin.reach(S, "relax-star-area", [], 1.5)
    with pytest.raises(ValueError, match="does not exist"):
        nnv.PosLin.reach(S, "relax-star", [], 1)
    # below 1 the host solves LPs first; the all-device entry point says so instead of guessing
    import ctypes
    from nnv_amd._lib import ORDER_AREA, check
    ctx = S.ctx
    raw_in, raw_out = (ctypes.c_void_p * 1)(S._h.h), (ctypes.c_void_p * 1)()
    with pytest.raises(ValueError, match="relaxFactor < 1"):
        check(ctx.lib.nnvhip_relu_relax(ctx.handle, ORDER_AREA, 0.5, 1, raw_in, raw_out))
    assert nnv.PosLin.reach(S, "relax-star-area", [], 0.5).nVar <= nnv.PosLin.reach(S, "relax-star-area", [], 1).nVar


@pytest.mark.parametrize("method", ["relax-star-area", "relax-star-random"])
def test_config1_full(nnv, method):
    margins = []
    run_both(1, method, margins=margins)
    assert min(margins) > 1e-12


def test_config2_full(nnv, oracle, capsys):
    margins = []
    dev, ora, net = run_both(2, "relax-star-area", margins=margins)
    dl, du = dev.estimateRanges()
    ol, ou = oracle.output_ranges(ora)
    assert_close_elementwise(dl, ol, "output lb")
    assert_close_elementwise(du, ou, "output ub")
    with capsys.disabled() if capsys is not None else contextlib.nullcontext():
        print("\ncfg2 classification margin per ReLU layer (min |bound| / max width):", ["%.2e" % m for m in margins])
    assert min(margins) > 1e-12


def test_config3_full(nnv, oracle, capsys):
    margins = []
    dev, ora, net = run_both(3, "relax-star-area", margins=margins)
    dl, du = dev.estimateRanges()
    ol, ou = oracle.output_ranges(ora)
    assert_close_elementwise(dl.reshape(-1), ol, "output lb")
    assert_close_elementwise(du.reshape(-1), ou, "output ub")
    with capsys.disabled() if capsys is not None else contextlib.nullcontext():
        print("\ncfg3 classification margin per ReLU layer (min |bound| / max width):", ["%.2e" % m for m in margins])
    assert min(margins) > 1e-12


def test_config4_shrunk(nnv):
    run_both(4, "relax-star-area", shrink=4)
    run_both(4, "relax-star-random", shrink=8)
    # ub-lb has exact mathematical ties across positions of a conv channel: order checked up to ties
    run_both(4, "relax-star-range", shrink=8, tie_tolerant=True)


def test_config5_shrunk_batched(nnv, oracle):
    dev, ora, net = run_both(5, "relax-star-area", shrink=4, check_constraints=False)
    assert len(dev) == len(ora) == 4
    run_both(5, "relax-star-random", shrink=8)


def test_out_of_memory_is_an_error_code_not_a_crash(nnv):
    # Star(lb, ub) with 2^20 free dimensions needs an 8.8 TB generator matrix: the library must
    # report NNVHIP_ERR_OOM (MemoryError here) and stay usable
    N = 1 << 20
    with pytest.raises(MemoryError):
        nnv.Star(np.zeros(N), np.ones(N))
    S = nnv.Star(np.zeros(4), np.ones(4))
    assert S.nVar == 4 and np.array_equal(S.estimateRanges()[1], np.ones(4))


def test_zero_width_dimensions_and_scalar_box(nnv, oracle):
    lb = np.array([0.5, -1.0, 2.0, 2.0])
    ub = np.array([0.5, 1.0, 2.0, 3.0])
    S = nnv.Star(lb, ub)
    E = oracle.star_from_box(lb, ub)
    assert S.nVar == 2 and np.array_equal(S.V, E.V)
    one = nnv.Star(np.array([1.0]), np.array([1.0]))         # numel(gens) == 1: the zero column stays
    assert one.nVar == 1 and np.array_equal(one.V, oracle.star_from_box([1.0], [1.0]).V)
    allfix = nnv.Star(np.array([1.0, 2.0]), np.array([1.0, 2.0]))
    assert allfix.nVar == 0 and np.array_equal(allfix.V, np.array([[1.0], [2.0]]))
    l, u = allfix.estimateRanges()
    assert np.array_equal(l, [1.0, 2.0]) and np.array_equal(u, [1.0, 2.0])
    R = nnv.PosLin.reach(allfix, "relax-star-area", [], 1)
    assert R.nVar == 0 and np.array_equal(R.V, allfix.V)


def _reach_in_subprocess(dense, k, method, shrink):
    """Output V / bounds of config k from a fresh process, with or without the structural-zero skipping
    of the FC map (the switch is read once per process)."""
    import json
    import os
    import subprocess
    import sys
    code = (
        "import json, sys, numpy as np, nnv_amd\n"
        "from nnv_amd.configs import make_config, device_input_sets\n"
        "cfg = make_config(%d, %d)\n"
        "net = nnv_amd.NN.from_config(cfg['layers'])\n"
        "out = net.reach(device_input_sets(cfg), {'reachMethod': '%s', 'relaxFactor': 1})\n"
        "outs = out if isinstance(out, (list, nnv_amd.SetArray)) else [out]\n"
        "res = []\n"
        "for o_ in outs:\n"
        "    V = np.asarray(o_.V); lb, ub = o_.estimateRanges()\n"
        "    res.append([V.reshape(-1, order='F').tolist(), np.asarray(lb).reshape(-1).tolist(), np.asarray(ub).reshape(-1).tolist()])\n"
        "json.dump(res, sys.stdout)\n" % (k, shrink, method))
    env = dict(os.environ)
    env.pop("NNVHIP_DENSE_AFFINE", None)
    if dense:
        env["NNVHIP_DENSE_AFFINE"] = "1"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, "-c", code], cwd=root, env=env, stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=200)
    assert p.returncode == 0, p.stderr.decode()[-2000:]
    return json.loads(p.stdout.decode())


@pytest.mark.parametrize("k,shrink", [(1, 1), (2, 1), (5, 64)])
def test_structural_zero_skipping_equals_dense_contraction(k, shrink):
    # W*[c V] with the one-hot columns gathered and the reset rows left out must give what the full
    # dense contraction gives: same columns bit for bit where only a gather is involved, and the
    # contracted columns up to the summation order of the kept rows
    a = _reach_in_subprocess(False, k, "relax-star-area", shrink)
    b = _reach_in_subprocess(True, k, "relax-star-area", shrink)
    assert len(a) == len(b)
    for (Va, la, ua), (Vb, lb_, ub_) in zip(a, b):
        Va, Vb = np.asarray(Va), np.asarray(Vb)
        assert Va.shape == Vb.shape
        scale = np.max(np.abs(Vb))
        assert np.max(np.abs(Va - Vb)) <= 1e-13 * scale
        assert np.array_equal(Va == 0, Vb == 0)
        assert np.allclose(la, lb_, rtol=0, atol=1e-12 * max(1.0, np.max(np.abs(lb_))))
        assert np.allclose(ua, ub_, rtol=0, atol=1e-12 * max(1.0, np.max(np.abs(ub_))))


def test_fc_on_sets_with_and_without_structure_hints(nnv, oracle):
    # the same matrices as a hand-built Star (no hints), as a box star (all generators one-hot) and as a
    # ReLU output (appended one-hot columns, reset rows), alone and mixed in one array
    rs = np.random.RandomState(77)
    N, M = 96, 40
    W, b = rs.randn(M, N), rs.randn(M)
    L = nnv.FullyConnectedLayer(W, b)
    lbv = -rs.rand(N)
    ubv = rs.rand(N)
    lbv[5] = ubv[5] = 0.25          # zero-width dimension: its generator column is dropped
    box_d, box_o = nnv.Star(lbv, ubv), oracle.star_from_box(lbv, ubv)
    Vh = rs.randn(N, 9)
    args = (Vh, np.zeros((1, 8)), np.zeros(1), -np.ones(8), np.ones(8))
    hand_d, hand_o = nnv.Star(*args), oracle.OStar(*args)
    W0, b0 = rs.randn(N, N), rs.randn(N)
    pre_d = nnv.FullyConnectedLayer(W0, b0).reach(box_d, "approx-star")
    relu_d = nnv.PosLin.reach(pre_d, "relax-star-area", [], 1)
    relu_o = oracle.reach_relaxed_star(oracle.affine_map(box_o, W0, b0), "relax-star-area", 1.0)
    for dset, oset, tag in ((box_d, box_o, "box"), (hand_d, hand_o, "hand"), (relu_d, relu_o, "relu")):
        R = L.reach(dset, "approx-star")
        E = oracle.affine_map(oset, W, b)
        assert_close(R.V, E.V, "fc on %s star" % tag)
        lb, ub = R.estimateRanges()
        elb, eub = oracle.estimate_ranges(E)
        assert_close(lb, elb, tag + " lb")
        assert_close(ub, eub, tag + " ub")
    outs = L.reach([relu_d, box_d, relu_d], "approx-star")     # array: not one arena, per-set launches
    for R, oset in zip(outs, (relu_o, box_o, relu_o)):
        assert_close(R.V, oracle.affine_map(oset, W, b).V, "fc on mixed array")


@pytest.mark.parametrize("k,shrink", [(1, 1), (2, 1), (3, 1), (5, 64)])
def test_configs_with_full_dense_contraction(nnv, k, shrink):
    # the same oracle parity with every FC / conv layer run as the full dense contraction
    ctx = nnv.default_context()
    ctx.set_dense_affine(True)
    try:
        run_both(k, "relax-star-area", shrink)
    finally:
        ctx.set_dense_affine(False)


def test_relu_output_consumers_that_need_every_column(nnv, oracle):
    # a ReLU output keeps its appended unit-vector columns implicit; ranges, another ReLU, a
    # row-wise layer and a property read must all see the full matrix
    rs = np.random.RandomState(91)
    N, n = 300, 40
    V, C, d, lb, ub = _rand_star_arrays(rs, N, n)
    S = nnv.Star(V, C, d, lb, ub)
    O = oracle.OStar(V, C, d, lb, ub)
    R = nnv.PosLin.reach(S, "relax-star-area", [], 1)
    E = oracle.reach_relaxed_star(O, "relax-star-area", 1.0)
    assert E.nVar > n                                   # some neurons cross
    rl, ru = R.estimateRanges()                         # before any read of R.V
    el, eu = oracle.estimate_ranges(E)
    assert_close(rl, el, "ranges of a ReLU output (lb)")
    assert_close(ru, eu, "ranges of a ReLU output (ub)")
    R2 = nnv.PosLin.reach(nnv.PosLin.reach(S, "relax-star-area", [], 1), "relax-star-range", [], 1)
    E2 = oracle.reach_relaxed_star(E, "relax-star-range", 1.0)
    assert np.array_equal(R2.V, E2.V)
    mean, var = rs.randn(N), rs.rand(N) + 0.5
    BN = nnv.BatchNormalizationLayer(NumChannels=N, TrainedMean=mean, TrainedVariance=var)
    R3 = BN.reach(nnv.PosLin.reach(S, "relax-star-area", [], 1), "approx-star")
    E3 = oracle.batchnorm_reach(E, mean, var, 1e-5, np.ones(N), np.zeros(N))
    assert np.array_equal(R3.V, E3.V)
    assert np.array_equal(R.V, E.V)                     # property read of the first output, last


@pytest.mark.parametrize("N,M", [(96, 40), (700, 300)])
def test_relu_output_whose_row_reset_is_still_pending(nnv, oracle, N, M):
    # a ReLU output shares its input's matrix until somebody needs the reset rows in memory: the FC map
    # must give the same set before and after that, alone and in an array, and the input set is untouched
    rs = np.random.RandomState(5 + N)
    W0, b0 = rs.randn(N, N), rs.randn(N)
    W, b = rs.randn(M, N), rs.randn(M)
    L = nnv.FullyConnectedLayer(W, b)
    lbv, ubv = -rs.rand(N), rs.rand(N)
    box_d, box_o = nnv.Star(lbv, ubv), oracle.star_from_box(lbv, ubv)
    pre_d = nnv.FullyConnectedLayer(W0, b0).reach(box_d, "approx-star")
    pre_o = oracle.affine_map(box_o, W0, b0)
    relu_o = oracle.reach_relaxed_star(pre_o, "relax-star-area", 1.0)
    E = oracle.affine_map(relu_o, W, b)
    assert relu_o.nVar > box_o.nVar
    relu_d = nnv.PosLin.reach(pre_d, "relax-star-area", [], 1)
    first = L.reach(relu_d, "approx-star")                      # reset pending: contraction over the kept rows
    assert_close(first.V, E.V, "fc on a ReLU output, reset pending")
    pair = L.reach([relu_d, nnv.PosLin.reach(pre_d, "relax-star-area", [], 1)], "approx-star")
    for R in pair:
        assert_close(R.V, E.V, "fc on an array of ReLU outputs, reset pending")
    assert np.array_equal(relu_d.V, relu_o.V)                   # the read runs the reset into a new buffer
    assert_close(pre_d.V, pre_o.V, "input of the ReLU after its output was written out")
    assert np.count_nonzero(np.asarray(pre_d.V)[:, 0] < 0) > 0  # ... still holds its negative rows
    second = L.reach(relu_d, "approx-star")
    assert_close(second.V, E.V, "fc on a ReLU output, rows in memory")
    el, eu = oracle.estimate_ranges(E)
    for R in (first, second):
        lb, ub = R.estimateRanges()
        assert_close(lb, el, "lb")
        assert_close(ub, eu, "ub")
    # a second ReLU directly on a pending output (no layer between)
    R2 = nnv.PosLin.reach(nnv.PosLin.reach(pre_d, "relax-star-area", [], 1), "relax-star-range", [], 1)
    E2 = oracle.reach_relaxed_star(relu_o, "relax-star-range", 1.0)
    assert np.array_equal(R2.V, E2.V)


def test_fc_after_a_relu_that_kept_no_row(nnv, oracle):
    # every neuron crossing or inactive: the columns the ReLU kept are all zero, so the next FC map has
    # nothing to contract over -- centre = bias, zeros, gathered columns; alone, in one arena, mixed with a
    # set that did keep rows, and without a bias
    rs = np.random.RandomState(12)
    n, N, M = 20, 400, 300                              # big enough for the structured route
    W0 = rs.randn(N, n)
    W1, b1 = rs.randn(M, N), rs.randn(M)
    wide_lb, wide_ub = -np.ones((n, 3)) * 50, np.ones((n, 3)) * 50
    wide_lb[:, 1], wide_ub[:, 1] = 0.5, 0.6              # the middle box is narrow: it keeps rows
    L0 = nnv.FullyConnectedLayer(W0, np.zeros(N))
    L1 = nnv.FullyConnectedLayer(W1, b1)
    boxes = nnv.Star.from_boxes(wide_lb, wide_ub)
    relu = nnv.PosLin.reach(L0.reach(boxes, "approx-star"), "relax-star-area", [], 1)
    outs = L1.reach(relu, "approx-star")
    kept = []
    for i, (R, X) in enumerate(zip(outs, relu)):
        O = oracle.reach_relaxed_star(oracle.affine_map(oracle.star_from_box(wide_lb[:, i], wide_ub[:, i]), W0, np.zeros(N)),
                                      "relax-star-area", 1.0)
        E = oracle.affine_map(O, W1, b1)
        ni, idx, _, _ = X.relu_info()
        kept.append(N - ni - idx.size)
        assert_close(R.V, E.V, "fc after relu, set %d" % i)
        lb, ub = R.estimateRanges()
        elb, eub = oracle.estimate_ranges(E)
        assert_close(lb, elb, "lb %d" % i)
        assert_close(ub, eub, "ub %d" % i)
        alone = L1.reach(nnv.PosLin.reach(L0.reach(nnv.Star(wide_lb[:, i], wide_ub[:, i]), "approx-star"),
                                          "relax-star-area", [], 1), "approx-star")
        if kept[-1] == 0:
            assert np.array_equal(alone.V, R.V)      # nothing is summed: bit for bit
        else:
            assert_close(alone.V, R.V, "alone against batched")
        nobias = nnv.PosLin.reach(L0.reach(nnv.Star(wide_lb[:, i], wide_ub[:, i]), "approx-star"),
                                  "relax-star-area", [], 1).affineMap(W1, None)
        assert_close(nobias.V, oracle.affine_map(O, W1, None).V, "no bias %d" % i)
        # a second ReLU on top: its ranges come from the sums the gather pass left
        R2 = nnv.PosLin.reach(R, "relax-star-range", [], 1)
        E2 = oracle.reach_relaxed_star(E, "relax-star-range", 1.0)
        assert R2.nVar == E2.nVar
        assert_close(R2.V, E2.V, "second relu %d" % i)
    assert kept[0] == 0 and kept[2] == 0 and kept[1] > 0


def test_ranges_of_an_array_in_one_call(nnv, oracle):
    rs = np.random.RandomState(3)
    lbs = rs.rand(30, 4) - 0.5
    ubs = lbs + rs.rand(30, 4) * 0.2
    W, b = rs.randn(17, 30), rs.randn(17)
    outs = nnv.FullyConnectedLayer(W, b).reach(nnv.Star.from_boxes(lbs, ubs), "approx-star")
    lb, ub = nnv.Star.estimateRanges_array(outs)
    assert lb.shape == (17, 4)
    for i, R in enumerate(outs):
        l, u = R.estimateRanges()
        assert np.array_equal(lb[:, i], l) and np.array_equal(ub[:, i], u)
        el, eu = oracle.estimate_ranges(oracle.affine_map(oracle.star_from_box(lbs[:, i], ubs[:, i]), W, b))
        assert_close(lb[:, i], el, "lb")
        assert_close(ub[:, i], eu, "ub")
    im = nnv.ImageStar(lbs[:, 0].reshape(5, 3, 2, order="F"), ubs[:, 0].reshape(5, 3, 2, order="F"))
    lb, ub = nnv.Star.estimateRanges_array([im])
    assert_close(lb[:, 0], lbs[:, 0], "image lb")          # centre -/+ half-width: equal up to rounding
    assert_close(ub[:, 0], ubs[:, 0], "image ub")
    assert nnv.Star.estimateRanges_array([])[0].size == 0


def test_more_sets_than_mailbox_words_and_the_array_limit(nnv, oracle):
    """Arrays beyond 8192 sets read their counts back through a copy instead of the per-set mailbox
    words; the result must not depend on which way the counts travel.  Beyond 65535 sets a call is
    refused with a shape error."""
    rs = np.random.RandomState(77)
    n_in, hidden, count = 4, 24, 8300
    W1, b1 = rs.randn(hidden, n_in), 0.3 * rs.randn(hidden)
    W2, b2 = rs.randn(3, hidden), 0.1 * rs.randn(3)
    centre = rs.rand(n_in, count)
    half = 0.05 + 0.2 * rs.rand(n_in, count)
    lbs, ubs = centre - half, centre + half
    net = nnv.NN([nnv.FullyConnectedLayer(W1, b1), nnv.ReluLayer(), nnv.FullyConnectedLayer(W2, b2)])
    opt = {"reachMethod": "relax-star-area", "relaxFactor": 1}
    outs = net.reach(nnv.Star.from_boxes(lbs, ubs), opt)
    assert len(outs) == count
    lb_all, ub_all = nnv.Star.estimateRanges_array(outs)
    layers = [{"type": "fc", "W": W1, "b": b1}, {"type": "relu"}, {"type": "fc", "W": W2, "b": b2}]
    for i in list(range(0, count, 517)) + [8191, 8192, count - 1]:
        E = oracle.nn_reach(layers, oracle.star_from_box(lbs[:, i], ubs[:, i]), "relax-star-area", 1.0)
        R = outs[i]
        assert R.nVar == E.nVar
        assert_close(np.asarray(R.V), E.V, "V of set %d" % i, RTOL)
        elb, eub = oracle.estimate_ranges(E)
        assert_close(lb_all[:, i], elb, "lb of set %d" % i, RTOL)
        assert_close(ub_all[:, i], eub, "ub of set %d" % i, RTOL)
        assert np.array_equal(np.asarray(R.C), E.C) or np.allclose(np.asarray(R.C), E.C, rtol=RTOL, atol=0)
    # the same sets in two smaller arrays (mailbox route): every set's bounds agree (the launch shapes,
    # hence the summation order of the products, differ with the array length)
    lo = net.reach(nnv.Star.from_boxes(lbs[:, :4150], ubs[:, :4150]), opt)
    hi = net.reach(nnv.Star.from_boxes(lbs[:, 4150:], ubs[:, 4150:]), opt)
    lb_lo, ub_lo = nnv.Star.estimateRanges_array(lo)
    lb_hi, ub_hi = nnv.Star.estimateRanges_array(hi)
    assert_close(np.hstack([lb_lo, lb_hi]), lb_all, "lb, split arrays", RTOL)
    assert_close(np.hstack([ub_lo, ub_hi]), ub_all, "ub, split arrays", RTOL)
    assert [s.nVar for s in lo] + [s.nVar for s in hi] == [s.nVar for s in outs]
    # too many sets for one call
    big = 65536
    tiny_lb = np.tile(np.array([[0.0], [0.1]]), (1, big))
    with pytest.raises(ValueError):
        nnv.ReluLayer().reach(nnv.Star.from_boxes(tiny_lb - 0.5, tiny_lb + 0.5), "relax-star-area", None, 1)


@pytest.mark.parametrize("count", [1, 3])
def test_columns_left_unwritten_are_written_on_any_first_read(nnv, oracle, count):
    """An FC map describes the columns it gathers from its weights and writes them only when somebody
    reads them.  Whatever is read first -- the FC output, the ReLU output that shares its matrix, the
    constraint rows that are rows of it, or nothing before the next layers ran -- every read must give
    the oracle's dense arrays, and exactly what the write-at-once mode gives."""
    rs = np.random.RandomState(91)
    n_in, h1, h2 = 100, 512, 256   # large enough for every FC map to gather (tiny products stay dense)
    L = [{"type": "fc", "W": rs.randn(h1, n_in) * 0.4, "b": 0.2 * rs.randn(h1)}, {"type": "relu"},
         {"type": "fc", "W": rs.randn(h2, h1) * 0.1, "b": 0.1 * rs.randn(h2)}, {"type": "relu"},
         {"type": "fc", "W": rs.randn(6, h2) * 0.2, "b": 0.1 * rs.randn(6)}]
    centre = rs.rand(n_in, count)
    half = 0.02 + 0.05 * rs.rand(n_in, count)
    lbs, ubs = centre - half, centre + half
    ctx = nnv.default_context()
    _, exp_sets = zip(*[oracle.nn_reach(L, oracle.star_from_box(lbs[:, i], ubs[:, i]), "relax-star-area", 1.0, keep=True)
                        for i in range(count)])

    def reach():
        net = nnv.NN.from_config(L)
        dev_in = nnv.Star.from_boxes(lbs, ubs) if count > 1 else nnv.Star(lbs[:, 0], ubs[:, 0])
        net.reach(dev_in, {"reachMethod": "relax-star-area", "relaxFactor": 1})
        return [[s] if count == 1 else list(s) for s in net.reachSet]

    def check(sets, layer, what):
        for i, S in enumerate(sets[layer]):
            E = exp_sets[i][layer]
            if what == "V":
                assert_close(np.asarray(S.V), E.V, "V of layer %d, set %d" % (layer, i), RTOL)
            else:
                assert_close(np.asarray(S.C), E.C, "C of layer %d, set %d" % (layer, i), RTOL)
                assert_close(np.asarray(S.d), E.d, "d of layer %d, set %d" % (layer, i), RTOL)

    orders = [[(0, "V"), (1, "V"), (2, "V"), (3, "V"), (4, "C"), (4, "V")],      # producers first
              [(4, "C"), (3, "V"), (1, "V"), (0, "V"), (2, "V")],                  # constraint rows first
              [(1, "V"), (3, "C"), (2, "V"), (0, "V")],                            # a ReLU output first
              [(2, "V"), (1, "C"), (0, "V")]]
    for order in orders:
        sets = reach()
        for layer, what in order:
            check(sets, layer, what)
    # the same reach with the columns written by the producing call: bit-identical reads
    lazy = reach()
    ctx.set_eager_columns(True)
    try:
        eager = reach()
    finally:
        ctx.set_eager_columns(False)
    for layer in range(len(L)):
        for A, B in zip(lazy[layer], eager[layer]):
            assert np.array_equal(np.asarray(A.V), np.asarray(B.V))
            assert np.array_equal(np.asarray(A.predicate_ub), np.asarray(B.predicate_ub))
    assert np.array_equal(np.asarray(lazy[-1][0].C), np.asarray(eager[-1][0].C))
    # ... and with the ReLU steps writing their whole output as well (nothing left for a first read)
    ctx.set_eager_columns(True)
    ctx.set_eager_relu(True)
    try:
        full = reach()
    finally:
        ctx.set_eager_columns(False)
        ctx.set_eager_relu(False)
    for layer in range(len(L)):
        for A, B in zip(lazy[layer], full[layer]):
            assert np.array_equal(np.asarray(A.V), np.asarray(B.V))
    assert np.array_equal(np.asarray(lazy[-1][0].C), np.asarray(full[-1][0].C))
    assert np.array_equal(np.asarray(lazy[-1][0].d), np.asarray(full[-1][0].d))


@pytest.mark.parametrize("degenerate", [0, 3])
def test_first_layer_centre_with_and_without_degenerate_dimensions(nnv, oracle, degenerate):
    """FC map of a box star: with a generator for every dimension the gather pass also forms W*c + b;
    with degenerate dimensions (no generator) the centre goes through the GEMM.  Both against the oracle,
    together with the bounds that are built on the centre."""
    rs = np.random.RandomState(123 + degenerate)
    K, M = 300, 520
    lb = rs.randn(K)
    ub = lb + 0.05 + 0.1 * rs.rand(K)
    ub[:degenerate] = lb[:degenerate]
    W, b = rs.randn(M, K) / np.sqrt(K), rs.randn(M)
    for bias in (b, None):
        L = nnv.FullyConnectedLayer(W, bias if bias is not None else np.zeros(M))
        R = L.reach(nnv.Star(lb, ub), "approx-star")
        E = oracle.affine_map(oracle.star_from_box(lb, ub), W, bias if bias is not None else np.zeros(M))
        assert R.nVar == K - degenerate
        lo, hi = R.estimateRanges()          # before V: the bounds come from the sums, the centre from its partials
        elo, ehi = oracle.estimate_ranges(E)
        assert_close(lo, elo, "lb", RTOL)
        assert_close(hi, ehi, "ub", RTOL)
        assert_close(np.asarray(R.V), E.V, "V", RTOL)
        # generator columns are plain copies of scaled weight columns: exact
        assert np.array_equal(np.asarray(R.V)[:, 1:], E.V[:, 1:])


def test_outer_zonotope_follows_the_reference(nnv, oracle):
    """Star.Z: Zono(center, gens) from Star(lb, ub) (set/Star.m:230-236), mapped by affineMap (:332-340), gone after
    the ReLU step (nn/funcs/PosLin.m:740) and for sets built from matrices or taken from an ImageStar."""
    o = oracle
    rs = np.random.RandomState(4)
    lb = rs.rand(6) - 0.5
    ub = lb + rs.rand(6)
    ub[3] = lb[3]                                   # a degenerate dimension: no generator for it
    S, O = nnv.Star(lb, ub), o.star_from_box(lb, ub)
    assert np.array_equal(S.Z.c, O.Z[0]) and np.array_equal(S.Z.V, O.Z[1])
    W1, b1, W2 = rs.randn(9, 6), rs.randn(9), rs.randn(4, 9)
    S1, O1 = S.affineMap(W1, b1), o.affine_map(O, W1, b1)
    S2, O2 = S1.affineMap(W2), o.affine_map(O1, W2)
    for A, B in ((S1, O1), (S2, O2)):
        assert_close(A.Z.c, B.Z[0], "Z.c", 1e-13)
        assert_close(A.Z.V, B.Z[1], "Z.V", 1e-13)
    R = nnv.PosLin.reach(S1, "relax-star-area", [], 1)
    assert R.Z is None and o.reach_relaxed_star(O1, "relax-star-area", 1.0).Z is None
    assert R.affineMap(W2).Z is None
    # an FC layer on the Star keeps it, the whole-network call too (every set in front of the first ReLU)
    net = nnv.NN.from_config([{"type": "fc", "W": W1, "b": b1}, {"type": "relu"}, {"type": "fc", "W": W2, "b": np.zeros(4)}])
    net.reach(S, {"reachMethod": "relax-star-area", "relaxFactor": 1})
    assert_close(net.reachSet[0].Z.V, O1.Z[1], "Z.V after the FC layer", 1e-13)
    assert net.reachSet[1].Z is None and net.reachSet[2].Z is None
    # sets built from matrices and Stars taken from an ImageStar have none
    assert nnv.Star(rs.randn(3, 3), np.zeros((1, 2)), np.zeros(1), [-1, -1], [1, 1]).Z is None
    assert nnv.ImageStar(np.zeros((2, 2, 1)), np.ones((2, 2, 1))).toStar().Z is None


def _relu_then_conv(nnv, oracle, rs, H, W, Cin, Cout, FH, FW, s, p, dil, n, count=1, spread=2.0):
    """ReLU step on ImageStars with rows of all three kinds, then a convolution; returns (device sets, oracle
    sets, launches of the apply pass while the convolution ran)."""
    ctx = nnv.default_context()
    Wt = rs.randn(FH, FW, Cin, Cout)
    b = rs.randn(Cout)
    dev_in, ora_in = [], []
    for _ in range(count):
        V = rs.randn(H, W, Cin, n + 1) * 0.3
        V[..., 0] = rs.randn(H, W, Cin) * spread          # centres spread so that many rows are clearly on or off
        lb, ub = -np.ones(n), np.ones(n)
        dev_in.append(nnv.ImageStar(V, np.zeros((1, n)), np.zeros(1), lb, ub))
        ora_in.append(oracle.OImageStar(V, np.zeros((1, n)), np.zeros(1), lb, ub))
    relu = nnv.ReluLayer()
    conv = nnv.Conv2DLayer(Wt, b, [p, p, p, p], [s, s], [dil, dil])
    mid = relu.reach(dev_in if count > 1 else dev_in[0], "relax-star-area", "single", 1)
    ctx.kernel_time(3)
    ctx.set_timing(2)
    try:
        out = conv.reach(mid, "relax-star-area", "single")
    finally:
        ctx.set_timing(0)
    applies = ctx.kernel_time(3)[1]
    exp_mid = [oracle.relu_layer_reach(o, "relax-star-area", 1.0) for o in ora_in]
    exp = [oracle.conv2d_reach(o, Wt, b, [p, p, p, p], [s, s], [dil, dil]) for o in exp_mid]
    return (list(out) if count > 1 else [out]), exp, applies, list(zip(list(mid) if count > 1 else [mid], exp_mid))


@pytest.mark.parametrize("H,W,Cin,Cout,FH,FW,s,p,dil,n,count", [
    (5, 5, 1, 1, 3, 3, 1, 0, 1, 2, 1), (7, 9, 3, 4, 3, 3, 1, 1, 1, 6, 1), (9, 7, 5, 20, 3, 3, 2, 0, 1, 11, 3),
    (11, 9, 2, 3, 3, 3, 1, 2, 2, 5, 1), (15, 15, 32, 64, 3, 3, 1, 1, 1, 20, 1), (13, 13, 7, 40, 5, 5, 2, 2, 1, 9, 2),
    (13, 12, 2, 5, 6, 6, 1, 2, 1, 4, 2)])   # the last one has more than 32 spatial taps: the general kernel
def test_conv_reads_through_a_pending_row_reset(nnv, oracle, H, W, Cin, Cout, FH, FW, s, p, dil, n, count):
    """The convolution after a ReLU step zeroes the reset rows as it loads them (Star.m:1442-1461 applied at
    the reader): same sets as the oracle's, no apply pass, and the ReLU's own output still reads correctly."""
    import os
    rs = np.random.RandomState(H * 100 + Cout)
    out, exp, applies, mid = _relu_then_conv(nnv, oracle, rs, H, W, Cin, Cout, FH, FW, s, p, dil, n, count)
    switched = nnv.default_context().switch_is_on("no_conv_mask", "eager_rows", "eager_tail", "dense_affine")
    if not switched:
        assert applies == 0
    for R, E in zip(out, exp):
        assert R.V.shape == E.V.shape
        compare_sets(R, E, "conv after ReLU")
    # the ReLU output, read afterwards, has its rows reset (first read runs the pass)
    for M, EM in mid:
        compare_sets(M, EM, "the ReLU output itself", True)


def test_conv_after_relu_on_an_image_too_large_for_the_row_mask(nnv, oracle):
    """135168 input rows and a 64-channel tile: the bit mask does not fit beside the operand tiles, the reset is
    run first."""
    import os
    rs = np.random.RandomState(8)
    out, exp, applies, _ = _relu_then_conv(nnv, oracle, rs, 64, 64, 33, 40, 3, 3, 2, 1, 1, 2, spread=100.0)
    if not nnv.default_context().switch_is_on("eager_rows", "eager_tail", "dense_affine"):
        assert applies == 1
    compare_sets(out[0], exp[0], "conv after ReLU, large image")


def test_filters_with_too_many_taps_are_refused(nnv):
    rs = np.random.RandomState(1)
    I = nnv.ImageStar(np.zeros((9, 9, 32, 2)), np.zeros((1, 1)), np.zeros(1), [-1.0], [1.0])
    with pytest.raises(ValueError, match="taps"):
        nnv.Conv2DLayer(rs.randn(8, 8, 32, 64), np.zeros(64)).reach(I, "relax-star-area")


def test_released_arrays_give_their_memory_back(nnv):
    """Arrays of 256 sets and more are let go lazily (while the library waits for the device); the pool's figures,
    a later reach and an element that was read out of the array before behave as if they had gone at once."""
    ctx = nnv.default_context()
    rs = np.random.RandomState(5)
    n_in, hidden, count = 6, 40, 700
    net = nnv.NN([nnv.FullyConnectedLayer(rs.randn(hidden, n_in), rs.randn(hidden)), nnv.ReluLayer(),
                  nnv.FullyConnectedLayer(rs.randn(5, hidden), rs.randn(5))])
    opt = {"reachMethod": "relax-star-area", "relaxFactor": 1}
    lbs = rs.rand(n_in, count) - 0.5
    ubs = lbs + 0.2
    net.reach(nnv.Star.from_boxes(lbs[:, :300], ubs[:, :300]), opt)   # the layers' weights (and what arrays derive from them) are on the device now
    net.reachSet = []
    ctx.synchronize()
    used0, _ = ctx.pool_stats()
    ins = nnv.Star.from_boxes(lbs, ubs)
    outs = net.reach(ins, opt)
    kept = outs[3]                       # an element read out of the array owns its handle
    lb_kept, ub_kept = kept.estimateRanges()
    used1, _ = ctx.pool_stats()
    assert used1 > used0
    del outs, ins
    net.reachSet = []
    used2, _ = ctx.pool_stats()
    assert used0 < used2 < used1         # everything but what `kept` holds on to is back in the pool
    # a second reach runs while the first one's arrays may still be queued for release, with the same result
    outs2 = net.reach(nnv.Star.from_boxes(lbs, ubs), opt)
    lb2, ub2 = outs2[3].estimateRanges()
    assert np.array_equal(lb2, lb_kept) and np.array_equal(ub2, ub_kept)
    assert np.array_equal(np.asarray(kept.V), np.asarray(outs2[3].V))
    del outs2, kept
    net.reachSet = []
    ctx.synchronize()
    assert ctx.pool_stats()[0] == used0


@pytest.mark.parametrize("method", ["relax-star-area", "relax-star-random"])
@pytest.mark.parametrize("shape,specs", [
    # (FH, FW, Cout, stride, padding [t b l r], dilation) per convolution, a ReLU after each but the last
    ((9, 8, 2), [(3, 3, 5, 1, [1, 1, 1, 1], 1), (3, 3, 6, 2, [0, 0, 0, 0], 1), (2, 3, 4, 1, [1, 0, 2, 1], 2), (1, 1, 3, 1, [0, 0, 0, 0], 1)]),
    ((16, 16, 3), [(3, 3, 20, 1, [1, 1, 1, 1], 1), (5, 5, 33, 2, [2, 2, 2, 2], 1), (3, 3, 40, 1, [0, 0, 0, 0], 1), (3, 3, 8, 2, [1, 1, 1, 1], 1)]),
    ((12, 20, 1), [(3, 1, 4, 1, [0, 0, 0, 0], 1), (1, 3, 4, 1, [0, 0, 1, 1], 1), (3, 3, 4, 3, [1, 1, 1, 1], 1)])])
def test_chains_of_convolutions_keep_generator_images_inside_their_windows(nnv, oracle, method, shape, specs):
    """Generators of a box ImageStar are single pixels; every convolution widens their images by its filter's
    reach, and the device computes them inside those windows only.  Every layer's set against the oracle (zero
    pattern included), over strides, asymmetric padding, dilation, windows cut by the image border, and a final
    fully connected layer that reads the whole images."""
    rs = np.random.RandomState(shape[0] * 7 + len(specs))
    H, W, C = shape
    layers = []
    h, w, c = H, W, C
    for i, (fh, fw, co, st, pad, dil) in enumerate(specs):
        Wt = rs.randn(fh, fw, c, co) * np.sqrt(2.0 / (fh * fw * c))
        L = {"type": "conv", "W": Wt, "b": 0.1 * rs.randn(co), "padding": pad, "stride": [st, st], "dilation": [dil, dil]}
        layers.append(L)
        h, w = oracle.conv2d_output_size(h, w, fh, fw, pad, [st, st], [dil, dil])
        c = co
        layers.append({"type": "relu"})
    layers.append({"type": "fc", "W": rs.randn(7, h * w * c) / np.sqrt(h * w * c), "b": rs.randn(7)})
    x = rs.rand(H * W * C)
    cfg = {"name": "conv chain %dx%dx%d" % shape, "kind": "image", "image_shape": shape, "layers": layers,
           "lb": x - 0.05, "ub": x + 0.05}
    run_cfg(cfg, method)


def test_an_input_image_set_is_mapped_again_and_again(nnv, oracle):
    """The stamp pass of a convolution looks the column of a pixel up in a table; for a box ImageStar that table is
    made by the first convolution that maps the set and kept on the set's handle.  The same input set through two
    networks with different first layers, twice each: every reach must give the same sets as the first one, and
    the first one the oracle's."""
    rs = np.random.RandomState(4242)
    H, W, C = 11, 9, 2
    x = rs.rand(H, W, C)
    lb, ub = x - 0.03, x + 0.03
    lb[3, 4, 1] = ub[3, 4, 1] = x[3, 4, 1]          # a pixel without a generator
    dev_in = nnv.ImageStar(lb, ub)
    ora_in = oracle.image_star_from_bounds(lb, ub)

    def net_layers(fh, fw, co, st):
        c1 = {"type": "conv", "W": rs.randn(fh, fw, C, co) * np.sqrt(2.0 / (fh * fw * C)), "b": 0.1 * rs.randn(co),
              "padding": [1, 1, 1, 1], "stride": [st, st], "dilation": [1, 1]}
        h, w = oracle.conv2d_output_size(H, W, fh, fw, [1, 1, 1, 1], [st, st], [1, 1])
        c2 = {"type": "conv", "W": rs.randn(3, 3, co, 5) * np.sqrt(2.0 / (9 * co)), "b": 0.1 * rs.randn(5),
              "padding": [0, 0, 0, 0], "stride": [1, 1], "dilation": [1, 1]}
        h2, w2 = oracle.conv2d_output_size(h, w, 3, 3, [0, 0, 0, 0], [1, 1], [1, 1])
        return [c1, {"type": "relu"}, c2, {"type": "relu"}, {"type": "fc", "W": rs.randn(4, h2 * w2 * 5) / 10.0, "b": rs.randn(4)}]

    opts = {"reachMethod": "relax-star-area", "relaxFactor": 1}
    for spec in ((3, 3, 6, 1), (2, 3, 4, 2)):
        layers = net_layers(*spec)
        net = nnv.NN.from_config(layers, "same input, %dx%d filters" % spec[:2])
        ora_out, _ = oracle.nn_reach(layers, ora_in, "relax-star-area", 1.0, keep=True)
        first = None
        for _ in range(3):
            out = net.reach(dev_in, opts)
            V = flat_V(out).copy()
            if first is None:
                first = V
                assert_close(V, flat_V(ora_out), "output set of the first reach")
            else:
                assert np.array_equal(V, first)
