"""Full-size GPU checks of configs 4 and 5 through size-independent properties (the CPU oracle would
take minutes there): structure of every ReLU output, containment of concrete forward passes
(the reference's own soundness criterion, tests/soundness/soundness_test_utils.m:228-322, done
constructively), per-set equivalence of the batched pass, and determinism."""
import numpy as np
import pytest

from nnv_amd.configs import make_config
from oracle import nnv_oracle as o
from tests.gpu_util import assert_close, assert_close_elementwise, classification_margin, flat_V, input_sets

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def nnv():
    import nnv_amd
    nnv_amd.default_context()
    return nnv_amd


def _check_relu_structure(pre, post, what):
    """post = ReLU(pre): inactive + crossing rows of the old columns are zero, active rows untouched,
    new columns one-hot at the crossing neurons, new predicate bounds [0, ub]."""
    Vp, Vq = flat_V(pre), flat_V(post)
    lb, ub = (x.reshape(-1, order="F") for x in pre.estimateRanges())
    ni, idx, clb, cub = post.relu_info()
    n_old = Vp.shape[1] - 1
    m = idx.size
    assert Vq.shape == (Vp.shape[0], n_old + 1 + m), what
    inactive = ub <= 0
    crossing = (lb < 0) & (ub > 0)
    assert ni == int(inactive.sum()) and m == int(crossing.sum()), what
    assert np.array_equal(np.sort(idx), np.flatnonzero(crossing)), what
    keep = ~(inactive | crossing)
    assert np.array_equal(Vq[keep, :n_old + 1], Vp[keep]), what
    assert not Vq[~keep, :n_old + 1].any(), what
    new = Vq[:, n_old + 1:]
    assert np.array_equal(new[idx, np.arange(m)], np.ones(m)) and new.sum() == m, what
    plb = post.pred_lb if hasattr(post, "pred_lb") else post.predicate_lb
    pub = post.pred_ub if hasattr(post, "pred_ub") else post.predicate_ub
    assert not plb[n_old:].any() and np.array_equal(pub[n_old:], ub[idx]), what
    assert np.array_equal(clb, lb[idx]) and np.array_equal(cub, ub[idx]), what
    return idx


def _area_order_ok(lb, ub, idx):
    key = 0.5 * (np.abs(ub[idx]) * np.abs(lb[idx]))
    d = np.diff(key)
    return np.all(d <= 0) and np.all(np.diff(idx)[d == 0] > 0)     # descending, ties by ascending index


def test_config4_full_structure_and_containment(nnv):
    cfg = make_config(4)
    dev_in, _ = input_sets(cfg)
    net = nnv.NN.from_config(cfg["layers"], cfg["name"])
    out = net.reach(dev_in, {"reachMethod": "relax-star-area", "relaxFactor": 1})
    sets = [dev_in] + net.reachSet
    for li, L in enumerate(cfg["layers"]):
        if L["type"] == "relu":
            idx = _check_relu_structure(sets[li], sets[li + 1], "cfg4 layer %d" % (li + 1))
            lb, ub = (x.reshape(-1, order="F") for x in sets[li].estimateRanges())
            assert _area_order_ok(lb, ub, idx), "cfg4 layer %d: new-predicate order" % (li + 1)
    # containment: concrete images from the input box land inside the output set for the predicate
    # vector alpha' = [alpha; ReLU outputs of the crossing neurons], and inside the output bounds
    sh = cfg["image_shape"]
    lbv, ubv = cfg["lb"], cfg["ub"]
    rs = np.random.RandomState(7)
    alphas = [np.ones(lbv.size), -np.ones(lbv.size)] + [rs.uniform(-1, 1, lbv.size) for _ in range(2)]
    crossing_lists = [s.relu_info()[1] if L["type"] == "relu" else None for L, s in zip(cfg["layers"], net.reachSet)]
    Vout = flat_V(out)
    olb, oub = (x.reshape(-1, order="F") for x in out.estimateRanges())
    for a0 in alphas:
        x = (0.5 * (lbv + ubv) + 0.5 * (ubv - lbv) * a0).reshape(sh, order="F")
        alpha = a0.copy()
        for L, cl in zip(cfg["layers"], crossing_lists):
            x = o.evaluate([L], x)
            if cl is not None:
                alpha = np.r_[alpha, x.reshape(-1, order="F")[cl]]
        y = x.reshape(-1, order="F")
        got = Vout[:, 0] + Vout[:, 1:] @ alpha
        assert_close(got, y, "cfg4 containment: c + V*alpha' reproduces the concrete output", 1e-9)
        assert np.all(y >= olb - 1e-9) and np.all(y <= oub + 1e-9)
        pub = out.pred_ub
        plb = out.pred_lb
        assert np.all(alpha <= pub + 1e-12) and np.all(alpha >= plb - 1e-12)
    # the triangle constraints hold for alpha' (checked on the last ReLU's rows, taken from the dense C)
    assert out.C.shape[0] == 1 + 3 * sum(c.size for c in crossing_lists if c is not None)


def test_config5_full_batched_equals_single(nnv):
    cfg = make_config(5)
    stars, _ = input_sets(cfg)
    assert len(stars) == 1024
    net = nnv.NN.from_config(cfg["layers"], cfg["name"])
    outs = net.reach(stars, {"reachMethod": "relax-star-area", "relaxFactor": 1})
    assert len(outs) == 1024
    from nnv_amd import _lib
    import ctypes as C
    ctx = outs[0].ctx
    N = outs[0].dim
    lb = np.empty((N, 1024), order="F")
    ub = np.empty((N, 1024), order="F")
    arr = (C.c_void_p * 1024)(*[s._h.h for s in outs])
    _lib.check(ctx.lib.nnvhip_estimate_ranges_batch(ctx.handle, 1024, arr, _lib.ptr(lb), _lib.ptr(ub)))
    assert np.all(lb <= ub)
    # every sub-box is contained in the original box, so its output bounds are too (monotonicity)
    big = nnv.NN.from_config(cfg["layers"]).reach(nnv.Star(cfg["lb"], cfg["ub"]),
                                                  {"reachMethod": "relax-star-area", "relaxFactor": 1})
    # a single-set reach of selected sub-boxes is bit-identical to its slot in the batched pass:
    # classification, new-predicate order, V, predicate bounds, bounds
    boxes = o.box_partition(cfg["lb"], cfg["ub"], cfg["partition"]["indexes"], cfg["partition"]["numbers"])
    for i in (0, 1, 517, 1023):
        one_net = nnv.NN.from_config(cfg["layers"])
        one = one_net.reach(nnv.Star(boxes[i][0], boxes[i][1]), {"reachMethod": "relax-star-area", "relaxFactor": 1})
        for li, L in enumerate(cfg["layers"]):
            a, b = one_net.reachSet[li], net.reachSet[li][i]
            if L["type"] == "relu":
                ia, ib = a.relu_info(), b.relu_info()
                assert ia[0] == ib[0] and np.array_equal(ia[1], ib[1]), "set %d layer %d" % (i, li + 1)
        assert_close(one.V, outs[i].V, "set %d output V" % i)
        l1, u1 = one.estimateRanges()
        assert_close(l1, lb[:, i], "set %d lb" % i)
        assert_close(u1, ub[:, i], "set %d ub" % i)
    # full-size oracle parity of two slots of the batched pass: classification and new-predicate
    # order bit-exact at every ReLU, generators and per-set output bounds within RTOL
    for i in (3, 900):
        ora_out, ora_sets = o.nn_reach(cfg["layers"], o.star_from_box(*boxes[i]), "relax-star-area", 1.0, keep=True)
        prev = o.star_from_box(*boxes[i])
        for li, L in enumerate(cfg["layers"]):
            if L["type"] == "relu":
                plb, pub = o.estimate_ranges(prev)
                m1, m2 = o.relax_classify(plb, pub, "relax-star-area")
                ni, idx, _, _ = net.reachSet[li][i].relu_info()
                assert ni == m1.size and np.array_equal(idx, m2), "set %d layer %d vs oracle" % (i, li + 1)
            prev = ora_sets[li]
        assert_close(outs[i].V, ora_out.V, "set %d output V vs oracle" % i)
        ol, ou = o.estimate_ranges(ora_out)
        assert_close(lb[:, i], ol, "set %d lb vs oracle" % i)
        assert_close(ub[:, i], ou, "set %d ub vs oracle" % i)
    # concrete corner of sub-box 517 lands inside its bounds
    l517, u517 = boxes[517]
    y = o.evaluate(cfg["layers"], u517)
    assert np.all(y >= lb[:, 517] - 1e-9) and np.all(y <= ub[:, 517] + 1e-9)
    del big


def test_config5_full_shortcuts_of_the_summing_pass_change_no_bit(nnv):
    """Config 5 at full size (batches of sixteen sets per block of the pass that sums the second FC layer's unwritten
    pieces, runs of equal sets across and inside batches) with the pass's shortcuts on and off, and a second time
    with them on: every ReLU step's counts and crossing lists, all output matrices and all output bounds are the same
    to the bit; and the layer's matrices, written when first read after the reach, equal those of the mode that
    writes them inside the call."""
    cfg = make_config(5)
    stars, _ = input_sets(cfg)
    opts = {"reachMethod": "relax-star-area", "relaxFactor": 1}
    ctx = nnv.default_context()
    from nnv_amd import _lib
    import ctypes as C

    def run(read=()):
        net = nnv.NN.from_config(cfg["layers"], cfg["name"])
        outs = net.reach(stars, opts)
        N = outs[0].dim
        lb, ub = np.empty((N, 1024), order="F"), np.empty((N, 1024), order="F")
        arr = (C.c_void_p * 1024)(*[s._h.h for s in outs])
        _lib.check(ctx.lib.nnvhip_estimate_ranges_batch(ctx.handle, 1024, arr, _lib.ptr(lb), _lib.ptr(ub)))
        infos = [[net.reachSet[li][i].relu_info() for i in (0, 255, 256, 700, 1023)]
                 for li, L in enumerate(cfg["layers"]) if L["type"] == "relu"]
        Vs = [np.asarray(outs[i].V).copy() for i in (0, 15, 16, 511, 1023)]
        mats = [np.asarray(net.reachSet[2][i].V).copy() for i in read]   # the second FC layer's sets
        return lb, ub, infos, Vs, mats

    was = {nm: ctx.switches.get(nm, False) for nm in ("no_sum_shortcuts", "eager_cols")}
    try:
        ctx.set_switch("no_sum_shortcuts", False)
        a = run(read=(1023, 0, 300))
        ctx.set_switch("no_sum_shortcuts", True)
        b = run()
        ctx.set_switch("no_sum_shortcuts", False)
        c = run()
        ctx.set_switch("eager_cols", True)
        e = run(read=(1023, 0, 300))
    finally:
        for nm, v in was.items():
            ctx.set_switch(nm, v)
    for x in (b, c):
        assert np.array_equal(a[0], x[0]) and np.array_equal(a[1], x[1])
        for ia, ix in zip(a[2], x[2]):
            for p, q in zip(ia, ix):
                assert p[0] == q[0] and np.array_equal(p[1], q[1])
        for p, q in zip(a[3], x[3]):
            assert np.array_equal(p, q)
    for p, q in zip(a[4], e[4]):
        assert np.array_equal(p, q)


def test_reach_is_deterministic(nnv):
    cfg = make_config(2)
    net = nnv.NN.from_config(cfg["layers"])
    opts = {"reachMethod": "relax-star-range", "relaxFactor": 1}
    a = net.reach(nnv.Star(cfg["lb"], cfg["ub"]), opts)
    Va, la = a.V, a.estimateRanges()[0]
    b = net.reach(nnv.Star(cfg["lb"], cfg["ub"]), opts)
    assert np.array_equal(Va, b.V) and np.array_equal(la, b.estimateRanges()[0])   # no atomics on fp data


def test_config4_full_against_the_recorded_oracle(nnv):
    # The CPU oracle's answers for configuration 4 at full size (100 s and several GB on the host, recorded once by
    # tests/golden/make_fullsize_fixtures.py): inactive counts and crossing lists in new-predicate order must match
    # exactly, sampled entries of every layer's generator matrix and the output ranges within the tolerance.
    import os
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "cfg4_fullsize_relax_star_area.npz"))
    cfg = make_config(4)
    assert int(gold["n_layers"][0]) == len(cfg["layers"])
    dev_in, _ = input_sets(cfg)
    net = nnv.NN.from_config(cfg["layers"], cfg["name"])
    out = net.reach(dev_in, {"reachMethod": "relax-star-area", "relaxFactor": 1})
    for li, (L, s) in enumerate(zip(cfg["layers"], net.reachSet)):
        what = "cfg4 layer %d (%s)" % (li + 1, L["type"])
        if L["type"] == "relu":
            ni, idx, _, _ = s.relu_info()
            assert ni == int(gold["inactive_%d" % li][0]), what + ": inactive count"
            assert np.array_equal(idx, gold["crossing_%d" % li]), what + ": crossing list / order"
        V = flat_V(s)
        assert tuple(V.shape) == tuple(int(v) for v in gold["shape_%d" % li]), what + ": shape"
        got = V[gold["rows_%d" % li], gold["cols_%d" % li]]
        assert_close(got, gold["vals_%d" % li], what + ": sampled entries of V", 1e-9)
        del V
    olb, oub = (x.reshape(-1, order="F") for x in out.estimateRanges())
    assert_close(olb, gold["out_lb"], "cfg4 output lb", 1e-9)
    assert_close(oub, gold["out_ub"], "cfg4 output ub", 1e-9)


def test_config5_full_against_the_recorded_oracle(nnv, capsys):
    """All 1024 sets of configuration 5 against what the CPU oracle computes for each sub-box on its own (recorded by
    tests/golden/make_fullsize_fixtures.py): per set and ReLU layer the inactive count, the number of crossing
    neurons and the crossing list in new-predicate order (by a 64-bit hash) exactly; the output ranges entry by entry;
    every pre-ReLU bound close to zero (the ones whose sign decides a class) with the oracle's sign; and the
    classification margins of the device's own bounds next to the oracle's."""
    import hashlib
    import os
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "cfg5_fullsize_relax_star_area.npz"))
    cfg = make_config(5)
    stars, _ = input_sets(cfg)
    net = nnv.NN.from_config(cfg["layers"], cfg["name"])
    outs = net.reach(stars, {"reachMethod": "relax-star-area", "relaxFactor": 1})
    n_sets = len(outs)
    assert n_sets == gold["inactive"].shape[0] == 1024
    relu_layers = [int(v) for v in gold["relu_layers"]]
    assert relu_layers == [li for li, L in enumerate(cfg["layers"]) if L["type"] == "relu"]
    near_where, near_value = gold["near_zero_where"], gold["near_zero_value"]
    dev_margin = np.zeros((n_sets, len(relu_layers)))
    for r, li in enumerate(relu_layers):
        pre_lb, pre_ub = nnv.Star.estimateRanges_array(net.reachSet[li - 1])    # the ReLU's input: ranges cached by the step
        post = net.reachSet[li]
        for i in range(n_sets):
            ni, idx, clb, cub = post[i].relu_info()
            tag = "set %d ReLU layer %d" % (i, li + 1)
            assert ni == int(gold["inactive"][i, r]), tag + ": inactive count"
            assert idx.size == int(gold["crossing"][i, r]), tag + ": number of crossing neurons"
            h = np.frombuffer(hashlib.blake2b(np.ascontiguousarray(idx, dtype="<i4").tobytes(), digest_size=8).digest(), dtype="<u8")[0]
            assert h == gold["crossing_hash"][i, r], tag + ": crossing list / new-predicate order"
            assert np.array_equal(clb, pre_lb[idx, i]) and np.array_equal(cub, pre_ub[idx, i]), tag
            dev_margin[i, r] = classification_margin(pre_lb[:, i], pre_ub[:, i])
            # the bound the oracle found closest to zero: same sign, same value
            k, upper = int(gold["margin_neuron"][i, r]), int(gold["margin_upper"][i, r])
            got = (pre_ub if upper else pre_lb)[k, i]
            exp = gold["margin_value"][i, r]
            assert abs(got - exp) <= 1e-12 * gold["scale"][i, r] and np.sign(got) == np.sign(exp), tag + ": closest bound"
        sel = near_where[:, 1] == r
        for (i, _, k, upper), exp in zip(near_where[sel], near_value[sel]):
            got = (pre_ub if upper else pre_lb)[k, i]
            assert np.sign(got) == np.sign(exp) and abs(got - exp) <= 1e-12 * gold["scale"][i, r], \
                "set %d ReLU layer %d neuron %d: bound near zero, expected %.3e got %.3e" % (i, li + 1, k, exp, got)
    lb, ub = nnv.Star.estimateRanges_array(outs)
    assert_close_elementwise(lb.T, gold["out_lb"], "output lb of all 1024 sets")
    assert_close_elementwise(ub.T, gold["out_ub"], "output ub of all 1024 sets")
    with capsys.disabled():
        print("\ncfg5 classification margins per ReLU layer (min over 1024 sets): device %s, oracle %s; %d bounds below 1e-6 of scale"
              % (np.array2string(dev_margin.min(axis=0), precision=3), np.array2string(gold["margin"].min(axis=0), precision=3),
                 near_value.size))
    assert np.all(dev_margin.min(axis=0) > 0)
