"""Random layer sequences on the GPU against the oracle: the structure marks the layers hand to one
another (one-hot columns, kept-row lists, pending row resets, implicit columns, pending range sums)
meet here in orders no fixed configuration exercises."""
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


def _fc(rs, out, inp, scale=1.0):
    return {"type": "fc", "W": rs.randn(out, inp) * scale / np.sqrt(inp), "b": rs.randn(out) * 0.2}


def _bn(rs, n):
    return {"type": "batchnorm", "mean": rs.randn(n) * 0.1, "var": rs.rand(n) + 0.5, "eps": 1e-5,
            "scale": rs.rand(n) + 0.5, "offset": rs.randn(n) * 0.1}


def _random_fc_sequence(rs, n_in):
    """fc / relu / batchnorm in random order; consecutive ReLUs and FCs are allowed on purpose."""
    layers, width = [], n_in
    for _ in range(rs.randint(4, 9)):
        kind = rs.choice(["fc", "fc", "relu", "relu", "bn"])
        if kind == "fc":
            out = int(rs.choice([24, 150, 300, 420]))
            layers.append(_fc(rs, out, width, scale=float(rs.choice([0.5, 2.0, 6.0]))))
            width = out
        elif kind == "relu":
            layers.append({"type": "relu"})
        else:
            layers.append(_bn(rs, width))
    layers.append(_fc(rs, 7, width))
    return layers


def _compare(nnv, oracle, layers, dev_in, ora_in, method, tol=1e-9):
    net = nnv.NN.from_config(layers)
    out = net.reach(dev_in, {"reachMethod": method, "relaxFactor": 1})
    exp, exp_sets = oracle.nn_reach(layers, ora_in, method, 1.0, keep=True)
    outs = out if isinstance(out, (list, nnv.SetArray)) else [out]
    exps = exp if isinstance(exp, list) else [exp]
    assert len(outs) == len(exps)
    for R, E in zip(outs, exps):
        EV = E.V.reshape(-1, E.V.shape[-1], order="F") if E.V.ndim == 4 else E.V
        RV = np.asarray(R.V)
        RV = RV.reshape(-1, RV.shape[-1], order="F") if RV.ndim == 4 else RV
        assert RV.shape == EV.shape
        assert_close(RV, EV, "output V", tol)
        lb, ub = R.estimateRanges()
        elb, eub = oracle.estimate_ranges(E) if hasattr(E, "predicate_lb") else oracle.image_star_estimate_ranges(E)
        assert_close(np.asarray(lb).reshape(-1, order="F"), np.asarray(elb).reshape(-1, order="F"), "lb", tol)
        assert_close(np.asarray(ub).reshape(-1, order="F"), np.asarray(eub).reshape(-1, order="F"), "ub", tol)
    # every intermediate set too, read after the whole reach has run (so the reads meet sets whose
    # row reset or appended columns were never needed by the next layer)
    # (of an array: its first, middle and last set - one read may write the matrices of many sets at once)
    for i, (rset, eset) in enumerate(zip(net.reachSet, exp_sets)):
        many = isinstance(rset, (list, nnv.SetArray))
        for k in (sorted({0, len(rset) // 2, len(rset) - 1}) if many else [None]):
            r0 = rset[k] if many else rset
            e0 = eset[k if many else 0] if isinstance(eset, list) else eset
            RV, EV = np.asarray(r0.V), e0.V
            if EV.ndim == 4:
                EV = EV.reshape(-1, EV.shape[-1], order="F")
                RV = RV.reshape(-1, RV.shape[-1], order="F")
            assert_close(RV, EV, "layer %d set %s V" % (i + 1, k), tol)
            assert np.array_equal(RV == 0, EV == 0), "layer %d set %s zero pattern" % (i + 1, k)


@pytest.mark.parametrize("seed", range(10))
def test_random_fc_sequences(nnv, oracle, seed):
    rs = np.random.RandomState(100 + seed)
    n_in = int(rs.choice([12, 40]))
    layers = _random_fc_sequence(rs, n_in)
    count = int(rs.choice([1, 1, 3]))
    centre = rs.rand(n_in, count)
    half = np.abs(rs.randn(n_in, count)) * rs.choice([0.02, 0.3, 3.0], size=(1, count))
    half[rs.randint(n_in), :] = 0.0                       # a zero-width dimension: its generator is dropped
    lbs, ubs = centre - half, centre + half
    method = ["relax-star-area", "relax-star-range", "relax-star-static"][seed % 3]
    if count == 1:
        dev_in, ora_in = nnv.Star(lbs[:, 0], ubs[:, 0]), oracle.star_from_box(lbs[:, 0], ubs[:, 0])
    else:
        dev_in = nnv.Star.from_boxes(lbs, ubs)
        ora_in = [oracle.star_from_box(lbs[:, i], ubs[:, i]) for i in range(count)]
    _compare(nnv, oracle, layers, dev_in, ora_in, method)


@pytest.mark.parametrize("seed", range(4))
def test_random_cnn_sequences(nnv, oracle, seed):
    rs = np.random.RandomState(200 + seed)
    H = W = int(rs.choice([8, 12]))
    cin = int(rs.choice([1, 3]))
    c1, c2 = int(rs.choice([4, 8])), int(rs.choice([4, 6]))
    s2 = int(rs.choice([1, 2]))
    layers = [{"type": "conv", "W": rs.randn(3, 3, cin, c1) * 0.4, "b": rs.randn(c1) * 0.1, "padding": [1, 1, 1, 1],
               "stride": [1, 1], "dilation": [1, 1]},
              {"type": "relu"}]
    if seed % 2 == 0:
        layers.append({"type": "relu"})                   # a ReLU straight on a ReLU output
    if seed % 2 == 1:
        layers.append(_bn(rs, c1))
    layers += [{"type": "conv", "W": rs.randn(3, 3, c1, c2) * 0.3, "b": rs.randn(c2) * 0.1, "padding": [0, 0, 0, 0],
                "stride": [s2, s2], "dilation": [1, 1]},
               {"type": "relu"}]
    Ho = (H - 3) // s2 + 1
    if seed >= 2 and Ho >= 2:
        layers.append({"type": "avgpool", "pool": [2, 2], "stride": [2, 2], "padding": [0, 0, 0, 0]})
        Ho = (Ho - 2) // 2 + 1
    layers += [_fc(rs, 30, Ho * Ho * c2, 2.0), {"type": "relu"}, _fc(rs, 5, 30)]
    x = rs.rand(H, W, cin)
    eps = float(rs.choice([0.01, 0.2]))
    dev_in = nnv.ImageStar(x - eps, x + eps)
    ora_in = oracle.image_star_from_bounds(x - eps, x + eps)
    _compare(nnv, oracle, layers, dev_in, ora_in, "relax-star-area")


ALL_RELAX = ["relax-star-area", "relax-star-range", "relax-star-static", "relax-star-random", "relax-star-bound",
             "relax-star-ub"]


@pytest.mark.parametrize("seed", range(300, 324))
def test_random_chains_of_convolutions(nnv, oracle, seed):
    """One to four convolutions of random geometry (filter 1..5, stride 1..3, dilation 1..2, asymmetric padding, 2 to
    40 output channels) on a box ImageStar with a different width per pixel (so that no two sort keys tie), with
    ReLUs, doubled ReLUs, batch normalisation, convolutions straight on convolutions and average pooling in between,
    most of them ending in two fully connected layers: every layer's set against the oracle, zero pattern included."""
    rs = np.random.RandomState(seed)
    H, W, c = int(rs.choice([6, 9, 12, 17])), int(rs.choice([6, 8, 13, 16])), int(rs.choice([1, 2, 3]))
    cin = c
    h, w = H, W
    layers = []
    for _ in range(int(rs.choice([1, 2, 3, 4]))):
        fh, fw = int(rs.choice([1, 2, 3, 5])), int(rs.choice([1, 2, 3, 5]))
        st = [int(rs.choice([1, 1, 2, 3])), int(rs.choice([1, 1, 2]))]
        dil = [int(rs.choice([1, 1, 2])), int(rs.choice([1, 1, 2]))]
        pad = [int(v) for v in rs.randint(0, 3, size=4)]
        ho = (h + pad[0] + pad[1] - (fh - 1) * dil[0] - 1) // st[0] + 1
        wo = (w + pad[2] + pad[3] - (fw - 1) * dil[1] - 1) // st[1] + 1
        if h + pad[0] + pad[1] - (fh - 1) * dil[0] - 1 < 0 or w + pad[2] + pad[3] - (fw - 1) * dil[1] - 1 < 0:
            fh = fw = 1
            st, dil, pad = [1, 1], [1, 1], [0, 0, 0, 0]
            ho, wo = h, w
        co = int(rs.choice([2, 5, 17, 33, 40]))
        layers.append({"type": "conv", "W": rs.randn(fh, fw, c, co) * np.sqrt(2.0 / (fh * fw * c)), "b": rs.randn(co) * 0.1,
                       "padding": pad, "stride": st, "dilation": dil})
        h, w, c = ho, wo, co
        r = rs.rand()
        if r < 0.7:
            layers.append({"type": "relu"})
            if rs.rand() < 0.15:
                layers.append({"type": "relu"})
        elif r < 0.85:
            layers += [_bn(rs, c), {"type": "relu"}]
        if rs.rand() < 0.15 and h >= 2 and w >= 2:
            layers.append({"type": "avgpool", "pool": [2, 2], "stride": [2, 2], "padding": [0, 0, 0, 0]})
            h, w = (h - 2) // 2 + 1, (w - 2) // 2 + 1
    if rs.rand() < 0.7:
        layers += [_fc(rs, 12, h * w * c, 2.0), {"type": "relu"}, _fc(rs, 4, 12)]
    x = rs.rand(H, W, cin)
    e = float(rs.choice([0.005, 0.05, 0.3])) * (0.5 + rs.rand(H, W, cin))
    lo, hi = x - e, x + e
    if rs.rand() < 0.3:
        k = rs.randint(lo.size)
        hi.reshape(-1)[k] = lo.reshape(-1)[k]
    _compare(nnv, oracle, layers, nnv.ImageStar(lo, hi), oracle.image_star_from_bounds(lo, hi), ALL_RELAX[seed % 6])


@pytest.mark.parametrize("wide,count,method", [(9000, 1, "relax-star-range"), (8200, 2, "relax-star-static"),
                                               (2049, 1, "relax-star-area"), (3000, 3, "relax-star-bound")])
def test_wide_layers_in_a_sequence(nnv, oracle, wide, count, method):
    # more than 2048 neurons: classification, sort and bounds run as separate multi-block kernels, and
    # the sets that come out of them feed batch normalisation, another ReLU and an FC layer
    rs = np.random.RandomState(wide)
    n_in = 10
    layers = [_fc(rs, wide, n_in, 3.0), {"type": "relu"}, _bn(rs, wide), {"type": "relu"}, _fc(rs, 300, wide, 2.0),
              {"type": "relu"}, _fc(rs, 5, 300)]
    centre = rs.rand(n_in, count)
    half = np.abs(rs.randn(n_in, count)) * 0.05
    lbs, ubs = centre - half, centre + half
    if count == 1:
        dev_in, ora_in = nnv.Star(lbs[:, 0], ubs[:, 0]), oracle.star_from_box(lbs[:, 0], ubs[:, 0])
    else:
        dev_in = nnv.Star.from_boxes(lbs, ubs)
        ora_in = [oracle.star_from_box(lbs[:, i], ubs[:, i]) for i in range(count)]
    _compare(nnv, oracle, layers, dev_in, ora_in, method)


@pytest.mark.parametrize("method", ["relax-star-area", "relax-star-static"])
def test_one_wide_set_through_the_tile_kernel(nnv, oracle, method):
    # one set with thousands of predicates whose row reset is pending: the FC layer after the ReLU contracts the
    # kept rows of 4201 columns into 520 outputs, enough 128 x 128 tiles for the kernel that arrays of sets use
    # (rows packed transposed, narrow last tile); a skinny layer with 20 outputs (two rows of 16) ends the net
    rs = np.random.RandomState(77)
    N, n = 300, 4200
    V = np.c_[rs.randn(N) * 2.0, rs.randn(N, n) * 5e-4]
    V[rs.choice(N, size=20, replace=False), 1:] = 0.0          # some neurons with a point range
    args = (V, np.zeros((1, n)), np.zeros(1), -np.ones(n), np.ones(n))
    layers = [{"type": "relu"}, _fc(rs, 520, N, 2.0), {"type": "relu"}, _fc(rs, 20, 520)]
    _compare(nnv, oracle, layers, nnv.Star(*args), oracle.OStar(*args), method)


@pytest.mark.parametrize("shapes,hidden", [(1, 300), (3, 300), (40, 300), (2, 1400)])
def test_arrays_of_boxes_that_share_their_half_widths(nnv, oracle, shapes, hidden):
    # 64 boxes with `shapes` different half-width vectors among them: sets of one shape gather the same scaled weight
    # columns, so the second FC layer reads their packed rows from one matrix per shape (up to 16 shapes; with more
    # every set packs its own rows).  201 columns per set: one whole 128-column tile and a 73-column remainder.
    # With 1400 hidden neurons a set keeps more than 512 rows: kept-row lists of more than 64 stages of eight.
    rs = np.random.RandomState(500 + shapes)
    n_in, count = 200, 64
    # (centres and half-widths on a binary grid: lb, ub and 0.5 * (ub - lb) are then exact, and sets of one shape
    # have the same half-widths to the bit, which is what the library looks for)
    widths = rs.randint(1, 128, size=(n_in, shapes)) / 4096.0
    widths[rs.randint(n_in), :] = 0.0 if shapes == 3 else widths[0, :]    # a degenerate dimension in one of the cases
    half = widths[:, np.arange(count) % shapes]
    centre = rs.randint(0, 1024, size=(n_in, count)) / 1024.0
    lbs, ubs = centre - half, centre + half
    assert np.array_equal(0.5 * (ubs - lbs), half)
    layers = [_fc(rs, hidden, n_in, 2.0), {"type": "relu"}, _fc(rs, 300, hidden, 2.0), {"type": "relu"}, _fc(rs, 6, 300)]
    dev_in = nnv.Star.from_boxes(lbs, ubs)
    ora_in = [oracle.star_from_box(lbs[:, i], ubs[:, i]) for i in range(count)]
    _compare(nnv, oracle, layers, dev_in, ora_in, "relax-star-area")


def _shared_product_launches(ctx, fn):
    """Runs fn with per-kernel timing on; returns (result, launches of the pass that writes sets as their group's
    shared product plus row differences)."""
    ctx.kernel_time(10)
    ctx.set_timing(2)
    try:
        res = fn()
    finally:
        ctx.set_timing(0)
    return res, ctx.kernel_time(10)[1]


@pytest.mark.parametrize("spread,shapes,expect", [(0.0, 1, True), (2e-3, 2, True), (2e-2, 3, True), (0.1, 2, None), (0.5, 2, False)])
def test_neighbouring_boxes_share_the_product_over_their_common_rows(nnv, oracle, spread, shapes, expect):
    """96 boxes around one centre, in `shapes` different half-width vectors.  The closer the centres, the more alike
    the rows the first ReLU keeps: the second FC layer then forms one product per shape over the rows most sets keep
    and adds, per set, the rows in which it differs (none at spread 0; 0-2; 1-9, more than the kernel looks up once
    per set; a few dozen at spread 0.1, where either route may be taken); far-apart boxes (66-118 rows) differ in too
    many rows and every set contracts over its own list.  Every set against the oracle either way, and the
    route that was taken is checked."""
    rs = np.random.RandomState(900 + shapes)
    n_in, count, hidden = 200, 96, 400
    widths = rs.randint(1, 64, size=(n_in, shapes)) / 8192.0
    half = widths[:, np.arange(count) % shapes]
    c0 = rs.randint(256, 768, size=(n_in, 1)) / 1024.0
    centre = c0 + np.round(rs.randn(n_in, count) * spread * 1024.0) / 1024.0
    lbs, ubs = centre - half, centre + half
    assert np.array_equal(0.5 * (ubs - lbs), half)
    layers = [_fc(rs, hidden, n_in, 2.0), {"type": "relu"}, _fc(rs, 260, hidden, 2.0), {"type": "relu"}, _fc(rs, 6, 260)]
    dev_in = nnv.Star.from_boxes(lbs, ubs)
    ora_in = [oracle.star_from_box(lbs[:, i], ubs[:, i]) for i in range(count)]
    ctx = nnv.default_context()
    _, launches = _shared_product_launches(ctx, lambda: _compare(nnv, oracle, layers, dev_in, ora_in, "relax-star-area"))
    if expect is not None and not ctx.switch_is_on("no_row_deltas", "dense_affine", "eager_tail"):
        assert (launches > 0) == expect, "spread %g: %d launches of the shared-product pass" % (spread, launches)


@pytest.mark.parametrize("then", ["relu", "fc", "batchnorm", "relu_relu"])
def test_matrices_a_layer_leaves_unwritten_read_the_same_later(nnv, oracle, then):
    """An FC layer over neighbouring boxes that forms its outputs as shared product plus row differences stores, by
    default, only their centres and range sums: the ReLU step behind it needs no more, and the next FC layer reads
    only rows that step keeps.  Whoever does read the matrices first (a fetch, a layer that is not a ReLU step, an
    FC layer behind two ReLU steps) has all sets of the call written by the same pass.  Against the "every column
    written at once" mode: every matrix of the layer is the same to the bit, whether read early, late or only after
    the next layers ran, and when it is read changes no bit of the bounds or of the sets two layers on; the pass
    runs once inside the layer and once more at the first read, not again at the second."""
    rs = np.random.RandomState(2300)
    n_in, count, hidden = 200, 96, 400
    widths = rs.randint(1, 64, size=(n_in, 2)) / 8192.0
    half = widths[:, np.arange(count) % 2]
    c0 = rs.randint(256, 768, size=(n_in, 1)) / 1024.0
    centre = c0 + np.round(rs.randn(n_in, count) * 2e-3 * 1024.0) / 1024.0
    lbs, ubs = centre - half, centre + half
    fc1, fc2, fc3 = _fc(rs, hidden, n_in, 2.0), _fc(rs, 260, hidden, 2.0), _fc(rs, 9, 260)
    tails = {"relu": [{"type": "relu"}, fc3], "fc": [fc3, {"type": "relu"}],
             "batchnorm": [_bn(rs, 260), {"type": "relu"}, fc3],
             "relu_relu": [{"type": "relu"}, {"type": "relu"}, fc3]}
    layers = [fc1, {"type": "relu"}, fc2] + tails[then]
    ctx = nnv.default_context()
    L = nnv.NN.from_config(layers, "unwritten matrices").Layers
    opts = ("relax-star-area", [], 1, None, "linprog")

    def passes():
        return ctx.kernel_time(10)[1]

    def run(read_first):
        s = nnv.Star.from_boxes(lbs, ubs)
        for layer in L[:2]:
            s = layer.reach(s, *opts)
        ctx.set_timing(2)
        try:
            passes()
            t = L[2].reach(s, *opts)
            n_layer = passes()
            early = [np.asarray(a.V).copy() for a in t] if read_first else None
            n_early = passes()
            u = t
            for layer in L[3:]:
                u = layer.reach(u, *opts)
            n_next = passes()
            outs = [np.asarray(a.V).copy() for a in u]
            bounds = [tuple(np.asarray(x).copy() for x in a.estimateRanges()) for a in t]
            n_rest = passes()
            late = [np.asarray(t[k].V).copy() for k in (count - 1, 0, count // 2)]
            n_late = passes()
            again = np.asarray(t[3].V).copy()
            n_again = passes()
        finally:
            ctx.set_timing(0)
        return dict(early=early, outs=outs, bounds=bounds, late=late, again=again, n=(n_layer, n_early, n_next, n_rest, n_late, n_again))

    a = run(False)
    b = run(True)
    was = ctx.switches.get("eager_cols", False)
    ctx.set_switch("eager_cols", True)
    try:
        e = run(True)
    finally:
        ctx.set_switch("eager_cols", was)
    for p, q in zip(a["outs"], b["outs"]):                               # read early or late: nothing else changes
        assert np.array_equal(p, q)
    for (l0, u0), (l1, u1) in zip(a["bounds"], b["bounds"]):
        assert np.array_equal(l0, l1) and np.array_equal(u0, u1)
    for x in (a, b):                                                     # the matrices themselves, whenever written
        for p, q in zip(x["late"], e["late"]):
            assert np.array_equal(p, q)
        assert np.array_equal(x["again"], e["again"])
        # (the other mode sums the bounds of these matrices in another order: equal to rounding, not to the bit)
        for (l0, u0), (l1, u1) in zip(x["bounds"], e["bounds"]):
            assert_close(l0, l1, "lb", 1e-11)
            assert_close(u0, u1, "ub", 1e-11)
    for p, q in zip(b["early"], e["early"]):
        assert np.array_equal(p, q)
    for k, idx in enumerate((count - 1, 0, count // 2)):
        assert np.array_equal(b["late"][k], b["early"][idx])
    if not ctx.switch_is_on("eager_cols", "dense_affine", "eager_tail", "no_row_deltas", "eager_rows"):
        assert e["n"][0] == 1 and sum(e["n"][1:]) == 0, e["n"]           # everything written inside the layer
        assert b["n"][:2] == (1, 1) and sum(b["n"][2:]) == 0, b["n"]     # ... at the first read
        assert a["n"][:2] == (1, 0) and sum(a["n"][2:]) == 1 and a["n"][5] == 0, a["n"]   # ... by whoever reads first
    # and against the oracle, all layers
    _compare(nnv, oracle, layers, nnv.Star.from_boxes(lbs, ubs), [oracle.star_from_box(lbs[:, i], ubs[:, i]) for i in range(count)],
             "relax-star-area")


@pytest.mark.parametrize("spread,shapes", [(0.0, 1), (2e-3, 2), (2e-2, 3)])
def test_shortcuts_of_the_pass_that_sums_unwritten_pieces_change_no_bit(nnv, oracle, spread, shapes):
    """The pass that sums the pieces of an FC layer's outputs without storing them sums a piece once for a run of sets
    that agree in their row differences and predicate bounds (at spread 0 all 96 sets do; further out, the sets of
    one shape that differ from their group's list in nothing or in the same rows), and leaves out half of the
    products where every predicate's bounds mirror each other (boxes: always).  With the shortcuts switched off -
    every set summed in full, with both bounds - the layer's bounds and the sets two layers on are the same to
    the bit."""
    rs = np.random.RandomState(2400 + shapes)
    n_in, count, hidden = 200, 96, 400
    widths = rs.randint(1, 64, size=(n_in, shapes)) / 8192.0
    half = widths[:, np.arange(count) % shapes]
    c0 = rs.randint(256, 768, size=(n_in, 1)) / 1024.0
    centre = c0 + np.round(rs.randn(n_in, count) * spread * 1024.0) / 1024.0
    lbs, ubs = centre - half, centre + half
    layers = [_fc(rs, hidden, n_in, 2.0), {"type": "relu"}, _fc(rs, 260, hidden, 2.0), {"type": "relu"}, _fc(rs, 6, 260)]
    ctx = nnv.default_context()
    L = nnv.NN.from_config(layers, "shortcuts").Layers
    opts = ("relax-star-area", [], 1, None, "linprog")

    def run():
        s = nnv.Star.from_boxes(lbs, ubs)
        for layer in L[:2]:
            s = layer.reach(s, *opts)
        ctx.set_timing(2)
        try:
            ctx.kernel_time(10)
            t = L[2].reach(s, *opts)
            passes = ctx.kernel_time(10)[1]
        finally:
            ctx.set_timing(0)
        bounds = [tuple(np.asarray(x).copy() for x in a.estimateRanges()) for a in t]
        u = L[4].reach(L[3].reach(t, *opts), *opts)
        return passes, bounds, [np.asarray(a.V).copy() for a in u]

    was = ctx.switches.get("no_sum_shortcuts", False)
    ctx.set_switch("no_sum_shortcuts", False)
    try:
        p0, b0, v0 = run()
        ctx.set_switch("no_sum_shortcuts", True)
        p1, b1, v1 = run()
    finally:
        ctx.set_switch("no_sum_shortcuts", was)
    for (l0, u0), (l1, u1) in zip(b0, b1):
        assert np.array_equal(l0, l1) and np.array_equal(u0, u1)
    for a, b in zip(v0, v1):
        assert np.array_equal(a, b)
    if not ctx.switch_is_on("no_row_deltas", "dense_affine", "eager_tail"):
        assert p0 == 1 and p1 == 1, (p0, p1)
    _compare(nnv, oracle, layers, nnv.Star.from_boxes(lbs, ubs), [oracle.star_from_box(lbs[:, i], ubs[:, i]) for i in range(count)],
             "relax-star-area")


@pytest.mark.parametrize("count,half_width", [(1, 0.02), (1, 3.0), (5, 0.3)])
def test_a_relu_on_top_of_a_relu_lists_its_rows_anew(nnv, oracle, count, half_width):
    """ReLU, ReLU, FC: the second step keeps the rows whose neurons crossed in the first (their range is now
    [0, ub]), rows the first step's reset zeroed -- whatever is remembered about where the kept rows' columns came
    from does not hold for them, and the FC layer behind must read them as they are in memory.  From narrow boxes
    (few neurons cross) to wide ones (nearly all do), one set and an array, with a second pair further down."""
    rs = np.random.RandomState(1700 + count)
    n_in = 90
    layers = [_fc(rs, 300, n_in, 2.0), {"type": "relu"}, {"type": "relu"}, _fc(rs, 150, 300, 2.0), {"type": "relu"},
              {"type": "relu"}, {"type": "relu"}, _fc(rs, 7, 150)]
    centre = rs.rand(n_in, count)
    half = np.abs(rs.randn(n_in, count)) * half_width
    lbs, ubs = centre - half, centre + half
    if count == 1:
        dev_in, ora_in = nnv.Star(lbs[:, 0], ubs[:, 0]), oracle.star_from_box(lbs[:, 0], ubs[:, 0])
    else:
        dev_in = nnv.Star.from_boxes(lbs, ubs)
        ora_in = [oracle.star_from_box(lbs[:, i], ubs[:, i]) for i in range(count)]
    for method in ("relax-star-area", "relax-star-random"):
        _compare(nnv, oracle, layers, dev_in, ora_in, method)


@pytest.mark.parametrize("count", [1, 40])
def test_relu_steps_that_append_their_predicate_bounds_in_place(nnv, oracle, count):
    """A ReLU step leaves room behind the predicate bounds it writes, and a later step whose input ends exactly
    there appends its own in place instead of copying the old ones.  Seven ReLU steps in a row behind FC layers of
    different widths (the room runs out on the way and a step copies again), every set of every layer against the
    oracle; then two different steps applied to one and the same set, in both orders, and a third to the set before
    it: nobody sees what another step appended behind the entries that are his."""
    rs = np.random.RandomState(2500 + count)
    n_in = 30
    widths = [64, 64, 96, 64, 48, 200, 64]
    layers, prev = [], n_in
    for wd in widths:
        layers += [_fc(rs, wd, prev, 2.5), {"type": "relu"}]
        prev = wd
    layers.append(_fc(rs, 5, prev))
    centre = rs.rand(n_in, count)
    half = np.abs(rs.randn(n_in, count)) * 0.4
    lbs, ubs = centre - half, centre + half
    if count == 1:
        dev_in, ora_in = nnv.Star(lbs[:, 0], ubs[:, 0]), oracle.star_from_box(lbs[:, 0], ubs[:, 0])
    else:
        dev_in = nnv.Star.from_boxes(lbs, ubs)
        ora_in = [oracle.star_from_box(lbs[:, i], ubs[:, i]) for i in range(count)]
    for method in ("relax-star-area", "relax-star-static"):
        _compare(nnv, oracle, layers, dev_in, ora_in, method)
    # one set, several steps
    L = nnv.NN.from_config(layers, "in place").Layers
    opts = ("relax-star-area", [], 1, None, "linprog")

    def bounds(sets):
        sets = sets if isinstance(sets, (list, nnv.SetArray)) else [sets]
        return [(np.asarray(t.predicate_lb).copy(), np.asarray(t.predicate_ub).copy()) for t in sets]

    ctx = nnv.default_context()
    lazy = not ctx.switch_is_on("eager_rows", "eager_tail", "dense_affine")  # (a step that writes rows or columns at once sizes its arrays exactly)
    c0 = ctx.relu_bounds_counts()
    s1 = L[1].reach(L[0].reach(dev_in, *opts), *opts)        # the first step's output: room behind its bounds
    f2 = L[2].reach(s1, *opts)
    b_s1, b_f2 = bounds(s1), bounds(f2)
    c1 = ctx.relu_bounds_counts()
    a = L[3].reach(f2, *opts)                                # appends in place
    c2 = ctx.relu_bounds_counts()
    b_a = bounds(a)
    b = L[3].reach(f2, "relax-star-range", [], 1, None, "linprog")   # the same input again: the room is taken
    other = L[3].reach(L[2].reach(s1, *opts), *opts)        # ... and for an equal input made afresh from the set before
    c3 = ctx.relu_bounds_counts()
    assert (c1[0] - c0[0], c1[1] - c0[1]) == (0, count)
    if lazy:
        assert (c2[0] - c1[0], c2[1] - c1[1]) == (count, 0) and (c3[0] - c2[0], c3[1] - c2[1]) == (0, 2 * count)
    for (l0, u0), (l1, u1) in zip(b_s1, bounds(s1)):
        assert np.array_equal(l0, l1) and np.array_equal(u0, u1)
    for (l0, u0), (l1, u1) in zip(b_f2, bounds(f2)):
        assert np.array_equal(l0, l1) and np.array_equal(u0, u1)
    for (l0, u0), (l1, u1) in zip(b_a, bounds(a)):
        assert np.array_equal(l0, l1) and np.array_equal(u0, u1)
    for (l0, u0), (l1, u1), (l2, u2) in zip(b_a, bounds(b), bounds(other)):
        # the same crossing neurons in another order: the same multiset of new bounds behind the same old ones
        assert len(l0) == len(l1) and np.array_equal(np.sort(u0), np.sort(u1))
        assert np.array_equal(l0, l2) and np.array_equal(u0, u2)      # the same step on an equal input: the same bounds


@pytest.mark.parametrize("seed", [318, 456, 620, 690, 717, 720, 800, 843, 855, 892])
def test_random_fc_sequences_that_once_failed(nnv, oracle, seed):
    """Random FC / ReLU / batch-normalisation sequences over one, two or five boxes of widths from 0.005 to 3, the
    six relax-star methods in turn: the seeds of a longer run of this generator on which an earlier build of the
    library gave wrong sets (all of them hold a ReLU step directly on top of another one)."""
    rs = np.random.RandomState(seed)
    n_in = int(rs.choice([5, 12, 40, 90]))
    layers = _random_fc_sequence(rs, n_in)
    count = int(rs.choice([1, 2, 5]))
    centre = rs.rand(n_in, count)
    half = np.abs(rs.randn(n_in, count)) * rs.choice([0.005, 0.02, 0.3, 3.0], size=(1, count))
    if rs.rand() < 0.5:
        half[rs.randint(n_in), :] = 0.0
    lbs, ubs = centre - half, centre + half
    method = ["relax-star-area", "relax-star-range", "relax-star-static", "relax-star-random", "relax-star-bound",
              "relax-star-ub"][seed % 6]
    if count == 1:
        dev_in, ora_in = nnv.Star(lbs[:, 0], ubs[:, 0]), oracle.star_from_box(lbs[:, 0], ubs[:, 0])
    else:
        dev_in = nnv.Star.from_boxes(lbs, ubs)
        ora_in = [oracle.star_from_box(lbs[:, i], ubs[:, i]) for i in range(count)]
    _compare(nnv, oracle, layers, dev_in, ora_in, method)


@pytest.mark.parametrize("count", [64, 100, 40])
def test_a_hint_about_the_next_fc_layer_changes_no_bit(nnv, oracle, count):
    """NN.reach tells the library which FC layer follows a ReLU step over an array of at least 64 sets; the step then
    queues that layer's range-sum product of the columns it appends behind its classification, and the FC call
    takes it from the sets instead of forming it.  With the hint, without it (the layers called one by one), with a
    hint that does not come true (another FC layer of the same shape is applied), and for an array too small for
    it: the same sets and the same bounds to the bit, and the oracle's to tolerance; where the hint is taken the FC
    call launches one matrix product less."""
    rs = np.random.RandomState(2100 + count)
    n_in, hidden = 60, 320
    half = rs.randint(1, 64, size=(n_in, count)) / 1024.0
    centre = rs.randint(0, 1024, size=(n_in, count)) / 1024.0
    lbs, ubs = centre - half, centre + half
    layers = [_fc(rs, hidden, n_in, 2.0), {"type": "relu"}, _fc(rs, 290, hidden, 2.0), {"type": "relu"}, _fc(rs, 6, 290)]
    other = nnv.NN.from_config([_fc(rs, 290, hidden, 2.0)], "another layer of the same shape").Layers[0]
    ctx = nnv.default_context()
    net = nnv.NN.from_config(layers, "hint")
    L = net.Layers
    opts = ("relax-star-area", [], 1, None, "linprog")

    def run(hint, second=None):
        s = nnv.Star.from_boxes(lbs, ubs)
        s = L[0].reach(s, *opts)
        if hint is not None:
            ctx.hint_next_fc(hint._weights(ctx))
        s = L[1].reach(s, *opts)
        ctx.kernel_time(0)
        ctx.set_timing(2)
        try:
            t = (second or L[2]).reach(s, *opts)
        finally:
            ctx.set_timing(0)
        gemms = ctx.kernel_time(0)[1]
        u = L[3].reach(t, *opts)
        bounds = [tuple(np.asarray(x).copy() for x in a.estimateRanges()) for a in t]
        return gemms, bounds, [np.asarray(a.V).copy() for a in u]

    g0, b0, v0 = run(None)
    g1, b1, v1 = run(L[2])
    g2, b2, v2 = run(other, second=L[2])         # hinted at a layer that is not the one applied
    for (l0, u0), (l1, u1), (l2, u2) in zip(b0, b1, b2):
        assert np.array_equal(l0, l1) and np.array_equal(u0, u1) and np.array_equal(l0, l2) and np.array_equal(u0, u2)
    for a, b, c_ in zip(v0, v1, v2):
        assert np.array_equal(a, b) and np.array_equal(a, c_)
    if not ctx.switch_is_on("eager_cols", "dense_affine", "eager_rows", "eager_tail"):
        assert g1 == (g0 - 1 if count >= 64 else g0), (g0, g1)
        assert g2 == g0
    # NN.reach gives the hint itself; against the oracle
    _compare(nnv, oracle, layers, nnv.Star.from_boxes(lbs, ubs), [oracle.star_from_box(lbs[:, i], ubs[:, i]) for i in range(count)],
             "relax-star-area")
