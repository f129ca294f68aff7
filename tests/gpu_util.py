"""Helpers shared by the GPU parity tests: run a configuration through the HIP library (via the
NNV-mirror classes, i.e. through the C ABI) and through the CPU oracle, and compare."""
import numpy as np

from nnv_amd import NN, ImageStar, Star
from nnv_amd.configs import make_config
from oracle import nnv_oracle as o

RTOL = 1e-9  # north-star tolerance for fp64 values (relative to the array's scale)


class DeviceDoubles:
    """`count` doubles of device memory owned by the test (hipMalloc through the HIP runtime the library
    itself is linked against), for entry points that take device pointers."""

    def __init__(self, count, fill=np.nan):
        import ctypes as C
        from nnv_amd import _lib
        _lib.load()                                   # brings the runtime into the process
        self._hip = C.CDLL("libamdhip64.so.7")
        self.count = int(count)
        p = C.c_void_p()
        assert self._hip.hipMalloc(C.byref(p), C.c_size_t(8 * self.count)) == 0
        self.ptr = p
        host = np.full(self.count, fill, dtype=np.float64)
        assert self._hip.hipMemcpy(self.ptr, host.ctypes.data_as(C.c_void_p), C.c_size_t(8 * self.count), 1) == 0   # host to device

    def get(self):
        import ctypes as C
        host = np.empty(self.count, dtype=np.float64)
        assert self._hip.hipMemcpy(host.ctypes.data_as(C.c_void_p), self.ptr, C.c_size_t(8 * self.count), 2) == 0   # device to host
        return host

    def __del__(self):
        try:
            self._hip.hipFree(self.ptr)
        except Exception:
            pass


def assert_close(got, exp, what, rtol=RTOL):
    got = np.asarray(got)
    exp = np.asarray(exp)
    assert got.shape == exp.shape, "%s: shape %s vs %s" % (what, got.shape, exp.shape)
    if exp.size == 0:
        return
    scale = max(np.max(np.abs(exp)), 1e-300)
    err = np.max(np.abs(got - exp))
    assert err <= rtol * scale, "%s: max abs err %.3e (scale %.3e, rel %.3e)" % (what, err, scale, err / scale)


def assert_close_elementwise(got, exp, what, rtol=RTOL, atol_of_scale=1e-12):
    """Entry by entry: |got - exp| <= rtol * |exp| + atol_of_scale * max|exp|, and the same sign wherever the expected
    entry is not zero.  The absolute term covers sums that cancel (a bound near zero is a difference of large
    terms; its error is that of the terms), the sign is what a classification depends on."""
    got = np.asarray(got, dtype=np.float64)
    exp = np.asarray(exp, dtype=np.float64)
    assert got.shape == exp.shape, "%s: shape %s vs %s" % (what, got.shape, exp.shape)
    if exp.size == 0:
        return
    scale = max(np.max(np.abs(exp)), 1e-300)
    err = np.abs(got - exp)
    bad = err > rtol * np.abs(exp) + atol_of_scale * scale
    assert not bad.any(), "%s: %d entries off, worst |err| %.3e at expected value %.3e (scale %.3e)" % (
        what, int(bad.sum()), float(err[bad].max()), float(exp[bad][np.argmax(err[bad])]), scale)
    flipped = (exp != 0) & (np.sign(got) != np.sign(exp))
    assert not flipped.any(), "%s: %d entries changed sign, e.g. expected %.3e got %.3e" % (
        what, int(flipped.sum()), float(exp[flipped][0]), float(got[flipped][0]))


def classification_margin(lb, ub):
    """min(|lb|, |ub|) over the neurons of a layer, relative to the largest bound: how far the closest bound is
    from changing a neuron's class."""
    lb, ub = np.asarray(lb), np.asarray(ub)
    scale = max(np.max(np.abs(lb)), np.max(np.abs(ub)), 1e-300)
    return float(min(np.min(np.abs(lb)), np.min(np.abs(ub))) / scale)


def input_sets(cfg):
    """Build the device input set(s) and the oracle's, exactly as Star(lb,ub)/ImageStar(lb,ub)."""
    if "partition" in cfg:
        boxes = o.box_partition(cfg["lb"], cfg["ub"], cfg["partition"]["indexes"], cfg["partition"]["numbers"])
        lbs = np.stack([b[0] for b in boxes], axis=1)
        ubs = np.stack([b[1] for b in boxes], axis=1)
        return Star.from_boxes(lbs, ubs), [o.star_from_box(l, u) for (l, u) in boxes]
    if cfg["kind"] == "image":
        sh = cfg["image_shape"]
        lb = cfg["lb"].reshape(sh, order="F")
        ub = cfg["ub"].reshape(sh, order="F")
        return ImageStar(lb, ub), o.image_star_from_bounds(lb, ub)
    return Star(cfg["lb"], cfg["ub"]), o.star_from_box(cfg["lb"], cfg["ub"])


def flat_V(S):
    V = np.asarray(S.V)
    return V.reshape(-1, V.shape[-1], order="F") if V.ndim == 4 else V


def nvar(S):
    return S.numPred if hasattr(S, "numPred") else S.nVar


def compare_sets(dev, ora, what, check_constraints=True):
    """Values within RTOL; shapes, one-hot/zero structure exact."""
    Vd, Vo = flat_V(dev), flat_V(ora)
    assert Vd.shape == Vo.shape, "%s: V shape %s vs %s" % (what, Vd.shape, Vo.shape)
    assert_close(Vd, Vo, what + ".V")
    assert np.array_equal(Vd == 0, Vo == 0) or np.max(np.abs(Vd[(Vd == 0) != (Vo == 0)])) < 1e-9 * np.max(np.abs(Vo)), what + ": zero pattern"
    plb = dev.pred_lb if hasattr(dev, "pred_lb") else dev.predicate_lb
    pub = dev.pred_ub if hasattr(dev, "pred_ub") else dev.predicate_ub
    olb = ora.pred_lb if hasattr(ora, "pred_lb") else ora.predicate_lb
    oub = ora.pred_ub if hasattr(ora, "pred_ub") else ora.predicate_ub
    assert_close(plb, olb, what + ".pred_lb")
    assert_close(pub, oub, what + ".pred_ub")
    if check_constraints:
        assert dev.C.shape == ora.C.shape, "%s: C shape %s vs %s" % (what, dev.C.shape, ora.C.shape)
        assert_close(dev.C, ora.C, what + ".C")
        assert_close(dev.d, ora.d, what + ".d")


def sort_key(lb, ub, method):
    if method == "relax-star-range":
        return ub - lb
    if method == "relax-star-area":
        return 0.5 * (np.abs(ub) * np.abs(lb))
    return None


def run_both(k, method="relax-star-area", shrink=1, check_constraints=True, margins=None, tie_tolerant=False):
    """Reach config k on the device and in the oracle; compare every layer's set.

    Classification parity (bit-exact): inactive counts, crossing index lists in new-predicate order.
    Returns (device output, oracle output, NN object)."""
    return run_cfg(make_config(k, shrink), method, check_constraints, margins, tie_tolerant)


def run_cfg(cfg, method="relax-star-area", check_constraints=True, margins=None, tie_tolerant=False):
    """run_both for a configuration dictionary (name, kind, layers, lb, ub[, image_shape, partition])."""
    dev_in, ora_in = input_sets(cfg)
    net = NN.from_config(cfg["layers"], cfg["name"])
    dev_out = net.reach(dev_in, {"reachMethod": method, "relaxFactor": 1})
    ora_out, ora_sets = o.nn_reach(cfg["layers"], ora_in, method, 1.0, keep=True)
    batched = not isinstance(dev_in, (Star, ImageStar))
    for li, (L, dset, oset) in enumerate(zip(cfg["layers"], net.reachSet, ora_sets)):
        dl = dset if batched else [dset]
        ol = oset if batched else [oset]
        prev = (ora_sets[li - 1] if li > 0 else ora_in)
        pl = prev if batched else [prev]
        assert len(dl) == len(ol)
        for si, (ds, os_, ps) in enumerate(zip(dl, ol, pl)):
            tag = "%s layer %d (%s) set %d" % (cfg["name"], li + 1, L["type"], si)
            if L["type"] == "relu":
                pstar = ps.to_star() if isinstance(ps, o.OImageStar) else ps
                lb, ub = o.estimate_ranges(pstar)
                m1, m2 = o.relax_classify(lb, ub, method)
                ni, idx, clb, cub = ds.relu_info()
                if margins is not None:
                    margins.append(float(np.min(np.minimum(np.abs(lb), np.abs(ub)) / max(np.max(np.abs(ub - lb)), 1e-300))))
                # the device's own bounds of the ReLU's input, entry by entry: a bound near zero must keep its sign
                dprev = (net.reachSet[li - 1] if li > 0 else dev_in)
                dprev = dprev[si] if batched else dprev
                dlb, dub = (np.asarray(x).reshape(-1, order="F") for x in dprev.estimateRanges())
                assert_close_elementwise(dlb, lb, tag + ": lb of the ReLU's input")
                assert_close_elementwise(dub, ub, tag + ": ub of the ReLU's input")
                assert ni == m1.size, "%s: inactive count %d vs %d" % (tag, ni, m1.size)
                if tie_tolerant and not np.array_equal(idx, m2):
                    # Sort keys that are equal in exact arithmetic (e.g. ub-lb of a conv layer under a
                    # uniform input box) are ordered by rounding noise, in any implementation.  Accept
                    # an order that is a valid descending sort of the oracle's keys up to RTOL; later
                    # layers are then column-permuted, so the comparison stops here.
                    assert np.array_equal(np.sort(idx), np.sort(m2)), "%s: crossing set differs" % tag
                    key = sort_key(lb, ub, method)[idx]
                    assert np.all(np.diff(key) <= RTOL * np.max(np.abs(key))), "%s: not a descending order" % tag
                    return dev_out, ora_out, net
                assert np.array_equal(idx, m2), "%s: crossing index list / order differs" % tag
                assert_close(clb, lb[m2], tag + ".lb(crossing)")
                assert_close(cub, ub[m2], tag + ".ub(crossing)")
            # only materialise C on the sets where it changed (after a ReLU) to keep the test fast
            compare_sets(ds, os_, tag, check_constraints and L["type"] == "relu")
    return dev_out, ora_out, net
