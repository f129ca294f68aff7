"""CPU checks of the host-side mirror of NNV's classes: argument validation, error strings, option
parsing and the Box arithmetic - everything that does not need a device call."""
import numpy as np
import pytest

from nnv_amd.configs import conv_out_hw, count_updates, make_config
from nnv_amd.layers import RELAX_ORDER, Conv2DLayer, FullyConnectedLayer
from nnv_amd.nn import NN
from nnv_amd.sets import Box
from oracle import nnv_oracle as o


def test_box_matches_oracle_arithmetic():
    lb = np.array([0.1, -1.0, 2.0, 2.0])
    ub = np.array([0.4, 1.0, 2.0, 3.5])
    b = Box(lb, ub)
    c, g = o.box_generators(lb, ub)
    assert np.array_equal(b.center, c) and np.array_equal(b.generators, g)
    assert b.generators.shape == (4, 3)          # the zero-width dimension has no generator
    parts = b.partition([0, 3], [2, 3])
    ref = o.box_partition(lb, ub, [0, 3], [2, 3])
    assert len(parts) == 6
    for p, (l, u) in zip(parts, ref):
        assert np.array_equal(p.lb, l) and np.array_equal(p.ub, u)
    with pytest.raises(ValueError, match="Inconsistent dimensions"):
        Box([0, 1], [1])
    with pytest.raises(ValueError, match="index in part_indexes"):
        b.partition([7], [2])


def test_layer_constructors_validate_like_nnv():
    with pytest.raises(ValueError, match="weight matrix and bias vector"):
        FullyConnectedLayer(np.ones((3, 2)), np.ones(4))
    with pytest.raises(ValueError, match="one column"):
        FullyConnectedLayer(np.ones((3, 2)), np.ones((3, 2)))
    L = FullyConnectedLayer("fc", np.ones((3, 2)), np.ones((3, 1)))
    assert (L.InputSize, L.OutputSize, L.Name) == (2, 3, "fc")
    assert np.array_equal(L.evaluate([1.0, 2.0]), [4.0, 4.0, 4.0])
    with pytest.raises(ValueError, match="filter weights and filter biases"):
        Conv2DLayer(np.ones((3, 3, 2, 4)), np.ones(3))
    C = Conv2DLayer(np.ones((3, 3, 2, 4)), np.ones(4), [1, 1, 1, 1], [2, 2], [1, 1])
    assert (C.NumChannels, C.NumFilters, C.FilterSize) == (2, 4, [3, 3])
    assert C.output_size(32, 32) == (16, 16)
    assert C.output_size(15, 15) == conv_out_hw(15, 15, {"W": np.ones((3, 3, 2, 4)), "padding": [1, 1, 1, 1],
                                                           "stride": [2, 2], "dilation": [1, 1]})


def test_reach_options_validation():
    net = NN([])
    with pytest.raises(ValueError, match="specify a relax factor"):
        net.validate_reach_options({"reachMethod": "relax-star-area"})
    with pytest.raises(ValueError, match="between 0 and 1"):
        net.validate_reach_options({"reachMethod": "relax-star-area", "relaxFactor": 1.5})
    opts = net.validate_reach_options({"reachMethod": "relax-star-area", "relaxFactor": 1, "numCores": 8})
    assert opts["numCores"] == 1 and opts["reachOption"] == "single"      # nn/NN.m:1227-1231
    with pytest.raises(TypeError, match="Wrong input set type"):
        net.reach(np.zeros(3), {"reachMethod": "relax-star-area", "relaxFactor": 1})


def test_relax_orders_cover_the_six_variants():
    assert sorted(RELAX_ORDER) == sorted(o.RELAX_METHODS)
    assert RELAX_ORDER["relax-star-area"] != RELAX_ORDER["relax-star-range"]
    assert len({RELAX_ORDER[m] for m in ("relax-star-bound", "relax-star-ub", "relax-star-random", "relax-star-static")}) == 1


def test_configs_are_reproducible_and_sized():
    a, b = make_config(2), make_config(2)
    assert np.array_equal(a["layers"][0]["W"], b["layers"][0]["W"]) and np.array_equal(a["lb"], b["lb"])
    assert [L["W"].shape for L in a["layers"] if L["type"] == "fc"] == [(1024, 784), (1024, 1024), (1024, 1024), (10, 1024)]
    c5 = make_config(5)
    assert np.array_equal(c5["layers"][0]["W"], a["layers"][0]["W"]) and len(c5["partition"]["indexes"]) == 10
    c4 = make_config(4)
    assert c4["image_shape"] == (32, 32, 3) and c4["layers"][8]["W"].shape == (512, 7 * 7 * 64)
    c3 = make_config(3)
    assert c3["layers"][4]["W"].shape == (100, 14 * 14 * 32)
    assert abs(np.std(a["layers"][2]["W"]) - np.sqrt(2.0 / 1024)) < 1e-3
    assert count_updates([(3, 4), (2, 1)]) == 3 * 5 + 2 * 2


class _HostStar:
    """Stands where a device Star would: ranges and LP bounds of an oracle star, so the host-side
    bookkeeping of the relaxFactor < 1 heuristics can be checked without a GPU."""

    def __init__(self, S):
        self.S = S

    def estimateRanges(self):
        return o.estimate_ranges(self.S)

    def getMaxs(self, idx, *_):
        return o.get_maxs(self.S, idx)

    def getMins(self, idx, *_):
        return o.get_mins(self.S, idx)


@pytest.mark.parametrize("method", sorted(RELAX_ORDER))
@pytest.mark.parametrize("rf", [0.0, 0.3, 0.5, 1.0])
def test_relax_factor_bookkeeping_hands_the_device_the_oracles_lists(monkeypatch, method, rf):
    # which neurons are reset, which cross with which bounds, and in which order: the lists the host code
    # passes to the device step must be the ones the restatement of PosLin.reach_relaxed_star_* builds
    from nnv_amd import layers
    rs = np.random.RandomState(4)
    n, N = 5, 30
    I = o.star_from_box(-rs.rand(n) - 0.2, rs.rand(n) + 0.2)
    S = o.affine_map(o.reach_relaxed_star(o.affine_map(I, rs.randn(N, n), rs.randn(N) * 0.3), "relax-star-area", 1.0),
                     rs.randn(N, N) * 0.5, rs.randn(N) * 0.3)
    seen = {}

    def capture(star, index, lb, ub, reset=()):
        seen.update(index=np.asarray(index), lb=np.asarray(lb), ub=np.asarray(ub), reset=np.asarray(reset))
        return o.multiple_step_reach_star_approx_at_one(o.reset_row(star.S, np.asarray(reset, dtype=int)), index, lb, ub)

    monkeypatch.setattr(layers.PosLin, "multipleStepReachStarApprox_at_one", staticmethod(capture))
    got = layers._relaxed_star_lp(_HostStar(S), method, rf, rng=np.random.RandomState(8))
    want = o.reach_relaxed_star_lp(S, method, rf, np.random.RandomState(8))
    assert np.array_equal(got.V, want.V) and np.array_equal(got.C, want.C) and np.array_equal(got.d, want.d)
    assert np.array_equal(got.predicate_ub, want.predicate_ub)
    assert np.all(seen["lb"] < 0) and np.all(seen["ub"] > 0)          # what the device step insists on
    assert len(set(seen["index"]) & set(seen["reset"])) == 0
    assert len(set(seen["index"])) == seen["index"].size


def test_partition_bounds_is_the_partition():
    rs = np.random.RandomState(2)
    lb = rs.rand(9) - 0.5
    ub = lb + rs.rand(9) * 0.3 + 0.01
    b = Box(lb, ub)
    for idx, nums in (([0, 3, 7], [2, 3, 2]), ([4], [5]), ([1, 2], [1, 4]), ([8, 0], [3, 3])):
        boxes = b.partition(idx, nums)
        lbs, ubs = b.partition_bounds(idx, nums)
        assert lbs.shape == (9, len(boxes))
        assert np.array_equal(lbs, np.stack([x.lb for x in boxes], axis=1))
        assert np.array_equal(ubs, np.stack([x.ub for x in boxes], axis=1))
        ref = o.box_partition(lb, ub, idx, nums)
        assert np.array_equal(lbs, np.stack([r[0] for r in ref], axis=1))
    with pytest.raises(ValueError, match="index in part_indexes"):
        b.partition_bounds([9], [2])


def test_precision_and_device_switches_of_a_set():
    from nnv_amd.sets import _change_device, _change_precision
    marker = object()
    assert _change_precision(marker, "double") is marker
    with pytest.raises(ValueError, match="double precision only"):
        _change_precision(marker, "single")
    with pytest.raises(ValueError, match="Only single or double"):
        _change_precision(marker, "half")
    assert _change_device(marker, "cpu") is marker and _change_device(marker, "gpu") is marker
    with pytest.raises(ValueError, match="'cpu' or 'gpu'"):
        _change_device(marker, "tpu")


class _CountingCtx:
    """Stands where a device context would: records which handles are released and how."""

    def __init__(self):
        self.single, self.bulk = [], []

    def release_set(self, h):
        self.single.append(h)

    def release_sets(self, count, raw):
        self.bulk.append([raw[i] for i in range(count) if raw[i]])


def test_set_array_makes_objects_on_demand_and_releases_every_handle_once():
    import ctypes as C
    import gc
    from nnv_amd.sets import ImageStar, SetArray, Star
    ctx = _CountingCtx()
    raw = (C.c_void_p * 5)(11, 12, 13, 14, 15)
    arr = SetArray(ctx, raw, [None, (2, 2, 1), None, None, None])
    assert len(arr) == 5 and arr._items is None            # nothing wrapped yet
    assert arr.handles() is raw
    b = arr[1]
    assert isinstance(b, ImageStar) and (b.height, b.width, b.numChannel) == (2, 2, 1)
    assert arr[1] is b and arr[-4] is b                     # one object per element
    e = arr[-1]
    assert type(e) is Star and e._h.h == 15
    with pytest.raises(IndexError):
        arr[5]
    assert [s._h.h for s in arr[2:4]] == [13, 14]           # a slice is a plain list of the elements
    del arr
    gc.collect()
    # the array released what nobody read (11), in one call; 13 and 14 died with the slice's list
    assert ctx.bulk == [[11]]
    assert sorted(ctx.single) == [13, 14]
    del b, e
    gc.collect()
    assert sorted(ctx.single) == [12, 13, 14, 15]
    # an array nobody looked into goes in one call
    ctx2 = _CountingCtx()
    arr2 = SetArray(ctx2, (C.c_void_p * 3)(1, 2, 3))
    assert [type(s) for s in arr2] == [Star] * 3 and ctx2.single == []
    arr3 = SetArray(ctx2, (C.c_void_p * 3)(4, 5, 6))
    del arr3
    gc.collect()
    assert ctx2.bulk == [[4, 5, 6]]
    # an array of boxes hands each element its own column of the bound matrices (Star(lb, ub) keeps them as
    # state_lb / state_ub, set/Star.m:232-233)
    lbs = np.asfortranarray(np.arange(6.0).reshape(3, 2))
    ubs = lbs + 1.0
    boxes = SetArray(ctx2, (C.c_void_p * 2)(7, 8), state=(lbs, ubs))
    assert np.array_equal(boxes[1].state_lb, [1.0, 3.0, 5.0]) and np.array_equal(boxes[1].state_ub, [2.0, 4.0, 6.0])
    assert boxes[0].state_lb.base is not None and np.array_equal(boxes[0].state_lb, lbs[:, 0])
