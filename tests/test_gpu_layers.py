"""GPU parity of the further affine layers (batch normalisation, average pooling, flatten, input
normalisation, ImageStar.affineMap, LayerS) through the C ABI, against the oracle."""
import numpy as np
import pytest

from oracle import nnv_oracle as o
from nnv_amd.configs import make_extended_cnn
from tests.gpu_util import RTOL, assert_close, compare_sets, input_sets

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def nnv():
    import nnv_amd
    return nnv_amd


def _pair(nnv, rs, H, W, C, n):
    V = rs.randn(H, W, C, n + 1)
    Cm, d = rs.randn(2, n), rs.rand(2) + 5.0
    plb, pub = -rs.rand(n) - 0.5, rs.rand(n) + 0.5
    return nnv.ImageStar(V, Cm, d, plb, pub), o.OImageStar(V, Cm, d, plb, pub)


@pytest.mark.parametrize("H,W,C,n", [(4, 5, 3, 4), (28, 28, 1, 40), (15, 15, 32, 130), (1, 1, 64, 7)])
def test_batchnorm_imagestar(nnv, H, W, C, n):
    rs = np.random.RandomState(H * W + C)
    D, O = _pair(nnv, rs, H, W, C, n)
    mean, var, scale, offset, eps = rs.randn(C), rs.rand(C) + 0.1, rs.randn(C), rs.randn(C), 1e-5
    L = nnv.BatchNormalizationLayer(NumChannels=C, TrainedMean=mean.reshape(1, 1, C), TrainedVariance=var.reshape(1, 1, C),
                                    Epsilon=eps, Scale=scale.reshape(1, 1, C), Offset=offset.reshape(1, 1, C))
    R = L.reach(D, "relax-star-area", "single", 1)
    E = o.batchnorm_reach(O, mean, var, eps, scale, offset)
    assert (R.height, R.width, R.numChannel) == (H, W, C)
    assert np.array_equal(R.V, E.V)      # same operations in the same order: bit-identical
    compare_sets(R, E, "batchnorm")
    # input untouched, bounds follow
    assert np.array_equal(D.V, O.V)
    lb, ub = R.estimateRanges()
    elb, eub = o.image_star_estimate_ranges(E)
    assert_close(lb, elb, "lb")
    assert_close(ub, eub, "ub")


def test_batchnorm_star_and_array(nnv):
    rs = np.random.RandomState(9)
    N, n = 37, 5
    mean, var, scale, offset = rs.randn(N), rs.rand(N) + 0.1, rs.randn(N), rs.randn(N)
    L = nnv.BatchNormalizationLayer(NumChannels=N, TrainedMean=mean, TrainedVariance=var, Scale=scale, Offset=offset)
    devs, oras = [], []
    for _ in range(3):
        V = rs.randn(N, n + 1)
        args = (V, np.zeros((1, n)), np.zeros(1), -np.ones(n), np.ones(n))
        devs.append(nnv.Star(*args))
        oras.append(o.OStar(*args))
    outs = L.reach(devs, "approx-star")
    for R, O in zip(outs, oras):
        E = o.batchnorm_reach(O, mean, var, 1e-5, scale, offset)
        assert np.array_equal(R.V, E.V)
    with pytest.raises(ValueError, match="Unknown reachability method"):
        L.reach(devs[0], "fancy-star")


@pytest.mark.parametrize("H,W,C,n,pool,stride,pad", [
    (4, 4, 1, 3, (2, 2), (2, 2), (0, 0, 0, 0)), (5, 5, 3, 6, (3, 3), (2, 2), (0, 0, 0, 0)),
    (28, 28, 1, 1, (6, 4), (4, 4), (1, 1, 0, 0)), (9, 8, 4, 50, (3, 2), (1, 2), (1, 0, 0, 1)),
    (32, 32, 16, 200, (2, 2), (2, 2), (0, 0, 0, 0)), (15, 15, 8, 33, (3, 3), (2, 2), (1, 1, 1, 1))])
def test_avgpool(nnv, H, W, C, n, pool, stride, pad):
    rs = np.random.RandomState(H + 7 * W + C)
    D, O = _pair(nnv, rs, H, W, C, n)
    L = nnv.AveragePooling2DLayer(list(pool), list(stride), list(pad))
    R = L.reach(D, "relax-star-range", "single", 1)
    E = o.avgpool2d_reach(O, pool, stride, pad)
    assert (R.height, R.width, R.numChannel) == E.V.shape[:3]
    assert np.array_equal(R.V, E.V)      # same summation order: bit-identical
    compare_sets(R, E, "avgpool")


def test_avgpool_known_answer_and_errors(nnv):
    # tests/nn/layers/AveragePooling2DLayer/test_layers_averagePooling.m:14-23 as a one-point set
    I = np.array([[1, 0, 2, 3], [4, 6, 6, 8], [3, 1, 1, 0], [1, 2, 2, 4]], dtype=float)
    S = nnv.ImageStar(I, I)
    R = nnv.AveragePooling2DLayer([2, 2], [2, 2], [0, 0, 0, 0]).reach(S, "approx-star")
    assert np.array_equal(R.V[:, :, 0, 0], [[11 / 4, 19 / 4], [7 / 4, 7 / 4]])
    with pytest.raises(TypeError, match="The input is not an ImageStar object"):
        nnv.AveragePooling2DLayer().reach(nnv.Star([0.0], [1.0]), "approx-star")
    with pytest.raises(ValueError, match="Invalid pool size"):
        nnv.AveragePooling2DLayer([2, 2, 2], [1, 1], [0, 0, 0, 0])


@pytest.mark.parametrize("ftype", ["nnet.cnn.layer.FlattenLayer", "nnet.keras.layer.FlattenCStyleLayer",
                                   "nnet.onnx.layer.FlattenLayer"])
@pytest.mark.parametrize("H,W,C,n", [(2, 2, 2, 3), (7, 5, 3, 20), (16, 16, 32, 100)])
def test_flatten(nnv, ftype, H, W, C, n):
    rs = np.random.RandomState(H + W + C)
    D, O = _pair(nnv, rs, H, W, C, n)
    R = nnv.FlattenLayer("flat", ftype).reach(D, "relax-star-area")
    E = o.flatten_reach(O, ftype)
    assert (R.height, R.width, R.numChannel) == (1, 1, H * W * C)
    assert np.array_equal(R.V, E.V)
    compare_sets(R, E, "flatten")
    S = nnv.Star([0.0, 1.0], [1.0, 2.0])
    assert nnv.FlattenLayer("flat", ftype).reach(S, "approx-star") is S
    with pytest.raises(ValueError, match="Unknown type of flatten layer"):
        nnv.FlattenLayer("flat", "other").reach(D, "approx-star")


@pytest.mark.parametrize("nrm,kw", [("none", {}), ("zerocenter", {"mean": "image"}), ("zerocenter", {"mean": "channel"}),
                                    ("zscore", {"mean": "channel", "std": True}),
                                    ("rescale-zero-one", {}), ("rescale-zero-one", {"mn": -2.0, "mx": 6.0}),
                                    ("rescale-symmetric", {}), ("rescale-symmetric", {"mn": -2.0, "mx": 6.0})])
def test_image_input_layer(nnv, nrm, kw):
    rs = np.random.RandomState(11)
    H, W, C, n = 6, 5, 3, 9
    D, O = _pair(nnv, rs, H, W, C, n)
    mean = rs.randn(H, W, C) if kw.get("mean") == "image" else rs.randn(1, 1, C) if kw.get("mean") else None
    std = rs.rand(C) + 0.5 if kw.get("std") else None
    L = nnv.ImageInputLayer("in", [H, W, C], nrm, "auto", mean, std, kw.get("mn"), kw.get("mx"))
    R = L.reach(D, "relax-star-area")
    E = o.image_input_reach(O, nrm, mean, std, kw.get("mn"), kw.get("mx"))
    assert np.array_equal(R.V, E.V)
    compare_sets(R, E, "imageinput " + nrm)
    with pytest.raises(TypeError, match="Input is not an ImageStar"):
        L.reach(nnv.Star([0.0], [1.0]), "approx-star")


def test_image_star_affine_map(nnv):
    rs = np.random.RandomState(12)
    D, O = _pair(nnv, rs, 5, 4, 3, 6)
    for scale, offset in ((2.5, None), (rs.randn(1, 1, 3), rs.randn(1, 1, 3)), (None, rs.randn(5, 4, 3)), (None, None)):
        R = D.affineMap(scale, offset)
        E = o.image_star_affine_map(O, scale, offset)
        assert np.array_equal(R.V, E.V)
    with pytest.raises(ValueError, match="Inconsistent number of channels"):
        D.affineMap(rs.randn(1, 1, 2), None)


def test_layers_wrapper(nnv):
    rs = np.random.RandomState(13)
    W, b = rs.randn(20, 6), rs.randn(20)
    lbv, ubv = -rs.rand(6), rs.rand(6)
    for f in ("purelin", "poslin"):
        R = nnv.LayerS(W, b, f).reach(nnv.Star(lbv, ubv), "relax-star-area", None, 1)
        E = o.layers_reach(o.star_from_box(lbv, ubv), W, b, f, "relax-star-area")
        compare_sets(R, E, "LayerS " + f)
    with pytest.raises(ValueError, match="Unknown reachability analysis method"):
        nnv.LayerS(W, b, "poslin").reach(nnv.Star(lbv, ubv), "nonsense")
    with pytest.raises(ValueError, match="Inconsistent dimensions"):
        nnv.LayerS(W, b[:5], "poslin")


@pytest.mark.parametrize("method", ["relax-star-area", "relax-star-random"])
def test_cnn_with_all_layers_end_to_end(nnv, method):
    cfg = make_extended_cnn(16, 3)
    dev_in, ora_in = input_sets(cfg)
    net = nnv.NN.from_config(cfg["layers"], cfg["name"])
    dev = net.reach(dev_in, {"reachMethod": method, "relaxFactor": 1})
    ora, ora_sets = o.nn_reach(cfg["layers"], ora_in, method, 1.0, keep=True)
    prev = ora_in
    for li, (L, ds, os_) in enumerate(zip(cfg["layers"], net.reachSet, ora_sets)):
        tag = "layer %d (%s)" % (li + 1, L["type"])
        if L["type"] == "relu":
            ps = prev.to_star() if isinstance(prev, o.OImageStar) else prev
            lb, ub = o.estimate_ranges(ps)
            m1, m2 = o.relax_classify(lb, ub, method)
            ni, idx, _, _ = ds.relu_info()
            assert ni == m1.size and np.array_equal(idx, m2), tag
        compare_sets(ds, os_, tag, check_constraints=False)
        prev = os_
    compare_sets(dev, ora, "output", check_constraints=True)
    # containment of sampled concrete outputs in the reported bounds
    lb, ub = dev.estimateRanges()
    rs = np.random.RandomState(0)
    for _ in range(5):
        x = (cfg["lb"] + (cfg["ub"] - cfg["lb"]) * rs.rand(cfg["lb"].size)).reshape(cfg["image_shape"], order="F")
        y = o.evaluate(cfg["layers"], x).reshape(-1)
        assert np.all(y >= lb.reshape(-1) - 1e-9) and np.all(y <= ub.reshape(-1) + 1e-9)


# ---- the reduceMem suffix of the ReLU layer (nn/layers/ReluLayer.m:107-146) -------------------------------
@pytest.mark.parametrize("H,W,C,n", [(6, 5, 1, 9), (4, 4, 3, 6), (28, 28, 1, 50)])
def test_relu_reduce_mem(nnv, H, W, C, n):
    rs = np.random.RandomState(H + 10 * C)
    D, O = _pair(nnv, rs, H, W, C, n)
    R = nnv.ReluLayer().reach(D, "relax-star-area-reduceMem", "single", 1)
    E = o.relu_layer_reach(O, "relax-star-area-reduceMem", 1.0)
    assert (R.height, R.width, R.numChannel) == (H, W, C)
    assert R.numPred == E.numPred
    # the box is built from the estimated ranges of the ReLU's output, which the device and the oracle sum in
    # different orders: values to rounding, structure (which entries are zero, generator order) exactly
    assert_close(R.V, E.V, "reduceMem V", 1e-12)
    assert np.array_equal(np.asarray(R.V) == 0, E.V == 0)
    assert np.array_equal(R.C, E.C) and np.array_equal(R.d, E.d)
    assert np.array_equal(R.pred_lb, E.pred_lb) and np.array_equal(R.pred_ub, E.pred_ub)
    assert_close(R.im_lb, E.im_lb, "im_lb", 1e-12)
    assert_close(R.im_ub, E.im_ub, "im_ub", 1e-12)
    # the set goes on through the network like any other
    Wt = rs.randn(3, 3, C, 2)
    conv = nnv.Conv2DLayer(Wt, rs.randn(2), [1, 1, 1, 1], [1, 1], [1, 1])
    R2 = conv.reach(R, "relax-star-area")
    E2 = o.conv2d_reach(E, Wt, conv.Bias, (1, 1, 1, 1), (1, 1), (1, 1))
    assert_close(R2.V, E2.V, "conv after reduceMem")


def test_relu_reduce_mem_degenerate_and_star_inputs(nnv):
    # every neuron inactive: the output is the zero set, l = u = 0, no predicate at all
    V = np.zeros((3, 3, 1, 3))
    V[..., 0] = -1.0
    V[..., 1] = 0.1
    D = nnv.ImageStar(V, np.zeros((1, 2)), np.zeros(1), -np.ones(2), np.ones(2))
    O = o.OImageStar(V, np.zeros((1, 2)), np.zeros(1), -np.ones(2), np.ones(2))
    R = nnv.ReluLayer().reach(D, "relax-star-range-reduceMem", "single", 1)
    E = o.relu_layer_reach(O, "relax-star-range-reduceMem", 1.0)
    assert R.numPred == E.numPred == 0
    assert np.array_equal(np.asarray(R.V), E.V)
    with pytest.raises(ValueError, match="This reachability method does not exist"):
        nnv.ReluLayer().reach(D.toStar(), "relax-star-area-reduceMem", "single", 1)
