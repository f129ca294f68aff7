"""Pins the oracle's restatements of the further affine layers (batch normalisation, average
pooling, flatten, input normalisation, LayerS) by the reference's known answers where it has any
and otherwise by what the mathematics fixes."""
import numpy as np
import pytest
import torch

from oracle import nnv_oracle as o


def _image_star(rs, H, W, C, n):
    V = rs.randn(H, W, C, n + 1)
    return o.OImageStar(V, np.zeros((1, n)), np.zeros(1), -np.ones(n), np.ones(n))


def _affine_consistent(reach, evaluate, I, tol=1e-12):
    """reach(I).c == evaluate(c) and reach(I).v_j == evaluate(c + v_j) - evaluate(c)."""
    R = reach(I)
    c = I.V[..., 0]
    yc = evaluate(c)
    assert np.allclose(R.V[..., 0].reshape(-1, order="F"), np.asarray(yc).reshape(-1, order="F"), rtol=0, atol=tol)
    for j in range(1, I.V.shape[-1]):
        yj = evaluate(c + I.V[..., j]) - yc
        assert np.allclose(R.V[..., j].reshape(-1, order="F"), np.asarray(yj).reshape(-1, order="F"), rtol=0, atol=tol)
    return R


def test_avgpool_reference_known_answers():
    # tests/nn/layers/AveragePooling2DLayer/test_layers_averagePooling.m:14-23
    I = np.array([[1, 0, 2, 3], [4, 6, 6, 8], [3, 1, 1, 0], [1, 2, 2, 4]], dtype=float)
    Y = o.avgpool2d_tensor(I[:, :, None, None], (2, 2), (2, 2), (0, 0, 0, 0))[:, :, 0, 0]
    assert np.array_equal(Y, [[(1 + 0 + 4 + 6) / 4, (2 + 3 + 6 + 8) / 4], [(3 + 1 + 1 + 2) / 4, (1 + 0 + 2 + 4) / 4]])
    # :41-56: 5x5x3 volume, 3x3 window, stride 2 -> window sums / 9 within 10 eps
    vol = np.zeros((5, 5, 3))
    vol[:, :, 0] = [[0, 0, 2, 0, 0], [1, 2, 0, 2, 0], [0, 0, 2, 2, 0], [0, 2, 2, 2, 2], [2, 2, 2, 1, 1]]
    vol[:, :, 1] = [[1, 2, 2, 1, 2], [2, 1, 2, 0, 2], [2, 2, 2, 0, 1], [1, 1, 1, 0, 0], [1, 0, 2, 2, 1]]
    vol[:, :, 2] = [[0, 0, 2, 2, 1], [0, 2, 1, 1, 2], [0, 2, 0, 0, 1], [0, 2, 1, 0, 1], [1, 2, 1, 0, 0]]
    y = o.avgpool2d_tensor(vol[:, :, :, None], (3, 3), (2, 2), (0, 0, 0, 0))[:, :, :, 0]
    assert y.shape == (2, 2, 3)
    for i in range(3):
        for j in range(2):
            for k in range(2):
                assert abs(y[j, k, i] - vol[2 * j:2 * j + 3, 2 * k:2 * k + 3, i].sum() / 9) <= 10 * np.finfo(float).eps
    # :94-101: a 28x28 image, pool [6 4], stride [4 4], padding [1 1 0 0] gives a 7x7 map
    assert o.avgpool2d_output_size(28, 28, (6, 4), (1, 1, 0, 0), (4, 4)) == (7, 7)


@pytest.mark.parametrize("pool,stride,pad", [((2, 2), (2, 2), (0, 0, 0, 0)), ((3, 3), (2, 2), (1, 1, 1, 1)),
                                             ((3, 2), (1, 2), (1, 0, 0, 1)), ((6, 4), (4, 4), (1, 1, 0, 0))])
def test_avgpool_border_rule_against_library(pool, stride, pad):
    # MatConvNet averages over the cells inside the image: sum-pool / count-pool of torch
    rs = np.random.RandomState(1)
    X = rs.randn(9, 8, 3, 2)
    Y = o.avgpool2d_tensor(X, pool, stride, pad)
    t = torch.from_numpy(np.ascontiguousarray(np.transpose(X, (3, 2, 0, 1))))
    padded = torch.nn.functional.pad(t, (pad[2], pad[3], pad[0], pad[1]))
    ones = torch.nn.functional.pad(torch.ones_like(t), (pad[2], pad[3], pad[0], pad[1]))
    ref = torch.nn.functional.avg_pool2d(padded, pool, stride) / torch.nn.functional.avg_pool2d(ones, pool, stride)
    assert np.allclose(Y, np.transpose(ref.numpy(), (2, 3, 1, 0)), rtol=0, atol=1e-14)


def test_avgpool_reach_is_evaluate_on_every_image():
    rs = np.random.RandomState(2)
    I = _image_star(rs, 7, 6, 2, 3)
    args = ((3, 2), (2, 1), (1, 0, 0, 1))
    _affine_consistent(lambda S: o.avgpool2d_reach(S, *args),
                       lambda x: o.avgpool2d_tensor(x[:, :, :, None], *args)[:, :, :, 0], I)
    with pytest.raises(TypeError):
        o.avgpool2d_reach(o.star_from_box([0.0], [1.0]), *args)


def test_batchnorm_formula_and_reach():
    rs = np.random.RandomState(3)
    mean, var, scale, offset, eps = rs.randn(3), rs.rand(3) + 0.1, rs.randn(3), rs.randn(3), 1e-5
    x = rs.randn(4, 5, 3)
    y = o.batchnorm_evaluate(x, mean, var, eps, scale, offset)
    ref = torch.nn.functional.batch_norm(torch.from_numpy(np.transpose(x, (2, 0, 1))[None]), torch.from_numpy(mean),
                                         torch.from_numpy(var), torch.from_numpy(scale), torch.from_numpy(offset),
                                         False, 0.0, eps)
    assert np.allclose(y, np.transpose(ref[0].numpy(), (1, 2, 0)), rtol=0, atol=1e-13)
    I = _image_star(rs, 4, 5, 3, 4)
    _affine_consistent(lambda S: o.batchnorm_reach(S, mean, var, eps, scale, offset),
                       lambda v: o.batchnorm_evaluate(v, mean, var, eps, scale, offset), I)
    # the reference's own test shape: mean 0.5, variance 0.1, unit scale (test_BatchNormalizationLayer.m:36-66)
    IS = o.image_star_from_bounds(np.arange(8.0).reshape(2, 2, 2) - 0.1, np.arange(8.0).reshape(2, 2, 2) + 0.1)
    R = o.batchnorm_reach(IS, [0.5, 0.5], [0.1, 0.1], 1e-5, [1, 1], [0, 0])
    assert np.allclose(R.V[:, :, :, 0], (np.arange(8.0).reshape(2, 2, 2) - 0.5) / np.sqrt(0.1 + 1e-5))
    # Star branch (:332-349): bias only on the centre
    S = o.OStar(rs.randn(3, 5), np.zeros((1, 4)), np.zeros(1), -np.ones(4), np.ones(4))
    RS = o.batchnorm_reach(S, mean, var, eps, scale, offset)
    l = scale / np.sqrt(var + eps)
    assert np.allclose(RS.V[:, 1:], S.V[:, 1:] * l[:, None]) and np.allclose(RS.V[:, 0], S.V[:, 0] * l + offset - mean * l)


def test_flatten_orders_by_hand():
    IM = np.zeros((2, 2, 2))
    IM[:, :, 0] = [[1, 2], [3, 4]]
    IM[:, :, 1] = [[5, 6], [7, 8]]
    # MATLAB reshape: column-major; Keras: permute [3 2 1] first (channel fastest, then column, then row);
    # ONNX: permute [2 1 3] (row-major inside each channel)
    assert o.flatten_evaluate(IM, "nnet.cnn.layer.FlattenLayer").reshape(-1).tolist() == [1, 3, 2, 4, 5, 7, 6, 8]
    assert o.flatten_evaluate(IM, "nnet.keras.layer.FlattenCStyleLayer").reshape(-1).tolist() == [1, 5, 2, 6, 3, 7, 4, 8]
    assert o.flatten_evaluate(IM, "nnet.onnx.layer.FlattenLayer").reshape(-1).tolist() == [1, 2, 3, 4, 5, 6, 7, 8]
    assert o.flatten_evaluate(IM, "nnet.cnn.layer.FlattenLayer").shape == (1, 1, 8)   # test_FlattenLayer.m:38-50
    with pytest.raises(ValueError):
        o.flatten_evaluate(IM, "something else")
    rs = np.random.RandomState(4)
    I = _image_star(rs, 3, 4, 2, 3)
    for t in ("nnet.cnn.layer.FlattenLayer", "nnet.keras.layer.FlattenCStyleLayer", "nnet.onnx.layer.FlattenInto2dLayer"):
        R = _affine_consistent(lambda S: o.flatten_reach(S, t), lambda v: o.flatten_evaluate(v, t), I)
        assert (R.height, R.width, R.numChannel) == (1, 1, 24)      # test_FlattenLayer.m:104-112
        for j in range(4):  # a pure permutation: values are moved, never changed
            assert np.array_equal(R.V[0, 0, :, j], o.flatten_evaluate(I.V[:, :, :, j], t).reshape(-1))
    S = o.star_from_box([0.0, 1.0], [1.0, 2.0])
    assert o.flatten_reach(S, "nnet.cnn.layer.FlattenLayer") is S


@pytest.mark.parametrize("nrm,kw", [("none", {}), ("zerocenter", {"mean": "image"}), ("zerocenter", {"mean": "channel"}),
                                    ("zscore", {"mean": "channel", "std": True}),
                                    ("rescale-zero-one", {}), ("rescale-zero-one", {"mn": -2.0, "mx": 6.0}),
                                    ("rescale-symmetric", {}), ("rescale-symmetric", {"mn": -2.0, "mx": 6.0})])
def test_image_input_normalisations(nrm, kw):
    rs = np.random.RandomState(5)
    H, W, C = 4, 3, 2
    mean = rs.randn(H, W, C) if kw.get("mean") == "image" else rs.randn(1, 1, C) if kw.get("mean") else None
    std = rs.rand(C) + 0.5 if kw.get("std") else None
    I = _image_star(rs, H, W, C, 3)
    args = (nrm, mean, std, kw.get("mn"), kw.get("mx"))
    _affine_consistent(lambda S: o.image_input_reach(S, *args), lambda v: o.image_input_evaluate(v, *args), I)
    # closed forms
    x = rs.rand(H, W, C) * 255
    y = o.image_input_evaluate(x, *args)
    if nrm == "rescale-zero-one" and not kw:
        assert np.allclose(y, x / 255)
    if nrm == "rescale-symmetric" and kw:
        assert np.allclose(y, 2 * (x + 2.0) / 8.0 - 1)
    with pytest.raises(ValueError):
        o.image_input_evaluate(x, "whiten")


def test_layers_wrapper():
    rs = np.random.RandomState(6)
    W, b = rs.randn(4, 3), rs.randn(4)
    S = o.star_from_box(-np.ones(3), np.ones(3))
    lin = o.layers_reach(S, W, b, "purelin", "relax-star-area")
    assert np.array_equal(lin.V, o.affine_map(S, W, b).V)
    rel = o.layers_reach(S, W, b, "poslin", "relax-star-area")
    ref = o.reach_relaxed_star(o.affine_map(S, W, b), "relax-star-area", 1.0)
    assert np.array_equal(rel.V, ref.V) and np.array_equal(rel.C, ref.C)
    with pytest.raises(ValueError):
        o.layers_reach(S, W, b, "tansig", "relax-star-area")


# ---- the reduceMem suffix of the ReLU layer (nn/layers/ReluLayer.m:107-146) ---------------------------------
def test_reduce_mem_single_channel_is_the_box_of_the_ranges_in_pixel_row_order():
    """One channel: the statements build exactly ImageStar(l, u) of the estimated ranges, except that the
    generators come in row-major pixel order (i1 outer, i2 inner) instead of MATLAB's column-major one."""
    rs = np.random.RandomState(0)
    l = rs.rand(3, 4, 1) - 0.5
    u = l + rs.rand(3, 4, 1)
    u[1, 2, 0] = l[1, 2, 0]                     # a degenerate pixel: no generator, not counted
    I = o.image_star_from_bounds(l, u)
    I.im_lb = I.im_ub = None                    # (ranges are then recomputed from V: l, u up to rounding)
    R = o.relu_reduce_mem(I)
    rl, ru = o.image_star_estimate_ranges(I)
    assert R.numPred == 11 and R.V.shape == (3, 4, 1, 12)
    assert np.array_equal(R.V[..., 0], 0.5 * (ru + rl))
    order = [(i1, i2) for i1 in range(3) for i2 in range(4) if (i1, i2) != (1, 2)]
    for g, (i1, i2) in enumerate(order):
        col = R.V[..., 1 + g]
        assert col[i1, i2, 0] == 0.5 * (ru[i1, i2, 0] - rl[i1, i2, 0])
        assert np.count_nonzero(col) == 1
    assert np.array_equal(R.C, np.zeros((1, 11))) and np.array_equal(R.d, np.zeros(1))
    assert np.array_equal(R.pred_lb, -np.ones(11)) and np.array_equal(R.pred_ub, np.ones(11))
    assert R.im_lb is not None and np.array_equal(R.im_lb, rl) and np.array_equal(R.im_ub, ru)
    # closed form: the new set's own ranges are centre -/+ half-width
    R.im_lb = R.im_ub = None
    bl, bu = o.image_star_estimate_ranges(R)
    assert np.allclose(bl, rl, rtol=0, atol=1e-15) and np.allclose(bu, ru, rtol=0, atol=1e-15)


def test_reduce_mem_with_channels_follows_the_reference_statements():
    """Hand-written 2 x 1 x 2 case.  v(i1,i2) reads channel 1 only; its value goes to every channel of the pixel;
    n counts elements, so one generator per pixel is filled and the others stay zero."""
    l = np.array([[[0.0, -1.0]], [[2.0, 3.0]]])       # l(:,:,1) = [0; 2], l(:,:,2) = [-1; 3]
    u = np.array([[[4.0, 1.0]], [[2.0, 5.0]]])        # u(:,:,1) = [4; 2], u(:,:,2) = [ 1; 5]
    I = o.image_star_from_bounds(l, u)
    R = o.relu_reduce_mem(I)
    # l - u is non-zero for three elements -> n = 3; pixel (1,1): v = 2 -> generator 1 = 2 on both channels;
    # pixel (2,1): v(2,1) = 0 on channel 1 -> no generator although channel 2 has width 2
    assert R.numPred == 3
    exp = np.zeros((2, 1, 2, 4))
    exp[:, 0, 0, 0] = [2.0, 2.0]
    exp[:, 0, 1, 0] = [0.0, 4.0]
    exp[0, 0, :, 1] = 2.0
    assert np.array_equal(R.V, exp)


def test_reduce_mem_routing_by_set_type():
    rs = np.random.RandomState(1)
    lb = rs.rand(4, 4, 1) - 0.6
    I = o.image_star_from_bounds(lb, lb + 0.5)
    A = o.relu_layer_reach(I, "relax-star-area-reduceMem")
    B = o.relu_reduce_mem(o.relu_reach(I, "relax-star-area"))
    assert np.array_equal(A.V, B.V)
    with pytest.raises(ValueError, match="This reachability method does not exist"):
        o.relu_layer_reach(I.to_star(), "relax-star-area-reduceMem")
