"""Synthetic benchmark configurations for the relax-star reach path.

Five seeded network + input-set definitions.  All draws come from
``numpy.random.RandomState(1000 + k)`` (the frozen legacy MT19937 stream), in this order:
the input point ``x`` first (uniform), then for every affine layer in network order its
weight tensor (standard normal, filled in MATLAB column-major order, scaled by
sqrt(2 / fan_in)) followed by its bias (standard normal scaled by 0.1, i.e. variance 0.01).

Layer dictionaries use NNV's own array layouts:
  fc:   W is Out x In, b is Out                       (FullyConnectedLayer.Weights / .Bias)
  conv: W is FH x FW x Cin x Cout, b is Cout,
        padding [t b l r], stride [sh sw], dilation [dh dw]   (Conv2DLayer properties,
        code/nnv/engine/nn/layers/Conv2DLayer.m:15-33)
  relu: no parameters
"""
from __future__ import annotations

import numpy as np

BIAS_SIGMA = 0.1


def _fc(rs, n_out, n_in):
    W = rs.randn(n_out * n_in).reshape((n_out, n_in), order="F") * np.sqrt(2.0 / n_in)
    b = rs.randn(n_out) * BIAS_SIGMA
    return {"type": "fc", "W": W, "b": b}


def _conv(rs, fh, fw, cin, cout, stride, pad):
    fan_in = fh * fw * cin
    W = rs.randn(fh * fw * cin * cout).reshape((fh, fw, cin, cout), order="F") * np.sqrt(2.0 / fan_in)
    b = rs.randn(cout) * BIAS_SIGMA
    return {"type": "conv", "W": W, "b": b, "padding": [pad, pad, pad, pad],
            "stride": [stride, stride], "dilation": [1, 1]}


def _relu():
    return {"type": "relu"}


def conv_out_hw(h, w, layer):
    """Feature-map size, code/nnv/engine/nn/layers/Conv2DLayer.m:1134-1135."""
    fh, fw = layer["W"].shape[:2]
    t, b, l, r = layer["padding"]
    sh, sw = layer["stride"]
    dh, dw = layer["dilation"]
    ho = (h + t + b - (fh - 1) * dh - 1) // sh + 1
    wo = (w + l + r - (fw - 1) * dw - 1) // sw + 1
    return ho, wo


def fc_net(rs, widths):
    layers = []
    for i in range(len(widths) - 1):
        layers.append(_fc(rs, widths[i + 1], widths[i]))
        if i < len(widths) - 2:
            layers.append(_relu())
    return layers


def make_config(k: int, shrink: int = 1):
    """Return a dict {name, layers, kind, lb, ub[, image_shape][, partition]} for config k (1..5).

    ``shrink`` > 1 divides hidden widths / channel counts (and for k = 5 the number of
    bisected dimensions) so the CPU checker finishes in seconds; shrink = 1 is the full size.
    """
    rs = np.random.RandomState(1000 + k)
    if k == 1:
        c = rs.rand(5) - 0.5
        layers = fc_net(rs, [5] + [max(50 // shrink, 4)] * 6 + [5])
        return {"name": "cfg1_fc_5x50x6x5", "kind": "star", "layers": layers,
                "lb": c - 0.02, "ub": c + 0.02}
    if k in (2, 5):
        # config 5 reuses config 2's network and box (seed 1002)
        rs = np.random.RandomState(1002)
        n_in = 784 if shrink == 1 else max(784 // shrink, 16)
        hid = max(1024 // shrink, 8)
        x = rs.rand(n_in)
        layers = fc_net(rs, [n_in, hid, hid, hid, 10])
        cfg = {"name": "cfg2_fc_784_1024x3_10", "kind": "star", "layers": layers,
               "lb": x - 0.02, "ub": x + 0.02}
        if k == 5:
            ndim = 10 if shrink == 1 else max(2, 10 // shrink)
            cfg["name"] = "cfg5_bab_%d_boxes" % (2 ** ndim)
            # all widths are equal, so the "widest" dimensions are the first ones (stable order);
            # Box.partition order: first listed index varies slowest
            cfg["partition"] = {"indexes": list(range(ndim)), "numbers": [2] * ndim}
        return cfg
    if k == 3:
        hw = 28 if shrink == 1 else max(28 // shrink, 6)
        c1, c2, f = max(16 // shrink, 2), max(32 // shrink, 2), max(100 // shrink, 4)
        x = rs.rand(hw * hw)
        conv1 = _conv(rs, 3, 3, 1, c1, 1, 1)
        conv2 = _conv(rs, 3, 3, c1, c2, 2, 1)
        h1, w1 = conv_out_hw(hw, hw, conv1)
        h2, w2 = conv_out_hw(h1, w1, conv2)
        layers = [conv1, _relu(), conv2, _relu(), _fc(rs, f, h2 * w2 * c2), _relu(), _fc(rs, 10, f)]
        eps = 1.0 / 255.0
        return {"name": "cfg3_cnn_28x28x1", "kind": "image", "image_shape": (hw, hw, 1),
                "layers": layers, "lb": x - eps, "ub": x + eps}
    if k == 4:
        hw = 32 if shrink == 1 else max(32 // shrink, 10)
        ca, cb, f = max(32 // shrink, 2), max(64 // shrink, 2), max(512 // shrink, 4)
        x = rs.rand(hw * hw * 3)
        conv1 = _conv(rs, 3, 3, 3, ca, 1, 1)
        conv2 = _conv(rs, 3, 3, ca, ca, 2, 0)
        conv3 = _conv(rs, 3, 3, ca, cb, 1, 1)
        conv4 = _conv(rs, 3, 3, cb, cb, 2, 0)
        h, w = hw, hw
        for L in (conv1, conv2, conv3, conv4):
            h, w = conv_out_hw(h, w, L)
        layers = [conv1, _relu(), conv2, _relu(), conv3, _relu(), conv4, _relu(),
                  _fc(rs, f, h * w * cb), _relu(), _fc(rs, 10, f)]
        eps = 2.0 / 255.0
        return {"name": "cfg4_cnn_32x32x3", "kind": "image", "image_shape": (hw, hw, 3),
                "layers": layers, "lb": x - eps, "ub": x + eps}
    raise ValueError("config index must be 1..5")


def make_extended_cnn(hw=16, cin=3, seed=2001):
    """A CNN that strings together the further affine layers around the relax-star ReLU:
    ImageInputLayer (zscore) -> conv 3x3x8 -> BatchNormalization -> ReLU -> AveragePooling 2x2/2 ->
    conv 3x3x16 -> ReLU -> AveragePooling 3x3/2 pad 1 -> Flatten (Keras C-style) -> FC 32 -> ReLU -> FC 10."""
    rs = np.random.RandomState(seed)
    x = rs.rand(hw * hw * cin)
    c1, c2 = 8, 16
    conv1 = _conv(rs, 3, 3, cin, c1, 1, 1)
    bn = {"type": "batchnorm", "mean": 0.1 * rs.randn(c1), "var": rs.rand(c1) + 0.5, "eps": 1e-5,
          "scale": 1.0 + 0.1 * rs.randn(c1), "offset": 0.1 * rs.randn(c1)}
    pool1 = {"type": "avgpool", "pool": [2, 2], "stride": [2, 2], "padding": [0, 0, 0, 0]}
    conv2 = _conv(rs, 3, 3, c1, c2, 1, 1)
    pool2 = {"type": "avgpool", "pool": [3, 3], "stride": [2, 2], "padding": [1, 1, 1, 1]}
    h = hw // 2
    h2 = (h + 2 - 3) // 2 + 1
    flat = {"type": "flatten", "flatten_type": "nnet.keras.layer.FlattenCStyleLayer"}
    inp = {"type": "imageinput", "normalization": "zscore", "input_size": [hw, hw, cin],
           "mean": rs.rand(1, 1, cin), "std": 0.5 + rs.rand(cin)}
    layers = [inp, conv1, bn, _relu(), pool1, conv2, _relu(), pool2, flat,
              _fc(rs, 32, h2 * h2 * c2), _relu(), _fc(rs, 10, 32)]
    eps = 1.0 / 255.0
    return {"name": "cnn_with_norm_pool_flatten_%dx%dx%d" % (hw, hw, cin), "kind": "image", "image_shape": (hw, hw, cin),
            "layers": layers, "lb": x - eps, "ub": x + eps}


def count_updates(layer_shapes):
    """Generator-neuron updates of one reach: sum over layer steps of N_out * (n_out + 1)."""
    return int(sum(int(N) * (int(n) + 1) for (N, n) in layer_shapes))


def device_input_sets(cfg, ctx=None):
    """Input set(s) of a config on the device, built as NNV builds them: Star(lb, ub) /
    ImageStar(lb, ub) (set/Star.m:220-237, set/ImageStar.m:302-343), and for the partitioned
    config Box.partition (set/Box.m:96-139) followed by one Star per sub-box."""
    from .sets import Box, ImageStar, Star
    if "partition" in cfg:
        lbs, ubs = Box(cfg["lb"], cfg["ub"]).partition_bounds(cfg["partition"]["indexes"], cfg["partition"]["numbers"])
        return Star.from_boxes(lbs, ubs, ctx=ctx)
    if cfg["kind"] == "image":
        sh = cfg["image_shape"]
        return ImageStar(cfg["lb"].reshape(sh, order="F"), cfg["ub"].reshape(sh, order="F"), ctx=ctx)
    return Star(cfg["lb"], cfg["ub"], ctx=ctx)
