"""FullyConnectedLayer / Conv2DLayer / ReluLayer / PosLin with NNV's reach signatures.

``layer.reach(in_sets, method, option, relaxFactor, dis_opt, lp_solver)`` accepts one set or a
list of sets (NNV's set arrays) and returns the same; the whole array is processed by one batched
device call.  Only the relax-star methods at relaxFactor = 1 are available for the ReLU.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from ._lib import ORDER_AREA, ORDER_INDEX, ORDER_RANGE, check, f64, ptr
from .sets import ImageStar, Star, _Handle

RELAX_ORDER = {
    "relax-star-range": ORDER_RANGE,   # nn/funcs/PosLin.m:934-936
    "relax-star-area": ORDER_AREA,     # :1049-1052
    "relax-star-bound": ORDER_INDEX,   # :1167-1232
    "relax-star-ub": ORDER_INDEX,      # :1326-1397
    "relax-star-random": ORDER_INDEX,  # :1488-1492
    "relax-star-static": ORDER_INDEX,  # :1604-1605
}
_AFFINE_STAR_METHODS = ("approx-star", "exact-star", "abs-dom")


def _as_list(sets):
    single = not isinstance(sets, (list, tuple))
    return ([sets] if single else list(sets)), single


def _handles_array(sets):
    arr = (C.c_void_p * len(sets))()
    for i, s in enumerate(sets):
        arr[i] = s._h.h
    return arr


def _wrap_like(inputs, ctx, raw, shape_fn=None):
    outs = []
    for s, h in zip(inputs, raw):
        hd = _Handle(h, ctx)
        if isinstance(s, ImageStar):
            outs.append(ImageStar(_handle=hd, shape=shape_fn(s)))
        else:
            outs.append(Star(_handle=hd))
    return outs


class FullyConnectedLayer:
    """nn/layers/FullyConnectedLayer.m: y = W*x + b."""

    def __init__(self, *args):
        if len(args) == 3:
            name, W, b = args
            if not isinstance(name, str):
                raise ValueError("Name is not char")
        elif len(args) == 2:
            W, b = args
            name = "fully_connected_layer"
        else:
            raise ValueError("Invalid number of inputs (should be 0, 2 or 3)")
        W = np.asarray(W, dtype=np.float64)
        b = np.asarray(b, dtype=np.float64)
        if b.ndim == 2 and b.shape[1] != 1:
            raise ValueError("Bias vector should have one column")
        b = b.reshape(-1)
        if W.ndim != 2 or W.shape[0] != b.shape[0]:
            raise ValueError("Inconsistent dimension between the weight matrix and bias vector")
        self.Name = name
        self.Weights = W
        self.Bias = b
        self.InputSize = W.shape[1]
        self.OutputSize = W.shape[0]
        self._dev = {}

    def evaluate(self, x):
        return self.Weights @ np.asarray(x, dtype=np.float64).reshape(-1, order="F") + self.Bias

    class _Weights:
        def __init__(self, ctx, W, b):
            self.ctx = ctx
            h = C.c_void_p()
            Wf = f64(W)
            bf = None if b is None else f64(b)
            check(ctx.lib.nnvhip_fc_create(ctx.handle, ptr(Wf), ptr(bf), W.shape[0], W.shape[1], C.byref(h)))
            self.h = h

        def __del__(self):
            try:
                self.ctx.lib.nnvhip_fc_destroy(self.h)
            except Exception:
                pass

    @staticmethod
    def _map(ctx, W, b, sets, weights=None):
        weights = weights or FullyConnectedLayer._Weights(ctx, W, b)
        out = (C.c_void_p * len(sets))()
        check(ctx.lib.nnvhip_affine_fc(ctx.handle, weights.h, len(sets), _handles_array(sets), out))
        return _wrap_like(sets, ctx, out, lambda s: (1, 1, W.shape[0]))

    def _weights(self, ctx):
        if ctx not in self._dev:
            self._dev[ctx] = FullyConnectedLayer._Weights(ctx, self.Weights, self.Bias)
        return self._dev[ctx]

    def reach_star_single_input(self, in_image):
        return self.reach_star_multipleInputs([in_image], None)[0]

    def reach_star_multipleInputs(self, inputs, option=None):
        """nn/layers/FullyConnectedLayer.m:295-316, 476-512."""
        if option not in (None, "", "single", "parallel") and not (isinstance(option, (list, tuple)) and len(option) == 0):
            raise ValueError("Unknown computation option, should be parallel or single")
        if not inputs:
            return []
        for s in inputs:
            if not isinstance(s, (Star, ImageStar)):
                raise TypeError("Input set is not an ImageStar or Star")
            if isinstance(s, ImageStar) and s.height * s.width * s.numChannel != self.InputSize:
                raise ValueError("Inconsistency between the size of the input image and the InputSize of the network")
        ctx = inputs[0].ctx
        return FullyConnectedLayer._map(ctx, self.Weights, self.Bias, inputs, self._weights(ctx))

    def reach(self, in_images, method="approx-star", option=None, relaxFactor=0, dis_opt=None, lp_solver="linprog"):
        """nn/layers/FullyConnectedLayer.m:162-220 (arguments after `option` are ignored)."""
        sets, single = _as_list(in_images)
        if method in _AFFINE_STAR_METHODS or "relax-star" in method:
            out = self.reach_star_multipleInputs(sets, option)
        elif method == "approx-zono":
            raise NotImplementedError("zonotope reachability is outside this library")
        else:
            raise ValueError("Unknown reachability method")
        return out[0] if single else out


class Conv2DLayer:
    """nn/layers/Conv2DLayer.m: cross-correlation, weights FH x FW x Cin x Cout, padding [t b l r]."""

    def __init__(self, *args):
        name = "convolutional_2d_layer"
        padding, stride, dilation = [0, 0, 0, 0], [1, 1], [1, 1]
        if len(args) == 2:
            W, b = args
        elif len(args) == 5:
            W, b, padding, stride, dilation = args
        elif len(args) == 6:
            name, W, b, padding, stride, dilation = args
            if not isinstance(name, str):
                raise ValueError("Layer name should be a char array")
        else:
            raise ValueError("Invalid number of inputs (should be 2, 5, or 6)")
        W = np.asarray(W, dtype=np.float64)
        if W.ndim == 2:
            W = W[:, :, None, None]
        elif W.ndim == 3:
            W = W[:, :, :, None]
        if W.ndim != 4:
            raise ValueError("Invalid weights array")
        b = np.asarray(b, dtype=np.float64).reshape(-1)
        if b.size != W.shape[3]:
            raise ValueError("Inconsistency between filter weights and filter biases")
        padding = [int(x) for x in np.asarray(padding).reshape(-1)]
        if len(padding) == 1:
            padding = padding * 4
        if len(padding) != 4:
            raise ValueError("Invalid padding matrix")
        stride = [int(x) for x in np.asarray(stride).reshape(-1)]
        if len(stride) == 1:
            stride = stride * 2
        if len(stride) != 2:
            raise ValueError("Invalid stride matrix")
        dilation = [int(x) for x in np.asarray(dilation).reshape(-1)]
        if len(dilation) == 1:
            dilation = dilation * 2
        if len(dilation) != 2:
            raise ValueError("Invalid dilation matrix")
        self.Name = name
        self.Weights = W
        self.Bias = b
        self.FilterSize = [W.shape[0], W.shape[1]]
        self.NumChannels = W.shape[2]
        self.NumFilters = W.shape[3]
        self.PaddingSize = padding
        self.Stride = stride
        self.DilationFactor = dilation
        self._dev = {}

    class _Weights:
        def __init__(self, ctx, layer):
            self.ctx = ctx
            h = C.c_void_p()
            W = f64(layer.Weights)
            b = f64(layer.Bias)
            I64x4 = C.c_int64 * 4
            I64x2 = C.c_int64 * 2
            check(ctx.lib.nnvhip_conv2d_create(ctx.handle, ptr(W), ptr(b), W.shape[0], W.shape[1], W.shape[2],
                                               W.shape[3], I64x4(*layer.PaddingSize), I64x2(*layer.Stride),
                                               I64x2(*layer.DilationFactor), C.byref(h)))
            self.h = h

        def __del__(self):
            try:
                self.ctx.lib.nnvhip_conv2d_destroy(self.h)
            except Exception:
                pass

    def _weights(self, ctx):
        if ctx not in self._dev:
            self._dev[ctx] = Conv2DLayer._Weights(ctx, self)
        return self._dev[ctx]

    def output_size(self, H, W):
        """Feature-map size, nn/layers/Conv2DLayer.m:1134-1135."""
        t, b, l, r = self.PaddingSize
        ho = (H + t + b - (self.FilterSize[0] - 1) * self.DilationFactor[0] - 1) // self.Stride[0] + 1
        wo = (W + l + r - (self.FilterSize[1] - 1) * self.DilationFactor[1] - 1) // self.Stride[1] + 1
        return ho, wo

    def reach_star_single_input(self, inp):
        return self.reach_star_multipleInputs([inp], "single")[0]

    def reach_star_multipleInputs(self, inputs, option="single"):
        """nn/layers/Conv2DLayer.m:559-601, 780, 862-886."""
        if option not in (None, "", "single", "parallel") and not (isinstance(option, (list, tuple)) and len(option) == 0):
            raise ValueError("Unknown computation option")
        if not inputs:
            return []
        for s in inputs:
            if not isinstance(s, ImageStar):
                raise TypeError("The input is not an ImageStar object")
            if s.numChannel != self.NumChannels:
                raise ValueError("Input set contains %d channels while the convolutional layers has %d channels"
                                 % (s.numChannel, self.NumChannels))
            if (s.height, s.width) != (inputs[0].height, inputs[0].width):
                raise ValueError("sets of one array must have the same image size")
        ctx = inputs[0].ctx
        H, W = inputs[0].height, inputs[0].width
        ho, wo = self.output_size(H, W)
        out = (C.c_void_p * len(inputs))()
        check(ctx.lib.nnvhip_affine_conv2d(ctx.handle, self._weights(ctx).h, H, W, len(inputs),
                                           _handles_array(inputs), out))
        return _wrap_like(inputs, ctx, out, lambda s: (ho, wo, self.NumFilters))

    def reach(self, in_images, method="approx-star", option="single", relaxFactor=0, dis_opt=None, lp_solver="linprog"):
        """nn/layers/Conv2DLayer.m:913-973."""
        sets, single = _as_list(in_images)
        if method in _AFFINE_STAR_METHODS or "relax-star" in method:
            out = self.reach_star_multipleInputs(sets, option)
        elif method == "approx-zono":
            raise NotImplementedError("zonotope reachability is outside this library")
        else:
            raise ValueError("Unknown reachability method")
        return out[0] if single else out


class PosLin:
    """nn/funcs/PosLin.m: the ReLU activation's reachability dispatcher (relax-star branches)."""

    @staticmethod
    def evaluate(x):
        return np.maximum(np.asarray(x, dtype=np.float64), 0)

    @staticmethod
    def reach(I, method="exact-star", option="parallel", relaxFactor=0, dis_opt=None, lp_solver="linprog"):
        """PosLin.reach, nn/funcs/PosLin.m:2073-2169."""
        sets, single = _as_list(I)
        if method in RELAX_ORDER:
            for s in sets:
                if not isinstance(s, Star):
                    raise TypeError("Input is not a star")
            if relaxFactor < 0 or relaxFactor > 1:
                raise ValueError("Invalid relax factor")
            if not sets:
                return []
            ctx = sets[0].ctx
            out = (C.c_void_p * len(sets))()
            check(ctx.lib.nnvhip_relu_relax(ctx.handle, RELAX_ORDER[method], float(relaxFactor), len(sets),
                                            _handles_array(sets), out))
            res = [Star(_handle=_Handle(h, ctx)) for h in out]
            if dis_opt == "display":
                for r in res:
                    ni, idx, _, _ = r.relu_info()
                    print("\n%d neurons with ub <= 0 are found by estimating ranges" % ni)
                    print("%d/%d neurons have lb < 0 & ub > 0" % (idx.size, r.dim))
                    print("Construct new star set, %d new predicate variables are introduced" % idx.size)
            return res[0] if single else res
        if method in ("exact-star", "exact-polyhedron", "approx-star", "approx-zono", "abs-dom"):
            raise NotImplementedError("only the relax-star methods are provided by this library (method '%s')" % method)
        raise ValueError("This reachability method does not exist")


class ReluLayer:
    """nn/layers/ReluLayer.m (+ ActivationFunctionLayer.m:108-172)."""

    def __init__(self, name="relu_layer"):
        self.Name = name

    def evaluate(self, x):
        return PosLin.evaluate(x)

    def reach_star_single_input(self, in_image, method, relaxFactor, dis_opt=None, lp_solver="linprog"):
        return self.reach_star_multipleInputs([in_image], method, None, relaxFactor, dis_opt, lp_solver)[0]

    def reach_star_multipleInputs(self, in_images, method, option, relaxFactor, dis_opt=None, lp_solver="linprog"):
        """nn/layers/ReluLayer.m:72-150, ActivationFunctionLayer.m:57-83: ImageStars go through
        toStar -> PosLin.reach -> toImageStar, which on the device is the same memory."""
        if option not in (None, "", "single", "parallel") and not (isinstance(option, (list, tuple)) and len(option) == 0):
            raise ValueError("Unknown computation option")
        for s in in_images:
            if not isinstance(s, (Star, ImageStar)):
                raise TypeError("input is not an ImageStar, Star or VolumeStar")
        if "reduceMem" in method:
            raise NotImplementedError("the reduceMem variants are outside this library")
        stars = [s.toStar() if isinstance(s, ImageStar) else s for s in in_images]
        res = PosLin.reach(stars, method, None, relaxFactor, dis_opt, lp_solver) if stars else []
        out = []
        for s, r in zip(in_images, res):
            out.append(r.toImageStar(s.height, s.width, s.numChannel) if isinstance(s, ImageStar) else r)
        return out

    def reach(self, in_images, method, option="single", relaxFactor=0, dis_opt=None, lp_solver="linprog"):
        """ActivationFunctionLayer.reach, nn/layers/ActivationFunctionLayer.m:108-172."""
        sets, single = _as_list(in_images)
        if method in _AFFINE_STAR_METHODS or "relax-star" in method:
            out = self.reach_star_multipleInputs(sets, method, option, relaxFactor, dis_opt, lp_solver)
        elif method == "approx-zono":
            raise NotImplementedError("zonotope reachability is outside this library")
        else:
            raise ValueError("Unsupported reachability method")
        return out[0] if single else out
