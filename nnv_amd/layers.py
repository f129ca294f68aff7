"""FullyConnectedLayer / Conv2DLayer / ReluLayer / PosLin with NNV's reach signatures.

``layer.reach(in_sets, method, option, relaxFactor, dis_opt, lp_solver)`` accepts one set or a
list of sets (NNV's set arrays) and returns the same; the whole array is processed by one batched
device call.  The ReLU offers the relax-star methods: at relaxFactor = 1 entirely on the device,
below 1 with the LPs of Star.getMaxs / getMins on the host, fed from the resident set.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from ._lib import ORDER_AREA, ORDER_INDEX, ORDER_RANGE, check, f64, ptr
from .sets import ImageStar, SetArray, Star, _Handle

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
    """(array of sets, whether a single set was given).  An array a layer returned stays as it is: its
    elements are only made into objects when somebody reads them."""
    if isinstance(sets, SetArray):
        return sets, False
    single = not isinstance(sets, (list, tuple))
    return ([sets] if single else list(sets)), single


def _handles_array(sets):
    if isinstance(sets, SetArray):
        return sets.handles()
    return (C.c_void_p * len(sets))(*[s._h.h for s in sets])


def _shapes(sets):
    """None when every set of the array is a Star; else one entry per set, None for a Star and
    (height, width, numChannel) for an ImageStar.  Anything else in the array is a TypeError."""
    if isinstance(sets, SetArray):
        return sets.shapes
    if all(type(s) is Star for s in sets):
        return None
    out = []
    for s in sets:
        if isinstance(s, ImageStar):
            out.append((s.height, s.width, s.numChannel))
        elif isinstance(s, Star):
            out.append(None)
        else:
            raise TypeError("not a Star or an ImageStar")
    return out


def _wrap_like(inputs, ctx, raw, out_shape=None):
    """The output array for the handles `raw`: a Star for a Star input, an ImageStar of `out_shape`
    (default: the input's own shape) for an ImageStar input."""
    if len(raw) == 1 and not isinstance(inputs, SetArray):   # one set: the object is wanted right away
        s, hd = inputs[0], _Handle(raw[0], ctx)
        if isinstance(s, ImageStar):
            return [ImageStar(_handle=hd, shape=out_shape or (s.height, s.width, s.numChannel))]
        return [Star._from_handle(hd)]
    shp = _shapes(inputs)
    if shp is not None and out_shape is not None:
        shp = [None if s is None else out_shape for s in shp]
    return SetArray(ctx, raw, shp)


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
        return _wrap_like(sets, ctx, out, (1, 1, W.shape[0]))

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
        if not len(inputs):
            return []
        try:
            shapes = _shapes(inputs)
        except TypeError:
            raise TypeError("Input set is not an ImageStar or Star") from None
        for shp in shapes or ():
            if shp is not None and shp[0] * shp[1] * shp[2] != self.InputSize:
                raise ValueError("Inconsistency between the size of the input image and the InputSize of the network")
        ctx = inputs.ctx if isinstance(inputs, SetArray) else inputs[0].ctx
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
        if not len(inputs):
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
        return _wrap_like(inputs, ctx, out, (ho, wo, self.NumFilters))

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
    def multipleStepReachStarApprox_at_one(I, index, lb, ub, reset=()):
        """PosLin.multipleStepReachStarApprox_at_one(I.resetRow(reset), index, lb, ub),
        nn/funcs/PosLin.m:685-742 with set/Star.m:1442-1461; all indices 0-based."""
        if not isinstance(I, Star):
            raise TypeError("Input is not a star")
        ctx = I.ctx
        reset = np.ascontiguousarray(np.asarray(reset).reshape(-1), dtype=np.int32)
        index = np.ascontiguousarray(np.asarray(index).reshape(-1), dtype=np.int32)
        lb, ub = f64(np.asarray(lb).reshape(-1)), f64(np.asarray(ub).reshape(-1))
        if lb.size != index.size or ub.size != index.size:
            raise ValueError("index, lb and ub must have the same length")
        out = (C.c_void_p * 1)()
        check(ctx.lib.nnvhip_relu_apply_lists(ctx.handle, I._h.h, reset.size, ptr(reset), index.size, ptr(index),
                                              ptr(lb), ptr(ub), out))
        return Star(_handle=_Handle(out[0], ctx))

    @staticmethod
    def reach_relaxed_star_lp(I, method, relaxFactor, option=None, dis_opt=None, lp_solver="linprog", rng=None):
        return _relaxed_star_lp(I, method, relaxFactor, option, dis_opt, lp_solver, rng)

    @staticmethod
    def reach(I, method="exact-star", option="parallel", relaxFactor=0, dis_opt=None, lp_solver="linprog"):
        """PosLin.reach, nn/funcs/PosLin.m:2073-2169."""
        sets, single = _as_list(I)
        if method in RELAX_ORDER:
            lazy = isinstance(sets, SetArray)
            if not (lazy and sets.shapes is None):
                for s in sets:
                    if not isinstance(s, Star):
                        raise TypeError("Input is not a star")
            if relaxFactor < 0 or relaxFactor > 1:
                raise ValueError("Invalid relax factor")
            if not len(sets):
                return []
            ctx = sets.ctx if lazy else sets[0].ctx
            if relaxFactor == 1:
                out = (C.c_void_p * len(sets))()
                check(ctx.lib.nnvhip_relu_relax(ctx.handle, RELAX_ORDER[method], float(relaxFactor), len(sets),
                                                _handles_array(sets), out))
                res = SetArray(ctx, out) if len(sets) > 1 or lazy else [Star._from_handle(_Handle(out[0], ctx))]
            else:
                # some bounds are tightened by LPs first: host LP solver fed from the resident set
                res = [PosLin.reach_relaxed_star_lp(s, method, relaxFactor, option, dis_opt, lp_solver) for s in sets]
            if dis_opt == "display" and relaxFactor == 1:
                for r in res:
                    ni, idx, _, _ = r.relu_info()
                    print("\n%d neurons with ub <= 0 are found by estimating ranges" % ni)
                    print("%d/%d neurons have lb < 0 & ub > 0" % (idx.size, r.dim))
                    print("Construct new star set, %d new predicate variables are introduced" % idx.size)
            return res[0] if single else res
        if method in ("exact-star", "exact-polyhedron", "approx-star", "approx-zono", "abs-dom"):
            raise NotImplementedError("only the relax-star methods are provided by this library (method '%s')" % method)
        raise ValueError("This reachability method does not exist")


def _matlab_round(x):
    return int(np.floor(x + 0.5))      # round(): halves away from zero, x >= 0 here


def _sort_descend(key):
    return np.argsort(-np.asarray(key), kind="stable")   # sort(..., 'descend') keeps ties in order


def _setdiff_stable(a, b):
    return a[~np.isin(a, b)] if len(b) else a


def _relaxed_star_lp(I, method, relaxFactor, option=None, dis_opt=None, lp_solver="linprog", rng=None):
    """The relaxFactor < 1 branches of PosLin.reach_relaxed_star_{range,area,bound,ub,random,static}
    (nn/funcs/PosLin.m:863-1650): n1 = round((1-relaxFactor)*#crossing) neurons, picked by the method's
    heuristic, get their upper (then lower) bound from an LP over the set's constraints; neurons whose
    optimised ub <= 0 are reset, those whose optimised lb >= 0 are left alone, and the rest go through
    the triangle relaxation with the tighter bounds.  Everything but the LPs runs on the device; the
    LPs get only the rows of V they need."""
    lb, ub = I.estimateRanges()
    map1 = np.flatnonzero(ub <= 0)
    map2 = np.flatnonzero((lb < 0) & (ub > 0))
    n1 = _matlab_round((1 - relaxFactor) * map2.size)
    N = map2.size
    if method in ("relax-star-range", "relax-star-area", "relax-star-random", "relax-star-static"):
        if method == "relax-star-range":            # PosLin.m:934-936
            midx = _sort_descend(ub[map2] - lb[map2])
            map21, map22 = map2[midx[:n1]], map2[midx[n1:]]
        elif method == "relax-star-area":           # :1049-1052
            midx = _sort_descend(0.5 * (np.abs(ub[map2]) * np.abs(lb[map2])))
            map21, map22 = map2[midx[:n1]], map2[midx[n1:]]
        elif method == "relax-star-random":         # :1488-1492 (randperm: not reproducible across libraries)
            rng = rng or np.random
            map21 = map2[rng.permutation(N)[:n1]]
            map22 = _setdiff_stable(map2, map21)
        else:                                       # :1604-1605
            map21, map22 = map2[:n1], map2[n1:]
        xmax = I.getMaxs(map21, option, dis_opt, lp_solver)
        map4 = map21[xmax <= 0]
        map11 = np.concatenate([map1, map4])
        map6, xmax1 = map21[xmax > 0], xmax[xmax > 0]
        xmin = I.getMins(map6, option, dis_opt, lp_solver)
        keep = xmin < 0
        index = np.concatenate([map22, map6[keep]])                     # map9
        lbs = np.concatenate([lb[map22], xmin[keep]])
        ubs = np.concatenate([ub[map22], xmax1[keep]])
    else:
        if method == "relax-star-bound":            # :1167-1176
            midx1 = _sort_descend(np.concatenate([ub[map2], np.abs(lb[map2])]))[:2 * n1]
            map21 = map2[midx1[midx1 < N]]
            map22 = map2[midx1[midx1 >= N] - N]
        else:                                       # relax-star-ub, :1326-1338
            midx_u = _sort_descend(ub[map2])
            midx_l = _sort_descend(np.abs(lb[map2]))
            if 2 * n1 <= N:
                map21, map22 = map2[midx_u[:2 * n1]], map2[:0]
            else:
                map21, map22 = map2[midx_u[:N]], map2[midx_l[:2 * n1 - N]]
        lb, ub = lb.copy(), ub.copy()
        map4 = map2[:0]
        if map21.size:
            xmax = I.getMaxs(map21, option, dis_opt, lp_solver)
            map4 = map21[xmax <= 0]
            ub[map21[xmax > 0]] = xmax[xmax > 0]
        map11 = np.concatenate([map1, map4])
        map23 = _setdiff_stable(map22, map4)
        map10 = map2[:0]
        if map23.size:
            xmin = I.getMins(map23, option, dis_opt, lp_solver)
            lb[map23[xmin < 0]] = xmin[xmin < 0]
            map10 = map23[xmin >= 0]
        index = _setdiff_stable(_setdiff_stable(map2, map4), map10)     # map24
        lbs, ubs = lb[index], ub[index]
    if dis_opt == "display":
        print("\n%d neurons with ub <= 0 are found by estimating ranges" % map1.size)
        print("(%d+%d =%d)/%d neurons have ub <= 0" % (map1.size, map4.size, map11.size, ub.size))
        print("%d/%d neurons have lb < 0 & ub > 0" % (index.size, ub.size))
        print("Construct new star set, %d new predicate variables are introduced" % index.size)
    return PosLin.multipleStepReachStarApprox_at_one(I, index, lbs, ubs, reset=map11)


def _reduce_mem(image):
    """nn/layers/ReluLayer.m:119-146: the box-like ImageStar of the set's estimated ranges, built on the device."""
    ctx = image.ctx
    h, w, c = image.height, image.width, image.numChannel
    out = (C.c_void_p * 1)()
    lb = np.empty(h * w * c)
    ub = np.empty(h * w * c)
    check(ctx.lib.nnvhip_relu_reduce_mem(ctx.handle, image._h.h, h, w, c, out, ptr(lb), ptr(ub)))
    res = ImageStar(_handle=_Handle(C.c_void_p(out[0]), ctx), shape=(h, w, c))
    res.im_lb = lb.reshape((h, w, c), order="F")
    res.im_ub = ub.reshape((h, w, c), order="F")
    return res


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
        reduce_mem = "reduceMem" in method
        if reduce_mem:
            # nn/layers/ReluLayer.m:107-112: the suffix is split off for ImageStars only; a Star hands the whole
            # string to PosLin.reach, which does not know it
            in_images = list(in_images)
            if any(isinstance(s, Star) and not isinstance(s, ImageStar) for s in in_images):
                raise ValueError("This reachability method does not exist")
            method = "-".join(method.split("-")[:-1])
        if isinstance(in_images, SetArray) and method in RELAX_ORDER and relaxFactor == 1 and dis_opt != "display":
            # an array straight from the previous layer: no object per set is needed
            ctx, shapes = in_images.ctx, in_images.shapes
            out = (C.c_void_p * len(in_images))()
            if len(in_images):
                check(ctx.lib.nnvhip_relu_relax(ctx.handle, RELAX_ORDER[method], 1.0, len(in_images), in_images.handles(), out))
            return SetArray(ctx, out, None if shapes is None else list(shapes))
        for s in in_images:
            if not isinstance(s, (Star, ImageStar)):
                raise TypeError("input is not an ImageStar, Star or VolumeStar")
        stars = [s.toStar() if isinstance(s, ImageStar) else s for s in in_images]
        res = PosLin.reach(stars, method, None, relaxFactor, dis_opt, lp_solver) if stars else []
        out = []
        for s, r in zip(in_images, res):
            o = r.toImageStar(s.height, s.width, s.numChannel) if isinstance(s, ImageStar) else r
            out.append(_reduce_mem(o) if reduce_mem else o)
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
