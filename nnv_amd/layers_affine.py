"""Further affine layers of NNV's CNN pipelines with the reference's reach signatures:
BatchNormalizationLayer, AveragePooling2DLayer, FlattenLayer, ImageInputLayer and the legacy
LayerS wrapper.  Each is a single device pass over the generator matrix (or free, for reshapes)."""
from __future__ import annotations

import ctypes as C

import numpy as np

from ._lib import check, f64, ptr
from .layers import _AFFINE_STAR_METHODS, PosLin, _as_list, _handles_array, _wrap_like
from .sets import ImageStar, Star, _Handle

OP_ADD, OP_SUB, OP_MUL, OP_DIV = 0, 1, 2, 3
SCOPE_CENTRE, SCOPE_ALL = 0, 1


class RowMap:
    """A per-row affine program resident on the device (nnvhip_rowmap_create): a list of
    (op, scope, per-row operand) steps applied in order to the centre or to all columns."""

    def __init__(self, ctx, N, steps):
        self.ctx = ctx
        self.N = int(N)
        ops = np.asarray([s[0] for s in steps], dtype=np.int32)
        scopes = np.asarray([s[1] for s in steps], dtype=np.int32)
        params = f64(np.stack([np.broadcast_to(np.asarray(s[2], dtype=np.float64).reshape(-1), (self.N,)) for s in steps], axis=1))
        h = C.c_void_p()
        check(ctx.lib.nnvhip_rowmap_create(ctx.handle, self.N, len(steps), ptr(ops), ptr(scopes), ptr(params), C.byref(h)))
        self.h = h

    def __del__(self):
        try:
            self.ctx.lib.nnvhip_rowmap_destroy(self.h)
        except Exception:
            pass

    def apply(self, sets, out_shape=None):
        out = (C.c_void_p * len(sets))()
        check(self.ctx.lib.nnvhip_affine_rowmap(self.ctx.handle, self.h, len(sets), _handles_array(sets), out))
        return _wrap_like(sets, self.ctx, out, out_shape)


def _per_row(values, H, W, Cn):
    """Expand a scalar, a 1x1xC per-channel array or a full H x W x C image to the H*W*C rows of a
    flattened image (column-major: h fastest, then w, then channel)."""
    a = np.asarray(values, dtype=np.float64)
    if a.size == 1:
        return np.full(H * W * Cn, float(a.reshape(-1)[0]))
    if a.size == Cn and (a.ndim <= 1 or a.shape[:2] == (1, 1) or a.size == a.shape[-1]):
        return np.repeat(a.reshape(-1), H * W)
    if a.size == H * W * Cn:
        return a.reshape(-1, order="F")
    raise ValueError("Inconsistent number of channels between scale array and the ImageStar")


def image_star_affine_map(I: ImageStar, scale, offset) -> ImageStar:
    """ImageStar.affineMap(scale, offset), set/ImageStar.m:431-460."""
    H, W, Cn = I.height, I.width, I.numChannel
    steps = []
    if scale is not None and np.size(scale):
        if np.size(scale) not in (1, Cn):
            raise ValueError("Inconsistent number of channels between scale array and the ImageStar")
        steps.append((OP_MUL, SCOPE_ALL, _per_row(scale, H, W, Cn)))
    if offset is not None and np.size(offset):
        steps.append((OP_ADD, SCOPE_CENTRE, _per_row(offset, H, W, Cn)))
    if not steps:
        return ImageStar(_handle=I._h, shape=(H, W, Cn))
    return RowMap(I.ctx, H * W * Cn, steps).apply([I])[0]


ImageStar.affineMap = image_star_affine_map


class _RowMapLayer:
    """Shared plumbing: the row programme depends on the input's image shape, so it is built (and
    kept on the device) per (context, shape)."""

    def __init__(self):
        self._maps = {}

    def _steps(self, kind, H, W, Cn):
        raise NotImplementedError

    def _apply(self, sets):
        if not sets:
            return []
        first = sets[0]
        ctx = first.ctx
        if isinstance(first, ImageStar):
            key = (ctx, "image", first.height, first.width, first.numChannel)
            dims = (first.height, first.width, first.numChannel)
        else:
            key = (ctx, "star", first.dim)
            dims = (first.dim, 1, 1)
        for s in sets:
            same = (isinstance(s, ImageStar) and isinstance(first, ImageStar) and
                    (s.height, s.width, s.numChannel) == dims) or \
                   (isinstance(s, Star) and isinstance(first, Star) and s.dim == first.dim)
            if not same:
                raise ValueError("sets of one array must have the same image size")
        if key not in self._maps:
            steps = self._steps(key[1], *dims)
            self._maps[key] = RowMap(ctx, dims[0] * dims[1] * dims[2], steps) if steps else None
        m = self._maps[key]
        if m is None:
            return list(sets)
        return m.apply(sets)

    def _reach(self, in_images, method, option):
        if option not in (None, "", "single", "parallel") and not (isinstance(option, (list, tuple)) and len(option) == 0):
            raise ValueError("Unknown computation option")
        sets, single = _as_list(in_images)
        if method in _AFFINE_STAR_METHODS or "relax-star" in method:
            out = self.reach_star_multipleInputs(sets, option)
        elif method == "approx-zono":
            raise NotImplementedError("zonotope reachability is outside this library")
        else:
            raise ValueError("Unknown reachability method")
        return out[0] if single else out


class BatchNormalizationLayer(_RowMapLayer):
    """nn/layers/BatchNormalizationLayer.m: name/value constructor (:33-83)."""

    def __init__(self, **kw):
        super().__init__()
        self.Name = kw.get("Name", "BatchNormalizationLayer")
        self.NumChannels = kw.get("NumChannels")
        self.TrainedMean = None if kw.get("TrainedMean") is None else np.asarray(kw["TrainedMean"], dtype=np.float64)
        self.TrainedVariance = None if kw.get("TrainedVariance") is None else np.asarray(kw["TrainedVariance"], dtype=np.float64)
        self.Epsilon = float(kw.get("Epsilon", 0.00001))
        n = self.NumChannels if self.NumChannels is not None else (self.TrainedMean.size if self.TrainedMean is not None else 0)
        self.Offset = np.asarray(kw["Offset"], dtype=np.float64) if kw.get("Offset") is not None else np.zeros(n)
        self.Scale = np.asarray(kw["Scale"], dtype=np.float64) if kw.get("Scale") is not None else np.ones(n)
        if self.NumChannels is None:
            self.NumChannels = n

    def evaluate(self, x):
        """BatchNormalizationLayer.evaluate, :118-229."""
        x = np.asarray(x, dtype=np.float64)
        shp = (1, 1, -1) if x.ndim == 3 else x.shape
        m, v, s, o = (np.asarray(a, dtype=np.float64).reshape(shp) for a in
                      (self.TrainedMean, self.TrainedVariance, self.Scale, self.Offset))
        return s * ((x - m) / np.sqrt(v + self.Epsilon)) + o

    def _steps(self, kind, H, W, Cn):
        if self.TrainedMean is None or self.TrainedVariance is None:
            return []   # the reference leaves the set unchanged (:306, 331)
        if kind == "image":
            # :286-330, in this order: c - mean; all ./ sqrt(var + eps); all .* scale; c + offset
            return [(OP_SUB, SCOPE_CENTRE, _per_row(self.TrainedMean, H, W, Cn)),
                    (OP_DIV, SCOPE_ALL, _per_row(np.sqrt(self.TrainedVariance.reshape(-1) + self.Epsilon), H, W, Cn)),
                    (OP_MUL, SCOPE_ALL, _per_row(self.Scale, H, W, Cn)),
                    (OP_ADD, SCOPE_CENTRE, _per_row(self.Offset, H, W, Cn))]
        # Star, :332-349: l = scale ./ sqrt(var + eps); b = offset - mean .* l; V .* l; c + b
        l = self.Scale.reshape(-1) / np.sqrt(self.TrainedVariance.reshape(-1) + self.Epsilon)
        b = self.Offset.reshape(-1) - self.TrainedMean.reshape(-1) * l
        return [(OP_MUL, SCOPE_ALL, np.broadcast_to(l, (H,))), (OP_ADD, SCOPE_CENTRE, np.broadcast_to(b, (H,)))]

    def reach_star_single_input(self, in_image):
        return self.reach_star_multipleInputs([in_image], "single")[0]

    def reach_star_multipleInputs(self, in_images, option="single"):
        """:384-413."""
        for s in in_images:
            if not isinstance(s, (ImageStar, Star)):
                raise TypeError("Input is not a Star, ImageStar or VolumeStar")
        return self._apply(list(in_images))

    def reach(self, in_images, method="approx-star", option=None, relaxFactor=0, dis_opt=None, lp_solver="linprog"):
        """:498-556."""
        return self._reach(in_images, method, option)


class ImageInputLayer(_RowMapLayer):
    """nn/layers/ImageInputLayer.m: (InputSize[, Normalization]) or all eight properties (:16-40)."""

    def __init__(self, *args):
        super().__init__()
        self.Name = "ImageInputLayer"
        self.InputSize = []
        self.Normalization = "none"
        self.NormalizationDimension = "auto"
        self.Mean = self.StandardDeviation = self.Min = self.Max = None
        if len(args) == 1:
            self.InputSize = args[0]
        elif len(args) == 2:
            self.InputSize, self.Normalization = args
        elif len(args) == 8:
            (self.Name, self.InputSize, self.Normalization, self.NormalizationDimension, self.Mean,
             self.StandardDeviation, self.Min, self.Max) = args
        elif len(args) != 0:
            raise ValueError("Wrong number of inputs, it must be 0,1,2, or 8.")

    def evaluate(self, x):
        """:60-117."""
        x = np.asarray(x, dtype=np.float64)
        nrm = self.Normalization
        has_range = self.Min is not None and self.Max is not None
        if nrm == "none":
            return x
        if nrm == "zerocenter":
            return x - np.asarray(self.Mean, dtype=np.float64)
        if nrm == "zscore":
            return (x - np.asarray(self.Mean, dtype=np.float64)) / np.asarray(self.StandardDeviation, dtype=np.float64).reshape(1, 1, -1)
        if nrm == "rescale-zero-one":
            return (x - self.Min) / (self.Max - self.Min) if has_range else x / 255
        if nrm == "rescale-symmetric":
            return 2 * (x - self.Min) / (self.Max - self.Min) - 1 if has_range else 2 * x / 255 - 1
        raise ValueError("The normalization method is not supported yet.")

    def _steps(self, kind, H, W, Cn):
        """:121-166: each branch is a chain of ImageStar.affineMap calls and whole-V scalings."""
        nrm = self.Normalization
        has_range = self.Min is not None and self.Max is not None
        row = lambda a: _per_row(a, H, W, Cn)  # noqa: E731
        if nrm == "none":
            return []
        if nrm == "zerocenter":
            return [(OP_ADD, SCOPE_CENTRE, row(-np.asarray(self.Mean, dtype=np.float64)))]
        if nrm == "zscore":
            return [(OP_ADD, SCOPE_CENTRE, row(-np.asarray(self.Mean, dtype=np.float64))),
                    (OP_DIV, SCOPE_ALL, row(np.asarray(self.StandardDeviation, dtype=np.float64).reshape(-1)))]
        if nrm == "rescale-zero-one":
            if has_range:
                return [(OP_ADD, SCOPE_CENTRE, row(-np.float64(self.Min))),
                        (OP_MUL, SCOPE_ALL, row(1.0 / (np.float64(self.Max) - np.float64(self.Min))))]
            return [(OP_MUL, SCOPE_ALL, row(1 / 255))]
        if nrm == "rescale-symmetric":
            if has_range:
                return [(OP_ADD, SCOPE_CENTRE, row(-np.float64(self.Min))),
                        (OP_MUL, SCOPE_ALL, row(2.0 / (np.float64(self.Max) - np.float64(self.Min)))),
                        (OP_ADD, SCOPE_CENTRE, row(-1.0))]
            return [(OP_MUL, SCOPE_ALL, row(2 / 255)), (OP_ADD, SCOPE_CENTRE, row(-1.0))]
        raise ValueError("The normalization method is not supported yet.")

    def reach_star_single_input(self, in_image):
        return self.reach_star_multipleInputs([in_image], "single")[0]

    def reach_star_multipleInputs(self, in_images, option="single"):
        for s in in_images:
            if not isinstance(s, ImageStar):
                raise TypeError("Input is not an ImageStar")
        return self._apply(list(in_images))

    def reach(self, in_images, method="approx-star", option=None, relaxFactor=0, dis_opt=None, lp_solver="linprog"):
        return self._reach(in_images, method, option)


class AveragePooling2DLayer:
    """nn/layers/AveragePooling2DLayer.m: ([name,] poolSize [h w], stride [sh sw], padding [t b l r])."""

    def __init__(self, *args):
        self.Name = "average_pooling_2d_layer"
        pool, stride, padding = [2, 2], [1, 1], [0, 0, 0, 0]
        if len(args) == 4:
            self.Name, pool, stride, padding = args
            if not isinstance(self.Name, str):
                raise ValueError("Name is not char")
        elif len(args) == 3:
            pool, stride, padding = args
        elif len(args) != 0:
            raise ValueError("Invalid number of inputs (should be 0, 3 or 4)")
        pool, stride, padding = (np.asarray(a).reshape(-1) for a in (pool, stride, padding))
        if pool.size != 2:
            raise ValueError("Invalid pool size")
        if stride.size != 2:
            raise ValueError("Invalid stride")
        if padding.size != 4:
            raise ValueError("Invalide padding size")
        self.PoolSize = [int(x) for x in pool]
        self.Stride = [int(x) for x in stride]
        self.PaddingSize = [int(x) for x in padding]
        self._dev = {}

    class _Dev:
        def __init__(self, ctx, layer):
            self.ctx = ctx
            h = C.c_void_p()
            check(ctx.lib.nnvhip_avgpool2d_create(ctx.handle, (C.c_int64 * 2)(*layer.PoolSize), (C.c_int64 * 2)(*layer.Stride),
                                                  (C.c_int64 * 4)(*layer.PaddingSize), C.byref(h)))
            self.h = h

        def __del__(self):
            try:
                self.ctx.lib.nnvhip_avgpool2d_destroy(self.h)
            except Exception:
                pass

    def output_size(self, H, W):
        """get_size_averageMap, :396-418."""
        t, b, l, r = self.PaddingSize
        return (H + t + b - self.PoolSize[0]) // self.Stride[0] + 1, (W + l + r - self.PoolSize[1]) // self.Stride[1] + 1

    def reach_star_single_input(self, inp):
        return self.reach_star_multipleInputs([inp], "single")[0]

    def reach_star_multipleInputs(self, inputs, option="single"):
        """:424-463."""
        if option not in (None, "", "single", "parallel") and not (isinstance(option, (list, tuple)) and len(option) == 0):
            raise ValueError("Unknown computation option, should be parallel or single")
        if not inputs:
            return []
        for s in inputs:
            if not isinstance(s, ImageStar):
                raise TypeError("The input is not an ImageStar object")
            if (s.height, s.width, s.numChannel) != (inputs[0].height, inputs[0].width, inputs[0].numChannel):
                raise ValueError("sets of one array must have the same image size")
        ctx = inputs[0].ctx
        if ctx not in self._dev:
            self._dev[ctx] = AveragePooling2DLayer._Dev(ctx, self)
        H, W, Cn = inputs[0].height, inputs[0].width, inputs[0].numChannel
        ho, wo = self.output_size(H, W)
        out = (C.c_void_p * len(inputs))()
        check(ctx.lib.nnvhip_affine_avgpool2d(ctx.handle, self._dev[ctx].h, H, W, len(inputs), _handles_array(inputs), out))
        return _wrap_like(inputs, ctx, out, (ho, wo, Cn))

    def reach(self, in_images, method="approx-star", option="single", relaxFactor=0, dis_opt=None, lp_solver="linprog"):
        """:550-608."""
        sets, single = _as_list(in_images)
        if method in _AFFINE_STAR_METHODS or "relax-star" in method:
            out = self.reach_star_multipleInputs(sets, option)
        elif method == "approx-zono":
            raise NotImplementedError("zonotope reachability is outside this library")
        else:
            raise ValueError("Unknown reachability method")
        return out[0] if single else out


class FlattenLayer:
    """nn/layers/FlattenLayer.m; Type selects MATLAB-style (a reshape), Keras C-style or ONNX flatten."""

    ONNX_TYPES = ("nnet.onnx.layer.FlattenLayer", "nnet.onnx.layer.FlattenInto2dLayer", "nnet.onnx.layer.Flatten3dInto2dLayer")

    def __init__(self, name="FlattenLayer", Type=""):
        if not isinstance(name, str):
            raise ValueError("Invalid name, should be a charracter array")
        self.Name = name
        self.Type = Type

    def _source_rows(self, H, W, Cn):
        """Row r of the flattened image reads row source[r] of the column-major H x W x C image
        (None = identity).  :118-170."""
        idx = np.arange(H * W * Cn).reshape((H, W, Cn), order="F")
        if self.Type == "nnet.cnn.layer.FlattenLayer":
            return None
        if self.Type == "nnet.keras.layer.FlattenCStyleLayer":
            return np.transpose(idx, (2, 1, 0)).reshape(-1, order="F")
        if self.Type in FlattenLayer.ONNX_TYPES:
            return np.transpose(idx, (1, 0, 2)).reshape(-1, order="F")
        raise ValueError("Unknown type of flatten layer")

    def evaluate(self, image):
        image = np.asarray(image, dtype=np.float64)
        if image.ndim != 3:
            raise ValueError("Invalid input.")
        src = self._source_rows(*image.shape)
        flat = image.reshape(-1, order="F")
        return (flat if src is None else flat[src]).reshape(1, 1, -1)

    def reach_single_input(self, in_set):
        return self.reach_multipleInputs([in_set], "single")[0]

    def reach_multipleInputs(self, inputs, option="single"):
        """:178-199, 204-243: ImageStar H x W x C -> ImageStar 1 x 1 x N; Stars pass through."""
        if option not in (None, "", "single", "parallel") and not (isinstance(option, (list, tuple)) and len(option) == 0):
            raise ValueError("Unknown computation option, should be parallel or single")
        if not inputs:
            return []
        if isinstance(inputs[0], Star):
            return list(inputs)
        for s in inputs:
            if not isinstance(s, ImageStar):
                raise TypeError("Invalid input set (ImageStar, ImageZono or VolumeStar)")
            if (s.height, s.width, s.numChannel) != (inputs[0].height, inputs[0].width, inputs[0].numChannel):
                raise ValueError("sets of one array must have the same image size")
        H, W, Cn = inputs[0].height, inputs[0].width, inputs[0].numChannel
        N = H * W * Cn
        src = self._source_rows(H, W, Cn)
        if src is None:  # column-major reshape: the same device buffer
            return [ImageStar(_handle=s._h, shape=(1, 1, N)) for s in inputs]
        ctx = inputs[0].ctx
        src = np.ascontiguousarray(src, dtype=np.int32)
        out = (C.c_void_p * len(inputs))()
        check(ctx.lib.nnvhip_permute_rows(ctx.handle, N, ptr(src), len(inputs), _handles_array(inputs), out))
        return _wrap_like(inputs, ctx, out, (1, 1, N))

    def reach(self, in_images, method="approx-star", option="single", relaxFactor=0, dis_opt=None, lp_solver="linprog"):
        """:246-300."""
        sets, single = _as_list(in_images)
        if method in _AFFINE_STAR_METHODS or "relax-star" in method or method == "approx-zono":
            out = self.reach_multipleInputs(sets, option)
        else:
            raise ValueError("Unknown reachability method")
        return out[0] if single else out


class LayerS:
    """Legacy fully-connected layer with its activation, nn/layers/LayerS.m: LayerS(W, b, f)."""

    def __init__(self, W, b, f, gamma=0):
        W = np.asarray(W, dtype=np.float64)
        b = np.asarray(b, dtype=np.float64)
        if W.shape[0] != b.reshape(-1, 1).shape[0]:
            raise ValueError("Inconsistent dimensions between Weights matrix and bias vector")
        if gamma >= 1:
            raise ValueError("Invalid parameter for leakyReLU, gamma should be <= 1")
        from .layers import FullyConnectedLayer
        self.W, self.b, self.f, self.gamma = W, b.reshape(-1), f, gamma
        self.N = W.shape[0]
        self._fc = FullyConnectedLayer(W, self.b)

    def evaluate(self, x):
        y = self.W @ np.asarray(x, dtype=np.float64).reshape(-1) + self.b
        if self.f == "poslin":
            return np.maximum(y, 0)
        if self.f in ("purelin", "softmax"):
            return y
        raise ValueError("Unknown or unsupported activation function")

    def reach(self, I, method, option=None, relaxFactor=0, dis_opt=None, lp_solver="linprog"):
        """LayerS.reach, :120-262: affineMap(W, b) then the activation's reach."""
        known = ("exact-star", "approx-star", "approx-star-fast", "approx-zono", "abs-dom", "exact-polyhedron",
                 "approx-star-split", "approx-star-no-split", "approx-rstar-0", "approx-rstar-2", "approx-rstar-4")
        if method not in known and "relax-star" not in method:
            raise ValueError("Unknown reachability analysis method")
        sets, single = _as_list(I)
        mapped = self._fc.reach_star_multipleInputs(sets, option)
        if self.f in ("purelin", "softmax"):
            out = mapped
        elif self.f == "poslin":
            out = PosLin.reach(mapped, method, None, relaxFactor, dis_opt, lp_solver)
        else:
            raise NotImplementedError("activation '%s' is outside this library" % self.f)
        return out[0] if single else out
