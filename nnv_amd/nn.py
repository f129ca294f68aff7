"""NN: the network container whose reach loop drives the layers (nn/NN.m:189-278, 1529-1551)."""
from __future__ import annotations

import time

import numpy as np

from .layers import Conv2DLayer, FullyConnectedLayer, ReluLayer
from .layers_affine import (AveragePooling2DLayer, BatchNormalizationLayer, FlattenLayer, ImageInputLayer,
                            LayerS)
from .sets import ImageStar, SetArray, Star, _Handle
from .verify import HalfSpace, verify_specification


class NN:
    def __init__(self, layers, name="nn"):
        self.Layers = list(layers)
        self.numLayers = len(self.Layers)
        self.Name = name
        self.reachMethod = "approx-star"
        self.relaxFactor = 0
        self.reachOption = []
        self.numCores = 1
        self.dis_opt = None
        self.lp_solver = "linprog"
        self.reachSet = []
        self.reachTime = []

    @staticmethod
    def from_config(layer_dicts, name="nn"):
        """Build from the layer dictionaries of nnv_amd.configs."""
        layers = []
        for L in layer_dicts:
            if L["type"] == "fc":
                layers.append(FullyConnectedLayer(L["W"], L["b"]))
            elif L["type"] == "conv":
                layers.append(Conv2DLayer(L["W"], L["b"], L.get("padding", [0, 0, 0, 0]), L.get("stride", [1, 1]),
                                          L.get("dilation", [1, 1])))
            elif L["type"] == "relu":
                layers.append(ReluLayer())
            elif L["type"] == "batchnorm":
                layers.append(BatchNormalizationLayer(NumChannels=np.size(L["mean"]), TrainedMean=L["mean"],
                                                      TrainedVariance=L["var"], Epsilon=L["eps"], Scale=L["scale"],
                                                      Offset=L["offset"]))
            elif L["type"] == "avgpool":
                layers.append(AveragePooling2DLayer(L["pool"], L["stride"], L["padding"]))
            elif L["type"] == "flatten":
                layers.append(FlattenLayer("FlattenLayer", L["flatten_type"]))
            elif L["type"] == "imageinput":
                layers.append(ImageInputLayer("ImageInputLayer", L.get("input_size", []), L["normalization"], "auto",
                                              L.get("mean"), L.get("std"), L.get("min"), L.get("max")))
            elif L["type"] == "layers":
                layers.append(LayerS(L["W"], L["b"], L["f"]))
            else:
                raise ValueError("unknown layer type %r" % (L["type"],))
        return NN(layers, name)

    def validate_reach_options(self, reachOptions):
        """nn/NN.m:1203-1233."""
        reachOptions = dict(reachOptions)
        method = reachOptions["reachMethod"]
        if "relax-star" in method:
            if "relaxFactor" not in reachOptions:
                raise ValueError("Please, specify a relax factor value to perform relax-star reachability analysis")
            if reachOptions["relaxFactor"] < 0 or reachOptions["relaxFactor"] > 1:
                raise ValueError("Invalid relaxFactor. The value of relax factor must be between 0 and 1")
        if "exact" not in method:
            reachOptions["reachOption"] = "single"
            reachOptions["numCores"] = 1
        return reachOptions

    def reach(self, inputSet, reachOptions=None):
        """nn/NN.m:189-278: inputSet is a Star / ImageStar or a list of them."""
        probe = inputSet[0] if isinstance(inputSet, (list, tuple, SetArray)) and len(inputSet) else inputSet
        if not isinstance(probe, (Star, ImageStar)):
            raise TypeError('Wrong input set type. Input set must be of type "Star", "ImageStar", "VolumeStar", "ImageZono", or "Zono"')
        if reachOptions is not None:
            if not isinstance(reachOptions, dict):
                raise TypeError("The reachability parameters must be specified as a struct.")
            reachOptions = self.validate_reach_options(reachOptions)
        else:
            reachOptions = {}
        if "reachMethod" in reachOptions:
            self.reachMethod = reachOptions["reachMethod"]
        self.numCores = reachOptions.get("numCores", 1)
        if "relaxFactor" in reachOptions:
            self.relaxFactor = reachOptions["relaxFactor"]
        self.dis_opt = reachOptions.get("dis_opt", None)
        if "lp_solver" in reachOptions:
            self.lp_solver = reachOptions["lp_solver"]
        return self.reach_noConns(inputSet)

    def reach_noConns(self, inSet):
        """nn/NN.m:1529-1551: layer loop; keeps every layer's output set and its wall time."""
        # the sets of an earlier reach are let go once the first layers of this one are queued on the
        # device: releasing thousands of handles then costs no device time
        earlier = self.reachSet
        self.reachSet = [None] * self.numLayers
        self.reachTime = [0.0] * self.numLayers
        rs = inSet
        ctx = rs.ctx if isinstance(rs, SetArray) else (rs[0] if isinstance(rs, (list, tuple)) else rs).ctx
        timed = self.dis_opt == "display"
        if not timed and self._reach_in_one_call(inSet, ctx):
            return self.reachSet[-1]
        last = len(self.Layers) - 1
        for i, layer in enumerate(self.Layers):
            if timed:
                print("Reachability for layer %d :" % (i + 1))
                ctx.synchronize()
            t0 = time.perf_counter()
            # the set that is handed back is written in full by the layer that produces it (the sets in
            # between write columns nobody reads only when somebody does)
            eager = i == last and not ctx.eager_columns
            if eager:
                ctx.set_eager_columns(True)
            # an array of sets in front of a ReLU step that an FC layer follows: the library is told, and queues
            # the part of that layer's range estimate that needs only the step's classes behind the classification
            if (isinstance(layer, ReluLayer) and i < last and isinstance(self.Layers[i + 1], FullyConnectedLayer)
                    and isinstance(rs, (list, tuple, SetArray)) and len(rs) >= 64):
                ctx.hint_next_fc(self.Layers[i + 1]._weights(ctx))
            try:
                rs = layer.reach(rs, self.reachMethod, self.reachOption, self.relaxFactor, self.dis_opt, self.lp_solver)
            finally:
                if eager:
                    ctx.set_eager_columns(False)
            if timed:
                ctx.synchronize()
            self.reachTime[i] = time.perf_counter() - t0
            self.reachSet[i] = rs
            earlier = None
        return rs

    def _reach_in_one_call(self, inSet, ctx):
        """The layer loop above as one library call (nnvhip_reach_layers) when the network consists of fully
        connected, convolutional and ReLU layers and the method is a relax-star one at relaxFactor = 1: the same
        layer operations in the same order, without a round trip through Python between them.  Fills reachSet
        (reachTime stays zero: per-layer times need the loop, dis_opt = 'display').  False: not applicable."""
        import ctypes as C
        from . import _lib
        from .layers import RELAX_ORDER, _as_list, _handles_array, _shapes
        if self.reachMethod not in RELAX_ORDER or self.relaxFactor != 1 or not self.Layers:
            return False
        if not all(type(L) in (FullyConnectedLayer, Conv2DLayer, ReluLayer) for L in self.Layers):
            return False
        if self.reachOption not in (None, "", "single", "parallel") and not (isinstance(self.reachOption, (list, tuple)) and not self.reachOption):
            return False
        sets, single = _as_list(inSet)
        if not len(sets):
            return False
        if len(sets) >= 64:
            # a large array: its layers take milliseconds, the loop's Python costs nothing next to them, and the loop
            # lets go of the previous reach's thousands of handles while the first layer runs (here they would go
            # after the call, with the device idle)
            return False
        try:
            shapes = _shapes(sets)
        except TypeError:
            return False
        if shapes is not None and any(s is None or s != shapes[0] for s in shapes):
            return False       # mixed arrays take the general loop
        shape = None if shapes is None else shapes[0]
        dim = sets[0].dim if shape is None else shape[0] * shape[1] * shape[2]   # dimension of the current layer's input
        n, count = len(self.Layers), len(sets)
        kind = (C.c_int32 * n)()
        layer = (C.c_void_p * n)()
        hw = (C.c_int64 * (2 * n))()
        out_shapes = []
        for i, L in enumerate(self.Layers):
            if type(L) is FullyConnectedLayer:
                if dim != L.InputSize:
                    return False   # the loop raises the reference's error
                kind[i], layer[i] = 0, L._weights(ctx).h
                shape = None if shape is None else (1, 1, L.OutputSize)
                dim = L.OutputSize
            elif type(L) is Conv2DLayer:
                if shape is None or shape[2] != L.NumChannels:
                    return False
                kind[i], layer[i] = 1, L._weights(ctx).h
                hw[2 * i], hw[2 * i + 1] = shape[0], shape[1]
                ho, wo = L.output_size(shape[0], shape[1])
                if ho < 1 or wo < 1:
                    return False
                shape = (ho, wo, L.NumFilters)
                dim = ho * wo * L.NumFilters
            else:
                kind[i], layer[i] = 2, None
            out_shapes.append(shape)
        out = (C.c_void_p * (n * count))()
        _lib.check(ctx.lib.nnvhip_reach_layers(ctx.handle, n, kind, layer, hw, RELAX_ORDER[self.reachMethod], 1.0, count,
                                               _handles_array(sets), out))
        for i in range(n):
            raw = (C.c_void_p * count)(*out[i * count:(i + 1) * count])
            shp = out_shapes[i]
            if single:
                hd = _Handle(raw[0], ctx)
                self.reachSet[i] = Star._from_handle(hd) if shp is None else ImageStar(_handle=hd, shape=shp)
            else:
                self.reachSet[i] = SetArray(ctx, raw, None if shp is None else [shp] * count)
        return True

    # ---- robustness check (the consumer of the reach set) ---------------------------------
    def robustness_set(self, target, class_type="max"):
        """NN.robustness_set, nn/NN.m:1334-1368 (target is 0-based): one single-row HalfSpace per
        other class, the unsafe region "some other class scores at least as high"."""
        layer = self.Layers[-1]
        if not isinstance(layer, FullyConnectedLayer):
            raise ValueError("Output size is set to 0, but it must be >= 1")
        outSize = len(layer.Bias)
        if target >= outSize:
            raise ValueError("Target idx must be less than or equal to the output size of the NN.")
        G = np.delete(np.eye(outSize), target, axis=0)
        if class_type == "max":
            G = -G
            G[:, target] = 1.0
        elif class_type == "min":
            G[:, target] = -1.0
        return [HalfSpace(G[i:i + 1, :], [0.0]) for i in range(G.shape[0])]

    def checkRobust(self, outputSet, target):
        """NN.checkRobust, nn/NN.m:608-636: 1 robust, 2 unknown."""
        if not isinstance(target, (HalfSpace, list, tuple)):
            if isinstance(target, (int, np.integer)) or getattr(target, "ndim", 1) == 0:
                target = self.robustness_set(int(target), "max")
            else:
                raise ValueError("Target must be a HalfSpace (unsafe/not robust region) or as a scalar determining the output label target.")
        return verify_specification(outputSet, target)

    def verify_robustness(self, inputSet, reachOptions, target):
        """NN.verify_robustness, nn/NN.m:639-655.  The relax-star methods over-approximate, so an
        "unknown" (2) is never promoted to "not robust" (0)."""
        R = self.reach(inputSet, reachOptions)
        return self.checkRobust(R, target)
