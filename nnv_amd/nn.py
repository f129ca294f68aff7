"""NN: the network container whose reach loop drives the layers (nn/NN.m:189-278, 1529-1551)."""
from __future__ import annotations

import time

from .layers import Conv2DLayer, FullyConnectedLayer, ReluLayer
from .sets import ImageStar, Star


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
        probe = inputSet[0] if isinstance(inputSet, (list, tuple)) and inputSet else inputSet
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
        self.reachSet = [None] * self.numLayers
        self.reachTime = [0.0] * self.numLayers
        rs = inSet
        ctx = (rs[0] if isinstance(rs, (list, tuple)) else rs).ctx
        timed = self.dis_opt == "display"
        for i, layer in enumerate(self.Layers):
            if timed:
                print("Reachability for layer %d :" % (i + 1))
                ctx.synchronize()
            t0 = time.perf_counter()
            rs = layer.reach(rs, self.reachMethod, self.reachOption, self.relaxFactor, self.dis_opt, self.lp_solver)
            if timed:
                ctx.synchronize()
            self.reachTime[i] = time.perf_counter() - t0
            self.reachSet[i] = rs
        return rs
