"""nnv_amd: MI355X-native star-set reachability (the relax-star methods) behind NNV's API.

The compute path is the HIP library nnv_amd/libnnvhip.so (C ABI in include/nnvhip.h); these Python
classes mirror NNV's MATLAB classes for the path and call it through ctypes.
"""
from ._lib import Context, NNVHipError, NNVHipOutOfMemory, default_context  # noqa: F401
from .layers import Conv2DLayer, FullyConnectedLayer, PosLin, ReluLayer  # noqa: F401
from .layers_affine import (AveragePooling2DLayer, BatchNormalizationLayer, FlattenLayer,  # noqa: F401
                            ImageInputLayer, LayerS)
from .nn import NN  # noqa: F401
from .sets import Box, ImageStar, SetArray, Star, Zono  # noqa: F401
from .verify import HalfSpace, verify_specification  # noqa: F401
