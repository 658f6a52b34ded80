from .conv import MLUConv1d, MLUConv2d, MLUConv3d
from .linear import MLULinear
from .mlumodel import MLUModel

__all__ = ["MLUConv1d", "MLUConv2d", "MLUConv3d", "MLULinear", "MLUModel"]
