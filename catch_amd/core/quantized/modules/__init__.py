from .conv import MLUConv2d
from .linear import MLULinear
from .mlumodel import MLUModel

__all__ = ["MLUConv2d", "MLULinear", "MLUModel"]
