"""catch_amd -- MI355X-native fixed-point quantized inference behind the torch_mlu op surface.

Importing the package loads the in-tree HIP library (``lib/libcatchq.so``) and the PyTorch
extension that registers ``torch.ops.torch_mlu.conv2d`` / ``linear`` (and helpers).  There is
no fallback: if the native parts are missing the import fails and says how to build them.
"""
from . import _native

_native.load()

from .core import mlu_quantize  # noqa: E402
from .core.quantized import modules as quantized_modules  # noqa: E402

__all__ = ["mlu_quantize", "quantized_modules"]
