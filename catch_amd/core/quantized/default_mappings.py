"""Which float module classes the quantization tool replaces, and by what.

Same two names as the reference's table (torch_mlu/core/quantized/default_mappings.py) so that scripts
importing them keep working: ``DEFAULT_MLU_MODULE_MAPPING`` (float class -> quantized class; the string
key ``"Conv2d"`` serves models that register their own class under that name) and
``DEFAULT_QCONFIG_PROPAGATE_WHITE_LIST`` (the classes a qconfig is attached to).
"""
from torch import nn

from . import modules as _q

# (float class or registered name, quantized counterpart): one row per supported layer type
_PAIRS = (
    (nn.Conv1d, _q.MLUConv1d),
    (nn.Conv2d, _q.MLUConv2d),
    ("Conv2d", _q.MLUConv2d),
    (nn.Conv3d, _q.MLUConv3d),
    (nn.Linear, _q.MLULinear),
)

DEFAULT_MLU_MODULE_MAPPING = dict(_PAIRS)
DEFAULT_QCONFIG_PROPAGATE_WHITE_LIST = tuple(src for src, _ in _PAIRS)
