"""(activation observer factory, weight observer factory) pairs.
Counterpart of torch_mlu/core/quantized/qconfig.py."""
from torch.quantization import QConfig  # the pair type with its "pass a class, not an instance" check

from .observer import (NoopObserver, default_mlu_observer, mlu_activation_observer, mlu_norm_observer,
                       mlu_weight_observer, mlu_weight_per_channel_observer)


default_mlu_qconfig = QConfig(activation=default_mlu_observer, weight=default_mlu_observer)


def mlu_weight_qconfig(dtype):
    return QConfig(weight=mlu_weight_observer(dtype), activation=NoopObserver)


def mlu_activation_qconfig(dtype, qscheme):
    return QConfig(weight=NoopObserver, activation=mlu_activation_observer(dtype, qscheme))


def custom_mlu_qconfig(dtype, qscheme):
    return QConfig(weight=mlu_weight_observer(dtype), activation=mlu_activation_observer(dtype, qscheme))


def norm_mlu_qconfig(dtype, qscheme):
    return QConfig(weight=mlu_weight_observer(dtype), activation=mlu_norm_observer(dtype, qscheme))


def mlu_per_channel_qconfig(dtype, qscheme):
    return QConfig(weight=mlu_weight_per_channel_observer(dtype, qscheme),
                   activation=mlu_activation_observer(dtype, qscheme))
