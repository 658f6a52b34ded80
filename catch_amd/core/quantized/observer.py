"""Calibration observers: running min/max -> scale = qmax / absmax.

Counterpart of torch_mlu/core/quantized/observer.py (same class names, constructor arguments and
attributes so calibration scripts and checkpoints carry over):
  _MLUObserverBase._calculate_qparams         :113-140
  MLUMinMaxObserver                           :142-170
  MLUPerChannelMinMaxObserver                 :202-238
  factory helpers                             :293-325
"""
import math
import warnings
from functools import partial

import torch
import torch.nn as nn

from .qscheme import mlu_qscheme

_QMAX = {"int8": 127.0, "int16": 32767.0}


class _WithArgs(object):
    """Callable that builds an observer with preset keyword arguments (``Cls.with_args(...)``)."""

    def __init__(self, factory):
        self.p = factory

    def __call__(self, *args, **kwargs):
        return self.p(*args, **kwargs)

    def with_args(self, **kwargs):
        return _WithArgs(partial(self.p, **kwargs))

    def __repr__(self):
        return repr(self.p)


class Observer(nn.Module):
    def __init__(self, dtype):
        super().__init__()
        self.dtype = dtype

    def forward(self, x):  # pragma: no cover - interface
        raise NotImplementedError

    def calculate_qparams(self, **kwargs):  # pragma: no cover - interface
        raise NotImplementedError

    @classmethod
    def with_args(cls, **kwargs):
        return _WithArgs(partial(cls, **kwargs))


class _MLUObserverBase(Observer):
    def __init__(self, dtype="int8", qscheme=mlu_qscheme):
        super().__init__(dtype=dtype)
        self.qscheme = dict(mlu_qscheme)
        self.qscheme.update(qscheme)
        self.ncalls = 0

    def get_count(self):
        return self.qscheme["iteration"]

    def _accept(self):
        """An observer takes at most ``iteration`` batches; the call counter advances first."""
        if self.get_count() > self.ncalls:
            self.ncalls += 1
            return True
        print("[warning] It seems that evaluation reaches maxium img_num or iteration is in network. "
              "Quantization still works.")
        return False

    def _calculate_qparams(self, min_val, max_val):
        if max_val is None or min_val is None:
            warnings.warn("Must run observer before calling calculate_qparams. Returning default scale")
            return 1.0
        if math.isnan(max_val) or math.isnan(min_val):
            warnings.warn("Your network weight or input have nan value, which can't be quantized.")
            return 1.0
        assert min_val <= max_val, "min {} should be less than max {}".format(min_val, max_val)
        if self.dtype not in _QMAX:
            warnings.warn("Data type must be int8 or int16. Using default int8 data type")
        qmax = _QMAX.get(self.dtype, 127.0)
        absmax = max(float(max_val), -float(min_val))
        return qmax / absmax if absmax != 0 else 1.0

    def _calculate_per_channel_qparams(self, min_vals, max_vals):
        if min_vals is None or max_vals is None:
            warnings.warn("must run observer before calling calculate_qparams. Returning default scale")
            return torch.tensor([1.0]), torch.tensor([0])
        return [float(self._calculate_qparams(lo, hi)) for lo, hi in zip(min_vals, max_vals)]


class MLUMinMaxObserver(_MLUObserverBase):
    def __init__(self, dtype="int8", qscheme=mlu_qscheme):
        super().__init__(dtype=dtype, qscheme=qscheme)
        self.min_val = None
        self.max_val = None
        self.scale = None

    def forward(self, *args):
        if not self._accept():
            return
        x = args[0].detach()
        k = self.qscheme["data_scale"]
        lo, hi = torch.min(x).item() * k, torch.max(x).item() * k
        if self.min_val is None or self.max_val is None:
            self.min_val, self.max_val = lo, hi
        elif self.qscheme["use_avg"]:
            n = float(self.ncalls)
            self.min_val = (self.min_val * n + lo) / (n + 1)
            self.max_val = (self.max_val * n + hi) / (n + 1)
        else:
            self.min_val, self.max_val = min(lo, self.min_val), max(hi, self.max_val)

    def calculate_qparams(self):
        self.scale = self._calculate_qparams(self.min_val, self.max_val)

    def extra_repr(self):
        return "min_val={}, max_val={}".format(self.min_val, self.max_val)


class MLUPerChannelMinMaxObserver(_MLUObserverBase):
    """min/max per slice of dimension 0 (one scale per output channel of a weight)."""

    def __init__(self, dtype="int8", qscheme=mlu_qscheme, ch_axis=0):
        super().__init__(dtype=dtype, qscheme=qscheme)
        self.min_vals = None
        self.max_vals = None
        self.scales = None
        self.ch_axis = ch_axis

    def forward(self, x_orig):
        if not self._accept():
            return None
        if self.dtype in _QMAX:
            flat = torch.flatten(x_orig.detach(), start_dim=1)
            k = self.qscheme["data_scale"]
            lo, hi = torch.min(flat, 1)[0] * k, torch.max(flat, 1)[0] * k
            if self.min_vals is not None and self.max_vals is not None:
                lo = torch.min(lo, torch.as_tensor(self.min_vals, dtype=lo.dtype))
                hi = torch.max(hi, torch.as_tensor(self.max_vals, dtype=hi.dtype))
            self.min_vals, self.max_vals = lo.tolist(), hi.tolist()
            return x_orig

    def calculate_qparams(self):
        self.scales = self._calculate_per_channel_qparams(self.min_vals, self.max_vals)

    def extra_repr(self):
        return "min_val={}, max_val={}".format(self.min_vals, self.max_vals)


class MLULrnObserver(MLUMinMaxObserver):
    """Range observer of a local-response-normalisation input (observer.py:172-199 in the reference): the same
    running min / max as MLUMinMaxObserver, but the scale describes the squared values the layer sums."""

    def calculate_qparams(self):
        self.scale = self._calculate_qparams(self.min_val ** 2, self.max_val ** 2)


class MLUNormObserver(_MLUObserverBase):
    """Observer of an L2-normalisation input (observer.py:252-294 in the reference).  The layer squares its
    input (scaled by 1 / max) and takes the root of the channel sums; both intermediate tensors get a range,
    [min, max] of x'^2 and of sqrt(sum_c x'^2) + 1e-10, hence two scales."""

    def __init__(self, dtype="int8", qscheme=mlu_qscheme):
        super().__init__(dtype=dtype, qscheme=qscheme)
        self.boundary_1 = None
        self.boundary_2 = None
        self.scale = None

    def forward(self, x_orig):
        if not self._accept() or self.dtype not in _QMAX:
            return
        x = x_orig.detach()
        squares = (x * (1.0 / x.max().item())).pow(2)
        norms = squares.sum(dim=1).sqrt() + 1e-10
        new = ([squares.min().item(), squares.max().item()], [norms.min().item(), norms.max().item()])
        if self.boundary_1 is None or self.boundary_2 is None:
            self.boundary_1, self.boundary_2 = new
        else:
            self.boundary_1 = [min(self.boundary_1[0], new[0][0]), max(self.boundary_1[1], new[0][1])]
            self.boundary_2 = [min(self.boundary_2[0], new[1][0]), max(self.boundary_2[1], new[1][1])]

    def calculate_qparams(self):
        self.scale = [self._calculate_qparams(*self.boundary_1), self._calculate_qparams(*self.boundary_2)]

    def extra_repr(self):
        return "boundary_1={}, boundary_2={}".format(self.boundary_1, self.boundary_2)


class NoopObserver(Observer):
    def __init__(self, dtype=torch.float16):
        if dtype != torch.float16:
            raise ValueError("Only float16 quantization can be used without calibration process")
        super().__init__(dtype=dtype)

    def forward(self, x):
        return x

    def calculate_qparams(self):
        raise Exception("calculate_qparams should not be called for NoopObserver")


default_mlu_observer = MLUMinMaxObserver.with_args(dtype="int8", qscheme=mlu_qscheme)


def mlu_weight_observer(dtype):
    return MLUMinMaxObserver.with_args(dtype=dtype)


def mlu_activation_observer(dtype, qscheme):
    return MLUMinMaxObserver.with_args(dtype=dtype, qscheme=qscheme)


def mlu_minmax_observer(dtype, qscheme):
    return MLUMinMaxObserver.with_args(dtype=dtype, qscheme=qscheme)


def mlu_norm_observer(dtype, qscheme):
    return MLUNormObserver.with_args(dtype=dtype, qscheme=qscheme)


def mlu_lrn_observer(dtype, qscheme):
    return MLULrnObserver.with_args(dtype=dtype, qscheme=qscheme)


def mlu_weight_per_channel_observer(dtype, qscheme):
    return MLUPerChannelMinMaxObserver.with_args(dtype=dtype, qscheme=qscheme)


mlu_activation_observer_dict = {"minmax": mlu_minmax_observer}
