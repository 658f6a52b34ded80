"""Quantized convolution modules (counterpart of torch_mlu/core/quantized/modules/conv.py:
MLUConvNd :19, MLUConv2d :148, MLUConv1d :258, MLUConv3d :314).

On CPU tensors a module is the float convolution plus an input observer: that is the
calibration pass (conv.py:174-177 in the reference).  On device tensors it calls
``torch.ops.torch_mlu.conv2d`` / ``conv1d`` / ``conv3d`` with the packed q-params (conv.py:178-190,
276-286, 345-354)."""
import logging

import torch
import torch.nn.functional as F
from torch.nn.modules.conv import Conv1d as NNConv1d
from torch.nn.modules.conv import Conv2d as NNConv2d
from torch.nn.modules.conv import Conv3d as NNConv3d
from torch.nn.modules.utils import _pair, _single, _triple
from torch.nn.parameter import Parameter

from .mlumodel import MLUModel


class MLUConvNd(torch.nn.Module, MLUModel):
    # what differs between the 1-d, 2-d and 3-d modules
    _tuple = staticmethod(_pair)
    _nn_class = NNConv2d
    _float_conv = staticmethod(F.conv2d)
    _op_name = "conv2d"

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1, groups=1,
                 bias=True, padding_mode="zeros"):
        super().__init__()
        if in_channels % groups != 0:
            raise ValueError("in_channels must be divisible by groups")
        if out_channels % groups != 0:
            raise ValueError("out_channels    must be divisible by groups")
        self.in_channels, self.out_channels, self.groups = in_channels, out_channels, groups
        self.kernel_size, self.stride = self._tuple(kernel_size), self._tuple(stride)
        self.padding, self.dilation = self._tuple(padding), self._tuple(dilation)
        self.padding_mode = padding_mode
        self.weight = Parameter(torch.empty(out_channels, in_channels // groups, *self.kernel_size))
        if bias:
            self.bias = Parameter(torch.empty(out_channels))
        else:
            self.register_parameter("bias", None)
        self.scale = None
        self.quantized_mode = None
        self.use_symmetry = Parameter(torch.tensor([1]), requires_grad=False)
        self.input_std = None
        self.input_mean = None
        self.quant = False
        ref = self._nn_class(in_channels, out_channels, self.kernel_size, groups=groups, bias=bias)
        with torch.no_grad():
            self.weight.copy_(ref.weight)
            if bias:
                self.bias.copy_(ref.bias)

    # -- calibration ----------------------------------------------------------------------------
    def _float_forward(self, x):
        if self.padding_mode == "circular":
            pads = []
            for pd in reversed(self.padding):  # F.pad wants the last dimension first
                pads += [(pd + 1) // 2, pd // 2]
            x = F.pad(x, tuple(pads), mode="circular")
            return self._float_conv(x, self.weight, self.bias, self.stride, self._tuple(0), self.dilation, self.groups)
        return self._float_conv(x, self.weight, self.bias, self.stride, self.padding, self.dilation, self.groups)

    def forward(self, input):
        if input.device.type == "cpu":
            return self._float_forward(input)
        if self.input_std is not None:
            input = (input - self.input_mean) / self.input_std
        op = getattr(torch.ops.torch_mlu, self._op_name)
        return op(input, self.weight, self.bias, list(self.padding), list(self.stride), list(self.dilation),
                  self.groups, self.scale, self.quantized_mode)

    # -- checkpoint format (conv.py:77-131): the keys are written and read by MLUModel ------------------------
    def _save_to_state_dict(self, destination, prefix, keep_vars):
        super()._save_to_state_dict(destination, prefix, keep_vars)
        self.save_qparams(destination, prefix)

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                              error_msgs):
        super()._load_from_state_dict(state_dict, prefix, local_metadata, False, missing_keys, unexpected_keys,
                                      error_msgs)
        self.load_qparams(state_dict, prefix, self.out_channels, missing_keys, unexpected_keys)

    def extra_repr(self):
        return ("{in_channels}, {out_channels}, kernel_size={kernel_size}, stride={stride}, padding={padding}, "
                "dilation={dilation}, groups={groups}").format(**self.__dict__) + \
               ", scale={}, quantized_mode={}".format(self.scale, self.quantized_mode)

    def _apply(self, fn, recurse=True):
        kept = None if self.scale is None else self.scale.detach().clone()
        super()._apply(fn)
        self.keep_wide_scale(kept)
        return self

    def _get_name(self):
        return type(self).__name__

    @classmethod
    def from_float(cls, mod, gen_quant):
        assert isinstance(mod, cls._nn_class), "{} only works for nn.{} or its subclass".format(
            cls.__name__, cls._nn_class.__name__)
        assert hasattr(mod, "qconfig"), "Input float module must have qconfig defined"
        q = cls(mod.in_channels, mod.out_channels, mod.kernel_size, mod.stride, mod.padding, mod.dilation,
                mod.groups, mod.bias is not None, mod.padding_mode)
        q.set_weight_bias(mod.weight, mod.bias)
        if gen_quant:
            if cls is MLUConv3d:
                assert mod.qconfig.activation().qscheme["per_channel"] is False, \
                    "MLUConv3d does not support per_channel quantization, set per_channel False in qconfig!"
            if cls._op_name == "conv2d" and MLUConv2d.is_first_layer:
                conf = mod.qconfig.activation().qscheme
                if conf["firstconv"] is True:
                    assert conf["mean"] is not None and conf["std"] is not None, \
                        "You are using firstconv but forget setting mean or std, please set mean and std in qconfig!"
                    assert q.in_channels in [1, 3, 4], \
                        "firstconv needs 1 (GRAY), 3 (RGB) or 4 (RGBA) input channels, got {}".format(q.in_channels)
                    assert min(conf["mean"]) >= 0 and max(conf["mean"]) <= 1 and \
                        min(conf["std"]) >= 0 and max(conf["std"]) <= 1, \
                        "firstconv mean and std must lie in [0.0, 1.0] (they are multiplied by 255 when saved)"
                    if set(conf["mean"]) == {0} and set(conf["std"]) == {1}:
                        logging.warning("firstconv with default mean [0,0,0] and std [1,1,1]: check that this is intended")
                    q.set_mean_std(torch.Tensor(conf["mean"]), torch.Tensor(conf["std"]))
                MLUConv2d.is_first_layer = False
            q.start_calibration(mod.qconfig)
        return q


class MLUConv2d(MLUConvNd):
    """conv.py:148-256: [N, C, H, W] tensors, op ``torch_mlu::conv2d``"""
    # only the first convolution of a network may take the first-conv normalisation
    is_first_layer = True


class MLUConv1d(MLUConvNd):
    """conv.py:258-312: the same module over [N, C, L] tensors, op ``torch_mlu::conv1d``"""
    _tuple = staticmethod(_single)
    _nn_class = NNConv1d
    _float_conv = staticmethod(F.conv1d)
    _op_name = "conv1d"


class MLUConv3d(MLUConvNd):
    """conv.py:314-380: [N, C, D, H, W] tensors, op ``torch_mlu::conv3d``; per-tensor weights only"""
    _tuple = staticmethod(_triple)
    _nn_class = NNConv3d
    _float_conv = staticmethod(F.conv3d)
    _op_name = "conv3d"
