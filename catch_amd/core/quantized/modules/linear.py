"""Quantized Linear module (counterpart of torch_mlu/core/quantized/modules/linear.py)."""
import torch
import torch.nn.functional as F
from torch.nn.modules.linear import Linear as NNLinear
from torch.nn.parameter import Parameter

from .mlumodel import MLUModel


class MLULinear(torch.nn.Module, MLUModel):
    def __init__(self, in_features, out_features, bias=True):
        super().__init__()
        self.in_features, self.out_features = in_features, out_features
        ref = NNLinear(in_features, out_features, bias)
        self.weight = Parameter(ref.weight.detach().clone())
        if bias:
            self.bias = Parameter(ref.bias.detach().clone())
        else:
            self.register_parameter("bias", None)
        self.scale = None
        self.quantized_mode = None
        self.quant = False
        self.use_symmetry = Parameter(torch.tensor([1]), requires_grad=False)

    def forward(self, input):
        if input.device.type == "cpu":  # calibration pass: float arithmetic (linear.py:38-41)
            return F.linear(input, self.weight, self.bias)
        return torch.ops.torch_mlu.linear(input, self.weight, self.bias, self.scale, self.quantized_mode)

    def _save_to_state_dict(self, destination, prefix, keep_vars):
        super()._save_to_state_dict(destination, prefix, keep_vars)
        self.save_qparams(destination, prefix)

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                              error_msgs):
        super()._load_from_state_dict(state_dict, prefix, local_metadata, False, missing_keys, unexpected_keys,
                                      error_msgs)
        self.load_qparams(state_dict, prefix, self.out_features, missing_keys, unexpected_keys)

    def _apply(self, fn, recurse=True):
        kept = None if self.scale is None else self.scale.detach().clone()
        super()._apply(fn)
        self.keep_wide_scale(kept)
        return self

    def _get_name(self):
        return "MLULinear"

    def extra_repr(self):
        return "in_features={}, out_features={}, bias={}, scale={}, quantized_mode={}, quant={}".format(
            self.in_features, self.out_features, self.bias is not None, self.scale, self.quantized_mode, self.quant)

    @classmethod
    def from_float(cls, mod, gen_quant):
        assert type(mod) == NNLinear, "MLULinear only works for nn.Linear"
        assert hasattr(mod, "qconfig"), "Input float module must have qconfig defined"
        q = cls(mod.in_features, mod.out_features)
        q.set_weight_bias(mod.weight, mod.bias)
        if gen_quant:
            q.start_calibration(mod.qconfig)
        return q
