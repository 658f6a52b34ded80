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

    def _observer_forward_hook(self, module, inputs, output):
        return self.observer(*inputs)

    def _save_to_state_dict(self, destination, prefix, keep_vars):
        super()._save_to_state_dict(destination, prefix, keep_vars)
        if self.weight is not None:
            destination[prefix + "weight"] = self.weight
        if self.bias is not None:
            destination[prefix + "bias"] = self.bias
        if not self.quant:
            return
        weight_observer = self.qconfig.weight()
        weight_observer(self.weight)
        weight_observer.calculate_qparams()
        self.observer.calculate_qparams()
        self.set_quantized_mode(torch.Tensor([2 if self.observer.dtype == "int16" else 1]))
        destination[prefix + "quantized_mode"] = self.quantized_mode.data
        if weight_observer._get_name() == "MLUMinMaxObserver":
            self.set_scale(torch.tensor([self.observer.scale, weight_observer.scale]))
        else:
            destination[prefix + "quantized_by_channel"] = torch.tensor([1]).data
            destination[prefix + "scale_weight_per_channel"] = torch.tensor(weight_observer.scales).data
            self.set_scale(torch.tensor([self.observer.scale, 0.0]))
        destination[prefix + "scale"] = self.scale.data

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                              error_msgs):
        super()._load_from_state_dict(state_dict, prefix, local_metadata, False, missing_keys, unexpected_keys,
                                      error_msgs)
        if prefix + "scale" in state_dict:
            self.set_scale(state_dict[prefix + "scale"], state_dict.get(prefix + "scale_weight_per_channel"))
        if prefix + "quantized_mode" in state_dict:
            self.set_quantized_mode(state_dict[prefix + "quantized_mode"],
                                    state_dict.get(prefix + "quantized_by_channel"))
        if state_dict.get(prefix + "bias") is None:
            self.set_bias_with_zeros(self.out_features)
        for lst in (missing_keys, unexpected_keys):
            for k in [k for k in lst if k.startswith(prefix)]:
                lst.remove(k)

    def _apply(self, fn, recurse=True):
        # The reference has no override: .half() turns the q-params into half tensors, and its per-channel
        # derivation then runs in half as well.  That is followed for int8, where half holds every number of
        # that derivation.  int16 q-params stay fp32: 32767 / absmax exceeds the largest half for absmax < 0.5,
        # and half holds neither 32767 nor the integers above 2048.
        kept = None if self.scale is None else self.scale.detach().clone()
        super()._apply(fn)
        if kept is not None and self.scale is not None and self.scale.dtype != torch.float32:
            int8 = self.quantized_mode is not None and self.quantized_mode.numel() == 1 \
                and int(self.quantized_mode.flatten()[0]) in (1, 3)
            if not int8 or not bool(torch.isfinite(self.scale.float()).all()):
                self.scale = Parameter(kept.detach().to(device=self.scale.device, dtype=torch.float32),
                                       requires_grad=False)
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
            q.quant = True
            q.qconfig = mod.qconfig
            q.observer = q.qconfig.activation()
            q.register_forward_hook(q._observer_forward_hook)
        return q
