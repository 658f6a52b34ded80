"""Parameter plumbing shared by the quantized modules
(counterpart of torch_mlu/core/quantized/modules/mlumodel.py:41-64)."""
import warnings

import torch
from torch.nn.parameter import Parameter


def _frozen(t):
    return Parameter(t, requires_grad=False)


class MLUModel(object):
    def set_bias_with_zeros(self, out_channels):
        self.bias = Parameter(torch.zeros(out_channels))

    def set_weight_bias(self, w, b):
        if isinstance(w, Parameter):
            self.weight, self.bias = w, b
        else:
            self.weight = _frozen(w)
            self.bias = _frozen(b) if b is not None else None

    def set_scale(self, s, scales_channel=None):
        """q_scale packing: [s_in, s_w] or [s_in, 0, s_c0 .. s_c(Co-1)], fp32."""
        if scales_channel is not None:
            s = torch.cat((s, scales_channel)).float()
        self.scale = _frozen(s)

    def set_quantized_mode(self, q, q_channel=None):
        """q_mode: 1 int8, 2 int16; with per-channel weights 3 / 4; int32."""
        if not isinstance(q, torch.Tensor):
            warnings.warn("The quantized_mode is not a tensor, please use Tensor type!")
            q = torch.tensor(q, dtype=torch.int)
        if q_channel and q.item() in (1, 2):
            mode = torch.tensor([int(q.item()) + 2], dtype=torch.int)
        else:
            mode = q.int()
        self.quantized_mode = _frozen(mode)

    def set_mean_std(self, mean, std):
        if mean.dim() == 1:
            mean, std = mean.reshape(1, -1, 1, 1), std.reshape(1, -1, 1, 1)
        self.input_mean = _frozen(mean)
        self.input_std = _frozen(std)

    # ---- what the conv and linear modules share ------------------------------------------------------------
    # checkpoint format: weight, bias, scale, quantized_mode [, quantized_by_channel, scale_weight_per_channel,
    # input_mean, input_std] (torch_mlu/core/quantized/modules/conv.py:77-131, linear.py:53-103)

    def start_calibration(self, qconfig):
        """what from_float does for gen_quant: an observer on the module's input, fed by a forward hook"""
        self.quant = True
        self.qconfig = qconfig
        self.observer = qconfig.activation()
        self.register_forward_hook(lambda module, inputs, output: self.observer(*inputs))

    def save_qparams(self, destination, prefix):
        """the quantization keys of state_dict(): derived from the observers when the module is calibrating"""
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
        if weight_observer._get_name() == "MLUPerChannelMinMaxObserver":
            destination[prefix + "quantized_by_channel"] = torch.tensor([1])
            destination[prefix + "scale_weight_per_channel"] = torch.tensor(weight_observer.scales)
            self.set_scale(torch.tensor([self.observer.scale, 0.0]))
        else:
            self.set_scale(torch.tensor([self.observer.scale, weight_observer.scale]))
        destination[prefix + "scale"] = self.scale.data
        destination[prefix + "quantized_mode"] = self.quantized_mode.data
        if getattr(self, "input_std", None) is not None:
            destination[prefix + "input_mean"] = self.input_mean.data.mul(255)
            destination[prefix + "input_std"] = self.input_std.data.mul(255)

    def load_qparams(self, state_dict, prefix, out_channels, missing_keys, unexpected_keys):
        """the quantization keys of a checkpoint; all of them are optional, in both directions"""
        if prefix + "scale" in state_dict:
            self.set_scale(state_dict[prefix + "scale"], state_dict.get(prefix + "scale_weight_per_channel"))
        if prefix + "quantized_mode" in state_dict:
            self.set_quantized_mode(state_dict[prefix + "quantized_mode"],
                                    state_dict.get(prefix + "quantized_by_channel"))
        if prefix + "input_mean" in state_dict and prefix + "input_std" in state_dict:
            self.set_mean_std(state_dict[prefix + "input_mean"], state_dict[prefix + "input_std"])
        if state_dict.get(prefix + "bias") is None:
            self.set_bias_with_zeros(out_channels)
        for lst in (missing_keys, unexpected_keys):
            for k in [k for k in lst if k.startswith(prefix)]:
                lst.remove(k)

    def keep_wide_scale(self, kept):
        """After a conversion of the module's tensors (.half(), .to()): the reference has no override, so .half()
        turns the q-params into half tensors and its per-channel derivation then runs in half as well.  That is
        followed for int8, where half holds every number of that derivation.  int16 q-params stay fp32:
        32767 / absmax exceeds the largest half for absmax < 0.5, and half holds neither 32767 nor the integers
        above 2048.  kept: the scale as it was before the conversion."""
        if kept is None or self.scale is None or self.scale.dtype == torch.float32:
            return
        int8 = self.quantized_mode is not None and self.quantized_mode.numel() == 1 \
            and int(self.quantized_mode.flatten()[0]) in (1, 3)
        if not int8 or not bool(torch.isfinite(self.scale.float()).all()):
            self.scale = _frozen(kept.detach().to(device=self.scale.device, dtype=torch.float32))
