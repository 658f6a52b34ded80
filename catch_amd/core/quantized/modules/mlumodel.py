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
