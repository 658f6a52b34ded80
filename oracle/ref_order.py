"""The reference's own order of tensor operations on the per-channel path -- TEST INFRASTRUCTURE.

The per-channel branches of cnnl_conv2d and cnnl_linear are written out of elementwise tensor ops
(torch_mlu/csrc/aten/operators/cnnl/quantify.cpp:55-114, quantify_conv_forward.cpp:107-131,
linear.cpp:40-70,110-127), so every intermediate is rounded to the dtype of the tensors involved: for
a model converted with .half() that is fp16 for the parameter derivation (absmax, log2, position,
scale, new_scale, scale_factor), for the weight quotient w / scale_factor, for the convolution's
output, for output / new_scale and for output + bias.  This module restates those branches with CPU
torch tensors of the same dtypes, expression by expression, so torch's type promotion and per-op
rounding stand in for the device's; only the integer contraction itself is taken from the C oracle
(it is exact) and converted to the output dtype with one rounding, which is this build's assumption
about the vendor convolution (the vendor library's own rounding is not stated in the tree).

With fp32 tensors the functions here must reproduce oracle.per_channel_params / oracle.ops.conv2d bit
for bit: tests/test_oracle_pins.py checks that, which ties the C restatement and this one together.
"""
import numpy as np
import torch

from . import conv2d_nhwc, gemm_nt, pos_from_scale, quantize


def quantify_per_channel(weight, scale_data, bitwidth):
    """cnnl_quantify_per_channel(input, scale_data, bitwidth)          quantify.cpp:55-114
    weight [Co, ...] and scale_data [Co] torch CPU tensors (fp32 or fp16).
    -> (quantized weight int8/int16, new_pos [1], new_scale [Co]) in the dtypes the reference produces"""
    qmin, qmax = (-128.0, 127.0) if bitwidth == 8 else (-32768.0, 32767.0)
    # :64  the C++ operator/(Scalar, Tensor) fills a tensor with the scalar and divides (a true division;
    # Python's scalar / tensor would multiply by the reciprocal instead)
    absmax_pc = torch.full_like(scale_data, qmax) / scale_data
    log2_absmax = torch.log2(absmax_pc)                             # :71-72 (floating dtype: no cast)
    pos_pc = torch.floor(log2_absmax) - (bitwidth - 2)              # :82-84
    scale_pc = torch.pow(2.0, pos_pc)                               # :87
    scale_pc = scale_pc * (2.0 ** (bitwidth - 1) - 1) / absmax_pc   # :88
    new_pos = (pos_pc.max() + pos_pc.min()) / 2                     # :91
    new_pos = torch.round(new_pos).reshape(-1)                      # :92 (half to even)
    new_scale = scale_pc * torch.pow(2.0, new_pos - pos_pc)         # :95
    scale_factor = torch.pow(2.0, new_pos) / new_scale              # :98
    shape = [-1] + [1] * (weight.dim() - 1)
    tmp = torch.clamp(torch.round(weight / scale_factor.reshape(shape)), qmin, qmax)   # :104-105
    return tmp.to(torch.int8 if bitwidth == 8 else torch.int16), new_pos, new_scale


def _mode(q_mode):
    mode = int(np.asarray(q_mode).reshape(-1)[0])
    assert mode in (3, 4), "the per-channel branch is quantized_mode 3 or 4"
    return 8 if mode == 3 else 16


def conv2d_per_channel(x, weight, bias, padding, stride, dilation, groups, q_scale, q_mode):
    """The per-channel branch of cnnl_conv2d                           quantify_conv_forward.cpp:93-131
    x [N,Ci,H,W], weight [Co,Ci/g,kh,kw], bias [Co], q_scale [2+Co]: torch CPU tensors in the dtypes the
    module holds them (all fp16 after .half(), all fp32 otherwise).
    -> dict(y torch [N,Co,Ho,Wo], qx, qw (NHWC / OHWI numpy), acc, pos_x, new_pos, new_scale)"""
    bw = _mode(q_mode)
    scale_data = q_scale.to(torch.float32)                          # :94
    pos_x = pos_from_scale(bw, float(scale_data[0]))                # :96
    x_nhwc = np.ascontiguousarray(x.permute(0, 2, 3, 1).numpy())    # :62-63, 97 (scaling by 2^-pos is exact)
    qx = quantize(x_nhwc, bw, pos_x)
    w_ohwi = weight.permute(0, 2, 3, 1).contiguous()
    qw_t, new_pos, new_scale = quantify_per_channel(w_ohwi, q_scale[2:], bw)        # :112-114
    qw = qw_t.numpy()
    pos_w = int(new_pos.to(torch.float32)[0])                       # :119-120
    acc, ovf = conv2d_nhwc(qx, qw, tuple(padding), tuple(stride), tuple(dilation), groups)
    out = torch.from_numpy(np.ldexp(acc.astype(np.float64), pos_x + pos_w))
    out = out.to(torch.float32).to(x.dtype).permute(0, 3, 1, 2)     # :123-125 output in the input's dtype
    out = out / new_scale.reshape(1, -1, 1, 1)                      # :127
    out = out + bias.reshape(1, -1, 1, 1)                           # :129
    return dict(y=out, qx=qx, qw=qw, acc=acc, overflow=ovf, pos_x=pos_x, new_pos=pos_w, new_scale=new_scale)


def linear_per_channel(x, weight, bias, q_scale, q_mode):
    """The per-channel branch of cnnl_linear                           linear.cpp:40-70,110-127
    The matrix product's output is fp32 whatever the inputs are (matmul.cpp:72-74), so output / new_scale
    and + bias promote to fp32; only the parameters and the weight quotient are in the tensors' dtype."""
    bw = _mode(q_mode)
    scale_data = q_scale.to(torch.float32)
    pos_x = pos_from_scale(bw, float(scale_data[0]))
    x2 = np.ascontiguousarray(x.reshape(-1, x.shape[-1]).numpy())
    qx = quantize(x2, bw, pos_x)
    qw_t, new_pos, new_scale = quantify_per_channel(weight, q_scale[2:], bw)
    qw = qw_t.numpy()
    pos_w = int(new_pos.to(torch.float32)[0])
    acc, ovf = gemm_nt(qx, qw)
    out = torch.from_numpy(np.ldexp(acc.astype(np.float64), pos_x + pos_w)).to(torch.float32)
    out = out / new_scale.reshape(1, -1)                            # :56
    if bias is not None and bias.dim() != 0:
        out = out + bias                                            # :57-59
    out = out.reshape(tuple(x.shape[:-1]) + (weight.shape[0],))
    return dict(y=out, qx=qx, qw=qw, acc=acc, overflow=ovf, pos_x=pos_x, new_pos=pos_w, new_scale=new_scale)
