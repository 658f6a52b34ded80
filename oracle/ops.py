"""Oracle-level restatement of the two quantized ops -- TEST INFRASTRUCTURE.

Composes the C oracle's primitives in the order of the reference wrappers
  cnnl_conv2d   torch_mlu/csrc/aten/operators/cnnl/quantify_conv_forward.cpp:56-147
  cnnl_linear   torch_mlu/csrc/aten/operators/cnnl/linear.cpp:40-167
and returns every intermediate (quantized tensors, int32 accumulators) so that a
GPU result can be compared stage by stage.  Arrays are numpy; activations are
logical NCHW on input/output like the ops, NHWC inside.
"""
import numpy as np

from . import (conv2d_nhwc, epilogue, gemm_nt, per_channel_params, pos_from_scale, quantize,
               quantize_per_channel)


def decode_qparams(q_scale, q_mode):
    """-> dict(bw_x, bw_w, per_channel, pos_x, pos_w|None, new_scale|None, sf|None)

    Encoding A (q_mode.numel()==1): q_mode in {1:int8, 2:int16, 3:int8 per-channel,
    4:int16 per-channel}, q_scale = [s_in, s_w|0, s_c0..]  (quantify_conv_forward.cpp:77-131).
    Encoding B (q_mode.numel()==2): q_scale = [bw_in, bw_w], q_mode = [pos_in, pos_w] (:132-145).
    """
    q_scale = np.asarray(q_scale, dtype=np.float32).reshape(-1)
    q_mode = np.asarray(q_mode, dtype=np.int32).reshape(-1)
    if q_mode.size == 1:
        mode = int(q_mode[0])
        bw = 8 if mode in (1, 3) else 16
        per_channel = 2 < mode < 5
        d = dict(bw_x=bw, bw_w=bw, per_channel=per_channel, pos_x=pos_from_scale(bw, q_scale[0]),
                 pos_w=None, new_scale=None, sf=None)
        if per_channel:
            new_pos, new_scale, sf = per_channel_params(bw, q_scale[2:])
            d.update(pos_w=new_pos, new_scale=new_scale, sf=sf)
        else:
            d.update(pos_w=pos_from_scale(bw, q_scale[1]))
        return d
    return dict(bw_x=int(q_scale[0]), bw_w=int(q_scale[1]), per_channel=False, pos_x=int(q_mode[0]),
                pos_w=int(q_mode[1]), new_scale=None, sf=None)


def _quantize_weight(w, d):
    if d["per_channel"]:
        return quantize_per_channel(w, d["bw_w"], d["sf"])
    return quantize(w, d["bw_w"], d["pos_w"])


def conv2d(x, weight, bias, padding, stride, dilation, groups, q_scale, q_mode, act=0,
           resid=None):
    """x [N,Ci,H,W] fp32/fp16, weight [Co,Ci/g,kh,kw], bias [Co] or None.
    -> dict(y [N,Co,Ho,Wo] in x.dtype, qx NHWC, qw [Co,kh,kw,Ci/g], acc NHWC int32, overflow, ...)"""
    d = decode_qparams(q_scale, q_mode)
    x = np.asarray(x)
    out_dtype = np.float16 if x.dtype == np.float16 else np.float32
    x_nhwc = np.ascontiguousarray(np.transpose(x, (0, 2, 3, 1)))
    w_ohwi = np.ascontiguousarray(np.transpose(np.asarray(weight, dtype=np.float32), (0, 2, 3, 1)))
    qx = quantize(x_nhwc, d["bw_x"], d["pos_x"])
    qw = _quantize_weight(w_ohwi, d)
    acc, ovf = conv2d_nhwc(qx, qw, tuple(padding), tuple(stride), tuple(dilation), groups)
    b = None if bias is None else np.asarray(bias, dtype=np.float32)
    r = None if resid is None else np.ascontiguousarray(np.transpose(resid, (0, 2, 3, 1)))
    y = epilogue(acc, d["pos_x"] + d["pos_w"], d["new_scale"], b, r, act, out_dtype)
    d.update(qx=qx, qw=qw, acc=acc, overflow=ovf, y=np.transpose(y, (0, 3, 1, 2)))
    return d


def linear(x, weight, bias, q_scale, q_mode, act=0, out_dtype=np.float32):
    """x [..., K], weight [N,K]; output fp32 like the reference (matmul.cpp:72-74)
    unless out_dtype says otherwise."""
    d = decode_qparams(q_scale, q_mode)
    x = np.asarray(x)
    lead = x.shape[:-1]
    x2 = np.ascontiguousarray(x.reshape(-1, x.shape[-1]))
    qx = quantize(x2, d["bw_x"], d["pos_x"])
    qw = _quantize_weight(np.asarray(weight, dtype=np.float32), d)
    acc, ovf = gemm_nt(qx, qw)
    b = None if bias is None else np.asarray(bias, dtype=np.float32)
    y = epilogue(acc, d["pos_x"] + d["pos_w"], d["new_scale"], b, None, act, out_dtype)
    d.update(qx=qx, qw=qw, acc=acc, overflow=ovf, y=y.reshape(lead + (weight.shape[0],)))
    return d
