"""Oracle-level restatement of the two quantized ops -- TEST INFRASTRUCTURE.

Composes the C oracle's primitives in the order of the reference wrappers
  cnnl_conv2d   torch_mlu/csrc/aten/operators/cnnl/quantify_conv_forward.cpp:56-147
  cnnl_linear   torch_mlu/csrc/aten/operators/cnnl/linear.cpp:40-167
and returns every intermediate (quantized tensors, int32 accumulators) so that a
GPU result can be compared stage by stage.  Arrays are numpy; activations are
logical NCHW on input/output like the ops, NHWC inside.
"""
import numpy as np

from . import (conv2d_nhwc, conv_out_size, epilogue, gemm_nt, per_channel_params, pos_from_scale, quant_params,
               quantize, quantize_per_channel)


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


def decode_fractional(q_scale, q_mode, co):
    """Encoding A read the way the reference's graph mode reads it: every tensor (per-axis: every
    output channel) gets position and fractional scale from its own scale = qmax / absmax
    (setQuantizedParams / setQuantizedParamsPerAxis, torch_mlu/csrc/jit/utils/utils.cpp:81-167), so its
    step is absmax / qmax rather than a power of two.
    -> dict(bw, pos_x, scale_x, pos_c[], scale_c[], exp2, div[co]): a weight of channel c is
    q * 2^pos_c / scale_c; with P = max pos_c, an integer sum dequantizes as
    acc * 2^(pos_x + P) / div[c], div[c] = fp32(scale_x * scale_c * 2^(P - pos_c)).
    Parity unpinned beyond the parameters themselves: what the reference's graph backend computes from
    them bit by bit is inside a closed library; this applies the eager quantizer's stated formula
    q = sat(rne(x * scale * 2^-position)) with scale != 1 and the eager epilogue's order of operations."""
    q_scale = np.asarray(q_scale, dtype=np.float32).reshape(-1)
    mode = int(np.asarray(q_mode).reshape(-1)[0])
    bw = 8 if mode in (1, 3) else 16
    pos_x, scale_x, _ = quant_params(bw, q_scale[0])
    per = [quant_params(bw, s) for s in (q_scale[2:] if mode > 2 else q_scale[1:2])]
    pos_c = np.array([p for p, _, _ in per], np.int32)
    scale_c = np.array([f for _, f, _ in per], np.float32)
    top = int(pos_c.max())
    div = np.float32(scale_x) * np.ldexp(scale_c, top - pos_c).astype(np.float32)
    return dict(bw=bw, pos_x=pos_x, scale_x=scale_x, pos_c=pos_c, scale_c=scale_c, exp2=pos_x + top,
                div=np.ascontiguousarray(np.broadcast_to(div.astype(np.float32), (co,))))


def quantize_weight_fractional(w, d):
    """w [Co, ...]; one (position, scale) for the tensor or one per output channel"""
    if d["pos_c"].size == 1:
        return quantize(w, d["bw"], int(d["pos_c"][0]), float(d["scale_c"][0]))
    return np.stack([quantize(np.ascontiguousarray(w[c]), d["bw"], int(d["pos_c"][c]), float(d["scale_c"][c]))
                     for c in range(w.shape[0])])


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


def conv1d(x, weight, bias, padding, stride, dilation, groups, q_scale, q_mode):
    """x [N,Ci,L], weight [Co,Ci/g,k]: the module of core/quantized/modules/conv.py:258-312 in the
    reference; a 1-d convolution is the 2-d one over images with a single row.  -> y [N,Co,Lo]"""
    x, weight = np.asarray(x), np.asarray(weight)
    d = conv2d(x[:, :, None, :], weight[:, :, None, :], bias, (0, padding[0]), (1, stride[0]), (1, dilation[0]),
               groups, q_scale, q_mode)
    d["y"] = d["y"][:, :, 0, :]
    return d


def conv3d(x, weight, bias, padding, stride, dilation, groups, q_scale, q_mode):
    """x [N,Ci,D,H,W], weight [Co,Ci/g,kd,kh,kw] (core/quantized/modules/conv.py:314-380 in the
    reference).  A 3-d convolution is the sum over the kd depth taps of 2-d convolutions of input depth
    slices with the tap's 2-d filters: the integer sums are added tap by tap, slices outside the
    volume contribute nothing, and the result goes through the same epilogue.  -> y [N,Co,Do,Ho,Wo]"""
    d = decode_qparams(q_scale, q_mode)
    x = np.asarray(x)
    out_dtype = np.float16 if x.dtype == np.float16 else np.float32
    n, ci, dep, h, w = x.shape
    co, _, kd, kh, kw = weight.shape
    qx = quantize(np.ascontiguousarray(np.transpose(x, (0, 2, 3, 4, 1))), d["bw_x"], d["pos_x"])  # N D H W C
    w_all = np.ascontiguousarray(np.transpose(np.asarray(weight, dtype=np.float32), (0, 2, 3, 4, 1)))  # O D H W I
    qw = _quantize_weight(w_all.reshape(co, kd * kh, kw, -1), d).reshape(w_all.shape)
    do = conv_out_size(dep, kd, padding[0], stride[0], dilation[0])
    ho = conv_out_size(h, kh, padding[1], stride[1], dilation[1])
    wo = conv_out_size(w, kw, padding[2], stride[2], dilation[2])
    acc = np.zeros((n, do, ho, wo, co), np.int64)
    for od in range(do):
        for t in range(kd):
            z = od * stride[0] - padding[0] + t * dilation[0]
            if z < 0 or z >= dep:
                continue
            a, _ = conv2d_nhwc(np.ascontiguousarray(qx[:, z]), np.ascontiguousarray(qw[:, t]), tuple(padding[1:]),
                               tuple(stride[1:]), tuple(dilation[1:]), groups)
            acc[:, od] += a
    ovf = int(((acc > 2 ** 31 - 1) | (acc < -2 ** 31)).sum())
    b = None if bias is None else np.asarray(bias, dtype=np.float32)
    y = epilogue(acc, d["pos_x"] + d["pos_w"], d["new_scale"], b, None, 0, out_dtype)
    d.update(qx=qx, qw=qw, acc=acc, overflow=ovf, y=np.transpose(y, (0, 4, 1, 2, 3)))
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
