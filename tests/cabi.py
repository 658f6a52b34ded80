"""Thin test-side wrappers: call the C ABI of include/catchq.h on torch device tensors."""
import ctypes

import numpy as np
import torch

from catch_amd import _native
from catch_amd._native import ChainLink, ConvDesc, Epilogue, PointwiseHead, RequantStage, Shortcut, check

F32, F16 = 0, 1
_INT = {8: torch.int8, 16: torch.int16, 31: torch.int32, 32: torch.int32}


def lib():
    return _native.kernel_lib()


def stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def dt(t):
    return F16 if t.dtype == torch.float16 else F32


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


def quantize(x, bw, pos, scale=1.0):
    q = torch.empty(x.shape, dtype=_INT[bw], device=x.device)
    check(lib().catchq_quantize(ptr(x), dt(x), ptr(q), bw, x.numel(), pos, scale, stream()))
    return q


def quantize_devpos(x, bw, pos_t, scale_t=None):
    q = torch.empty(x.shape, dtype=_INT[bw], device=x.device)
    check(lib().catchq_quantize_devpos(ptr(x), dt(x), ptr(q), bw, x.numel(), ptr(pos_t), ptr(scale_t), stream()))
    return q


def quantize_nchw_to_nhwc(x, bw, pos, scale=1.0, cpad=None):
    n, c, h, w = x.shape
    cpad = cpad or c
    q = torch.empty((n, h, w, cpad), dtype=_INT[bw], device=x.device)
    check(lib().catchq_quantize_nchw_to_nhwc(ptr(x), dt(x), ptr(q), bw, n, c, h, w, cpad, pos, scale, stream()))
    return q


def quantize_param(x, bw, mode=2):
    sz = ctypes.c_size_t()
    check(lib().catchq_quantize_param_workspace_size(x.numel(), ctypes.byref(sz)))
    ws = torch.empty(max(sz.value, 4), dtype=torch.int8, device=x.device)
    absmax = torch.empty(1, dtype=torch.float32, device=x.device)
    pos = torch.empty(1, dtype=torch.int32, device=x.device)
    scale = torch.ones(1, dtype=torch.float32, device=x.device)
    off = torch.ones(1, dtype=torch.float32, device=x.device)
    check(lib().catchq_quantize_param(ptr(x), dt(x), x.numel(), bw, mode, ptr(ws), sz.value, ptr(absmax), ptr(pos),
                                      ptr(scale), ptr(off), stream()))
    return absmax, pos, scale, off


def quantize_per_channel(w, bw, sf):
    q = torch.empty(w.shape, dtype=_INT[bw], device=w.device)
    co = w.shape[0]
    check(lib().catchq_quantize_per_channel(ptr(w), dt(w), ptr(q), bw, co, w.numel() // max(co, 1), ptr(sf), stream()))
    return q


def dequantize(q, pos, scale=1.0, half=False):
    bits = q.element_size() * 8
    y = torch.empty(q.shape, dtype=torch.float16 if half else torch.float32, device=q.device)
    check(lib().catchq_dequantize(ptr(q), bits, ptr(y), F16 if half else F32, q.numel(), pos, scale, stream()))
    return y


def _epilogue(shape, device, exp2, chan_div, bias, resid, act, y_dtype, want_acc, q_bw, q_pos, q_scale,
              chan_rcp=None, act_slope=0.0, resid_after_act=False):
    e = Epilogue()
    e.act_slope, e.resid_after_act = act_slope, int(resid_after_act)
    out = {}
    e.exp2 = exp2
    e.chan_div, e.chan_rcp, e.bias, e.resid = ptr(chan_div), ptr(chan_rcp), ptr(bias), ptr(resid)
    e.act = act
    if y_dtype is not None:
        out["y"] = torch.empty(shape, dtype=y_dtype, device=device)
        e.y, e.y_dtype = ptr(out["y"]), (F16 if y_dtype == torch.float16 else F32)
    if want_acc:
        out["acc"] = torch.empty(shape, dtype=torch.int32, device=device)
        e.acc_out = ptr(out["acc"])
    if q_bw:
        out["q"] = torch.empty(shape, dtype=_INT[q_bw], device=device)
        e.q, e.q_bitwidth, e.q_position, e.q_scale = ptr(out["q"]), q_bw, q_pos, q_scale
    return e, out


def gemm_nt(a, b, exp2=0, chan_div=None, bias=None, act=0, y_dtype=torch.float32, want_acc=True, q_bw=0,
            q_pos=0, q_scale=1.0, chan_rcp=None):
    m, k = a.shape
    n = b.shape[0]
    e, out = _epilogue((m, n), a.device, exp2, chan_div, bias, None, act, y_dtype, want_acc, q_bw, q_pos, q_scale,
                       chan_rcp)
    check(lib().catchq_gemm_nt(ptr(a), a.element_size() * 8, ptr(b), b.element_size() * 8, m, n, k,
                               ctypes.byref(e), stream()))
    return out


def conv_desc(x_shape, w_shape, padding, stride, dilation, groups):
    n, h, w, ci = x_shape
    co, kh, kw, _ = w_shape
    return ConvDesc(n, h, w, ci, co, kh, kw, padding[0], padding[1], stride[0], stride[1], dilation[0],
                    dilation[1], groups)


def conv2d_nhwc(x, w, padding=(0, 0), stride=(1, 1), dilation=(1, 1), groups=1, exp2=0, chan_div=None, bias=None,
                resid=None, act=0, y_dtype=torch.float32, want_acc=True, q_bw=0, q_pos=0, q_scale=1.0,
                chan_rcp=None, act_slope=0.0, resid_after_act=False):
    d = conv_desc(x.shape, w.shape, padding, stride, dilation, groups)
    ho = lib().catchq_conv_out_size(d.h, d.kh, d.pad_h, d.stride_h, d.dil_h)
    wo = lib().catchq_conv_out_size(d.w, d.kw, d.pad_w, d.stride_w, d.dil_w)
    e, out = _epilogue((d.n, ho, wo, d.co), x.device, exp2, chan_div, bias, resid, act, y_dtype, want_acc, q_bw,
                       q_pos, q_scale, chan_rcp, act_slope, resid_after_act)
    check(lib().catchq_conv2d_nhwc(ptr(x), x.element_size() * 8, ptr(w), w.element_size() * 8, ctypes.byref(d),
                                   ctypes.byref(e), stream()))
    return out


def conv2d_shortcut_nhwc(x, w, sx, sw, sc_stride, sc_exp2, sc_chan_div=None, sc_bias=None, sc_chan_rcp=None, padding=(0, 0),
                         stride=(1, 1), dilation=(1, 1), exp2=0, chan_div=None, bias=None, act=0, y_dtype=torch.float32,
                         q_bw=0, q_pos=0, q_scale=1.0, chan_rcp=None, act_slope=0.0, resid_after_act=False):
    """-> (outputs, workspace bytes the library asked for)"""
    d = conv_desc(x.shape, w.shape, padding, stride, dilation, 1)
    ho = lib().catchq_conv_out_size(d.h, d.kh, d.pad_h, d.stride_h, d.dil_h)
    wo = lib().catchq_conv_out_size(d.w, d.kw, d.pad_w, d.stride_w, d.dil_w)
    e, out = _epilogue((d.n, ho, wo, d.co), x.device, exp2, chan_div, bias, None, act, y_dtype, False, q_bw, q_pos,
                       q_scale, chan_rcp, act_slope, resid_after_act)
    sc = Shortcut(ptr(sx), ptr(sw), sx.element_size() * 8, sw.element_size() * 8, sx.shape[1], sx.shape[2], sx.shape[3],
                  sc_stride, sc_exp2, ptr(sc_chan_div), ptr(sc_chan_rcp), ptr(sc_bias))
    need = ctypes.c_size_t()
    check(lib().catchq_conv2d_shortcut_workspace_size(x.element_size() * 8, w.element_size() * 8, ctypes.byref(d),
                                                      ctypes.byref(sc), ctypes.byref(need)))
    ws = torch.empty(max(need.value, 16), dtype=torch.int8, device=x.device)
    check(lib().catchq_conv2d_shortcut_nhwc(ptr(x), x.element_size() * 8, ptr(w), w.element_size() * 8, ctypes.byref(d),
                                            ctypes.byref(e), ctypes.byref(sc), ptr(ws), need.value, stream()))
    return out, need.value


def conv1x1_conv3x3_nhwc(x, w1, exp2_1, div1, rcp1, bias1, q_pos1, w, padding=(1, 1), stride=(1, 1), exp2=0, chan_div=None,
                         bias=None, act=0, y_dtype=None, q_bw=8, q_pos=0, q_scale=1.0, chan_rcp=None, sharing=0):
    """x [N,H,W,K1] int8, w1 [Cm,K1] int8 (1x1 + ReLU + requantization at q_pos1), w [Co,kh,kw,Cm] int8
    -> (outputs, workspace bytes the library asked for)"""
    d = conv_desc((x.shape[0], x.shape[1], x.shape[2], w.shape[3]), w.shape, padding, stride, (1, 1), 1)
    ho = lib().catchq_conv_out_size(d.h, d.kh, d.pad_h, d.stride_h, d.dil_h)
    wo = lib().catchq_conv_out_size(d.w, d.kw, d.pad_w, d.stride_w, d.dil_w)
    e, out = _epilogue((d.n, ho, wo, d.co), x.device, exp2, chan_div, bias, None, act, y_dtype, False, q_bw, q_pos,
                       q_scale, chan_rcp)
    e.sharing = sharing
    hd = PointwiseHead(ptr(w1), x.shape[3], exp2_1, ptr(div1), ptr(rcp1), ptr(bias1), q_pos1)
    need = ctypes.c_size_t()
    check(lib().catchq_conv1x1_conv3x3_workspace_size(ctypes.byref(hd), ctypes.byref(d), ctypes.byref(e), ctypes.byref(need)))
    ws = torch.empty(max(need.value, 16), dtype=torch.int8, device=x.device)
    check(lib().catchq_conv1x1_conv3x3_nhwc(ptr(x), ctypes.byref(hd), ptr(w), ctypes.byref(d), ctypes.byref(e), ptr(ws),
                                            need.value, stream()))
    return out, need.value


def inverted_residual_nhwc(x, expand, depthwise, w3, stride=1, exp2=0, chan_div=None, bias=None, resid=None, act=0,
                           y_dtype=None, q_bw=8, q_pos=0, chan_rcp=None, sharing=0):
    """x [N,H,W,Ci] int8; expand / depthwise: dicts with w (int8 [hid,Ci] / [hid,3,3]), exp2, chan_div, chan_rcp, bias,
    act, q_pos (device tensors); w3 [Co,hid] int8 -> (outputs of the projection, workspace bytes the library asked for)"""
    n, h, w, ci = x.shape
    hid, co = expand["w"].shape[0], w3.shape[0]
    ho = lib().catchq_conv_out_size(h, 3, 1, stride, 1)
    wo = lib().catchq_conv_out_size(w, 3, 1, stride, 1)
    e, out = _epilogue((n, ho, wo, co), x.device, exp2, chan_div, bias, resid, act, y_dtype, False, q_bw, q_pos, 1.0,
                       chan_rcp)
    e.sharing = sharing
    st = [RequantStage(ptr(s["w"]), s["exp2"], ptr(s["chan_div"]), ptr(s.get("chan_rcp")), ptr(s["bias"]), s["act"],
                       s["q_pos"]) for s in (expand, depthwise)]
    need = ctypes.c_size_t()
    check(lib().catchq_inverted_residual_workspace_size(n, h, w, ci, hid, co, stride, ctypes.byref(st[0]),
                                                        ctypes.byref(st[1]), ctypes.byref(e), ctypes.byref(need)))
    ws = torch.empty(max(need.value, 16), dtype=torch.int8, device=x.device)
    check(lib().catchq_inverted_residual_nhwc(ptr(x), n, h, w, ci, hid, co, stride, ctypes.byref(st[0]), ctypes.byref(st[1]),
                                              ptr(w3), ctypes.byref(e), ptr(ws), need.value, stream()))
    return out, need.value


def first_layers_nchw(x, x_pos, conv, k, stride=2, pad=3, pool=(3, 2, 1), x_scale=1.0, sharing=0):
    """x [N,C,H,W] fp32; conv: dict with w (int8 [Co,k,kw4,4], zero taps and channels included), exp2, chan_div, chan_rcp,
    bias, act, q_pos (device tensors) -> (pooled int8 [N,Hp,Wp,Co], workspace bytes the library asked for)"""
    n, c, h, w = x.shape
    co = conv["w"].shape[0]
    L = lib()
    hc, wc = L.catchq_conv_out_size(h, k, pad, stride, 1), L.catchq_conv_out_size(w, k, pad, stride, 1)
    hp, wp = L.catchq_conv_out_size(hc, pool[0], pool[2], pool[1], 1), L.catchq_conv_out_size(wc, pool[0], pool[2], pool[1], 1)
    st = RequantStage(ptr(conv["w"]), conv["exp2"], ptr(conv["chan_div"]), ptr(conv.get("chan_rcp")), ptr(conv["bias"]),
                      conv["act"], conv["q_pos"])
    need = ctypes.c_size_t()
    check(L.catchq_first_layers_workspace_size(n, c, h, w, co, k, k, stride, pad, ctypes.byref(st), pool[0], pool[1], pool[2],
                                               sharing, ctypes.byref(need)))
    ws = torch.empty(max(need.value, 16), dtype=torch.int8, device=x.device)
    q = torch.empty((n, hp, wp, co), dtype=torch.int8, device=x.device)
    check(L.catchq_first_layers_nchw(ptr(x), n, c, h, w, x_pos, x_scale, co, k, k, stride, pad, ctypes.byref(st), pool[0],
                                     pool[1], pool[2], ptr(q), sharing, ptr(ws), need.value, stream()))
    return q, need.value


def conv1x1_avgpool_nhwc(x, w, exp2=0, chan_div=None, bias=None, resid=None, act=0, chan_rcp=None, want_mean=True, q_bw=0,
                         q_pos=0, q_scale=1.0):
    """x [N,H,W,Ci] int8, w [Co,Ci] int8 -> ({"mean": fp32 [N,Co] or None, "q": int8 / int16 [N,Co] or None},
    workspace bytes the library asked for)"""
    n, hw, ci, co = x.shape[0], x.shape[1] * x.shape[2], x.shape[3], w.shape[0]
    e, _ = _epilogue((n, hw, 1, co), x.device, exp2, chan_div, bias, resid, act, None, False, 0, 0, 1.0, chan_rcp)
    need = ctypes.c_size_t()
    check(lib().catchq_conv1x1_avgpool_workspace_size(n, hw, ci, co, ctypes.byref(e), ctypes.byref(need)))
    ws = torch.empty(max(need.value, 16), dtype=torch.int8, device=x.device)
    mean = torch.empty((n, co), dtype=torch.float32, device=x.device) if want_mean else None
    q = torch.empty((n, co), dtype=_INT[q_bw], device=x.device) if q_bw else None
    check(lib().catchq_conv1x1_avgpool_nhwc(ptr(x), ptr(w), n, hw, ci, co, ctypes.byref(e), ptr(mean), ptr(q), q_bw, q_pos,
                                            q_scale, ptr(ws), need.value, stream()))
    return {"mean": mean, "q": q}, need.value


def conv1x1_chain_nhwc(links, want_y=True, want_q=True, q_pos=0, sharing=0):
    """links: dicts with x [N,H,W,Ci] int8, w [Co,Ci] int8, stride, exp2, chan_div, chan_rcp, bias (device tensors);
    links[0] is the projection shortcut.  -> {"y": fp32 or None, "q": int8 or None}"""
    n, co = links[0]["x"].shape[0], links[0]["w"].shape[0]
    s0 = links[0]["stride"]
    ho = lib().catchq_conv_out_size(links[0]["x"].shape[1], 1, 0, s0, 1)
    wo = lib().catchq_conv_out_size(links[0]["x"].shape[2], 1, 0, s0, 1)
    arr = (ChainLink * len(links))()
    for a, l in zip(arr, links):
        a.x, a.w = l["x"].data_ptr(), l["w"].data_ptr()
        a.in_h, a.in_w, a.ci = l["x"].shape[1], l["x"].shape[2], l["x"].shape[3]
        a.stride, a.exp2 = l["stride"], l["exp2"]
        for k in ("chan_div", "chan_rcp", "bias"):
            setattr(a, k, None if l.get(k) is None else l[k].data_ptr())
    dev_ = links[0]["x"].device
    y = torch.empty((n, ho, wo, co), dtype=torch.float32, device=dev_) if want_y else None
    q = torch.empty((n, ho, wo, co), dtype=torch.int8, device=dev_) if want_q else None
    check(lib().catchq_conv1x1_chain_nhwc(arr, len(links), n, ho, wo, co, ptr(y), ptr(q), q_pos, sharing, stream()))
    return {"y": y, "q": q}


def quantize_conv2d(x, pos_x, w, pos_w, x_bits=8, w_bits=8, padding=(0, 0), stride=(1, 1), dilation=(1, 1), groups=1,
                    bias=None):
    """x [N,H,W,Ci], w [Co,kh,kw,Ci/g] floating, pos_x / pos_w int32 device tensors of one element"""
    d = conv_desc(x.shape, w.shape, padding, stride, dilation, groups)
    ho = lib().catchq_conv_out_size(d.h, d.kh, d.pad_h, d.stride_h, d.dil_h)
    wo = lib().catchq_conv_out_size(d.w, d.kw, d.pad_w, d.stride_w, d.dil_w)
    need = ctypes.c_size_t()
    check(lib().catchq_quantize_conv2d_workspace_size(ctypes.byref(d), x_bits, w_bits, ctypes.byref(need)))
    ws = torch.empty(need.value, dtype=torch.int8, device=x.device)
    y = torch.empty((d.n, ho, wo, d.co), dtype=x.dtype, device=x.device)
    dt = lambda t: F16 if t.dtype == torch.float16 else F32
    check(lib().catchq_quantize_conv2d_nhwc(ptr(x), dt(x), ptr(pos_x), x_bits, ptr(w), dt(w), ptr(pos_w), w_bits,
                                            ctypes.byref(d), ptr(bias), ptr(y), dt(x), ptr(ws), need.value, stream()))
    return y


def conv_route(x_bits, w_bits, x_shape, w_shape, padding=(0, 0), stride=(1, 1), dilation=(1, 1), groups=1):
    d = conv_desc(x_shape, w_shape, padding, stride, dilation, groups)
    return lib().catchq_conv2d_route(x_bits, w_bits, ctypes.byref(d)).decode()
