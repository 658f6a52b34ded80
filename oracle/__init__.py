"""CPU oracle for the quantized hot path -- TEST INFRASTRUCTURE, not product code.

numpy/ctypes front end of ``catchq_oracle.c``.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this package; ``catch_amd`` never does.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcatchq_oracle.so")


def build(force=False):
    """Compile the C restatement with gcc (a few seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-B", "-C", _HERE, "libcatchq_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    c_i, c_i64, c_f, c_d, c_p = (ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_double,
                                 ctypes.c_void_p)
    ip, fp = ctypes.POINTER(c_i), ctypes.POINTER(c_f)
    sig = {
        "orc_num_threads": (c_i, []),
        "orc_set_num_threads": (None, [c_i]),
        "orc_f16_to_f32": (c_f, [ctypes.c_uint16]),
        "orc_f32_to_f16": (ctypes.c_uint16, [c_f]),
        "orc_pos_from_scale": (c_i, [c_i, c_f]),
        "orc_quant_params": (None, [c_i, c_f, ip, fp, fp]),
        "orc_calib_scale": (c_d, [c_i, c_d, c_d]),
        "orc_per_channel_params": (None, [c_i, c_p, c_i, ip, c_p, c_p]),
        "orc_quantize_param": (None, [c_f, c_i, ip, fp, fp]),
        "orc_absmax_f32": (c_f, [c_p, c_i64]),
        "orc_absmax_f16": (c_f, [c_p, c_i64]),
        "orc_quantize_f32": (None, [c_p, c_p, c_i, c_i64, c_i, c_f]),
        "orc_quantize_f16": (None, [c_p, c_p, c_i, c_i64, c_i, c_f]),
        "orc_quantize_nchw_to_nhwc_f32": (None, [c_p, c_p, c_i, c_i, c_i, c_i, c_i, c_i, c_i, c_f]),
        "orc_quantize_per_channel_f32": (None, [c_p, c_p, c_i, c_i, c_i64, c_p]),
        "orc_dequantize_f32": (None, [c_p, c_i, c_p, c_i64, c_i, c_f]),
        "orc_gemm_nt": (c_i64, [c_p, c_i, c_p, c_i, c_i64, c_i64, c_i64, c_p]),
        "orc_conv_out_size": (c_i, [c_i] * 5),
        "orc_conv2d_nhwc": (c_i64, [c_p, c_i, c_p, c_i] + [c_i] * 14 + [c_p]),
        "orc_epilogue_f32": (None, [c_p, c_i64, c_i64, c_i, c_p, c_p, c_p, c_i, c_p]),
        "orc_epilogue_f16": (None, [c_p, c_i64, c_i64, c_i, c_p, c_p, c_p, c_i, c_p]),
        "orc_global_avgpool_nhwc_f32": (None, [c_p, c_i, c_i, c_i, c_p]),
        "orc_maxpool_nhwc_f32": (None, [c_p, c_i, c_i, c_i, c_i, c_i, c_i, c_i, c_p]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


_lib = _load()

_INT = {8: np.int8, 16: np.int16, 31: np.int32, 32: np.int32}


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype=None):
    return np.ascontiguousarray(a, dtype=dtype)


def num_threads():
    return _lib.orc_num_threads()


def set_num_threads(n):
    _lib.orc_set_num_threads(int(n))


def f16_to_f32(h):
    return _lib.orc_f16_to_f32(int(h))


def f32_to_f16(f):
    return _lib.orc_f32_to_f16(float(np.float32(f)))


def pos_from_scale(bw, scale):
    return _lib.orc_pos_from_scale(bw, float(np.float32(scale)))


def quant_params(bw, scale):
    """-> (position, fractional scale, scale_factor)"""
    p, s, f = ctypes.c_int(), ctypes.c_float(), ctypes.c_float()
    _lib.orc_quant_params(bw, float(np.float32(scale)), ctypes.byref(p), ctypes.byref(s),
                          ctypes.byref(f))
    return p.value, np.float32(s.value), np.float32(f.value)


def calib_scale(bw, min_val, max_val):
    return _lib.orc_calib_scale(bw, float(min_val), float(max_val))


def per_channel_params(bw, scales):
    """-> (new_pos, new_scale[Co] fp32, scale_factor[Co] fp32)"""
    s = _c(scales, np.float32)
    ns, sf = np.empty_like(s), np.empty_like(s)
    p = ctypes.c_int()
    _lib.orc_per_channel_params(bw, _ptr(s), s.size, ctypes.byref(p), _ptr(ns), _ptr(sf))
    return p.value, ns, sf


def quantize_param(absmax, bw):
    p, s, o = ctypes.c_int(), ctypes.c_float(), ctypes.c_float()
    _lib.orc_quantize_param(float(np.float32(absmax)), bw, ctypes.byref(p), ctypes.byref(s),
                            ctypes.byref(o))
    return p.value, np.float32(s.value), np.float32(o.value)


def absmax(x):
    x = _c(x)
    if x.dtype == np.float16:
        return np.float32(_lib.orc_absmax_f16(_ptr(x), x.size))
    x = _c(x, np.float32)
    return np.float32(_lib.orc_absmax_f32(_ptr(x), x.size))


def quantize(x, bw, pos, scale=1.0):
    x = _c(x)
    q = np.empty(x.shape, _INT[bw])
    if x.dtype == np.float16:
        _lib.orc_quantize_f16(_ptr(x), _ptr(q), bw, x.size, int(pos), float(np.float32(scale)))
    else:
        x = _c(x, np.float32)
        _lib.orc_quantize_f32(_ptr(x), _ptr(q), bw, x.size, int(pos), float(np.float32(scale)))
    return q


def quantize_nchw_to_nhwc(x, bw, pos, scale=1.0, cpad=None):
    x = _c(x, np.float32)
    n, c, h, w = x.shape
    cpad = cpad or c
    q = np.empty((n, h, w, cpad), _INT[bw])
    _lib.orc_quantize_nchw_to_nhwc_f32(_ptr(x), _ptr(q), bw, n, c, h, w, cpad, int(pos),
                                       float(np.float32(scale)))
    return q


def quantize_per_channel(w, bw, sf):
    w = _c(w, np.float32)
    sf = _c(sf, np.float32)
    q = np.empty(w.shape, _INT[bw])
    co = w.shape[0]
    _lib.orc_quantize_per_channel_f32(_ptr(w), _ptr(q), bw, co, w.size // max(co, 1), _ptr(sf))
    return q


def dequantize(q, pos, scale=1.0):
    q = _c(q)
    bits = q.dtype.itemsize * 8
    y = np.empty(q.shape, np.float32)
    _lib.orc_dequantize_f32(_ptr(q), bits, _ptr(y), q.size, int(pos), float(np.float32(scale)))
    return y


def gemm_nt(a, b):
    """a [M,K], b [N,K] int8/int16 -> (acc int64 [M,N], number of sums outside int32)"""
    a, b = _c(a), _c(b)
    m, k = a.shape
    n, k2 = b.shape
    assert k == k2
    acc = np.empty((m, n), np.int64)
    ovf = _lib.orc_gemm_nt(_ptr(a), a.dtype.itemsize * 8, _ptr(b), b.dtype.itemsize * 8, m, n, k,
                           _ptr(acc))
    return acc, ovf


def conv_out_size(n, k, pad, stride, dil):
    return _lib.orc_conv_out_size(n, k, pad, stride, dil)


def conv2d_nhwc(x, w, padding=(0, 0), stride=(1, 1), dilation=(1, 1), groups=1):
    """x [N,H,W,Ci], w [Co,kh,kw,Ci/g] int8/int16 -> (acc int64 [N,Ho,Wo,Co], number of sums outside int32)"""
    x, w = _c(x), _c(w)
    n, h, wd, ci = x.shape
    co, kh, kw, cig = w.shape
    assert cig * groups == ci and co % groups == 0
    ho = conv_out_size(h, kh, padding[0], stride[0], dilation[0])
    wo = conv_out_size(wd, kw, padding[1], stride[1], dilation[1])
    acc = np.empty((n, ho, wo, co), np.int64)
    ovf = _lib.orc_conv2d_nhwc(_ptr(x), x.dtype.itemsize * 8, _ptr(w), w.dtype.itemsize * 8, n, h,
                               wd, ci, co, kh, kw, padding[0], padding[1], stride[0], stride[1],
                               dilation[0], dilation[1], groups, _ptr(acc))
    return acc, ovf


def leaky_relu(y, slope):
    """x > 0 ? x : x * slope in fp32 (one rounding), the elementwise op of torch.nn.LeakyReLU"""
    y = np.asarray(y, np.float32)
    return np.where(y > 0, y, y * np.float32(slope)).astype(np.float32)


def epilogue(acc, exp2, chan_div=None, bias=None, resid=None, act=0, out_dtype=np.float32, act_slope=0.0,
             resid_after_act=False):
    """acc [..., Co] integer sums -> fp32/fp16 [..., Co].  act 3 = leaky ReLU with act_slope;
    resid_after_act: act(v) + resid instead of act(v + resid).  Those two variants are composed
    here from the plain dequant+bias step and separate fp32 elementwise steps, the way a model
    built from the reference's ops runs them (activation and add are ops of their own there)."""
    if act == 3 or (resid_after_act and resid is not None):
        y = epilogue(acc, exp2, chan_div, bias, None if resid_after_act else resid, 0)
        if act == 3:
            y = leaky_relu(y, act_slope)
        elif act >= 1:
            y = np.where(y > 0, y, np.float32(0)).astype(np.float32)
            if act == 2:
                y = np.where(y < 6, y, np.float32(6)).astype(np.float32)
        if resid_after_act and resid is not None:
            y = (y + np.asarray(resid, np.float32).reshape(y.shape)).astype(np.float32)
        return y.astype(np.float16) if out_dtype == np.float16 else y
    acc = _c(acc, np.int64)
    co = acc.shape[-1]
    rows = acc.size // max(co, 1)
    cd = None if chan_div is None else _c(chan_div, np.float32)
    bs = None if bias is None else _c(bias, np.float32)
    rs = None if resid is None else _c(resid, np.float32)
    if out_dtype == np.float16:
        y = np.empty(acc.shape, np.uint16)
        _lib.orc_epilogue_f16(_ptr(acc), rows, co, int(exp2), _ptr(cd), _ptr(bs), _ptr(rs), int(act),
                              _ptr(y))
        return y.view(np.float16)
    y = np.empty(acc.shape, np.float32)
    _lib.orc_epilogue_f32(_ptr(acc), rows, co, int(exp2), _ptr(cd), _ptr(bs), _ptr(rs), int(act),
                          _ptr(y))
    return y


def maxpool_nhwc(x, k, stride, pad):
    x = _c(x, np.float32)
    n, h, w, c = x.shape
    ho, wo = (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1
    y = np.empty((n, ho, wo, c), np.float32)
    _lib.orc_maxpool_nhwc_f32(_ptr(x), n, h, w, c, k, stride, pad, _ptr(y))
    return y


def global_avgpool_nhwc(x):
    """x [N,H,W,C] fp32 -> [N,C]"""
    x = _c(x, np.float32)
    n, h, w, c = x.shape
    y = np.empty((n, c), np.float32)
    _lib.orc_global_avgpool_nhwc_f32(_ptr(x), n, h * w, c, _ptr(y))
    return y
