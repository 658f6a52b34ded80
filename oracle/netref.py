"""Oracle-level execution of a whole calibrated network -- TEST INFRASTRUCTURE.

Runs a layer list (catch_amd.nets) the *unfused* way the reference does: every conv / fc layer
quantizes its own fp32 input and its weight, runs the integer contraction, dequantizes, adds bias
(quantify_conv_forward.cpp:56-147, linear.cpp:72-167); residual add, activation, pooling are
separate float steps between the ops, as in a torch model built from the reference's modules.
Tensors are NHWC numpy arrays.  Returns every layer's quantized input, integer sums and fp32
output so that a GPU run can be compared stage by stage.
"""
import numpy as np

from . import (conv2d_nhwc, epilogue, gemm_nt, global_avgpool_nhwc, maxpool_nhwc, quantize,
               quantize_per_channel)
from .ops import decode_fractional, decode_qparams, quantize_weight_fractional

_ACT = {"none": 0, "relu": 1, "relu6": 2, "leaky": 3}
LEAKY_SLOPE = 0.1


def _key(name):
    return "mods." + name.replace(".", "_") + "."


def run(layers, sd, x_nchw, record=True, fractional_scale=False):
    """sd: dict of numpy arrays (weight [Co,Ci/g,kh,kw] / [N,K], bias, scale, quantized_mode).
    record=False keeps only the activations (no per-layer quantized inputs / integer sums).
    fractional_scale: quantize with position and fractional scale per tensor / per output channel
    (ops.decode_fractional) instead of the eager ops' power-of-two steps."""
    t = {"input": np.ascontiguousarray(np.transpose(np.asarray(x_nchw, np.float32), (0, 2, 3, 1)))}
    rec = {}
    for l in layers:
        if l.kind in ("conv", "fc"):
            k = _key(l.name)
            if fractional_scale:
                fr = decode_fractional(sd[k + "scale"], sd[k + "quantized_mode"], np.shape(sd[k + "weight"])[0])
                d = dict(bw_x=fr["bw"], pos_x=fr["pos_x"], pos_w=fr["exp2"] - fr["pos_x"], new_scale=fr["div"])
            else:
                d = decode_qparams(sd[k + "scale"], sd[k + "quantized_mode"])
            w = np.asarray(sd[k + "weight"], np.float32)
            b = sd.get(k + "bias")
            b = None if b is None else np.asarray(b, np.float32)
            x = t[l.src]
            if l.kind == "conv":
                w = np.ascontiguousarray(np.transpose(w, (0, 2, 3, 1)))
            else:
                x = x.reshape(x.shape[0], -1)
            if fractional_scale:
                qx = quantize(x, fr["bw"], fr["pos_x"], fr["scale_x"])
                qw = quantize_weight_fractional(w, fr)
            else:
                qx = quantize(x, d["bw_x"], d["pos_x"])
                qw = (quantize_per_channel(w, d["bw_w"], d["sf"]) if d["per_channel"]
                      else quantize(w, d["bw_w"], d["pos_w"]))
            if l.kind == "conv":
                acc, ovf = conv2d_nhwc(qx, qw, (l.pad, l.pad), (l.stride, l.stride), (1, 1), l.groups)
                resid = t[l.add] if l.add else None
            else:
                acc, ovf = gemm_nt(qx, qw)
                resid = None
            y = epilogue(acc, d["pos_x"] + d["pos_w"], d["new_scale"], b, resid, _ACT[l.act], act_slope=LEAKY_SLOPE,
                         resid_after_act=bool(l.add_after))
            if record:
                rec[l.name] = dict(qx=qx, qw=qw, acc=acc, y=y, overflow=ovf, pos_x=d["pos_x"], pos_w=d["pos_w"])
            t[l.name] = y
        elif l.kind == "maxpool":
            t[l.name] = maxpool_nhwc(t[l.src], l.k, l.stride, l.pad)
        elif l.kind == "gap":
            g = global_avgpool_nhwc(t[l.src])
            t[l.name] = g.reshape(g.shape[0], 1, 1, g.shape[1])
        elif l.kind == "upsample":
            t[l.name] = np.repeat(np.repeat(t[l.src], 2, axis=1), 2, axis=2)
        elif l.kind == "concat":
            t[l.name] = np.concatenate([t[s] for s in l.src], axis=3)
        else:
            raise ValueError(l.kind)
    return t, rec
