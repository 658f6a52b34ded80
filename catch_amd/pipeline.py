"""Fused int8/int16 execution of a calibrated network.

The drop-in ops (``torch_mlu::conv2d`` / ``linear``) take and return floating tensors, so a model
built from them writes every activation in fp32, reads it back, quantizes it, and runs ReLU and
the residual add as separate float kernels.  This module compiles the same network -- the layer
list of ``catch_amd.nets`` plus a checkpoint in the reference's format (``scale``,
``quantized_mode`` per layer) -- into a plan in which each convolution's epilogue applies
dequantization, bias, residual add and activation and writes the *next* layer's quantized input
directly; fp32 copies are written only where a residual branch, the global average pool or a
network output needs them.  Max pooling runs on the integers (quantization is monotonic).

Every value is computed by the same arithmetic, in the same order, as the unfused sequence
quantize -> integer conv -> dequant+bias -> add -> activation -> quantize, so all quantized
tensors, int32 accumulators and fp32 outputs are identical to it bit for bit.
"""
import ctypes

import numpy as np
import torch

from . import _native
from .nets import LEAKY_SLOPE, outputs_of

_ACT_CODE = {"none": 0, "relu": 1, "relu6": 2, "leaky": 3}
_PASS = ("maxpool", "upsample", "concat")


def _key(name):
    return "mods." + name.replace(".", "_") + "."


def pos_from_scale(bw, scale):
    p = ctypes.c_int()
    _native.check(_native.kernel_lib().catchq_pos_from_scale(int(bw), float(scale), ctypes.byref(p)), "position")
    return p.value


def quant_params(bw, scale):
    """scale (= qmax / absmax) -> (position, fractional scale in [1, 2)): the general form
    q = rne(x * scale_frac * 2^-position) whose step is absmax / qmax exactly
    (setQuantizedParams, torch_mlu/csrc/jit/utils/utils.cpp:81-118 in the reference)"""
    p, f, sf = ctypes.c_int(), ctypes.c_float(), ctypes.c_float()
    _native.check(_native.kernel_lib().catchq_quant_params(int(bw), float(scale), ctypes.byref(p), ctypes.byref(f),
                                                           ctypes.byref(sf)), "quant_params")
    return p.value, f.value


class _LayerQ(object):
    """decoded q-params and the quantized weight of one conv / fc layer"""
    __slots__ = ("bw_x", "bw_w", "pos_x", "scale_x", "pos_w", "qw", "chan_div", "bias", "exp2", "cpad", "groups")


def _pad16(c, bw=8):
    """device-side channel count of a tensor with c channels: the matrix-core routes want a 16-byte
    K chunk not to straddle filter taps, i.e. multiples of 16 channels for int8 activations (1..3
    channel inputs take 4: one pixel per dword) and of 8 for int16 activations"""
    if bw == 16:
        return (c + 7) // 8 * 8
    if c <= 4:
        return 4 if c < 4 else c
    return (c + 15) // 16 * 16


def _act_bits(layer, sd):
    """bit width of the layer's quantized input, from the checkpoint's q-param encoding"""
    k = _key(layer.name)
    mode = sd[k + "quantized_mode"].detach().cpu().reshape(-1)
    if mode.numel() == 1:
        return 8 if int(mode[0]) in (1, 3) else 16
    return int(sd[k + "scale"].detach().float().cpu()[0].item())


def _quantize_weight_fractional(w, bw, scales):
    """w [Co, ...] fp32 (dim 0 slowest in memory), scales: one (per tensor) or Co (per axis) values of
    qmax / absmax.  Each channel is quantized with its own (position, fractional scale)
    (setQuantizedParams / setQuantizedParamsPerAxis, jit/utils/utils.cpp:81-167 in the reference).
    -> (q, P, div): integer weights, the largest position P, and div[c] = scale_c * 2^(P - position_c),
    so that the real value of q[c, ...] is q * 2^P / div[c]."""
    co = w.shape[0]
    pf = [quant_params(bw, float(v)) for v in scales]
    if len(pf) == 1:
        q = torch.ops.torch_mlu.quantize(w, bw, pf[0][0], pf[0][1])
        pf = pf * co
    else:
        rows = w.reshape(co, -1)
        q = torch.stack([torch.ops.torch_mlu.quantize(rows[c], bw, pf[c][0], pf[c][1]) for c in range(co)])
        q = q.reshape(w.shape)
    top = max(p for p, _ in pf)
    div = np.array([np.ldexp(np.float32(f), top - p) for p, f in pf], dtype=np.float32)
    return q, top, div


def _decode(layer, sd, device, ci_dev, co_dev, fractional=False):
    """ci_dev / co_dev: channel counts of the layer's input / output tensors as laid out on the
    device (>= the real counts; extra channels are zeros: zero weights, zero bias, divisor 1).
    fractional: quantize with position *and* fractional scale (steps of exactly absmax / qmax) rather
    than with the power-of-two step the eager ops use."""
    q = _LayerQ()
    q.scale_x = 1.0
    k = _key(layer.name)
    w = sd[k + "weight"].to(device=device, dtype=torch.float32)
    scale = sd[k + "scale"].detach().float().cpu()
    mode = sd[k + "quantized_mode"].detach().cpu().to(torch.int32).reshape(-1)
    bias = sd.get(k + "bias")
    q.bias = None if bias is None else bias.to(device=device, dtype=torch.float32).contiguous()
    q.chan_div = None
    if layer.kind == "conv":
        w = w.contiguous(memory_format=torch.channels_last)  # memory [Co][kh][kw][Ci/g]
    if fractional:
        if mode.numel() != 1:
            raise ValueError("%s: a checkpoint of bit widths and positions holds no fractional scales" % layer.name)
        m = int(mode[0])
        bw = 8 if m in (1, 3) else 16
        q.bw_x = q.bw_w = bw
        q.pos_x, q.scale_x = quant_params(bw, scale[0].item())
        if layer.kind == "conv":  # [Co,kh,kw,Ci/g] contiguous: every channel is one run of memory
            w = w.permute(0, 2, 3, 1).contiguous()
        qw, q.pos_w, div = _quantize_weight_fractional(w, bw, scale[2:].tolist() if m > 2 else [scale[1].item()])
        if layer.kind == "conv":
            qw = qw.permute(0, 3, 1, 2)  # logical [Co,Ci/g,kh,kw] again, same memory
        q.chan_div = torch.from_numpy(np.float32(q.scale_x) * div).to(device)
    elif mode.numel() == 1:
        m = int(mode[0])
        bw = 8 if m in (1, 3) else 16
        q.bw_x = q.bw_w = bw
        q.pos_x = pos_from_scale(bw, scale[0].item())
        if m > 2:
            qw, new_pos, new_scale = torch.ops.torch_mlu.quantize_per_channel(w, scale[2:].to(device), bw)
            q.pos_w, q.chan_div = int(new_pos.item()), new_scale
        else:
            q.pos_w = pos_from_scale(bw, scale[1].item())
            qw = torch.ops.torch_mlu.quantize(w, bw, q.pos_w)
    else:
        q.bw_x, q.bw_w = int(scale[0].item()), int(scale[1].item())
        q.pos_x, q.pos_w = int(mode[0]), int(mode[1])
        qw = torch.ops.torch_mlu.quantize(w, q.bw_w, q.pos_w)
    q.exp2 = q.pos_x + q.pos_w
    q.cpad = ci_dev
    pad = torch.nn.functional.pad
    co = qw.shape[0]
    if layer.kind == "conv":
        qw = qw.permute(0, 2, 3, 1)  # [Co,kh,kw,Ci/g] view of the same memory
        depthwise = layer.groups > 1 and layer.groups == layer.ci == layer.co
        if layer.groups == 1 and ci_dev != layer.ci:
            qw = pad(qw, (0, ci_dev - layer.ci))
        if layer.groups > 1 and not depthwise and (ci_dev != layer.ci or co_dev != co):
            raise ValueError("grouped convolution %s needs unpadded channels" % layer.name)
        q.groups = co_dev if depthwise else layer.groups
    else:
        if ci_dev != layer.ci:
            qw = pad(qw, (0, ci_dev - layer.ci))
        q.groups = 1
    if co_dev != co:  # zero filters for the padding channels
        qw = pad(qw, (0, 0) * (qw.dim() - 1) + (0, co_dev - co))
        if q.bias is not None:
            q.bias = pad(q.bias, (0, co_dev - co))
        if q.chan_div is not None:
            q.chan_div = pad(q.chan_div, (0, co_dev - co), value=1.0)
    q.qw = qw.contiguous()
    return q


class FusedNet(object):
    def __init__(self, layers, state_dict, device="cuda", out_half=False, fuse_shortcuts=True,
                 fractional_scale=False, chain_links=None, fuse_heads=True, fuse_blocks=False,
                 fuse_first_layers=True, fuse_avgpool=True):
        """fractional_scale: quantize activations and weights with position and fractional scale -- the
        general form the reference's fused (graph) mode hands to its backend per tensor / per axis
        (jit/utils/utils.cpp:81-167) -- instead of the eager ops' power-of-two steps.
        chain_links: how far the residual branch of a stage of bottleneck blocks is recomputed from the
        blocks' int8 tensors instead of being stored and read back in fp32: a block whose chain back to the
        stage's projection shortcut has at most this many links (the shortcut counts as one) evaluates the
        whole chain inside its last convolution's launch (torch_mlu::qconv2d_chain); None picks the default
        rule (_default_chain_links), 0 switches the recomputation off.
        fuse_heads: a 1x1 convolution + ReLU whose only reader is a 3x3 convolution (the first two layers of a
        bottleneck block) runs inside that convolution's launch where the kernel library serves the shapes
        (torch_mlu::qconv2d_head); its int8 output is then never stored.
        fuse_blocks: an inverted-residual block (1x1 expansion, 3x3 depthwise, 1x1 linear projection, each hidden
        tensor read by the next layer only) runs as one launch (torch_mlu::qconv2d_irb) where the library's kernel
        serves the shape and the image is large enough for it to pay (block_fuses).  Off by default: the one-launch
        kernel is bound by the same vector arithmetic as the three launches, and with the batch in two parts on
        parallel streams, where one part's launches already fill the other's start-up gaps, MobileNetV2 at batch 128
        measured 2 % slower with it (one stream: 1.5 % faster).
        fuse_first_layers: the input quantizer, a few-channel first convolution + ReLU and the max pooling that is its
        only reader run as one launch (torch_mlu::qconv2d_first_layers) where the library's kernel serves the shape;
        neither the quantized image nor the convolution's output is then stored.
        fuse_avgpool: a 1x1 convolution whose only reader is the global average pooling runs inside the pooling's launch
        (torch_mlu::qconv2d_avgpool) where the library's kernel serves the shape; its fp32 output is then never stored."""
        self.layers = list(layers)
        self.device = torch.device(device)
        self.outputs = outputs_of(self.layers)
        self.out_half = out_half
        # channel counts: real (chan) and as laid out on the device (cdev)
        bw = _act_bits(self.layers[0], state_dict)
        self.chan, self.cdev = {"input": self.layers[0].ci}, {"input": _pad16(self.layers[0].ci, bw)}
        for l in self.layers:
            if l.kind == "conv":
                self.chan[l.name], self.cdev[l.name] = l.co, _pad16(l.co, bw)
            elif l.kind == "fc":
                self.chan[l.name] = self.cdev[l.name] = l.co
            elif l.kind == "concat":
                for s_ in l.src:
                    if self.chan[s_] != self.cdev[s_]:
                        raise ValueError("concat %s: source %s has padded channels" % (l.name, s_))
                self.chan[l.name] = self.cdev[l.name] = sum(self.chan[s_] for s_ in l.src)
            else:
                self.chan[l.name], self.cdev[l.name] = self.chan[l.src], self.cdev[l.src]
        self.q = {l.name: _decode(l, state_dict, self.device, self.cdev[l.src], self.cdev[l.name], fractional_scale)
                  for l in self.layers if l.kind in ("conv", "fc")}
        self._plan_demands()
        self._graph = None
        # A few-channel int8 network input feeding one k x k convolution: quantize it into a zero frame
        # (the convolution's padding, materialised) and pad the filter rows to whole groups of 4 taps,
        # so the first layer fetches filter rows with plain 16-byte loads on the matrix-core route.
        self.stem = None
        l0 = self.layers[0]
        users = [l for l in self.layers if l.src == "input" or (isinstance(l.src, tuple) and "input" in l.src)
                 or l.add == "input"]
        few = (self.q[l0.name].bw_x, self.cdev["input"]) in ((8, 4), (16, 8)) if l0.kind == "conv" else False
        if l0.kind == "conv" and l0.src == "input" and l0.groups == 1 and l0.k > 1 and users == [l0] and few:
            lq = self.q[l0.name]
            extra = (l0.k + 3) // 4 * 4 - l0.k
            if extra:
                lq.qw = torch.nn.functional.pad(lq.qw, (0, 0, 0, extra)).contiguous()  # [Co,kh,kw+extra,C]
            self.stem = dict(name=l0.name, pad=l0.pad, extra=extra)
        # Projection shortcuts (1x1 convolution, no activation, consumed only as the residual of one
        # convolution): evaluated inside that convolution's launch, their fp32 output is never stored.
        # shortcut_of: main layer name -> shortcut layer; a traced pass runs them as launches of their own.
        self.shortcut_of = {}
        if fuse_shortcuts:
            by_name = {l.name: l for l in self.layers}
            for l in self.layers:
                ds = by_name.get(l.add) if l.kind == "conv" and l.add else None
                if ds is None or ds.kind != "conv" or l.groups != 1:
                    continue
                readers = [m for m in self.layers
                           if m.src == ds.name or (isinstance(m.src, tuple) and ds.name in m.src) or m.add == ds.name]
                lq, dq = self.q[l.name], self.q[ds.name]
                if (ds.k == 1 and ds.pad == 0 and ds.groups == 1 and ds.act == "none" and not ds.add
                        and readers == [l] and ds.name not in self.outputs and not self.q_demand[ds.name]
                        and (lq.bw_x, lq.bw_w, dq.bw_x, dq.bw_w) == (8, 8, 8, 8)
                        and not (self.stem and self.stem["name"] in (l.name, ds.name))):
                    self.shortcut_of[l.name] = ds
        # Residual chains: chain_of[name] = [shortcut layer, last convolution of block 0, .., this layer]
        self.chain_of = {}
        if fuse_shortcuts and chain_links != 0:
            self._plan_chains(chain_links)
        # a shortcut has no launch of its own when its one reader, the first block's last convolution, evaluates it
        # itself (as a two-branch launch or as the head of a chain); later blocks' chains recompute it either way
        self._fused_away = set(ds.name for ds in self.shortcut_of.values())
        self._fused_away.update(links[0].name for links in self.chain_of.values()
                                if links[1].name in self.chain_of or links[1].name in self.shortcut_of)
        # Heads: head_of[3x3 layer name] = the 1x1 layer in front of it.  Whether a pair runs as one launch also
        # depends on the image size (head_fuses), known when a batch arrives.
        self.head_of = {}
        if fuse_heads:
            by_name = {l.name: l for l in self.layers}
            for l in self.layers:
                h = by_name.get(l.src) if l.kind == "conv" and isinstance(l.src, str) else None
                if h is None or h.kind != "conv" or l.name in self.chain_of or l.name in self.shortcut_of:
                    continue
                readers = [m for m in self.layers
                           if m.src == h.name or (isinstance(m.src, tuple) and h.name in m.src) or m.add == h.name]
                lq, hq = self.q[l.name], self.q[h.name]
                if (l.k == 3 and l.pad == 1 and l.stride == 1 and l.groups == 1 and not l.add
                        and h.k == 1 and h.pad == 0 and h.stride == 1 and h.groups == 1 and h.act == "relu" and not h.add
                        and readers == [l] and h.name not in self.outputs and not self.f_demand[h.name]
                        and self.q_demand[h.name] == [(8, lq.pos_x, 1.0)]
                        and (lq.bw_x, lq.bw_w, hq.bw_x, hq.bw_w) == (8, 8, 8, 8) and hq.scale_x == 1.0
                        and hq.chan_div is not None and hq.bias is not None and -64 <= hq.exp2 <= 64
                        and h.name not in self._fused_away and not (self.stem and self.stem["name"] in (l.name, h.name))):
                    self.head_of[l.name] = h
        self._head_names = set(h.name for h in self.head_of.values())
        # Inverted-residual blocks: block_of[projection layer name] = (expansion layer, depthwise layer).
        self.block_of = {}
        if fuse_blocks:
            by_name = {l.name: l for l in self.layers}

            def only_reader(a, b):
                readers = [m for m in self.layers
                           if m.src == a.name or (isinstance(m.src, tuple) and a.name in m.src) or m.add == a.name]
                return (readers == [b] and a.name not in self.outputs and not self.f_demand[a.name]
                        and self.q_demand[a.name] == [(8, self.q[b.name].pos_x, 1.0)])

            def inner_ok(a):
                aq = self.q[a.name]
                return (a.act in ("relu", "relu6") and not a.add and (aq.bw_x, aq.bw_w) == (8, 8) and aq.scale_x == 1.0
                        and aq.chan_div is not None and aq.bias is not None and -64 <= aq.exp2 <= 64
                        and a.name not in self._fused_away and a.name not in self._head_names
                        and not (self.stem and self.stem["name"] == a.name))
            for pl in self.layers:
                d = by_name.get(pl.src) if pl.kind == "conv" and isinstance(pl.src, str) else None
                x = by_name.get(d.src) if d is not None and d.kind == "conv" and isinstance(d.src, str) else None
                if x is None or x.kind != "conv" or pl.name in self.chain_of or pl.name in self.shortcut_of:
                    continue
                pq = self.q[pl.name]
                if (pl.k == 1 and pl.pad == 0 and pl.stride == 1 and pl.groups == 1 and pl.act == "none"
                        and not pl.add_after and (pq.bw_x, pq.bw_w) == (8, 8)
                        and d.k == 3 and d.pad == 1 and d.stride in (1, 2) and d.groups == d.ci == d.co and d.groups > 1
                        and x.k == 1 and x.pad == 0 and x.stride == 1 and x.groups == 1
                        and inner_ok(x) and inner_ok(d) and only_reader(x, d) and only_reader(d, pl)
                        and self.cdev[x.name] == self.cdev[d.name] == x.co):
                    self.block_of[pl.name] = (x, d)
        # First layers: first_pool = the max-pooling layer behind the few-channel first convolution, when the pooled
        # int8 tensor is all that anything reads of the two.
        self.first_pool = None
        if fuse_first_layers and self.stem:
            l0 = self.layers[0]
            lq = self.q[l0.name]
            readers = [m for m in self.layers
                       if m.src == l0.name or (isinstance(m.src, tuple) and l0.name in m.src) or m.add == l0.name]
            pool = readers[0] if len(readers) == 1 and readers[0].kind == "maxpool" else None
            if (pool is not None and l0.act in ("relu", "relu6") and not l0.add and (lq.bw_x, lq.bw_w) == (8, 8)
                    and lq.chan_div is not None and lq.bias is not None and -64 <= lq.exp2 <= 64
                    and self.cdev["input"] == 4 and len(self.q_demand["input"]) == 1
                    and not ({l0.name, pool.name} & set(self.outputs))
                    and not self.f_demand[l0.name] and not self.f_demand[pool.name]
                    and len(self.q_demand[pool.name]) == 1 and self.q_demand[pool.name][0][0] == 8
                    and self.q_demand[pool.name][0][2] == 1.0 and self.q_demand[l0.name] == self.q_demand[pool.name]):
                self.first_pool = pool
        # Global average pooling: pooled_conv[pooling layer name] = the 1x1 convolution in front of it, when nothing else
        # reads that convolution.
        self.pooled_conv = {}
        if fuse_avgpool:
            by_name = {l.name: l for l in self.layers}
            for g in self.layers:
                c = by_name.get(g.src) if g.kind == "gap" and isinstance(g.src, str) else None
                if c is None or c.kind != "conv":
                    continue
                cq = self.q[c.name]
                readers = [m for m in self.layers
                           if m.src == c.name or (isinstance(m.src, tuple) and c.name in m.src) or m.add == c.name]
                if (readers == [g] and c.k == 1 and c.pad == 0 and c.stride == 1 and c.groups == 1
                        and c.act in ("none", "relu", "relu6") and not c.add_after and (cq.bw_x, cq.bw_w) == (8, 8)
                        and cq.chan_div is not None and cq.bias is not None and -64 <= cq.exp2 <= 64
                        and c.name not in self.outputs and not self.q_demand[c.name]
                        and c.name not in self.chain_of and c.name not in self.shortcut_of and c.name not in self.block_of
                        and c.name not in self._fused_away and c.name not in self._head_names
                        and not (self.stem and self.stem["name"] == c.name)):
                    self.pooled_conv[g.name] = c
        self._pooled_names = set(c.name for c in self.pooled_conv.values())
        self._block_inner = {}
        for pname, (x, d) in self.block_of.items():
            self._block_inner[x.name] = pname
            self._block_inner[d.name] = pname

    def block_fuses(self, proj, n, h, w):
        """whether the inverted-residual block that ends in the layer `proj` runs as one launch over n images whose
        block input is h x w.  The one-launch kernel is bound by the same vector arithmetic as the three launches and
        saves their start-up and the hidden tensors' traffic: measured on MobileNetV2 it pays from 14 x 14 outputs
        on; smaller images leave it too few blocks."""
        if proj.name not in self.block_of:
            return False
        x, d = self.block_of[proj.name]
        ho, wo = (h - 1) // d.stride + 1, (w - 1) // d.stride + 1
        if ho * wo < 196:
            return False
        return bool(torch.ops.torch_mlu.inverted_residual_fuses(n, h, w, self.cdev[x.src], self.cdev[x.name],
                                                                self.cdev[proj.name], d.stride))

    def first_layers_fuse(self, n, c, h, w):
        """whether quantizer, first convolution and pooling run as one launch on a contiguous fp32 batch [n, c, h, w]"""
        if self.first_pool is None:
            return False
        l0, pool = self.layers[0], self.first_pool
        return bool(torch.ops.torch_mlu.first_layers_fuse(n, c, h, w, self.cdev[l0.name], l0.k, l0.stride, l0.pad, pool.k,
                                                          pool.stride, pool.pad))

    def avgpool_fuses(self, gap, n, h, w):
        """whether the 1x1 convolution in front of the pooling layer `gap` runs inside the pooling's launch over n images
        of h x w"""
        c = self.pooled_conv.get(gap.name)
        if c is None:
            return False
        return bool(torch.ops.torch_mlu.conv1x1_avgpool_fuses(n, h * w, self.cdev[c.src], self.cdev[c.name]))

    def head_fuses(self, head, n, h, w):
        """whether the 1x1 layer `head` and the 3x3 layer behind it run as one launch over n images of h x w"""
        if head.name not in self._head_names:
            return False
        main = next(l for l in self.layers if self.head_of.get(l.name) is head)
        return bool(torch.ops.torch_mlu.conv1x1_conv3x3_fuses(n, h, w, self.cdev[head.src], self.cdev[head.name],
                                                             self.cdev[main.name]))

    @staticmethod
    def _default_chain_links(co):
        """Longest chain worth recomputing.  A link costs 2*K matrix-core operations and ~7 vector
        operations per output element and saves 8 bytes of fp32 traffic; measured on ResNet-50 (224 x 224,
        32 images per launch) the trade pays for the first two blocks of the widest stage and for the
        projection blocks of the others."""
        return 3 if co <= 256 else 2

    def _plan_chains(self, chain_links):
        by_name = {l.name: l for l in self.layers}

        def pointwise(l, act, need_add):
            lq = self.q.get(l.name)
            return (l.kind == "conv" and l.k == 1 and l.pad == 0 and l.groups == 1 and l.act == act
                    and bool(l.add) == need_add and not l.add_after and lq is not None
                    and (lq.bw_x, lq.bw_w) == (8, 8) and lq.chan_div is not None and lq.bias is not None
                    and lq.scale_x == 1.0 and -64 <= lq.exp2 <= 64 and self.cdev[l.src] % 64 == 0
                    and not (self.stem and self.stem["name"] == l.name))

        for l in self.layers:
            if l.kind != "conv" or not l.add or l.stride != 1 or not pointwise(l, "relu", True):
                continue
            if self.out_half and l.name in self.outputs:
                continue
            links, cur = [l], l
            while True:
                r = by_name.get(cur.add)
                if r is None:
                    links = None
                    break
                if pointwise(r, "relu", True) and r.stride == 1:
                    links.append(r)
                    cur = r
                    continue
                if pointwise(r, "none", False) and r.name not in self.outputs:
                    readers = [m for m in self.layers
                               if m.src == r.name or (isinstance(m.src, tuple) and r.name in m.src) or m.add == r.name]
                    if readers == [cur]:
                        links.append(r)
                        break
                links = None
                break
            if links is None or len(links) > 8:
                continue
            limit = chain_links
            if limit is None:
                limit = self._default_chain_links(self.cdev[l.name])
            qd = self.q_demand[l.name]
            if len(links) > limit or len(qd) > 1 or (qd and (qd[0][0] != 8 or qd[0][2] != 1.0)):
                continue
            self.chain_of[l.name] = links[::-1]
            self.shortcut_of.pop(l.name, None)
        if self.chain_of:
            self._plan_demands()

    def padding(self, layer):
        """padding the layer's convolution call gets (the stem's lives in its input frame)"""
        if self.stem and layer.name == self.stem["name"]:
            return [0, 0]
        return [layer.pad, layer.pad]

    # which forms of every tensor are needed: 'f' (fp32 NHWC) and/or quantized at (bitwidth, position, scale)
    def _plan_demands(self):
        names = ["input"] + [l.name for l in self.layers]
        self.q_demand = {n: [] for n in names}
        self.f_demand = {n: False for n in names}
        for o in self.outputs:
            self.f_demand[o] = True

        def want_q(t, d):
            if d not in self.q_demand[t]:
                self.q_demand[t].append(d)

        for l in reversed(self.layers):
            if l.kind in ("conv", "fc"):
                lq = self.q[l.name]
                want_q(l.src, (lq.bw_x, lq.pos_x, lq.scale_x))
                if l.add and l.name not in getattr(self, "chain_of", {}):
                    self.f_demand[l.add] = True
            elif l.kind == "gap":
                self.f_demand[l.src] = True
            elif l.kind in _PASS:
                for s in ((l.src,) if isinstance(l.src, str) else l.src):
                    for d in self.q_demand[l.name]:
                        want_q(s, d)
                    self.f_demand[s] = self.f_demand[s] or self.f_demand[l.name]
        # a conv epilogue writes one quantized form; further ones are quantized from the fp32 copy
        for l in self.layers:
            if l.kind in ("conv", "fc") and len(self.q_demand[l.name]) > 1:
                self.f_demand[l.name] = True

    # ------------------------------------------------------------------------------------------
    def forward(self, x, trace=None, timers=None, keep=None):
        """x: [N,3,H,W] fp32 (NCHW) on the device.  trace: optional dict filled with, per conv/fc
        layer, its quantized input, int32 accumulators and fp32 output (as NHWC tensors).
        keep: optional dict that receives every tensor the plan itself produces, keyed (name, "f") for an
        fp32 (or fp16 output) NHWC tensor and (name, bitwidth, position, scale) for a quantized one -- the
        untraced plan's own launches, unlike trace, which asks every layer for extra outputs.
        timers: optional dict; every conv/fc launch is bracketed by a pair of events recorded on
        the current stream and the pair is appended to timers[layer name] (durations of the
        launches in their real sequence, caches as the previous layer left them)."""
        ops = torch.ops.torch_mlu
        env = {}
        tracing = trace is not None

        def tick(name):
            if timers is None:
                return None
            ev = torch.cuda.Event(enable_timing=True)
            ev.record()
            timers.setdefault(name, []).append(ev)
            return ev
        first_fused = set()
        if not tracing and x.dtype == torch.float32 and x.is_contiguous() and self.first_layers_fuse(*x.shape):
            l0, pool, d = self.layers[0], self.first_pool, self.q_demand["input"][0]
            lq, qd = self.q[l0.name], self.q_demand[self.first_pool.name][0]
            tick(l0.name)
            env[(pool.name,) + qd] = ops.qconv2d_first_layers(x, d[1], d[2], lq.qw, lq.exp2, lq.chan_div, lq.bias,
                                                              _ACT_CODE[l0.act], qd[1], l0.k, l0.stride, l0.pad, pool.k,
                                                              pool.stride, pool.pad)
            tick(l0.name)
            first_fused = {l0.name, pool.name}
        for d in self.q_demand["input"] if not first_fused else ():
            if self.stem:
                sp, h, w = self.stem["pad"], x.shape[2], x.shape[3]
                env[("input",) + d] = ops.quantize_nhwc_frame(x, d[0], d[1], self.cdev["input"], h + 2 * sp,
                                                              w + 2 * sp + self.stem["extra"], sp, sp, d[2])
            else:
                env[("input",) + d] = ops.quantize_nhwc(x, d[0], d[1], self.cdev["input"], d[2])
        skipped_heads = set()
        skipped_inner = set()
        pooled_inside = set()
        by_name = {l.name: l for l in self.layers}
        for l in self.layers:
            name = l.name
            if name in first_fused:
                continue
            if l.kind == "conv" and not tracing and name in self._pooled_names:
                lq = self.q[name]
                px = env[(l.src, lq.bw_x, lq.pos_x, lq.scale_x)]
                gap = next(g for g in self.layers if self.pooled_conv.get(g.name) is l)
                if self.avgpool_fuses(gap, px.shape[0], px.shape[1], px.shape[2]):
                    pooled_inside.add(name)  # computed inside the launch of the pooling behind it
                    continue
            if l.kind == "conv" and not tracing and name in self._block_inner:
                pl = by_name[self._block_inner[name]]
                x_, d_ = self.block_of[pl.name]
                if l is x_:
                    bx = env[(l.src, 8, self.q[name].pos_x, 1.0)]
                    if self.block_fuses(pl, bx.shape[0], bx.shape[1], bx.shape[2]):
                        skipped_inner.add(name)  # computed inside the launch of the block's projection
                        continue
                elif x_.name in skipped_inner:
                    skipped_inner.add(name)
                    continue
            if l.kind == "conv" and name in self.block_of and self.block_of[name][1].name in skipped_inner:
                x_, d_ = self.block_of[name]
                lq, xq, dq = self.q[name], self.q[x_.name], self.q[d_.name]
                qd = self.q_demand[name][0] if self.q_demand[name] else None
                want_y = self.f_demand[name] or qd is None
                resid = env[(l.add, "f")] if l.add else None
                tick(name)
                y, q = ops.qconv2d_irb(env[(x_.src, 8, xq.pos_x, 1.0)], xq.qw, xq.exp2, xq.chan_div, xq.bias,
                                       _ACT_CODE[x_.act], dq.pos_x, dq.qw, d_.stride, dq.exp2, dq.chan_div, dq.bias,
                                       _ACT_CODE[d_.act], lq.pos_x, lq.qw, lq.exp2, lq.chan_div, lq.bias, resid, want_y,
                                       self.out_half and name in self.outputs, qd[0] if qd else 0, qd[1] if qd else 0,
                                       qd[2] if qd else 1.0)
                tick(name)
                if want_y:
                    env[(name, "f")] = y
                if qd:
                    env[(name,) + qd] = q
                for dd in self.q_demand[name][1:]:
                    env[(name,) + dd] = ops.quantize(y, dd[0], dd[1], dd[2])
                continue
            if l.kind == "conv" and not tracing and name in self._fused_away:
                continue
            if l.kind == "conv" and not tracing and name in self._head_names:
                hx = env[(l.src, 8, self.q[name].pos_x, 1.0)]
                if self.head_fuses(l, hx.shape[0], hx.shape[1], hx.shape[2]):
                    skipped_heads.add(name)  # computed inside the launch of the 3x3 layer behind it
                    continue
            if l.kind == "conv" and name in self.head_of and self.head_of[name].name in skipped_heads:
                lq, h = self.q[name], self.head_of[name]
                hq = self.q[h.name]
                qd = self.q_demand[name][0] if self.q_demand[name] else None
                want_y = self.f_demand[name] or qd is None
                tick(name)
                y, q = ops.qconv2d_head(env[(h.src, 8, hq.pos_x, 1.0)], hq.qw, hq.exp2, hq.chan_div, hq.bias, lq.pos_x,
                                        lq.qw, lq.exp2, lq.chan_div, lq.bias, self.padding(l), [1, 1], [1, 1],
                                        _ACT_CODE[l.act], want_y, self.out_half and name in self.outputs,
                                        qd[0] if qd else 0, qd[1] if qd else 0, qd[2] if qd else 1.0, LEAKY_SLOPE)
                tick(name)
                if want_y:
                    env[(name, "f")] = y
                if qd:
                    env[(name,) + qd] = q
                for d in self.q_demand[name][1:]:
                    env[(name,) + d] = ops.quantize(y, d[0], d[1], d[2])
                continue
            if l.kind == "conv":
                lq = self.q[name]
                qx = env[(l.src, lq.bw_x, lq.pos_x, lq.scale_x)]
                qd = self.q_demand[name][0] if self.q_demand[name] else None
                want_y = self.f_demand[name] or tracing or qd is None
                ds = None if tracing else self.shortcut_of.get(name)
                chain = None if tracing else self.chain_of.get(name)
                tick(name)
                if chain is not None:
                    cq = [self.q[c.name] for c in chain]
                    y, q = ops.qconv2d_chain([env[(c.src, 8, k.pos_x, k.scale_x)] for c, k in zip(chain, cq)],
                                             [k.qw for k in cq], [c.stride for c in chain], [k.exp2 for k in cq],
                                             [k.chan_div for k in cq], [k.bias for k in cq], want_y,
                                             8 if qd else 0, qd[1] if qd else 0)
                    acc = None
                elif ds is not None:
                    dq = self.q[ds.name]
                    y, q = ops.qconv2d_shortcut(qx, lq.qw, lq.exp2, lq.chan_div, lq.bias,
                                                env[(ds.src, dq.bw_x, dq.pos_x, dq.scale_x)], dq.qw, ds.stride, dq.exp2,
                                                dq.chan_div, dq.bias, self.padding(l), [l.stride, l.stride], [1, 1],
                                                _ACT_CODE[l.act], want_y, self.out_half and name in self.outputs,
                                                qd[0] if qd else 0, qd[1] if qd else 0, qd[2] if qd else 1.0, LEAKY_SLOPE,
                                                bool(l.add_after))
                    acc = None
                else:
                    resid = env[(l.add, "f")] if l.add else None
                    y, q, acc = ops.qconv2d(qx, lq.qw, lq.exp2, lq.chan_div, lq.bias, resid, self.padding(l),
                                            [l.stride, l.stride], [1, 1], lq.groups, _ACT_CODE[l.act], want_y,
                                            self.out_half and name in self.outputs, tracing,
                                            qd[0] if qd else 0, qd[1] if qd else 0, qd[2] if qd else 1.0, LEAKY_SLOPE,
                                            bool(l.add_after))
                tick(name)
                if want_y:
                    env[(name, "f")] = y
                if qd:
                    env[(name,) + qd] = q
                for d in self.q_demand[name][1:]:
                    env[(name,) + d] = ops.quantize(y, d[0], d[1], d[2])
                if tracing:
                    trace[name] = dict(qx=qx, acc=acc, y=y)
                    if self.stem and name == self.stem["name"]:  # the image inside the frame
                        sp = self.stem["pad"]
                        trace[name]["qx_dev"] = qx
                        trace[name]["qx"] = qx[:, sp:qx.shape[1] - sp, sp:qx.shape[2] - sp - self.stem["extra"]].contiguous()
            elif l.kind == "fc":
                lq = self.q[name]
                qx = env[(l.src, lq.bw_x, lq.pos_x, lq.scale_x)]
                qx2 = qx.reshape(qx.shape[0], lq.qw.shape[1])  # not -1: an empty batch leaves it ambiguous
                tick(name)
                y, _, acc = ops.qlinear(qx2, lq.qw, lq.exp2, lq.chan_div, lq.bias, 0, True, False, tracing, 0, 0, 1.0)
                tick(name)
                env[(name, "f")] = y
                if tracing:
                    trace[name] = dict(qx=qx2, acc=acc, y=y)
            elif l.kind == "maxpool":
                for form in self._forms(name):
                    env[(name,) + form] = ops.maxpool_nhwc(env[(l.src,) + form], l.k, l.stride, l.pad)
            elif l.kind == "gap" and l.src in pooled_inside:
                c = self.pooled_conv[name]
                cq = self.q[c.name]
                qds = self.q_demand[name]
                want_mean = self.f_demand[name] or len(qds) != 1
                qd = qds[0] if qds else None
                tick(c.name)
                mean, q = ops.qconv2d_avgpool(env[(c.src, cq.bw_x, cq.pos_x, cq.scale_x)], cq.qw, cq.exp2, cq.chan_div, cq.bias,
                                              env[(c.add, "f")] if c.add else None, _ACT_CODE[c.act], want_mean,
                                              qd[0] if qd else 0, qd[1] if qd else 0, qd[2] if qd else 1.0)
                tick(c.name)
                if want_mean:
                    env[(name, "f")] = mean.reshape(mean.shape[0], 1, 1, mean.shape[1])
                if qd:
                    env[(name,) + qd] = q.reshape(q.shape[0], 1, 1, q.shape[1])
                for d in qds[1:]:
                    env[(name,) + d] = ops.quantize(env[(name, "f")], d[0], d[1], d[2])
            elif l.kind == "gap":
                if self.f_demand[name] or tracing or not self.q_demand[name]:
                    g = ops.global_avgpool_nhwc(env[(l.src, "f")])
                    env[(name, "f")] = g.reshape(g.shape[0], 1, 1, g.shape[1])
                    for d in self.q_demand[name]:
                        env[(name,) + d] = ops.quantize(env[(name, "f")], d[0], d[1], d[2])
                else:  # only quantized forms are read: pooled and quantized in one launch each
                    for d in self.q_demand[name]:
                        g = ops.global_avgpool_nhwc(env[(l.src, "f")], d[0], d[1], d[2])
                        env[(name,) + d] = g.reshape(g.shape[0], 1, 1, g.shape[1])
            elif l.kind == "upsample":
                for form in self._forms(name):
                    t = env[(l.src,) + form]
                    env[(name,) + form] = t.repeat_interleave(2, 1).repeat_interleave(2, 2)
            elif l.kind == "concat":
                for form in self._forms(name):
                    env[(name,) + form] = torch.cat([env[(s,) + form] for s in l.src], 3)
            else:
                raise ValueError(l.kind)
        if keep is not None:
            keep.update(env)
        outs = []
        for o in self.outputs:
            y = env[(o, "f")]
            if y.dim() == 4:  # logical NCHW over NHWC memory, padding channels dropped
                y = y.permute(0, 3, 1, 2)[:, :self.chan[o]]
            outs.append(y)
        return outs[0] if len(outs) == 1 else tuple(outs)

    __call__ = forward

    def _forms(self, name):
        forms = [tuple(d) for d in self.q_demand[name]]
        if self.f_demand[name]:
            forms.append(("f",))
        return forms

    # ------------------------------------------------------------------------------------------
    def capture(self, example, streams=1):
        """Record one forward pass into a HIP graph; returns (static_input, replay) where replay()
        re-runs the whole network on whatever static_input holds and returns the static output(s).

        streams > 1 splits the batch into that many parts, each recorded on a stream of its own (all of
        default priority) between a fork and a join: the images are independent, so the results are the
        same tensors, and the launches of one part fill the compute units that the other part's launches
        leave idle while they start up and drain."""
        static_in = example.clone()
        parts = max(1, min(int(streams), static_in.shape[0]))
        chunks = list(static_in.chunk(parts))
        side = [torch.cuda.Stream() for _ in chunks]
        # the launches recorded below will share the device: their tile shapes are chosen for a part of it (a hint
        # of this thread, handed to the kernel library with every call)
        before = torch.ops.torch_mlu.set_launch_sharing(len(chunks))
        try:
            return self._capture(static_in, chunks, side)
        finally:
            torch.ops.torch_mlu.set_launch_sharing(max(before, 1))

    def _capture(self, static_in, chunks, side):
        """Side streams only ever wait on the capturing stream (fork) and are only ever waited on by it (join).
        Waits between two side streams in both directions inside one capture ended a capture with a segmentation
        fault inside the runtime's end-of-capture call; nothing here may introduce such a wait."""
        cur0 = torch.cuda.current_stream()
        if len(set(s.cuda_stream for s in side)) != len(side) or any(s.cuda_stream == cur0.cuda_stream for s in side):
            raise ValueError("capture: every part needs a side stream of its own, distinct from the capturing stream")
        sample = None
        for st, c in zip(side, chunks):  # warm-up outside the capture, on the streams the graph will use
            st.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(st):
                for _ in range(2):
                    sample = self.forward(c)
        for st in side:
            torch.cuda.current_stream().wait_stream(st)
        torch.cuda.synchronize()
        # the whole batch's outputs, allocated outside the graph; every part fills its rows
        sample_outs = sample if isinstance(sample, tuple) else (sample,)
        whole = [torch.empty((static_in.shape[0],) + tuple(o.shape[1:]), dtype=o.dtype, device=o.device,
                             memory_format=torch.channels_last if o.dim() == 4 else torch.contiguous_format)
                 for o in sample_outs]  # feature maps stay NHWC in memory, like the parts' own outputs
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            if len(chunks) == 1:
                static_out = self.forward(static_in)
            else:
                # every part copies its outputs into its rows of the whole batch's outputs on its own stream
                cur = torch.cuda.current_stream()
                row = 0
                for st, c in zip(side, chunks):
                    st.wait_stream(cur)
                    with torch.cuda.stream(st):
                        out = self.forward(c)
                        for w_, o in zip(whole, out if isinstance(out, tuple) else (out,)):
                            w_[row:row + c.shape[0]].copy_(o)
                    row += c.shape[0]
                for st in side:
                    cur.wait_stream(st)
                static_out = tuple(whole) if isinstance(sample, tuple) else whole[0]
        self._graph = graph
        # the first replays of a new graph are slower (the executable graph is uploaded on first use): take them here
        for _ in range(8):
            graph.replay()
        torch.cuda.synchronize()

        def replay():
            graph.replay()
            return static_out

        return static_in, replay


def calibrate(float_net, x_cpu, dtype="int8", per_channel=True):
    """Run the reference-style calibration flow on the CPU and return the checkpoint
    (weights + scale / quantized_mode / scale_weight_per_channel per layer)."""
    from .core.mlu_quantize import quantize_dynamic_mlu
    spec = {"use_avg": False, "data_scale": 1.0, "per_channel": per_channel, "firstconv": False, "iteration": 1}
    calib = quantize_dynamic_mlu(float_net, spec, dtype=dtype, gen_quant=True)
    with torch.no_grad():
        calib(x_cpu)
    sd = calib.state_dict()
    # merge the per-channel scales the way the modules do when they load the checkpoint
    out = {}
    for k, v in sd.items():
        out[k] = v
    for k in list(sd.keys()):
        if k.endswith(".scale"):
            p = k[:-len("scale")]
            if p + "scale_weight_per_channel" in sd:
                out[k] = torch.cat((sd[k], sd[p + "scale_weight_per_channel"])).float()
                m = int(sd[p + "quantized_mode"].item())
                out[p + "quantized_mode"] = torch.tensor([m + 2 if m in (1, 2) else m], dtype=torch.int32)
    return out


def to_position_encoding(sd, bw_x=16, bw_w=8):
    """Rewrite a per-tensor checkpoint into the reference's second q-param encoding:
    ``scale = [bitwidth_input, bitwidth_weight]``, ``quantized_mode = [position_input,
    position_weight]`` (quantify_conv_forward.cpp:79-88), pure power-of-two quantization.  The
    activation range is recovered from the calibrated scale (scale = qmax / absmax), the weight
    range is the tensor's own max-abs."""
    out = dict(sd)
    for k in list(sd.keys()):
        if not k.endswith(".quantized_mode"):
            continue
        p = k[:-len("quantized_mode")]
        m = int(sd[k].reshape(-1)[0].item())
        qmax_cal = 127.0 if m in (1, 3) else 32767.0
        absmax_x = qmax_cal / float(sd[p + "scale"].reshape(-1)[0].item())
        absmax_w = float(sd[p + "weight"].abs().max().item())
        qx, qw = float(2 ** (bw_x - 1) - 1), float(2 ** (bw_w - 1) - 1)
        pos_x = pos_from_scale(bw_x, qx / absmax_x)
        pos_w = pos_from_scale(bw_w, qw / absmax_w if absmax_w > 0 else 1.0)
        out[p + "scale"] = torch.tensor([float(bw_x), float(bw_w)])
        out[k] = torch.tensor([pos_x, pos_w], dtype=torch.int32)
    return out
