"""Workload definitions for the quantized-inference benchmarks and parity tests.

A network is a list of ``Layer`` records (a tiny graph IR): every layer names its input tensor(s)
and produces one tensor under its own name.  From one description we build
  * ``FloatNet``      -- an ordinary torch.nn model (float reference, calibration, and the
                         module-swap drop-in flow through ``quantize_dynamic_mlu``),
  * the fused int8 plan of ``catch_amd.pipeline``,
so all of them are the same network by construction.

Architectures are written out here (torchvision is not a dependency): ResNet-18 / ResNet-50 v1.5
(stride on the 3x3), MobileNetV2 (width 1.0), Darknet-53 with three YOLOv3 heads.  Batch norm is
folded: with freshly initialised statistics (gamma=1, beta=0, mean=0, var=1) folding multiplies
the weights by 1/sqrt(1+eps) and leaves a zero bias.
"""
import math
from collections import namedtuple

import torch
import torch.nn as nn
import torch.nn.functional as F

Layer = namedtuple("Layer", "kind name src ci co k stride pad groups act add add_after")
Layer.__new__.__defaults__ = (None,) * 12

LEAKY_SLOPE = 0.1

BN_EPS = 1e-5


def conv(name, src, ci, co, k, stride=1, pad=None, groups=1, act="relu", add=None, add_after=False):
    """add: tensor added to the convolution's output, before the activation (ResNet) or, with
    add_after, after it (Darknet's shortcut layers)."""
    return Layer("conv", name, src, ci, co, k, stride, (k // 2) if pad is None else pad, groups, act, add,
                 bool(add_after))


def maxpool(name, src, k, stride, pad):
    return Layer("maxpool", name, src, None, None, k, stride, pad, None, None, None)


def gap(name, src):
    return Layer("gap", name, src)


def fc(name, src, ci, co):
    return Layer("fc", name, src, ci, co, None, None, None, None, "none", None)


def upsample(name, src):
    return Layer("upsample", name, src)


def concat(name, srcs):
    return Layer("concat", name, tuple(srcs))


# ----------------------------------------------------------------------------------------------
def resnet(depth, num_classes=1000):
    """ResNet v1.5: in a bottleneck the stride sits on the 3x3 convolution."""
    cfg = {18: ("basic", [2, 2, 2, 2]), 34: ("basic", [3, 4, 6, 3]), 50: ("bottleneck", [3, 4, 6, 3])}[depth]
    block, counts = cfg
    L = [conv("conv1", "input", 3, 64, 7, 2, 3), maxpool("pool1", "conv1", 3, 2, 1)]
    x, cin = "pool1", 64
    for stage, (n, width) in enumerate(zip(counts, [64, 128, 256, 512])):
        for i in range(n):
            stride = 2 if (i == 0 and stage > 0) else 1
            p = "l%d.%d." % (stage + 1, i)
            cout = width * (4 if block == "bottleneck" else 1)
            ident = x
            if stride != 1 or cin != cout:
                L.append(conv(p + "ds", x, cin, cout, 1, stride, 0, act="none"))
                ident = p + "ds"
            if block == "bottleneck":
                L.append(conv(p + "c1", x, cin, width, 1))
                L.append(conv(p + "c2", p + "c1", width, width, 3, stride))
                L.append(conv(p + "c3", p + "c2", width, cout, 1, act="relu", add=ident))
                x = p + "c3"
            else:
                L.append(conv(p + "c1", x, cin, width, 3, stride))
                L.append(conv(p + "c2", p + "c1", width, cout, 3, act="relu", add=ident))
                x = p + "c2"
            cin = cout
    L += [gap("gap", x), fc("fc", "gap", cin, num_classes)]
    return L


def mobilenet_v2(num_classes=1000):
    setting = [(1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2), (6, 320, 1, 1)]
    L = [conv("stem", "input", 3, 32, 3, 2, 1, act="relu6")]
    x, cin, b = "stem", 32, 0
    for t, c, n, s in setting:
        for i in range(n):
            stride = s if i == 0 else 1
            p = "b%d." % b
            hid = cin * t
            y = x
            if t != 1:
                L.append(conv(p + "exp", y, cin, hid, 1, act="relu6"))
                y = p + "exp"
            L.append(conv(p + "dw", y, hid, hid, 3, stride, 1, groups=hid, act="relu6"))
            L.append(conv(p + "proj", p + "dw", hid, c, 1, act="none", add=x if (stride == 1 and cin == c) else None))
            x, cin, b = p + "proj", c, b + 1
    L += [conv("head", x, cin, 1280, 1, act="relu6"), gap("gap", "head"), fc("fc", "gap", 1280, num_classes)]
    return L


def darknet53_yolov3(num_outputs=255):
    """Darknet-53 backbone + the three YOLOv3 detection heads (13/26/52 grids at 416x416)."""
    L = []
    cnt = [0]

    def cbl(src, ci, co, k, stride=1, act="leaky", add=None):
        cnt[0] += 1
        name = "c%d" % cnt[0]
        L.append(conv(name, src, ci, co, k, stride, k // 2, act=act, add=add, add_after=True))
        return name

    x = cbl("input", 3, 32, 3)
    cin = 32
    routes = {}
    for stage, (co, n) in enumerate([(64, 1), (128, 2), (256, 8), (512, 8), (1024, 4)]):
        x = cbl(x, cin, co, 3, 2)
        for _ in range(n):
            y = cbl(x, co, co // 2, 1)
            x = cbl(y, co // 2, co, 3, add=x)  # shortcut: input + leaky(conv), linear afterwards
        cin = co
        routes[stage] = x

    def head(src, ci, mid, tag):
        y = src
        c = ci
        for i in range(3):
            y = cbl(y, c, mid, 1)
            c = mid
            if i < 2:
                y = cbl(y, mid, mid * 2, 3)
                c = mid * 2
        branch = y
        y = cbl(y, mid, mid * 2, 3)
        cnt[0] += 1
        out = "yolo%s" % tag
        L.append(conv(out, y, mid * 2, num_outputs, 1, 1, 0, act="none"))
        return branch, out

    b13, _ = head(routes[4], 1024, 512, "13")
    u = cbl(b13, 512, 256, 1)
    L.append(upsample("up26", u))
    L.append(concat("cat26", ["up26", routes[3]]))
    b26, _ = head("cat26", 256 + 512, 256, "26")
    u = cbl(b26, 256, 128, 1)
    L.append(upsample("up52", u))
    L.append(concat("cat52", ["up52", routes[2]]))
    head("cat52", 128 + 256, 128, "52")
    return L


NETS = {"resnet18": lambda: resnet(18), "resnet50": lambda: resnet(50), "mobilenet_v2": mobilenet_v2,
        "darknet53_yolov3": darknet53_yolov3}


def outputs_of(layers):
    used = set()
    for l in layers:
        for s in ((l.src,) if isinstance(l.src, str) else (l.src or ())):
            used.add(s)
        if l.add:
            used.add(l.add)
    return [l.name for l in layers if l.name not in used]


def conv_macs(layers, n, h, w):
    """multiply-accumulates of the conv/fc layers for an n x 3 x h x w input"""
    shape = {"input": (h, w)}
    total = 0
    for l in layers:
        if l.kind == "conv":
            hi, wi = shape[l.src]
            ho, wo = (hi + 2 * l.pad - l.k) // l.stride + 1, (wi + 2 * l.pad - l.k) // l.stride + 1
            shape[l.name] = (ho, wo)
            total += n * ho * wo * l.co * (l.ci // l.groups) * l.k * l.k
        elif l.kind == "maxpool":
            hi, wi = shape[l.src]
            shape[l.name] = ((hi + 2 * l.pad - l.k) // l.stride + 1, (wi + 2 * l.pad - l.k) // l.stride + 1)
        elif l.kind == "gap":
            shape[l.name] = (1, 1)
        elif l.kind == "fc":
            shape[l.name] = (1, 1)
            total += n * l.ci * l.co
        elif l.kind == "upsample":
            hi, wi = shape[l.src]
            shape[l.name] = (hi * 2, wi * 2)
        elif l.kind == "concat":
            shape[l.name] = shape[l.src[0]]
    return total


# ----------------------------------------------------------------------------------------------
_ACT = {"none": lambda x: x, "relu": F.relu, "relu6": F.relu6, "leaky": lambda x: F.leaky_relu(x, LEAKY_SLOPE)}


class FloatNet(nn.Module):
    """The float model of a layer list: plain nn.Conv2d / nn.Linear children (so that
    ``quantize_dynamic_mlu`` can swap them) wired according to the description.  weight_std: one
    standard deviation for every layer, or "he" for sqrt(2 / fan_in) per layer, a quarter of that on
    convolutions whose output is added to a shortcut (keeps activations of deep stacks at unit scale)."""

    def __init__(self, layers, seed=0, weight_std=0.05):
        super().__init__()
        self.layers = list(layers)
        self.outputs = outputs_of(layers)
        g = torch.Generator().manual_seed(seed)
        mods = {}
        fold = 1.0 / math.sqrt(1.0 + BN_EPS)
        for l in self.layers:
            if l.kind == "conv":
                m = nn.Conv2d(l.ci, l.co, l.k, l.stride, l.pad, 1, l.groups, bias=True)
                with torch.no_grad():
                    std = weight_std
                    if weight_std == "he":  # the last convolution of a residual branch starts small
                        std = math.sqrt(2.0 / (l.ci // l.groups * l.k * l.k)) * (0.25 if l.add else 1.0)
                    m.weight.copy_(torch.randn(m.weight.shape, generator=g) * std * fold)
                    m.bias.zero_()
                mods[l.name.replace(".", "_")] = m
            elif l.kind == "fc":
                m = nn.Linear(l.ci, l.co, bias=True)
                with torch.no_grad():
                    std = math.sqrt(1.0 / l.ci) if weight_std == "he" else weight_std
                    m.weight.copy_(torch.randn(m.weight.shape, generator=g) * std)
                    m.bias.copy_(torch.randn(m.bias.shape, generator=g) * std)
                mods[l.name.replace(".", "_")] = m
        self.mods = nn.ModuleDict(mods)

    def module_of(self, name):
        return self.mods[name.replace(".", "_")]

    def forward(self, x, keep=False):
        t = {"input": x}
        for l in self.layers:
            if l.kind == "conv":
                y = self.module_of(l.name)(t[l.src])
                if l.add and not l.add_after:
                    y = y + t[l.add]
                y = _ACT[l.act](y)
                if l.add and l.add_after:
                    y = y + t[l.add]
            elif l.kind == "maxpool":
                y = F.max_pool2d(t[l.src], l.k, l.stride, l.pad)
            elif l.kind == "gap":
                y = t[l.src].mean((2, 3))
            elif l.kind == "fc":
                y = self.module_of(l.name)(t[l.src])
            elif l.kind == "upsample":
                y = F.interpolate(t[l.src], scale_factor=2, mode="nearest")
            elif l.kind == "concat":
                y = torch.cat([t[s] for s in l.src], 1)
            else:
                raise ValueError(l.kind)
            t[l.name] = y
        if keep:
            return t
        outs = [t[o] for o in self.outputs]
        return outs[0] if len(outs) == 1 else tuple(outs)
