"""Lowering of a traced model to the fused integer plan.

The reference's fusion mode converts the ``torch_mlu::conv2d`` / ``torch_mlu::linear`` nodes of a
TorchScript graph, together with their float neighbours, into one compiled network with the
quantization ranges taken from the nodes' ``q_scale`` / ``q_mode`` operands
(torch_mlu/csrc/jit/codegen/convertion/ops/conv.cpp:69-132,180-216; matmul.cpp:37-106,183-214).
This module is the counterpart for this build: it walks the frozen graph of a traced module,
maps

    torch_mlu::conv2d [-> aten::add] [-> relu | relu6 | hardtanh(0,6) | leaky_relu] [-> aten::add]
    torch_mlu::linear, aten::max_pool2d, aten::adaptive_avg_pool2d / aten::mean over (2,3),
    aten::upsample_nearest2d (x2), aten::cat over channels, shape-only ops after the pooling

onto the layer records of ``catch_amd.nets`` plus a checkpoint dictionary, and hands both to
``catch_amd.pipeline.FusedNet`` -- so a model prepared with ``quantize_dynamic_mlu`` and traced
with ``torch.jit.trace`` runs with int8/int16 activations between its layers and one HIP graph
instead of one float tensor per op.  Anything outside this vocabulary raises ``LoweringError``:
there is no silent fall-back.
"""
import torch

from .nets import LEAKY_SLOPE, Layer
from .pipeline import FusedNet


class LoweringError(RuntimeError):
    pass


_PASS_THROUGH = ("aten::flatten", "aten::view", "aten::reshape", "aten::contiguous", "aten::squeeze",
                 "aten::dropout", "aten::feature_dropout", "aten::detach", "aten::clone")
_IGNORED = ("prim::Constant", "prim::ListConstruct", "aten::size", "aten::Int", "prim::NumToTensor",
            "aten::mul", "aten::floor_divide", "aten::floordiv", "aten::ScalarImplicit")


def _const(value):
    """python value of a graph value that is a constant (or a list of constants), else None"""
    node = value.node()
    if node.kind() == "prim::Constant":
        return value.toIValue()
    if node.kind() == "prim::ListConstruct":
        items = [_const(v) for v in node.inputs()]
        return None if any(i is None for i in items) else items
    return None


def _need(value, what, node):
    c = _const(value)
    if c is None:
        raise LoweringError("%s of %s is not a constant of the frozen graph" % (what, node.kind()))
    return c


def _pair(v, what):
    v = list(v) if isinstance(v, (list, tuple)) else [v, v]
    if len(v) == 1:
        v = v * 2
    if len(v) != 2 or v[0] != v[1]:
        raise LoweringError("%s %s: only equal values for both image dimensions are supported" % (what, v))
    return int(v[0])


def graph_to_layers(graph):
    """-> (layers, state_dict, output_names) of a frozen TorchScript graph"""
    inputs = [v for v in graph.inputs() if v.type().kind() == "TensorType"]
    if len(inputs) != 1:
        raise LoweringError("expected one tensor input, found %d" % len(inputs))
    name_of = {inputs[0].unique(): "input"}   # id of a graph value -> tensor name of the plan
    recs, sd = [], {}                # layer records as dicts (mutable while neighbours are fused in)
    by_name = {}

    def uses(v):
        return len(v.uses())

    def src(v, node):
        if v.unique() not in name_of:
            raise LoweringError("%s consumes a value produced by an unsupported node (%s)" % (node.kind(), v.node().kind()))
        return name_of[v.unique()]

    def open_conv(v):
        """the conv record that produced v, if v is that record's current output and nothing else reads it"""
        r = by_name.get(name_of.get(v.unique()))
        if r is not None and r["kind"] == "conv" and r["out"] == v.unique() and uses(v) == 1:
            return r
        return None

    for node in graph.nodes():
        kind = node.kind()
        ins = list(node.inputs())
        if kind in _IGNORED:
            continue
        if kind in ("torch_mlu::conv2d", "torch_mlu::linear"):
            name = "n%d" % len(recs)
            w = _need(ins[1], "weight", node)
            b = _const(ins[2])
            off = 3 if kind == "torch_mlu::linear" else 7
            q_scale, q_mode = _need(ins[off], "q_scale", node), _need(ins[off + 1], "q_mode", node)
            key = "mods." + name + "."
            sd[key + "weight"] = w.detach()
            if b is not None and b.dim() == 1 and b.numel() == w.shape[0]:
                sd[key + "bias"] = b.detach()
            sd[key + "scale"] = q_scale.detach().float()
            sd[key + "quantized_mode"] = q_mode.detach().to(torch.int32)
            if kind == "torch_mlu::conv2d":
                pad = _pair(_need(ins[3], "padding", node), "padding")
                stride = _pair(_need(ins[4], "stride", node), "stride")
                if _pair(_need(ins[5], "dilation", node), "dilation") != 1:
                    raise LoweringError("dilated convolutions are not part of the plan vocabulary")
                groups = int(_need(ins[6], "groups", node))
                if w.shape[2] != w.shape[3]:
                    raise LoweringError("only square filters are supported, got %s" % (tuple(w.shape),))
                r = dict(kind="conv", name=name, src=src(ins[0], node), ci=int(w.shape[1]) * groups, co=int(w.shape[0]),
                         k=int(w.shape[2]), stride=stride, pad=pad, groups=groups, act="none", add=None,
                         add_after=False)
            else:
                r = dict(kind="fc", name=name, src=src(ins[0], node), ci=int(w.shape[1]), co=int(w.shape[0]), k=None,
                         stride=None, pad=None, groups=None, act="none", add=None, add_after=None)
            r["out"] = node.output().unique()
            recs.append(r)
            by_name[name] = r
            name_of[node.output().unique()] = name
            continue
        if kind in ("aten::relu", "aten::relu_", "aten::relu6", "aten::relu6_", "aten::hardtanh", "aten::hardtanh_",
                    "aten::leaky_relu", "aten::leaky_relu_"):
            r = open_conv(ins[0])
            if r is None or r["act"] != "none" or r["add_after"]:
                raise LoweringError("%s must directly follow a convolution (or its residual add)" % kind)
            if kind.startswith("aten::relu6"):
                act = "relu6"
            elif kind.startswith("aten::relu"):
                act = "relu"
            elif kind.startswith("aten::hardtanh"):
                lo, hi = float(_need(ins[1], "min", node)), float(_need(ins[2], "max", node))
                if (lo, hi) != (0.0, 6.0):
                    raise LoweringError("hardtanh(%g, %g): only (0, 6) = ReLU6 is supported" % (lo, hi))
                act = "relu6"
            else:
                slope = float(_need(ins[1], "negative_slope", node))
                if abs(slope - LEAKY_SLOPE) > 1e-12:
                    raise LoweringError("leaky_relu slope %g: the plan uses %g" % (slope, LEAKY_SLOPE))
                act = "leaky"
            r["act"] = act
            r["out"] = node.output().unique()
            name_of[node.output().unique()] = r["name"]
            continue
        if kind in ("aten::add", "aten::add_"):
            if len(ins) > 2 and float(_need(ins[2], "alpha", node)) != 1.0:
                raise LoweringError("add with alpha != 1")
            done = False
            # either operand may be the convolution the add is fused into; with two candidates (a block's
            # last convolution and its projection shortcut) take the one that runs later
            cands = [(a, b) for a, b in ((ins[0], ins[1]), (ins[1], ins[0]))
                     if open_conv(a) is not None and open_conv(a)["add"] is None and b.unique() in name_of]
            cands.sort(key=lambda ab: recs.index(open_conv(ab[0])))
            if cands:
                a, b = cands[-1]
                r = open_conv(a)
                r["add"] = name_of[b.unique()]
                r["add_after"] = r["act"] != "none"
                r["out"] = node.output().unique()
                name_of[node.output().unique()] = r["name"]
                done = True
            if not done:
                raise LoweringError("aten::add: one operand must be the (single-use) output of a convolution")
            continue
        if kind == "aten::max_pool2d":
            k = _pair(_need(ins[1], "kernel_size", node), "kernel_size")
            s_ = _need(ins[2], "stride", node)
            stride = _pair(s_, "stride") if s_ else k
            pad = _pair(_need(ins[3], "padding", node), "padding")
            if _pair(_need(ins[4], "dilation", node), "dilation") != 1 or bool(_need(ins[5], "ceil_mode", node)):
                raise LoweringError("max_pool2d: dilation / ceil_mode are not supported")
            r = dict(kind="maxpool", name="n%d" % len(recs), src=src(ins[0], node), ci=None, co=None, k=k, stride=stride,
                     pad=pad, groups=None, act=None, add=None, add_after=None)
        elif kind == "aten::adaptive_avg_pool2d":
            if [int(v) for v in _need(ins[1], "output_size", node)] != [1, 1]:
                raise LoweringError("adaptive_avg_pool2d: only the global (1, 1) form is supported")
            r = dict(kind="gap", name="n%d" % len(recs), src=src(ins[0], node))
        elif kind == "aten::mean":
            dims = sorted(int(d) % 4 for d in _need(ins[1], "dim", node))
            if dims != [2, 3]:
                raise LoweringError("mean over %s: only the spatial mean (2, 3) is supported" % dims)
            r = dict(kind="gap", name="n%d" % len(recs), src=src(ins[0], node))
        elif kind == "aten::upsample_nearest2d":
            si, so = ins[0].type().sizes(), node.output().type().sizes()
            if si and so:
                ok = so[2] == 2 * si[2] and so[3] == 2 * si[3]
            else:
                flat = []
                for v in ins[1:]:
                    c = _const(v)
                    flat += list(c) if isinstance(c, (list, tuple)) else [c]
                ok = [float(f) for f in flat if isinstance(f, float)] in ([2.0], [2.0, 2.0])
            if not ok:
                raise LoweringError("upsample_nearest2d: only a scale factor of 2 is supported")
            r = dict(kind="upsample", name="n%d" % len(recs), src=src(ins[0], node))
        elif kind == "aten::cat":
            parts = list(ins[0].node().inputs()) if ins[0].node().kind() == "prim::ListConstruct" else None
            if parts is None or int(_need(ins[1], "dim", node)) % 4 != 1:
                raise LoweringError("cat: only concatenation of a tensor list over channels is supported")
            r = dict(kind="concat", name="n%d" % len(recs), src=tuple(src(p, node) for p in parts))
        elif kind in _PASS_THROUGH:
            name_of[node.output().unique()] = src(ins[0], node)
            continue
        elif kind == "prim::TupleConstruct":
            continue
        else:
            raise LoweringError("node %s is outside the vocabulary of the fused plan" % kind)
        r["out"] = node.output().unique()
        recs.append(r)
        by_name[r["name"]] = r
        name_of[node.output().unique()] = r["name"]

    outs = []
    for o in graph.outputs():
        vals = list(o.node().inputs()) if o.node().kind() == "prim::TupleConstruct" else [o]
        outs += [src(v, o.node()) for v in vals]
    layers = [Layer(*[r.get(f) for f in Layer._fields]) for r in recs]
    return layers, sd, outs


def lower(module, example_input, device="cuda", out_half=False, fractional_scale=False):
    """module: an nn.Module whose quantized layers call torch_mlu::conv2d / linear (as prepared by
    ``quantize_dynamic_mlu`` and moved to the device), or an already traced ScriptModule.
    fractional_scale: give every tensor (every output channel of per-axis weights) position *and*
    fractional scale, the form in which the reference's converters hand the ranges to their backend
    (setQuantizedParams / setQuantizedParamsPerAxis, torch_mlu/csrc/jit/utils/utils.cpp:81-167);
    the default keeps the eager ops' power-of-two steps, so that the plan equals the traced module.
    Returns (FusedNet, layers).  The FusedNet's outputs come in the order of the traced outputs."""
    if not isinstance(module, torch.jit.ScriptModule):
        with torch.no_grad():
            module = torch.jit.trace(module.eval(), example_input, check_trace=False)
    frozen = torch.jit.freeze(module.eval())
    graph = frozen.inlined_graph
    layers, sd, outs = graph_to_layers(graph)
    fused = FusedNet(layers, sd, device=device, out_half=out_half, fractional_scale=fractional_scale)
    if list(fused.outputs) != outs:
        if sorted(fused.outputs) != sorted(outs):
            raise LoweringError("graph outputs %s do not match the plan's terminal tensors %s" % (outs, fused.outputs))
        fused.outputs = outs
    return fused, layers
