"""Parity at the sizes the benchmark runs: the launches of the untraced plan (specialised epilogues, fused
projection shortcuts, non-temporal stores, the tile shapes picked for a shared device) are checked layer by
layer against the oracle on sampled output rows, each layer fed with the plan's own input tensors, so the
oracle's work stays a few image rows per layer while every layer of the full-size network is covered."""
import sys

import numpy as np
import pytest
import torch

import oracle as orc
from oracle import netref

pytestmark = pytest.mark.gpu

if torch.cuda.is_available():
    import catch_amd  # noqa: F401
    from catch_amd import _native, nets, pipeline

torch.set_grad_enabled(False)
_ACT = {"none": 0, "relu": 1, "relu6": 2, "leaky": 3}


def note(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def _band(t, n, top, rows):
    """rows top .. top+rows-1 of image n of an NHWC device tensor as numpy, zeros outside the image"""
    h = t.shape[1]
    if hasattr(t, "head_q"):  # the output of a 1x1 convolution + ReLU + requantization that was never stored
        hq = t.head_q
        out = np.zeros((1, rows) + tuple(t.shape[2:]), dtype=np.int8)
        lo, hi = max(top, 0), min(top + rows, h)
        if hi > lo:
            acc, ovf = orc.conv2d_nhwc(t.src[n:n + 1, lo:hi].cpu().numpy(), hq.qw.cpu().numpy(), (0, 0), (1, 1), (1, 1), 1)
            assert ovf == 0
            out[0, lo - top:hi - top] = orc.quantize(orc.epilogue(acc, hq.exp2, _np(hq.chan_div), _np(hq.bias), None, 1),
                                                     8, t.q_pos)[0]
        return out
    out = np.zeros((1, rows) + tuple(t.shape[2:]), dtype={torch.int8: np.int8, torch.int16: np.int16}[t.dtype])
    lo, hi = max(top, 0), min(top + rows, h)
    if hi > lo:
        out[0, lo - top:hi - top] = t[n, lo:hi].cpu().numpy()
    return out


def _np(t):
    return None if t is None else t.detach().float().cpu().numpy()


def check_plan_rows(fused, x, images, rows_per_layer=3):
    """every tensor the untraced plan produced for `x`, against the oracle on sampled images / output rows"""
    keep = {}
    out = fused.forward(x, keep=keep)
    torch.cuda.synchronize()
    checked = 0
    heads_inside = 0
    for l in fused.layers:
        if l.kind == "conv":
            if l.name in fused._fused_away:
                continue  # evaluated inside its consumer's launch: covered there
            lq = fused.q[l.name]
            if l is fused.layers[0] and fused.first_pool is not None and ("input",) + tuple(fused.q_demand["input"][0]) not in keep:
                # quantizer, first convolution and pooling ran as one launch: the pooled tensor of the sampled images
                # against the oracle's four steps on the whole image
                d, pool = fused.q_demand["input"][0], fused.first_pool
                qd = fused.q_demand[pool.name][0]
                got = keep[(pool.name,) + tuple(qd)]
                for n in images:
                    qx = orc.quantize_nchw_to_nhwc(x[n:n + 1].cpu().numpy(), d[0], d[1], d[2], cpad=fused.cdev["input"])
                    acc, ovf = orc.conv2d_nhwc(qx, lq.qw.cpu().numpy()[:, :, :l.k], (l.pad, l.pad), (l.stride, l.stride), (1, 1), 1)
                    assert ovf == 0
                    q1 = orc.quantize(orc.epilogue(acc, lq.exp2, _np(lq.chan_div), _np(lq.bias), None, _ACT[l.act]), 8, qd[1])
                    want = orc.maxpool_nhwc(q1.astype(np.float32), pool.k, pool.stride, pool.pad).astype(np.int8)
                    assert np.array_equal(want, got[n:n + 1].cpu().numpy()), "first layers: image %d" % n
                    checked += 1
                continue
            if l.name in fused._pooled_names and (l.name, "f") not in keep:
                # computed inside the launch of the global average pooling behind it: the pooled values of the sampled
                # images against the oracle's convolution, epilogue, ordered mean and quantizer
                gap = next(g for g in fused.layers if fused.pooled_conv.get(g.name) is l)
                qx = keep[(l.src, lq.bw_x, lq.pos_x, lq.scale_x)]
                for n in images:
                    acc, ovf = orc.conv2d_nhwc(qx[n:n + 1].cpu().numpy(), lq.qw.cpu().numpy(), (0, 0), (1, 1), (1, 1), 1)
                    assert ovf == 0
                    resid = keep[(l.add, "f")][n:n + 1].float().cpu().numpy() if l.add else None
                    mean = orc.global_avgpool_nhwc(orc.epilogue(acc, lq.exp2, _np(lq.chan_div), _np(lq.bias), resid, _ACT[l.act]))
                    if (gap.name, "f") in keep:
                        assert np.array_equal(mean, keep[(gap.name, "f")][n:n + 1].reshape(mean.shape).cpu().numpy()), gap.name
                        checked += 1
                    for d in fused.q_demand[gap.name]:
                        got = keep[(gap.name,) + tuple(d)][n:n + 1].reshape(mean.shape).cpu().numpy()
                        assert np.array_equal(orc.quantize(mean, d[0], d[1], d[2]), got), gap.name
                        checked += 1
                continue
            if l.name in fused._head_names and (l.name, 8, fused.q_demand[l.name][0][1], 1.0) not in keep:
                continue  # a 1x1 head computed inside the launch of the 3x3 layer behind it: covered there
            head = fused.head_of.get(l.name)
            if head is not None and (l.src, lq.bw_x, lq.pos_x, lq.scale_x) not in keep:
                # this layer's input never reached memory: the oracle's head on the rows that are needed
                hq = fused.q[head.name]
                hx = keep[(head.src, hq.bw_x, hq.pos_x, hq.scale_x)]
                heads_inside += 1

                class _Virtual(object):  # rows of the head's output, computed on demand by _band
                    shape, dtype, head_q, src = (hx.shape[0], hx.shape[1], hx.shape[2], hq.qw.shape[0]), torch.int8, hq, hx
                    q_pos = lq.pos_x
                qx = _Virtual()
            else:
                qx = keep[(l.src, lq.bw_x, lq.pos_x, lq.scale_x)]
            qw = lq.qw.cpu().numpy()
            pad = fused.padding(l)[0]
            kh = qw.shape[1]
            ho_n = (qx.shape[1] + 2 * pad - kh) // l.stride + 1
            ds = fused.shortcut_of.get(l.name)
            chain = fused.chain_of.get(l.name)
            for n in images:
                for ho in sorted(set([0, ho_n // 2, ho_n - 1][:rows_per_layer])):
                    band = _band(qx, n, ho * l.stride - pad, kh)
                    acc, ovf = orc.conv2d_nhwc(band, qw, (0, pad), (l.stride, l.stride), (1, 1), lq.groups)
                    assert ovf == 0 and acc.shape[1] == 1, l.name
                    if chain is not None:
                        # the residual is the chain of the earlier blocks, shortcut first, evaluated on this row
                        resid = None
                        for i, c in enumerate(chain[:-1]):
                            cq = fused.q[c.name]
                            cx = keep[(c.src, cq.bw_x, cq.pos_x, cq.scale_x)]
                            cacc, covf = orc.conv2d_nhwc(_band(cx, n, ho * c.stride, 1), cq.qw.cpu().numpy(), (0, 0),
                                                         (c.stride, c.stride), (1, 1), 1)
                            assert covf == 0
                            resid = orc.epilogue(cacc, cq.exp2, _np(cq.chan_div), _np(cq.bias), resid, 0 if i == 0 else 1)
                    elif ds is not None:
                        dq = fused.q[ds.name]
                        sx = keep[(ds.src, dq.bw_x, dq.pos_x, dq.scale_x)]
                        sacc, _ = orc.conv2d_nhwc(_band(sx, n, ho * ds.stride, 1), dq.qw.cpu().numpy(), (0, 0),
                                                  (ds.stride, ds.stride), (1, 1), 1)
                        resid = orc.epilogue(sacc, dq.exp2, _np(dq.chan_div), _np(dq.bias))
                    elif l.add:
                        resid = keep[(l.add, "f")][n, ho:ho + 1][None].float().cpu().numpy()
                    else:
                        resid = None
                    y = orc.epilogue(acc, lq.exp2, _np(lq.chan_div), _np(lq.bias), resid, _ACT[l.act],
                                     act_slope=netref.LEAKY_SLOPE, resid_after_act=bool(l.add_after))
                    if (l.name, "f") in keep:
                        got = keep[(l.name, "f")][n, ho].cpu().numpy()
                        want = y[0, 0].astype(np.float16) if got.dtype == np.float16 else y[0, 0]
                        assert np.array_equal(want, got), "%s: image %d row %d, floating output" % (l.name, n, ho)
                        checked += 1
                    for d in fused.q_demand[l.name]:
                        got = keep[(l.name,) + tuple(d)][n, ho].cpu().numpy()
                        assert np.array_equal(orc.quantize(y[0, 0], d[0], d[1], d[2]), got), \
                            "%s: image %d row %d, quantized output at %s" % (l.name, n, ho, d)
                        checked += 1
        elif l.kind == "fc":
            lq = fused.q[l.name]
            qx = keep[(l.src, lq.bw_x, lq.pos_x, lq.scale_x)]
            rows = qx.reshape(qx.shape[0], -1)[list(images)].cpu().numpy()
            acc, ovf = orc.gemm_nt(rows, lq.qw.cpu().numpy())
            y = orc.epilogue(acc, lq.exp2, _np(lq.chan_div), _np(lq.bias))
            assert ovf == 0 and np.array_equal(y, keep[(l.name, "f")][list(images)].cpu().numpy()), l.name
            checked += 1
        elif l.kind == "maxpool":
            for form in fused._forms(l.name):
                if l is fused.first_pool and (l.src,) + form not in keep:
                    continue  # pooled inside the first convolution's launch: covered there
                src, got = keep[(l.src,) + form], keep[(l.name,) + form]
                for n in images:
                    want = orc.maxpool_nhwc(src[n:n + 1].float().cpu().numpy(), l.k, l.stride, l.pad)
                    assert np.array_equal(want, got[n:n + 1].float().cpu().numpy()), l.name
                    checked += 1
        elif l.kind == "gap" and (l.src, "f") not in keep:
            assert l.name in fused.pooled_conv  # pooled inside the launch that computes the convolution: covered there
        elif l.kind == "gap":
            src = keep[(l.src, "f")]
            mean = orc.global_avgpool_nhwc(src[list(images)].cpu().numpy())
            if (l.name, "f") in keep:
                assert np.array_equal(mean, keep[(l.name, "f")][list(images)].reshape(mean.shape).cpu().numpy()), l.name
            for d in fused.q_demand[l.name]:
                got = keep[(l.name,) + tuple(d)][list(images)].reshape(mean.shape).cpu().numpy()
                assert np.array_equal(orc.quantize(mean, d[0], d[1], d[2]), got), l.name
                checked += 1
        else:
            raise AssertionError("layer kind %s is not covered by this check" % l.kind)
    # the network input's quantized forms
    for d in fused.q_demand["input"]:
        if ("input",) + tuple(d) not in keep:
            assert fused.first_pool is not None  # quantized inside the first convolution's launch
            continue
        got = keep[("input",) + tuple(d)]
        for n in images:
            want = orc.quantize_nchw_to_nhwc(x[n:n + 1].cpu().numpy(), d[0], d[1], d[2], cpad=fused.cdev["input"])
            g = got[n:n + 1]
            if fused.stem:
                sp = fused.stem["pad"]
                inner = g[:, sp:g.shape[1] - sp, sp:g.shape[2] - sp - fused.stem["extra"]]
                assert int(g.abs().sum().item()) == int(inner.abs().sum().item())  # the frame is zeros
                g = inner
            assert np.array_equal(want, g.cpu().numpy())
    return out, checked


def _plan(arch, batch, calib, seed=0, weight_std=0.05):
    layers = nets.NETS[arch]()
    net = nets.FloatNet(layers, seed=seed, weight_std=weight_std).eval()
    x = torch.randn(batch, 3, 224, 224, generator=torch.Generator().manual_seed(1))
    sd = pipeline.calibrate(net, x[:calib], "int8", True)
    return layers, sd, x, pipeline.FusedNet(layers, sd)


def test_resnet50_at_the_benchmark_shapes():
    """ResNet-50 v1.5, 32 x 3 x 224 x 224 with the launches planned for a device shared by two (what each half
    of the benchmark's batch of 64 runs): every layer of the untraced plan on sampled rows of the first, a middle
    and the last image, and the logits of those images against the oracle's whole unfused network."""
    note("resnet50 bs32 224x224, launch sharing 2")
    layers, sd, x, fused = _plan("resnet50", 32, 4)
    before = torch.ops.torch_mlu.set_launch_sharing(2)
    try:
        logits, checked = check_plan_rows(fused, x.cuda(), (0, 17, 31))
    finally:
        torch.ops.torch_mlu.set_launch_sharing(max(before, 1))
    # the plan the benchmark runs: every stage's first block and the second block of the widest stage are residual chains,
    # and the 1x1 reductions of the widest stage run inside the launches of the 3x3 layers behind them
    assert checked > 300 and sorted(len(c) for c in fused.chain_of.values()) == [2, 2, 2, 2, 3] and not fused.shortcut_of
    assert sorted(n for n, h in fused.head_of.items() if fused.head_fuses(h, 32, 56, 56)) == ["l1.0.c2", "l1.1.c2", "l1.2.c2"]
    pick = [0, 31]
    t, _ = netref.run(layers, {k: v.detach().cpu().numpy() for k, v in sd.items()}, x[pick].numpy(), record=False)
    want = t[fused.outputs[0]].reshape(len(pick), -1)
    assert np.array_equal(want, logits[pick].cpu().numpy())
    # the graph the benchmark replays (two halves on two streams) returns the same logits
    static_in, replay = fused.capture(x.cuda(), streams=2)
    assert torch.equal(replay(), logits)


def test_mobilenet_v2_at_the_benchmark_shapes():
    """MobileNetV2, 64 x 3 x 224 x 224 planned for a device shared by two (half of the benchmark's 128)"""
    note("mobilenet_v2 bs64 224x224, launch sharing 2")
    layers, sd, x, fused = _plan("mobilenet_v2", 64, 4, seed=5, weight_std=0.2)
    before = torch.ops.torch_mlu.set_launch_sharing(2)
    try:
        logits, checked = check_plan_rows(fused, x.cuda(), (0, 63))
    finally:
        torch.ops.torch_mlu.set_launch_sharing(max(before, 1))
    assert checked > 200
    t, _ = netref.run(layers, {k: v.detach().cpu().numpy() for k, v in sd.items()}, x[:1].numpy(), record=False)
    assert np.array_equal(t[fused.outputs[0]].reshape(1, -1), logits[:1].cpu().numpy())


@pytest.mark.parametrize("m,n,k", [(4096, 3072, 768), (4096, 768, 3072)])
def test_standalone_linear_full_size_with_its_epilogue(m, n, k):
    """X[m,k], W[n,k] ~ N(0,1) (seeds 2, 3), bias N(0,1) (seed 4): X per-tensor int8, W per-channel int8, fp16
    output = ReLU(dequant + bias) -- the launch the benchmark times (256x256 / 128x128 tiles with the fp16
    ReLU epilogue), compared bit for bit on row blocks at the top, the middle, the bottom and at random."""
    note("standalone linear", m, n, k)
    ops = torch.ops.torch_mlu
    x = torch.randn(m, k, generator=torch.Generator().manual_seed(2))
    w = torch.randn(n, k, generator=torch.Generator().manual_seed(3))
    bias = torch.randn(n, generator=torch.Generator().manual_seed(4))
    s_x = 127.0 / x.abs().max().item()
    s_c = (127.0 / w.abs().amax(1)).float()
    pos_x = orc.pos_from_scale(8, s_x)
    new_pos, new_scale, sf = orc.per_channel_params(8, s_c.numpy())
    qx = ops.quantize(x.cuda(), 8, pos_x, 1.0)
    qw, gp, gs = ops.quantize_per_channel(w.cuda(), s_c.cuda(), 8)
    assert int(gp.item()) == new_pos and np.array_equal(gs.cpu().numpy(), new_scale)
    want_qw = orc.quantize_per_channel(w.numpy(), 8, sf)
    assert np.array_equal(want_qw, qw.cpu().numpy())
    y, _, _ = ops.qlinear(qx, qw, pos_x + new_pos, gs, bias.cuda(), 1, True, True, False, 0, 0, 1.0)
    assert y.dtype == torch.float16 and tuple(y.shape) == (m, n)
    r = np.random.default_rng(k)
    starts = [0, m // 2 - 32, m - 64] + [int(v) for v in r.integers(0, m - 64, 3)]
    yc = y.cpu().numpy()
    for s in starts:
        rows = slice(s, s + 64)
        want_qx = orc.quantize(x[rows].numpy(), 8, pos_x)
        assert np.array_equal(want_qx, qx[rows].cpu().numpy())
        acc, ovf = orc.gemm_nt(want_qx, want_qw)
        want = orc.epilogue(acc, pos_x + new_pos, new_scale, bias.numpy(), None, 1, np.float16)
        assert ovf == 0 and np.array_equal(want.view(np.uint16), yc[rows].view(np.uint16)), "rows %d.." % s
    assert (yc >= 0).all() and (yc > 0).mean() > 0.3  # ReLU applied, and not to everything
    # the same launch through the module-level op the reference defines (fp32 out, no activation)
    y32 = ops.linear(x.cuda(), w.cuda(), bias.cuda(), torch.cat([torch.tensor([s_x, 0.0]), s_c]).cuda(),
                     torch.tensor([3], dtype=torch.int32).cuda())
    assert torch.equal(torch.relu(y32).half(), y)


@pytest.mark.parametrize("m,n,k", [(4096, 2048, 2048), (4000, 2304, 2128), (8192, 8192, 8192)])
def test_big_gemm_with_the_operands_in_separate_rings(m, n, k):
    """int8 GEMMs large enough for the 256 x 256 tile with long K, whose operands travel through rings of their own
    (two A slots, three B slots): the int32 sums and the fp32 epilogue on row blocks at the top, the middle, the
    ragged bottom and at random against the oracle; K ending inside a 128-byte step; uniformly random bytes (every
    digit pattern, sums near the int32 limits for the largest K)"""
    note("big gemm", m, n, k)
    r = np.random.default_rng(m + n + k)
    lim = 128 if k <= 4096 else 64  # the int32 sum of 8192 products of full-range bytes could overflow
    a = r.integers(-lim, lim, (m, k)).astype(np.int8)
    b = r.integers(-128, 128, (n, k)).astype(np.int8)
    a[0, :], a[-1, :] = lim - 1, -lim
    b[0, :], b[-1, :] = 127, -128
    div = r.uniform(0.6, 3.5, n).astype(np.float32)
    bias = r.standard_normal(n).astype(np.float32)
    import cabi
    out = cabi.gemm_nt(cabi.dev(a), cabi.dev(b), exp2=-12, chan_div=cabi.dev(div), bias=cabi.dev(bias), act=0,
                       y_dtype=torch.float32, want_acc=True, chan_rcp=cabi.dev(np.float32(1) / div))
    acc_g, y_g = out["acc"].cpu().numpy(), out["y"].cpu().numpy()
    starts = [0, m // 2 - 32, m - 64] + [int(v) for v in r.integers(0, m - 64, 2)]
    for s in starts:
        rows = slice(s, s + 64)
        acc, ovf = orc.gemm_nt(a[rows], b)
        assert ovf == 0 and np.array_equal(acc.astype(np.int32), acc_g[rows]), "rows %d.." % s
        assert np.array_equal(orc.epilogue(acc, -12, div, bias).view(np.uint32), y_g[rows].view(np.uint32)), "rows %d.." % s


def test_darknet53_yolov3_fp16_heads_at_416():
    """Darknet-53 + YOLOv3 heads, one 3 x 416 x 416 U(0,1) image, int16 activations x int8 weights, fp16
    outputs at the 13 / 26 / 52 grids: the heads the plan stores in half precision equal the oracle's fp32 head
    values rounded once to half, bit for bit, in the traced and in the untraced plan."""
    note("darknet53_yolov3 bs1 416x416 fp16 heads")
    layers = nets.darknet53_yolov3()
    net = nets.FloatNet(layers, seed=7, weight_std="he").eval()
    x = torch.rand(1, 3, 416, 416, generator=torch.Generator().manual_seed(8))
    sd = pipeline.to_position_encoding(pipeline.calibrate(net, x, "int16", False), 16, 8)
    fused = pipeline.FusedNet(layers, sd, out_half=True)
    t, rec = netref.run(layers, {k: v.detach().cpu().numpy() for k, v in sd.items()}, x.numpy())
    assert all(r["overflow"] == 0 for r in rec.values())
    trace = {}
    traced = fused.forward(x.cuda(), trace=trace)
    plain = fused.forward(x.cuda())
    torch.cuda.synchronize()
    assert [tuple(o.shape) for o in plain] == [(1, 255, 13, 13), (1, 255, 26, 26), (1, 255, 52, 52)]
    for name, a, b in zip(fused.outputs, traced, plain):
        want = t[name].astype(np.float16)
        for got in (a, b):
            assert got.dtype == torch.float16
            g = np.transpose(got.cpu().numpy(), (0, 2, 3, 1))
            assert np.array_equal(want.view(np.uint16), np.ascontiguousarray(g).view(np.uint16)), name
    # the integer sums of every layer, full resolution
    for l in layers:
        if l.kind == "conv":
            got = trace[l.name]["acc"].cpu().numpy()
            want = rec[l.name]["acc"].astype(np.int32)
            assert np.array_equal(want, got[..., :want.shape[-1]]), l.name


@pytest.mark.parametrize("arch,batch,side", [("mobilenet_v2", 128, 224), ("darknet53_yolov3", 16, 416), ("resnet50", 64, 224)])
def test_full_batch_graph_equals_its_images_alone(arch, batch, side):
    """The benchmark's whole batch through the graph the benchmark replays (two parts on two streams, tiles planned
    for a shared device): every output row of the first and last image of either part equals what the same plan
    returns for that image alone, bit for bit, and the first image alone equals the oracle's whole network.  The
    images are independent, so this carries the oracle's check to every batch position that the tile and band
    rules place differently (first / last tile of a launch, either stream)."""
    note("full batch", arch, batch, side)
    layers = nets.NETS[arch]()
    detector = arch == "darknet53_yolov3"
    net = nets.FloatNet(layers, seed=7 if detector else 5, weight_std="he" if detector else (0.2 if arch == "mobilenet_v2" else 0.05)).eval()
    g = torch.Generator().manual_seed(8)
    x = torch.rand(batch, 3, side, side, generator=g) if detector else torch.randn(batch, 3, side, side, generator=g)
    if detector:
        sd = pipeline.to_position_encoding(pipeline.calibrate(net, x[:1], "int16", False), 16, 8)
    else:
        sd = pipeline.calibrate(net, x[:4], "int8", True)
    fused = pipeline.FusedNet(layers, sd, out_half=detector)
    static_in, replay = fused.capture(x.cuda(), streams=2)
    out = replay()
    outs = out if isinstance(out, tuple) else (out,)
    half = batch // 2
    for n in (0, half - 1, half, batch - 1):
        alone = fused.forward(x[n:n + 1].cuda())
        alone = alone if isinstance(alone, tuple) else (alone,)
        for a, b in zip(alone, outs):
            assert torch.equal(a[0], b[n]), (arch, n)
    t, rec = netref.run(layers, {k: v.detach().cpu().numpy() for k, v in sd.items()}, x[:1].numpy(), record=False)
    for name, o in zip(fused.outputs, outs):
        got = o[:1].float().cpu().numpy()
        want = t[name]
        got = np.transpose(got, (0, 2, 3, 1)) if got.ndim == 4 else got.reshape(want.shape)
        want = want.astype(np.float16).astype(np.float32) if detector else want
        assert np.array_equal(want, got), name
