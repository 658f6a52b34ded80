"""Model-level parity: the fused int8 pipeline on the GPU against the oracle's unfused,
layer-by-layer execution of the same calibrated network -- every layer's quantized input and
int32 accumulators bit-exact, outputs within 1e-3 of their range (they are in fact identical),
and the module-swap drop-in flow against both."""
import sys

import numpy as np
import pytest
import torch

from oracle import netref

pytestmark = pytest.mark.gpu

if torch.cuda.is_available():
    import catch_amd  # noqa: F401
    from catch_amd import nets, pipeline
    from catch_amd.core.mlu_quantize import quantize_dynamic_mlu

torch.set_grad_enabled(False)


def note(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def np_sd(sd):
    return {k: v.detach().cpu().numpy() for k, v in sd.items()}


def check_against_oracle(layers, sd, x, fused, fractional_scale=False):
    t, rec = netref.run(layers, np_sd(sd), x.numpy(), fractional_scale=fractional_scale)
    trace = {}
    out = fused.forward(x.cuda(), trace=trace)
    torch.cuda.synchronize()
    for l in layers:
        if l.kind not in ("conv", "fc"):
            continue
        r, g = rec[l.name], trace[l.name]
        assert r["overflow"] == 0, l.name
        def real(t, want):  # drop the zero channels the device layout pads with
            t = t.cpu().numpy()
            if t.shape[-1] != want.shape[-1]:
                assert not t[..., want.shape[-1]:].any(), "padding channels of %s are not zero" % l.name
                t = t[..., :want.shape[-1]]
            return t.reshape(want.shape)
        assert np.array_equal(r["qx"], real(g["qx"], r["qx"])), "quantized input of " + l.name
        # the quantized weight as the plan holds it: the oracle's, plus zero padding (channels, taps of the stem's rows)
        qw = fused.q[l.name].qw.cpu().numpy()
        inner = tuple(slice(0, e) for e in r["qw"].shape)
        assert qw.dtype == r["qw"].dtype and np.array_equal(qw[inner], r["qw"]), "quantized weight of " + l.name
        assert np.count_nonzero(qw) == np.count_nonzero(r["qw"]), "weight padding of %s is not zero" % l.name
        assert np.array_equal(r["acc"].astype(np.int32), real(g["acc"], r["acc"])), "accumulators of " + l.name
        assert np.array_equal(r["y"], real(g["y"].float(), r["y"])), "output of " + l.name
    outs = out if isinstance(out, tuple) else (out,)
    for name, o in zip(fused.outputs, outs):
        want = t[name]
        got = o.float().cpu().numpy()
        got = np.transpose(got, (0, 2, 3, 1)) if got.ndim == 4 else got.reshape(want.shape)
        span = float(want.max() - want.min())
        assert np.abs(got - want).max() <= 1e-3 * span
    # the untraced run (fp32 copies only where needed) gives the same outputs
    out2 = fused.forward(x.cuda())
    outs2 = out2 if isinstance(out2, tuple) else (out2,)
    for a, b in zip(outs, outs2):
        assert torch.equal(a, b)
    return outs


@pytest.mark.parametrize("per_channel", [False, True])
def test_resnet18_bs1(per_channel):
    """ResNet-18, 1x3x224x224 N(0,1), weights N(0,0.05), int8 weights and activations."""
    note("resnet18", per_channel)
    layers = nets.resnet(18)
    net = nets.FloatNet(layers, seed=0).eval()
    x = torch.randn(1, 3, 224, 224, generator=torch.Generator().manual_seed(1))
    sd = pipeline.calibrate(net, x, "int8", per_channel)
    fused = pipeline.FusedNet(layers, sd)
    check_against_oracle(layers, sd, x, fused)


@pytest.mark.parametrize("per_channel", [False, True])
def test_resnet18_bs1_position_and_fractional_scale(per_channel):
    """The same network quantized the general way: position from max-abs plus a fractional scale per tensor
    (per output channel for per-axis weights), so that every step is absmax / qmax exactly."""
    note("resnet18 fractional scale", per_channel)
    layers = nets.resnet(18)
    net = nets.FloatNet(layers, seed=0).eval()
    x = torch.randn(1, 3, 224, 224, generator=torch.Generator().manual_seed(1))
    sd = pipeline.calibrate(net, x, "int8", per_channel)
    fused = pipeline.FusedNet(layers, sd, fractional_scale=True)
    assert 1.0 < fused.q["conv1"].scale_x < 2.0 and fused.shortcut_of
    (logits,) = check_against_oracle(layers, sd, x, fused, fractional_scale=True)
    # the fractional scale uses the whole integer range: the largest input value maps to +-127
    trace = {}
    fused.forward(x.cuda(), trace=trace)
    assert int(trace["conv1"]["qx"].abs().max()) == 127
    # and it is a different quantization from the power-of-two one
    (pow2,) = check_against_oracle(layers, sd, x, pipeline.FusedNet(layers, sd))
    assert not torch.equal(pow2, logits)
    _, replay = fused.capture(x.cuda())
    assert torch.equal(replay(), logits)


def test_fractional_scale_rejects_position_checkpoints():
    layers = nets.resnet(18)
    net = nets.FloatNet(layers, seed=0).eval()
    x = torch.randn(1, 3, 64, 64, generator=torch.Generator().manual_seed(1))
    sd = pipeline.to_position_encoding(pipeline.calibrate(net, x, "int8", False), 8, 8)
    with pytest.raises(ValueError, match="fractional"):
        pipeline.FusedNet(layers, sd, fractional_scale=True)


def test_resnet50_small_batch_and_graph_replay():
    note("resnet50 bs2 112x112")
    layers = nets.resnet(50)
    net = nets.FloatNet(layers, seed=0).eval()
    x = torch.randn(2, 3, 112, 112, generator=torch.Generator().manual_seed(2))
    sd = pipeline.calibrate(net, x, "int8", True)
    fused = pipeline.FusedNet(layers, sd)
    (logits,) = check_against_oracle(layers, sd, x, fused)
    # HIP graph: several replays, with eager work in between, all equal to the eager result
    static_in, replay = fused.capture(x.cuda())
    for i in range(3):
        static_in.copy_(x.cuda())
        out = replay()
        torch.cuda.synchronize()
        assert torch.equal(out, logits), "replay %d" % i
        _ = fused.forward(torch.randn(2, 3, 112, 112, device="cuda"))
        torch.cuda.synchronize()


@pytest.mark.parametrize("arch,batch,streams", [("resnet50", 5, 2), ("resnet50", 4, 3), ("darknet53_yolov3", 3, 2),
                                                ("resnet18", 2, 4)])
def test_graph_with_the_batch_on_parallel_streams(arch, batch, streams):
    """the batch split into parts that run on streams of their own inside one HIP graph (uneven parts, more
    streams than images, several outputs): every replay equals the single eager pass, new inputs included"""
    note("parallel streams", arch, batch, streams)
    layers = nets.NETS[arch]()
    det = arch.startswith("darknet")
    net = nets.FloatNet(layers, seed=0, weight_std="he" if det else 0.05).eval()
    g = torch.Generator().manual_seed(11)
    x = torch.rand(batch, 3, 64, 64, generator=g) if det else torch.randn(batch, 3, 64, 64, generator=g)
    sd = pipeline.calibrate(net, x, "int16" if det else "int8", not det)
    if det:
        sd = pipeline.to_position_encoding(sd, 16, 8)
    fused = pipeline.FusedNet(layers, sd, out_half=det)
    static_in, replay = fused.capture(x.cuda(), streams=streams)
    for i in range(4):
        xi = x.cuda() if i % 2 == 0 else (x.cuda() * 0.5 + 0.1)
        want = fused.forward(xi)
        static_in.copy_(xi)
        got = replay()
        torch.cuda.synchronize()
        want = want if isinstance(want, tuple) else (want,)
        got = got if isinstance(got, tuple) else (got,)
        assert len(want) == len(got)
        for a, b in zip(want, got):
            assert a.shape == b.shape and torch.equal(a, b), "replay %d" % i
        _ = fused.forward(torch.randn(batch, 3, 64, 64, device="cuda"))  # eager work between the replays
        torch.cuda.synchronize()


@pytest.mark.parametrize("depth,expect", [(18, ["l2.0.c2", "l3.0.c2", "l4.0.c2"]),
                                          (50, ["l1.0.c3", "l2.0.c3", "l3.0.c3", "l4.0.c3"])])
def test_projection_shortcuts_fused_into_block_end(depth, expect):
    """the projection shortcuts run inside the launch of the block's last convolution; logits identical to
    the plan that runs them as launches of their own (which the traced pass checks against the oracle)"""
    note("shortcut fusion, resnet", depth)
    layers = nets.resnet(depth)
    net = nets.FloatNet(layers, seed=3).eval()
    x = torch.randn(3, 3, 96, 96, generator=torch.Generator().manual_seed(4))
    sd = pipeline.calibrate(net, x, "int8", True)
    fused = pipeline.FusedNet(layers, sd)
    plain = pipeline.FusedNet(layers, sd, fuse_shortcuts=False)
    # (a bottleneck block's shortcut is the first link of a residual chain, a basic block's one half of a two-branch launch)
    inside = dict(fused.shortcut_of, **{n: c[0] for n, c in fused.chain_of.items() if len(c) == 2})
    assert sorted(inside) == expect and not plain.shortcut_of and not plain.chain_of
    assert sorted(l.name for l in inside.values()) == [e.rsplit(".", 1)[0] + ".ds" for e in expect]
    timers = {}
    a = fused.forward(x.cuda(), timers=timers)
    b = plain.forward(x.cuda())
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    assert not any(n.endswith(".ds") for n in timers)  # no launch of their own
    check_against_oracle(layers, sd, x, fused)


@pytest.mark.parametrize("limit", [None, 0, 2, 3, 8])
def test_resnet50_residual_chains(limit):
    """Blocks whose residual branch is recomputed from int8 tensors inside their last convolution's launch
    (chain_links): every tensor the plan still produces equals the block-by-block plan's, the logits equal the
    oracle's; with 8 links every block of every stage is a chain and no fp32 tensor is left between blocks."""
    note("residual chains, resnet50, limit", limit)
    layers = nets.resnet(50)
    net = nets.FloatNet(layers, seed=8).eval()
    x = torch.randn(3, 3, 96, 96, generator=torch.Generator().manual_seed(9))
    sd = pipeline.calibrate(net, x, "int8", True)
    fused = pipeline.FusedNet(layers, sd, chain_links=limit)
    plain = pipeline.FusedNet(layers, sd, chain_links=0, fuse_avgpool=False)
    lens = {n: len(c) for n, c in fused.chain_of.items()}
    if limit == 0:
        assert not lens and sorted(fused.shortcut_of) == ["l1.0.c3", "l2.0.c3", "l3.0.c3", "l4.0.c3"]
    elif limit == 2:
        assert lens == {"l1.0.c3": 2, "l2.0.c3": 2, "l3.0.c3": 2, "l4.0.c3": 2} and not fused.shortcut_of
    elif limit == 8:
        assert len(lens) == 16 and lens["l3.5.c3"] == 7 and lens["l4.2.c3"] == 4 and not fused.shortcut_of
        assert not any(fused.f_demand[n] for n in lens if n != "l4.2.c3")
    else:
        assert lens["l1.0.c3"] == 2 and lens["l1.1.c3"] == 3 and "l1.2.c3" not in lens
    for name, c in fused.chain_of.items():
        assert c[-1].name == name and c[0].name.endswith(".ds") and [l.name[:2] for l in c] == [name[:2]] * len(c)
    ka, kb = {}, {}
    a = fused.forward(x.cuda(), keep=ka)
    b = plain.forward(x.cuda(), keep=kb)
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    for key, t in ka.items():
        assert torch.equal(t, kb[key]), key
    check_against_oracle(layers, sd, x, fused)


def test_mobilenet_v2_small():
    """MobileNetV2: depthwise stencil kernel, ReLU6, linear bottlenecks with residual adds, channel
    counts (24, 144) that the device layout pads to multiples of 16."""
    note("mobilenet_v2 bs2 96x96")
    layers = nets.mobilenet_v2()
    net = nets.FloatNet(layers, seed=5, weight_std=0.2).eval()
    x = torch.randn(2, 3, 96, 96, generator=torch.Generator().manual_seed(6))
    sd = pipeline.calibrate(net, x, "int8", True)
    fused = pipeline.FusedNet(layers, sd)
    assert fused.cdev["b1.proj"] == 32 and fused.chan["b1.proj"] == 24
    check_against_oracle(layers, sd, x, fused)


def test_mobilenet_v2_blocks_in_one_launch():
    """fuse_blocks: inverted-residual blocks as one launch each (torch_mlu::qconv2d_irb).  At 224 x 224 the blocks
    with 28 x 28 and 14 x 14 outputs and hidden channel counts the kernel serves run fused; every tensor the plan still
    produces, and the logits, equal the layer-by-layer plan's bit for bit, and that plan equals the oracle."""
    note("mobilenet_v2 bs2 224x224, fused blocks")
    layers = nets.mobilenet_v2()
    net = nets.FloatNet(layers, seed=5, weight_std=0.2).eval()
    x = torch.randn(2, 3, 224, 224, generator=torch.Generator().manual_seed(6))
    sd = pipeline.calibrate(net, x, "int8", True)
    fused = pipeline.FusedNet(layers, sd, fuse_blocks=True)
    plain = pipeline.FusedNet(layers, sd)
    assert sorted(fused.block_of) == sorted("b%d.proj" % b for b in range(1, 17)) and not plain.block_of
    ka, kb, timers = {}, {}, {}
    a = fused.forward(x.cuda(), keep=ka, timers=timers)
    b = plain.forward(x.cuda(), keep=kb)
    torch.cuda.synchronize()
    one_launch = sorted(int(n[1:].split(".")[0]) for n in fused.block_of if n[:-4] + "dw" not in timers)
    assert one_launch == list(range(4, 13)), one_launch  # b4 .. b12: hidden channels a multiple of 32, 196 outputs and more
    for bnum in one_launch:
        assert "b%d.exp" % bnum not in timers and ("b%d.exp" % bnum, 8) not in [k[:2] for k in ka]
    assert torch.equal(a, b)
    for key, t in ka.items():
        assert torch.equal(t, kb[key]), key
    check_against_oracle(layers, sd, x, plain)


def test_resnet50_first_layers_in_one_launch():
    """fuse_first_layers (the default): input quantizer, 7x7 convolution + ReLU and 3x3 max pooling as one launch
    (torch_mlu::qconv2d_first_layers).  Neither the quantized image nor the convolution's output is produced; every other
    tensor of the plan, and the logits, equal those of the plan that runs the three launches, bit for bit, eagerly and
    from a captured graph, and that plan equals the oracle."""
    note("resnet50 bs3 96x96, first layers in one launch")
    layers = nets.resnet(50)
    net = nets.FloatNet(layers, seed=11, weight_std=0.05).eval()
    x = torch.randn(3, 3, 96, 96, generator=torch.Generator().manual_seed(12))
    sd = pipeline.calibrate(net, x, "int8", True)
    fused = pipeline.FusedNet(layers, sd)
    plain = pipeline.FusedNet(layers, sd, fuse_first_layers=False)
    assert fused.first_pool is not None and fused.first_pool.name == "pool1" and plain.first_pool is None
    assert fused.first_layers_fuse(3, 3, 96, 96) and not fused.first_layers_fuse(3, 3, 96, 98)
    ka, kb, timers = {}, {}, {}
    a = fused.forward(x.cuda(), keep=ka, timers=timers)
    b = plain.forward(x.cuda(), keep=kb)
    torch.cuda.synchronize()
    missing = sorted(set(kb) - set(ka))
    assert [k[0] for k in missing] == ["conv1", "input"] and set(ka) <= set(kb), missing
    assert torch.equal(a, b)
    for key, t in ka.items():
        assert torch.equal(t, kb[key]), key
    static_in, replay = fused.capture(x.cuda())
    for i in range(2):
        static_in.copy_(x.cuda())
        assert torch.equal(replay(), b), "replay %d" % i
        _ = fused.forward(torch.randn(3, 3, 96, 96, device="cuda"))  # eager work between the replays
        torch.cuda.synchronize()
    # a width the one-launch kernel does not take: the same plan falls back to the three launches
    x2 = torch.randn(2, 3, 64, 62, generator=torch.Generator().manual_seed(13)).cuda()
    assert torch.equal(fused.forward(x2), plain.forward(x2))
    check_against_oracle(layers, sd, x, plain)


@pytest.mark.parametrize("arch", ["resnet50", "mobilenet_v2"])
def test_last_convolution_inside_the_average_pooling(arch):
    """fuse_avgpool (the default): the 1x1 convolution in front of the global average pooling runs inside the pooling's
    launch (torch_mlu::qconv2d_avgpool) at 7 x 7; its fp32 output is not produced, every other tensor of the plan and the
    logits equal those of the plan with the two launches, eagerly and from a captured graph on two streams; at a
    resolution whose last feature map has more than 64 pixels the same plan runs the two launches."""
    note(arch, "bs4 224x224, last convolution inside the average pooling")
    layers = nets.NETS[arch]()
    net = nets.FloatNet(layers, seed=21, weight_std=0.2 if arch == "mobilenet_v2" else 0.05).eval()
    x = torch.randn(4, 3, 224, 224, generator=torch.Generator().manual_seed(22))
    sd = pipeline.calibrate(net, x, "int8", True)
    fused = pipeline.FusedNet(layers, sd)
    plain = pipeline.FusedNet(layers, sd, fuse_avgpool=False)
    (gname, conv), = fused.pooled_conv.items()
    assert not plain.pooled_conv and conv.k == 1
    ka, kb = {}, {}
    a = fused.forward(x.cuda(), keep=ka)
    b = plain.forward(x.cuda(), keep=kb)
    torch.cuda.synchronize()
    assert sorted(set(kb) - set(ka)) == [(conv.name, "f")] and set(ka) <= set(kb)
    assert torch.equal(a, b)
    for key, t in ka.items():
        assert torch.equal(t, kb[key]), key
    static_in, replay = fused.capture(x.cuda(), streams=2)
    for i in range(2):
        static_in.copy_(x.cuda())
        assert torch.equal(replay(), b), "replay %d" % i
        _ = fused.forward(torch.randn(4, 3, 224, 224, device="cuda"))  # eager work between the replays
        torch.cuda.synchronize()
    x2 = torch.randn(2, 3, 288, 288, generator=torch.Generator().manual_seed(23)).cuda()  # 9 x 9 at the end
    k2 = {}
    assert torch.equal(fused.forward(x2, keep=k2), plain.forward(x2)) and (conv.name, "f") in k2


def test_darknet53_yolov3_int16_activations():
    """Darknet-53 + three YOLOv3 heads with int16 activations x int8 weights in the reference's
    [bitwidths],[positions] q-param encoding: leaky ReLU, shortcut adds after the activation,
    upsample + concat on the integers, 255-channel heads (padded to 256 on the device)."""
    note("darknet53_yolov3 bs1 64x64 int16 x int8")
    layers = nets.darknet53_yolov3()
    net = nets.FloatNet(layers, seed=7, weight_std="he").eval()
    x = torch.rand(1, 3, 64, 64, generator=torch.Generator().manual_seed(8))
    sd = pipeline.to_position_encoding(pipeline.calibrate(net, x, "int16", False), 16, 8)
    fused = pipeline.FusedNet(layers, sd, out_half=False)
    assert fused.cdev["input"] == 8 and fused.cdev["yolo13"] == 256
    assert fused.q["c2"].bw_x == 16 and fused.q["c2"].bw_w == 8
    outs = check_against_oracle(layers, sd, x, fused)
    assert [tuple(o.shape) for o in outs] == [(1, 255, 2, 2), (1, 255, 4, 4), (1, 255, 8, 8)]


def test_dropin_modules_match_fused_pipeline():
    """quantize_dynamic_mlu flow (torch_mlu::conv2d/linear + ATen relu/add/pool in float) gives
    the same logits as the fused plan, up to the global-average-pool summation order."""
    note("drop-in vs fused")
    layers = nets.resnet(18)
    net = nets.FloatNet(layers, seed=3).eval()
    x = torch.randn(2, 3, 96, 96, generator=torch.Generator().manual_seed(4))
    spec = {"use_avg": False, "data_scale": 1.0, "per_channel": True, "firstconv": False}
    calib = quantize_dynamic_mlu(net, spec, dtype="int8", gen_quant=True)
    calib(x)
    ckpt = calib.state_dict()
    qnet = quantize_dynamic_mlu(net)
    qnet.load_state_dict(ckpt)
    got = qnet.to("cuda")(x.cuda())
    fused = pipeline.FusedNet(layers, pipeline.calibrate(net, x, "int8", True))
    want = fused.forward(x.cuda())
    span = (want.max() - want.min()).item()
    assert (got - want).abs().max().item() <= 1e-3 * span


def test_pool_kernels():
    note("pool kernels")
    import oracle as orc
    g = np.random.default_rng(0)
    for shape, k, s, p in (((2, 9, 11, 64), 3, 2, 1), ((1, 8, 8, 6), 2, 2, 0), ((2, 7, 7, 16), 3, 1, 1)):
        x = g.standard_normal(shape).astype(np.float32)
        want = orc.maxpool_nhwc(x, k, s, p)
        got = torch.ops.torch_mlu.maxpool_nhwc(torch.from_numpy(x).cuda(), k, s, p).cpu().numpy()
        assert np.array_equal(want, got)
        q = orc.quantize(x, 8, -5)
        gq = torch.ops.torch_mlu.maxpool_nhwc(torch.from_numpy(q).cuda(), k, s, p).cpu().numpy()
        assert np.array_equal(orc.quantize(want, 8, -5), gq)  # pooling commutes with quantization
        q16 = orc.quantize(x, 16, -12)
        gq16 = torch.ops.torch_mlu.maxpool_nhwc(torch.from_numpy(q16).cuda(), k, s, p).cpu().numpy()
        assert np.array_equal(orc.quantize(want, 16, -12), gq16)
    # the whole int8 / int16 range (the int8 kernel compares packed bytes), windows hanging over every border
    for shape, k, s, p in (((2, 13, 10, 32), 3, 2, 1), ((1, 9, 12, 32), 2, 2, 0), ((2, 5, 6, 16), 3, 1, 0),
                           ((1, 11, 11, 48), 5, 2, 2), ((1, 4, 4, 16), 2, 1, 1), ((3, 1, 1, 16), 3, 2, 1)):
        for bits, dt in ((8, np.int8), (16, np.int16)):
            q = g.integers(-2 ** (bits - 1), 2 ** (bits - 1), shape).astype(dt)
            q[0, 0, 0, :4] = (-2 ** (bits - 1), 2 ** (bits - 1) - 1, -1, 0)
            want = orc.maxpool_nhwc(q.astype(np.float32), k, s, p).astype(dt)
            got = torch.ops.torch_mlu.maxpool_nhwc(torch.from_numpy(q).cuda(), k, s, p).cpu().numpy()
            assert np.array_equal(want, got), (shape, k, s, p, bits)
    x = (g.standard_normal((3, 7, 7, 130)) * 100).astype(np.float32)
    got = torch.ops.torch_mlu.global_avgpool_nhwc(torch.from_numpy(x).cuda()).cpu().numpy()
    assert np.array_equal(orc.global_avgpool_nhwc(x), got)


def test_global_avgpool_with_fused_quantizer():
    """the pooled-and-quantized launch equals pooling then quantizing, at unit and fractional scale, int8 and int16"""
    import oracle as orc
    g = np.random.default_rng(5)
    x = (g.standard_normal((3, 7, 7, 130)) * 40).astype(np.float32)
    mean = orc.global_avgpool_nhwc(x)
    for bw, pos, scale in ((8, -1, 1.0), (8, 0, 1.3720703125), (16, -9, 1.0), (16, -8, 1.9990234375)):
        got = torch.ops.torch_mlu.global_avgpool_nhwc(torch.from_numpy(x).cuda(), bw, pos, scale).cpu().numpy()
        assert np.array_equal(orc.quantize(mean, bw, pos, scale), got), (bw, pos, scale)
    with pytest.raises(RuntimeError, match="bitwidth not support"):
        torch.ops.torch_mlu.global_avgpool_nhwc(torch.from_numpy(x).cuda(), 12, 0, 1.0)
