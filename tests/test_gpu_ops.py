"""GPU tests of the drop-in ops torch.ops.torch_mlu.{conv2d,linear} and of the module-swap flow,
replaying the reference's own test grids (test/magicmind/op_test/test_conv.py:103-156,
test/magicmind/op_test/test_matmul.py:116-174, test/magicmind/test_quantization.py:42-72) with
the CPU oracle as the exact expectation and the reference's rel-RMS <= 0.02 vs float as a
secondary check."""
import math
import sys
from itertools import product

import numpy as np
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

import oracle as orc
from oracle import ops as oops
from oracle import ref_order

pytestmark = pytest.mark.gpu

if torch.cuda.is_available():
    import catch_amd  # noqa: F401  (registers the ops)
    from catch_amd.core.mlu_quantize import quantize_dynamic_mlu

torch.set_grad_enabled(False)


def note(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def rel_rms(a, b):  # test/common_utils.py:514-522
    a, b = a.astype(np.float64), b.astype(np.float64)
    return math.sqrt(((a - b) ** 2).sum() / (a ** 2).sum())


def same_bits(a, b):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    return a.shape == b.shape and a.dtype == b.dtype and np.array_equal(a.view(np.uint8), b.view(np.uint8))


def calibrate(model, x, bw, per_channel):
    qconfig = {"use_avg": False, "data_scale": 1.0, "per_channel": per_channel, "firstconv": False}
    calib = quantize_dynamic_mlu(model, qconfig, dtype=bw, gen_quant=True)
    calib(x)
    return calib.state_dict()


@pytest.mark.parametrize("bias,bw,per_channel,half",
                         list(product([True, False], ["int8", "int16"], [True, False], [False, True])))
def test_conv2d_qint_grid(bias, bw, per_channel, half):
    note("conv2d_qint", bias, bw, per_channel, half)
    torch.manual_seed(11)
    model = nn.Sequential(nn.Conv2d(64, 64, 3, 3, 3, 1, 1, bias)).eval().float()
    x = torch.randn(3, 64, 24, 24)
    want_float = model(x).numpy()
    ckpt = calibrate(model, x, bw, per_channel)
    qmodel = quantize_dynamic_mlu(model)
    qmodel.load_state_dict(ckpt)
    conv = qmodel[0]
    assert conv.quantized_mode.item() == {("int8", False): 1, ("int16", False): 2, ("int8", True): 3,
                                          ("int16", True): 4}[(bw, per_channel)]
    assert conv.scale.numel() == (2 + 64 if per_channel else 2)
    xin = x.half() if half else x
    if half:
        qmodel.half()
    qmodel.to("cuda")
    got = qmodel(xin.to("cuda"))
    assert got.shape == (3, 64, 10, 10) and got.dtype == xin.dtype
    assert got.is_contiguous(memory_format=torch.channels_last)
    b = conv.bias.detach().float().cpu().numpy()
    # .half() turns the q-params into half tensors too, as in the reference, unless half cannot hold them
    # (int16 scales of weights below 0.5 are inf there: those stay fp32)
    assert (conv.scale.dtype == torch.float16) == (half and bw == "int8")  # int16 q-params stay fp32
    if half and per_channel and conv.scale.dtype == torch.float16:
        # the reference's all-half order (quantify.cpp:55-114 and quantify_conv_forward.cpp:123-129 on half
        # tensors): same integers bit for bit
        r = ref_order.conv2d_per_channel(xin, conv.weight.detach().cpu(), conv.bias.detach().cpu(), (3, 3), (3, 3),
                                         (1, 1), 1, conv.scale.detach().cpu(), conv.quantized_mode.cpu().numpy())
        q, new_pos, new_scale = torch.ops.torch_mlu.quantize_per_channel(conv.weight.detach(), conv.scale.detach()[2:], 8)
        assert same_bits(r["qw"], q.permute(0, 2, 3, 1).contiguous().cpu().numpy())
        assert int(new_pos.item()) == r["new_pos"] and torch.equal(new_scale.cpu(), r["new_scale"])
        # ... and the output: rounded to half after the scaling, after `/ new_scale` and after `+ bias`
        assert same_bits(r["y"].contiguous(memory_format=torch.channels_last).numpy(),
                         got.contiguous(memory_format=torch.channels_last).cpu().numpy())
    else:
        ref = oops.conv2d(xin.numpy(), conv.weight.detach().float().cpu().numpy(), b, (3, 3), (3, 3), (1, 1), 1,
                          conv.scale.detach().float().cpu().numpy(), conv.quantized_mode.cpu().numpy())
        # a half model carries half weights: the oracle sees the same rounded values
        assert same_bits(ref["y"], got.cpu().numpy())
    assert rel_rms(want_float, got.float().cpu().numpy()) <= 0.02


@pytest.mark.parametrize("bias,ni,ci,co", list(product([True, False], [1, 10, 20], [10, 50, 100], [25, 75, 125])))
def test_linear_qint_grid(bias, ni, ci, co):
    note("linear_qint", bias, ni, ci, co)
    torch.manual_seed(ni * 1000 + ci * 10 + co)
    model = nn.Sequential(nn.Linear(ci, co, bias)).eval().float()
    x = torch.rand(ni, ci)
    want_float = model(x).numpy()
    for bw, per_channel, half in product(["int8", "int16"], [True, False], [False, True]):
        ckpt = calibrate(model, x, bw, per_channel)
        qmodel = quantize_dynamic_mlu(model)
        qmodel.load_state_dict(ckpt)
        lin = qmodel[0]
        xin = x.half() if half else x
        if half:
            qmodel.half()
        qmodel.to("cuda")
        got = qmodel(xin.to("cuda"))
        assert got.dtype == torch.float32 and got.shape == (ni, co)  # fp32 whatever the input type
        if half and per_channel and lin.scale.dtype == torch.float16:
            # all-half parameters and weight quotient, fp32 output arithmetic (linear.cpp:54-59 after matmul.cpp:72-74):
            # nothing is left to tolerance
            r = ref_order.linear_per_channel(xin, lin.weight.detach().cpu(), lin.bias.detach().cpu(),
                                             lin.scale.detach().cpu(), lin.quantized_mode.cpu().numpy())
            assert same_bits(r["y"].numpy(), got.cpu().numpy()), (bw, per_channel, half)
        else:
            ref = oops.linear(xin.numpy(), lin.weight.detach().float().cpu().numpy(),
                              lin.bias.detach().float().cpu().numpy(), lin.scale.detach().float().cpu().numpy(),
                              lin.quantized_mode.cpu().numpy())
            assert same_bits(ref["y"], got.cpu().numpy()), (bw, per_channel, half)
        assert rel_rms(want_float, got.cpu().numpy()) <= 0.02, (bw, per_channel, half)


def test_linear_leading_dims_and_no_bias_tensor():
    note("linear leading dims")
    torch.manual_seed(3)
    w = torch.randn(48, 32) * 0.1
    x = torch.randn(2, 5, 32)
    q_scale = torch.tensor([127 / x.abs().max().item(), 127 / w.abs().max().item()])
    q_mode = torch.tensor([1], dtype=torch.int32)
    zero_dim_bias = torch.tensor(0.0)  # bias.dim() == 0 means "no bias" (linear.cpp:57)
    got = torch.ops.torch_mlu.linear(x.cuda(), w.cuda(), zero_dim_bias.cuda(), q_scale.cuda(), q_mode.cuda())
    ref = oops.linear(x.numpy(), w.numpy(), None, q_scale.numpy(), q_mode.numpy())
    assert got.shape == (2, 5, 48) and same_bits(ref["y"], got.cpu().numpy())
    with pytest.raises(RuntimeError, match="we only support the  dim of weight is 2"):
        torch.ops.torch_mlu.linear(x.cuda(), w.cuda()[None], zero_dim_bias.cuda(), q_scale.cuda(), q_mode.cuda())


def test_conv2d_cnnl_encoding_int16_act_int8_weight():
    """q_scale = [bitwidth_in, bitwidth_w], q_mode = [pos_in, pos_w] (quantify_conv_forward.cpp:132-145)"""
    note("conv2d encoding B")
    torch.manual_seed(5)
    x = torch.rand(2, 32, 13, 13)
    w = torch.randn(48, 32, 3, 3) * 0.05
    b = torch.randn(48)
    q_scale = torch.tensor([16.0, 8.0])
    q_mode = torch.tensor([-14, -9], dtype=torch.int32)
    got = torch.ops.torch_mlu.conv2d(x.cuda(), w.cuda(), b.cuda(), [1, 1], [1, 1], [1, 1], 1, q_scale, q_mode)
    ref = oops.conv2d(x.numpy(), w.numpy(), b.numpy(), (1, 1), (1, 1), (1, 1), 1, q_scale.numpy(), q_mode.numpy())
    assert ref["overflow"] == 0 and ref["qx"].dtype == np.int16 and ref["qw"].dtype == np.int8
    assert same_bits(ref["y"], got.cpu().numpy())
    want = F.conv2d(x, w, b, 1, 1).numpy()
    assert rel_rms(want, got.cpu().numpy()) <= 0.02


@pytest.mark.parametrize("groups,ci,co", [(2, 4, 16), (8, 8, 8), (32, 32, 32), (2, 64, 64), (4, 64, 80)])  # the last two: one GEMM per group on the matrix cores
def test_conv2d_groups_and_layouts(groups, ci, co):
    note("conv2d groups", groups, ci, co)
    torch.manual_seed(groups)
    x = torch.randn(2, ci, 12, 12)
    w = torch.randn(co, ci // groups, 3, 3) * 0.2
    b = torch.randn(co)
    wf = w.reshape(co, -1)
    q_scale = torch.cat([torch.tensor([127 / x.abs().max().item(), 0.0]), 127 / wf.abs().max(1)[0]])
    q_mode = torch.tensor([3], dtype=torch.int32)
    ref = oops.conv2d(x.numpy(), w.numpy(), b.numpy(), (1, 1), (2, 2), (1, 1), groups, q_scale.numpy(), q_mode.numpy())
    for xin in (x.cuda(), x.cuda().contiguous(memory_format=torch.channels_last), x.cuda().transpose(2, 3).contiguous().transpose(2, 3)):
        got = torch.ops.torch_mlu.conv2d(xin, w.cuda(), b.cuda(), [1, 1], [2, 2], [1, 1], groups, q_scale.cuda(), q_mode.cuda())
        assert same_bits(ref["y"], got.cpu().numpy())
    with pytest.raises(RuntimeError, match="Input's dim must greater than 2!"):
        torch.ops.torch_mlu.conv2d(x.cuda()[0, 0], w.cuda(), b.cuda(), [1, 1], [2, 2], [1, 1], groups, q_scale.cuda(), q_mode.cuda())


def test_weight_cache_follows_inplace_updates():
    note("weight cache")
    torch.manual_seed(8)
    x = torch.randn(1, 16, 8, 8).cuda()
    w = (torch.randn(16, 16, 3, 3) * 0.1).cuda()
    b = torch.zeros(16).cuda()
    q_scale = torch.tensor([127 / 4.0, 127 / 0.5]).cuda()
    q_mode = torch.tensor([1], dtype=torch.int32).cuda()
    args = ([1, 1], [1, 1], [1, 1], 1)
    y1 = torch.ops.torch_mlu.conv2d(x, w, b, *args, q_scale, q_mode)
    y1b = torch.ops.torch_mlu.conv2d(x, w, b, *args, q_scale, q_mode)  # served from the cache
    assert torch.equal(y1, y1b)
    w.mul_(0.5)  # bumps the version counter -> re-quantized
    y2 = torch.ops.torch_mlu.conv2d(x, w, b, *args, q_scale, q_mode)
    ref = oops.conv2d(x.cpu().numpy(), w.cpu().numpy(), None, (1, 1), (1, 1), (1, 1), 1, q_scale.cpu().numpy(),
                      q_mode.cpu().numpy())
    assert same_bits(ref["y"], y2.cpu().numpy()) and not torch.equal(y1, y2)
    q_scale[0] = 127 / 8.0  # parameter change is seen too
    y3 = torch.ops.torch_mlu.conv2d(x, w, b, *args, q_scale, q_mode)
    ref = oops.conv2d(x.cpu().numpy(), w.cpu().numpy(), None, (1, 1), (1, 1), (1, 1), 1, q_scale.cpu().numpy(),
                      q_mode.cpu().numpy())
    assert same_bits(ref["y"], y3.cpu().numpy())


def test_weight_cache_sees_swapped_storage_and_host_qparams_by_content():
    """what identity and version cannot tell: a `.data =` swap of q_scale (same tensor object, same version,
    new storage), q-params that live on the host and change in place under inference mode (no version
    counter), and entries of weights that no longer exist"""
    note("weight cache: data swap, host q-params, purge")
    torch.manual_seed(9)
    ops = torch.ops.torch_mlu
    x = torch.randn(1, 16, 8, 8).cuda()
    w = (torch.randn(16, 16, 3, 3) * 0.1).cuda()
    b = torch.zeros(16).cuda()
    args = ([1, 1], [1, 1], [1, 1], 1)
    q_mode = torch.tensor([1], dtype=torch.int32).cuda()

    def want(q_scale):
        return oops.conv2d(x.cpu().numpy(), w.cpu().numpy(), None, (1, 1), (1, 1), (1, 1), 1, q_scale.cpu().numpy(), [1])["y"]
    q_scale = torch.tensor([127 / 4.0, 127 / 0.5]).cuda()
    assert same_bits(want(q_scale), ops.conv2d(x, w, b, *args, q_scale, q_mode).cpu().numpy())
    ver = q_scale._version
    q_scale.data = torch.tensor([127 / 16.0, 127 / 0.5]).cuda()
    assert q_scale._version == ver
    assert same_bits(want(q_scale), ops.conv2d(x, w, b, *args, q_scale, q_mode).cpu().numpy())
    with torch.inference_mode():
        hs = torch.tensor([127 / 4.0, 127 / 0.5])       # host q-params, inference tensors: version 0 for ever
        hm = torch.tensor([1], dtype=torch.int32)
        wi, xi, bi = w.clone(), x.clone(), b.clone()
        y1 = ops.conv2d(xi, wi, bi, *args, hs, hm)
        hs[0] = 127 / 32.0
        y2 = ops.conv2d(xi, wi, bi, *args, hs, hm)
    assert same_bits(want(torch.tensor([127 / 4.0, 127 / 0.5])), y1.cpu().numpy())
    assert same_bits(want(torch.tensor([127 / 32.0, 127 / 0.5])), y2.cpu().numpy())
    # entries of dead weights go at the next miss, not when 4096 of them have piled up
    ops.clear_weight_cache()
    for i in range(5):
        wt = (torch.randn(16, 16, 3, 3) * 0.1).cuda()
        ops.conv2d(x, wt, b, *args, q_scale, q_mode)
        del wt
    assert ops.weight_cache_size() <= 2


def test_cpu_tensors_are_refused():
    note("cpu refused")
    x, w, b = torch.randn(1, 4, 4, 4), torch.randn(4, 4, 1, 1), torch.zeros(4)
    with pytest.raises((RuntimeError, NotImplementedError)):
        torch.ops.torch_mlu.conv2d(x, w, b, [0, 0], [1, 1], [1, 1], 1, torch.tensor([1.0, 1.0]),
                                   torch.tensor([1], dtype=torch.int32))


class _SmallNet(nn.Module):  # test/magicmind/test_quantization.py:22-40
    def __init__(self, ci):
        super().__init__()
        self.block1 = nn.Sequential(nn.Conv2d(ci, 16, 3, 1, 0, 1, 1, bias=False), nn.BatchNorm2d(16, affine=False),
                                    nn.ReLU())

    def forward(self, x):
        y = self.block1(x)
        z = F.max_pool2d(y + y, 2)
        return torch.transpose(z, 0, 3)


@pytest.mark.parametrize("ci", [1, 3, 10])
def test_quantized_model(ci):
    note("quantized model", ci)
    torch.manual_seed(ci)
    net = _SmallNet(ci).eval().float()
    x = torch.rand(1, ci, 64, 64)
    want = net(x).numpy()
    ckpt = calibrate(net, x, "int8", True)
    qnet = quantize_dynamic_mlu(net)
    qnet.load_state_dict(ckpt)
    qnet = qnet.to("cuda")
    got = qnet(x.to("cuda"))
    assert rel_rms(want, got.cpu().numpy()) <= 0.02
    # the reference runs this model through torch.jit.trace (test_quantization.py:66-70): the traced module, with
    # the torch_mlu::conv2d nodes in its graph, gives the eager result
    traced = torch.jit.trace(qnet, x.to("cuda"), check_trace=False)
    assert "torch_mlu::conv2d" in str(traced.inlined_graph)
    assert torch.equal(traced(x.to("cuda")), got)


def test_helper_ops():
    note("helper ops")
    torch.manual_seed(2)
    x = torch.randn(3, 5, 7, 9).cuda()
    q = torch.ops.torch_mlu.quantize(x, 8, -5)
    assert same_bits(orc.quantize(x.cpu().numpy(), 8, -5), q.cpu().numpy())
    pos, scale, off = torch.ops.torch_mlu.quantize_param(x, 8, 1)
    p, s, _ = orc.quantize_param(orc.absmax(x.cpu().numpy()), 8)
    assert pos.item() == p and np.float32(scale.item()) == s
    assert same_bits(torch.ops.torch_mlu.quantize_dev(x, 8, pos).cpu().numpy(), orc.quantize(x.cpu().numpy(), 8, p))
    w = (torch.randn(6, 5, 3, 3) * 0.1).cuda()
    s_c = 127 / w.reshape(6, -1).abs().max(1)[0]
    qw, new_pos, new_scale = torch.ops.torch_mlu.quantize_per_channel(w, s_c, 8)
    op, ons, osf = orc.per_channel_params(8, s_c.cpu().numpy())
    assert new_pos.item() == op and same_bits(ons, new_scale.cpu().numpy())
    assert same_bits(orc.quantize_per_channel(w.cpu().numpy(), 8, osf), qw.cpu().numpy())
    d = torch.ops.torch_mlu.dequantize(q, -5)
    assert same_bits(orc.dequantize(q.cpu().numpy(), -5), d.cpu().numpy())
    a = torch.randint(-128, 128, (9, 32), dtype=torch.int8).cuda()
    b = torch.randint(-128, 128, (11, 32), dtype=torch.int8).cuda()
    acc, _ = orc.gemm_nt(a.cpu().numpy(), b.cpu().numpy())
    assert same_bits(orc.epilogue(acc, -7), torch.ops.torch_mlu.mm_q(a, -3, b, -4).cpu().numpy())


def test_quantize_conv2d_op_matches_conv2d_op():
    """torch_mlu::quantize_conv2d (positions as device tensors) against torch_mlu::conv2d with the same
    positions given through the [bitwidths],[positions] q-param encoding."""
    note("quantize_conv2d op")
    torch.manual_seed(11)
    x = torch.randn(2, 16, 9, 9, device="cuda")
    w = torch.randn(24, 16, 3, 3, device="cuda") * 0.2
    b = torch.randn(24, device="cuda")
    px = torch.tensor([-5], dtype=torch.int32, device="cuda")
    pw = torch.tensor([-8], dtype=torch.int32, device="cuda")
    got = torch.ops.torch_mlu.quantize_conv2d(x, px, w, pw, b, [1, 1], [1, 1], [1, 1], 1, 8, 8)
    want = torch.ops.torch_mlu.conv2d(x, w, b, [1, 1], [1, 1], [1, 1], 1, torch.tensor([8., 8.]),
                                      torch.tensor([-5, -8], dtype=torch.int32))
    assert got.shape == want.shape == (2, 24, 9, 9)
    assert torch.equal(got, want)
    with pytest.raises(Exception):
        torch.ops.torch_mlu.quantize_conv2d(x, px.cpu(), w, pw, b, [1, 1], [1, 1], [1, 1], 1, 8, 8)


@pytest.mark.parametrize("bw,per_channel,half", [("int8", False, False), ("int8", True, True), ("int16", True, False)])
def test_conv1d_module_swap(bw, per_channel, half):
    """nn.Conv1d -> MLUConv1d -> torch_mlu::conv1d (core/quantized/modules/conv.py:258-312 in the reference)"""
    note("conv1d module", bw, per_channel, half)
    torch.manual_seed(21)
    model = nn.Sequential(nn.Conv1d(24, 40, 5, 2, 3, 2, 2, True)).eval().float()
    x = torch.randn(3, 24, 77)
    want_float = model(x).numpy()
    ckpt = calibrate(model, x, bw, per_channel)
    qmodel = quantize_dynamic_mlu(model)
    qmodel.load_state_dict(ckpt)
    conv = qmodel[0]
    assert type(conv).__name__ == "MLUConv1d"
    xin = x.half() if half else x
    if half:
        qmodel.half()
    got = qmodel.to("cuda")(xin.to("cuda"))
    assert got.shape == want_float.shape and got.dtype == xin.dtype
    if half and per_channel:
        # all-half model: the reference's half tensor ops (the 1-d convolution as images of one row)
        assert conv.scale.dtype == torch.float16
        r = ref_order.conv2d_per_channel(xin[:, :, None, :], conv.weight.detach().cpu()[:, :, None, :],
                                         conv.bias.detach().cpu(), (0, 3), (1, 2), (1, 2), 2, conv.scale.detach().cpu(),
                                         conv.quantized_mode.cpu().numpy())
        assert same_bits(r["y"][:, :, 0, :].contiguous().numpy(), got.cpu().contiguous().numpy())
    else:
        ref = oops.conv1d(xin.numpy(), conv.weight.detach().float().cpu().numpy(), conv.bias.detach().float().cpu().numpy(),
                          (3,), (2,), (2,), 2, conv.scale.detach().float().cpu().numpy(), conv.quantized_mode.cpu().numpy())
        assert same_bits(ref["y"], got.cpu().numpy())
    assert rel_rms(want_float, got.float().cpu().numpy()) <= 0.02


CONV3D_CASES = [
    # N, Ci, D, H, W, Co, k, pad, stride, dil, groups
    (2, 16, 6, 12, 12, 32, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 1),
    (1, 12, 7, 9, 10, 8, (2, 3, 1), (1, 0, 1), (2, 1, 2), (2, 1, 1), 2),
    (2, 8, 5, 10, 10, 24, (1, 3, 3), (0, 1, 1), (1, 2, 2), (1, 1, 1), 1),   # depth folds into the batch (a view)
    (2, 8, 5, 10, 10, 24, (1, 3, 3), (1, 1, 1), (2, 1, 1), (1, 1, 1), 1),   # kd == 1 with depth stride and padding
    (1, 32, 4, 6, 6, 16, (3, 1, 1), (0, 0, 0), (1, 1, 1), (1, 1, 1), 1),    # kh == kw == 1
]


@pytest.mark.parametrize("case", CONV3D_CASES)
@pytest.mark.parametrize("bw,half", [("int8", False), ("int16", False), ("int8", True)])
def test_conv3d_module_swap(case, bw, half):
    """nn.Conv3d -> MLUConv3d -> torch_mlu::conv3d (core/quantized/modules/conv.py:314-380 in the reference)"""
    note("conv3d module", case, bw, half)
    n, ci, d, h, w, co, k, pad, stride, dil, g = case
    torch.manual_seed(co + d)
    model = nn.Sequential(nn.Conv3d(ci, co, k, stride, pad, dil, g, True)).eval().float()
    x = torch.randn(n, ci, d, h, w)
    want_float = model(x).numpy()
    ckpt = calibrate(model, x, bw, False)
    qmodel = quantize_dynamic_mlu(model)
    qmodel.load_state_dict(ckpt)
    conv = qmodel[0]
    assert type(conv).__name__ == "MLUConv3d"
    xin = x.half() if half else x
    if half:
        qmodel.half()
    got = qmodel.to("cuda")(xin.to("cuda"))
    assert got.shape == want_float.shape and got.dtype == xin.dtype
    ref = oops.conv3d(xin.numpy(), conv.weight.detach().float().cpu().numpy(), conv.bias.detach().float().cpu().numpy(),
                      pad, stride, dil, g, conv.scale.detach().float().cpu().numpy(), conv.quantized_mode.cpu().numpy())
    assert same_bits(ref["y"], got.cpu().numpy())
    assert rel_rms(want_float, got.float().cpu().numpy()) <= 0.02


def test_conv3d_refuses_per_channel_calibration_and_bad_shapes():
    note("conv3d errors")
    model = nn.Sequential(nn.Conv3d(4, 4, 3)).eval()
    qconfig = {"use_avg": False, "data_scale": 1.0, "per_channel": True, "firstconv": False}
    with pytest.raises(AssertionError, match="per_channel"):
        quantize_dynamic_mlu(model, qconfig, dtype="int8", gen_quant=True)
    x = torch.randn(1, 4, 2, 5, 5).cuda()
    w = torch.randn(4, 4, 3, 3, 3).cuda()
    q_scale, q_mode = torch.tensor([30.0, 30.0]).cuda(), torch.tensor([1], dtype=torch.int32).cuda()
    with pytest.raises(RuntimeError, match="Calculated output size is too small"):
        torch.ops.torch_mlu.conv3d(x, w, torch.zeros(4).cuda(), [0, 0, 0], [1, 1, 1], [1, 1, 1], 1, q_scale, q_mode)
    with pytest.raises(RuntimeError, match="expects 5-d"):
        torch.ops.torch_mlu.conv3d(x[0], w, torch.zeros(4).cuda(), [0, 0, 0], [1, 1, 1], [1, 1, 1], 1, q_scale, q_mode)
    with pytest.raises(RuntimeError, match="expects 3-d"):
        torch.ops.torch_mlu.conv1d(x, w, torch.zeros(4).cuda(), [0], [1], [1], 1, q_scale, q_mode)


@pytest.mark.parametrize("ci,k,pad,stride,dil,mode", [
    (3, 7, 3, 2, 1, 1), (3, 3, 1, 1, 1, 3), (1, 5, 2, 2, 1, 1), (2, 3, 0, 1, 1, 3), (3, 3, 1, 1, 2, 1),
    (3, 3, 1, 2, 1, 2), (1, 3, 1, 1, 1, 4), (3, (3, 5), (1, 2), (1, 2), (2, 1), 1)])
def test_conv2d_few_input_channels(ci, k, pad, stride, dil, mode):
    """images of 1-3 channels: the op frames / pads them for the matrix-core routes (int8: zero frame + fourth
    channel + filter rows of whole groups of 4 taps; int16: eight channels); same integers, same outputs"""
    note("conv2d few channels", ci, k, pad, stride, dil, mode)
    torch.manual_seed(ci * 10 + mode)
    two = lambda v: (v, v) if isinstance(v, int) else tuple(v)
    k, pad, stride, dil = two(k), two(pad), two(stride), two(dil)
    x = torch.randn(2, ci, 40, 44)
    w = torch.randn(24, ci, *k) * 0.2
    b = torch.randn(24)
    qmax = 127.0 if mode in (1, 3) else 32767.0
    if mode > 2:
        q_scale = torch.cat([torch.tensor([qmax / x.abs().max().item(), 0.0]), qmax / w.reshape(24, -1).abs().max(1)[0]])
    else:
        q_scale = torch.tensor([qmax / x.abs().max().item(), qmax / w.abs().max().item()])
    q_mode = torch.tensor([mode], dtype=torch.int32)
    ref = oops.conv2d(x.numpy(), w.numpy(), b.numpy(), pad, stride, dil, 1, q_scale.numpy(), q_mode.numpy())
    wc, qs, qm = w.cuda(), q_scale.cuda(), q_mode.cuda()  # the same tensor objects in every call: cache hits
    for xin in (x.cuda(), x.cuda().contiguous(memory_format=torch.channels_last)):
        got = torch.ops.torch_mlu.conv2d(xin, wc, b.cuda(), list(pad), list(stride), list(dil), 1, qs, qm)
        assert same_bits(ref["y"], got.cpu().numpy())
    # the same weight with another dilation: the cached, laid-out weight must not be reused blindly
    dil2 = (1, 2) if dil[1] == 1 else (1, 1)
    ref2 = oops.conv2d(x.numpy(), w.numpy(), b.numpy(), pad, stride, dil2, 1, q_scale.numpy(), q_mode.numpy())
    got2 = torch.ops.torch_mlu.conv2d(x.cuda(), wc, b.cuda(), list(pad), list(stride), list(dil2), 1, qs, qm)
    assert same_bits(ref2["y"], got2.cpu().numpy())
    got = torch.ops.torch_mlu.conv2d(x.cuda(), wc, b.cuda(), list(pad), list(stride), list(dil), 1, qs, qm)
    assert same_bits(ref["y"], got.cpu().numpy())


@pytest.mark.parametrize("k,co,h,w", [(1, 1, 101, 130), (3, 37, 120, 150), (7, 64, 100, 333), (10, 100, 160, 104)])
def test_conv2d_first_qint(k, co, h, w):
    """test/magicmind/op_test/test_conv.py:160-229 in the reference: an RGBA image with raw 0..255 pixel values goes
    to the device, the module normalises it with the mean / std recorded at calibration (firstconv), half input,
    stride (1, 4), padding (2, 2); rel-RMS <= 0.02 against the float model on the normalised image"""
    note("conv2d first conv", k, co, h, w)
    torch.manual_seed(k * 100 + co)
    mean, std = [0.485, 0.456, 0.406, 0.449], [0.229, 0.224, 0.225, 0.226]
    raw = torch.randint(0, 255, (1, 4, h, w)).float()
    x_cpu = (raw / 255.0 - torch.tensor(mean).view(1, 4, 1, 1)) / torch.tensor(std).view(1, 4, 1, 1)
    model = nn.Sequential(nn.Conv2d(4, co, k, (1, 4), (2, 2), (1, 1), 1, True)).eval().float()
    want_float = model(x_cpu).numpy()
    qconfig = {"use_avg": False, "data_scale": 1.0, "mean": mean, "std": std, "firstconv": True, "per_channel": True}
    calib = quantize_dynamic_mlu(model, qconfig, dtype="int8", gen_quant=True)
    calib(x_cpu)
    ckpt = calib.state_dict()
    np.testing.assert_allclose(ckpt["0.input_mean"].flatten().numpy(), np.array(mean) * 255, rtol=1e-6)
    qmodel = quantize_dynamic_mlu(model)
    qmodel.load_state_dict(ckpt)
    qmodel.half().to("cuda")
    conv = qmodel[0]
    got = qmodel(raw.half().to("cuda"))
    assert got.dtype == torch.float16 and got.shape == want_float.shape
    assert rel_rms(want_float, got.float().cpu().numpy()) <= 0.02
    # exact: the oracle on the tensor the module hands to the op
    x_norm = ((raw.half().cuda() - conv.input_mean) / conv.input_std)
    assert x_norm.dtype == torch.float16
    # the all-half model against the reference's half tensor ops: same integers, same output bits
    assert conv.scale.dtype == torch.float16
    r = ref_order.conv2d_per_channel(x_norm.cpu(), conv.weight.detach().cpu(), conv.bias.detach().cpu(), (2, 2), (1, 4),
                                     (1, 1), 1, conv.scale.detach().cpu(), conv.quantized_mode.cpu().numpy())
    q = torch.ops.torch_mlu.quantize_per_channel(conv.weight.detach(), conv.scale.detach()[2:], 8)[0]
    assert same_bits(r["qw"], q.permute(0, 2, 3, 1).contiguous().cpu().numpy())
    assert same_bits(r["y"].contiguous().numpy(), got.cpu().contiguous().numpy())


def test_conv2d_half_per_channel_overflows_to_inf_like_the_reference():
    """all-half per-channel convolution whose scaled integer sum exceeds 65504: the reference's vendor convolution
    returns half, so the value is inf before `/ new_scale` and `+ bias` see it (quantify_conv_forward.cpp:123-129);
    the fp32 quotient would have been finite"""
    note("conv2d half per-channel overflow")
    torch.manual_seed(5)
    co, ci = 16, 256
    # channel 0: one large tap (a wide weight range, so the shared position sits well above the other channels' own);
    # channels 1..7: 256 small positive taps on a positive input: the sum times new_scale (about 15.6) passes 65504
    # although the quotient (about 7700) does not; channels 8..15: the same taps with alternating signs, small sums
    w = torch.zeros(co, ci, 1, 1)
    w[0, 0] = 60.0
    w[1:8] = 0.5 + 0.01 * torch.rand(7, ci, 1, 1)
    sign = torch.tensor([1.0, -1.0]).repeat(ci // 2).reshape(1, ci, 1, 1)
    w[8:] = (0.5 + 0.01 * torch.rand(8, ci, 1, 1)) * sign
    w = w.half()
    x = (torch.rand(2, ci, 5, 5) * 60.0 + 30.0).half()
    bias = torch.randn(co).half()
    s_x = 127.0 / x.float().abs().max().item()
    s_w = 127.0 / w.float().reshape(co, -1).abs().amax(1)
    q_scale = torch.cat([torch.tensor([s_x, 0.0]), s_w]).half()
    q_mode = torch.tensor([3], dtype=torch.int32)
    r = ref_order.conv2d_per_channel(x, w, bias, (0, 0), (1, 1), (1, 1), 1, q_scale, q_mode.numpy())
    got = torch.ops.torch_mlu.conv2d(x.cuda(), w.cuda(), bias.cuda(), [0, 0], [1, 1], [1, 1], 1, q_scale.cuda(), q_mode.cuda())
    want = r["y"]
    assert torch.isinf(want[:, 1:8]).all() and torch.isfinite(want[:, 0]).all() and torch.isfinite(want[:, 8:]).all()
    assert same_bits(want.contiguous().numpy(), got.cpu().contiguous().numpy())


def test_empty_batches():
    """zero images / zero rows: the ops return empty tensors of the right shape and dtype, nothing is launched"""
    note("empty batches")
    w = torch.randn(8, 4, 3, 3)
    q_scale = torch.tensor([20.0, 30.0])
    q_mode = torch.tensor([1], dtype=torch.int32)
    for dt in (torch.float32, torch.float16):
        x = torch.zeros(0, 4, 9, 9, dtype=dt, device="cuda")
        y = torch.ops.torch_mlu.conv2d(x, w.cuda().to(dt), torch.zeros(8, device="cuda", dtype=dt), [1, 1], [2, 2], [1, 1], 1,
                                       q_scale.cuda(), q_mode.cuda())
        assert tuple(y.shape) == (0, 8, 5, 5) and y.dtype == dt
    xl = torch.zeros(0, 16, device="cuda")
    yl = torch.ops.torch_mlu.linear(xl, torch.randn(5, 16, device="cuda"), torch.zeros(5, device="cuda"), q_scale.cuda(),
                                    q_mode.cuda())
    assert tuple(yl.shape) == (0, 5)
    yl = torch.ops.torch_mlu.linear(torch.zeros(3, 0, 16, device="cuda"), torch.randn(5, 16, device="cuda"),
                                    torch.zeros(5, device="cuda"), q_scale.cuda(), q_mode.cuda())
    assert tuple(yl.shape) == (3, 0, 5)
    q = torch.ops.torch_mlu.quantize(torch.zeros(0, 7, device="cuda"), 8, -3)
    assert tuple(q.shape) == (0, 7) and q.dtype == torch.int8
    p = torch.ops.torch_mlu.maxpool_nhwc(torch.zeros(0, 8, 8, 16, dtype=torch.int8, device="cuda"), 3, 2, 1)
    assert tuple(p.shape) == (0, 4, 4, 16)
    g = torch.ops.torch_mlu.global_avgpool_nhwc(torch.zeros(0, 7, 7, 32, device="cuda"))
    assert tuple(g.shape) == (0, 32)
    y1 = torch.ops.torch_mlu.conv1d(torch.zeros(0, 4, 20, device="cuda"), torch.randn(6, 4, 3, device="cuda"),
                                    torch.zeros(6, device="cuda"), [1], [1], [1], 1, q_scale.cuda(), q_mode.cuda())
    assert tuple(y1.shape) == (0, 6, 20)
    y3 = torch.ops.torch_mlu.conv3d(torch.zeros(0, 4, 5, 6, 6, device="cuda"), torch.randn(6, 4, 3, 3, 3, device="cuda"),
                                    torch.zeros(6, device="cuda"), [1, 1, 1], [1, 1, 1], [1, 1, 1], 1, q_scale.cuda(),
                                    q_mode.cuda())
    assert tuple(y3.shape) == (0, 6, 5, 6, 6)
    m = torch.ops.torch_mlu.mm_q(torch.zeros(0, 16, dtype=torch.int8, device="cuda"), -3,
                                 torch.zeros(5, 16, dtype=torch.int8, device="cuda"), -4)
    assert tuple(m.shape) == (0, 5)
    # the fused plan on an empty batch
    from catch_amd import nets, pipeline
    layers = nets.resnet(18)
    net = nets.FloatNet(layers, seed=0).eval()
    xc = torch.randn(1, 3, 64, 64, generator=torch.Generator().manual_seed(1))
    fused = pipeline.FusedNet(layers, pipeline.calibrate(net, xc, "int8", True))
    out = fused.forward(torch.zeros(0, 3, 64, 64, device="cuda"))
    assert tuple(out.shape) == (0, 1000)
    torch.cuda.synchronize()


def test_strided_inputs_equal_their_contiguous_copies():
    """sliced / transposed / expanded views as input, weight and bias: same results as dense copies"""
    note("strided inputs")
    g = torch.Generator().manual_seed(21)
    big = torch.randn(3, 16, 12, 20, generator=g).cuda()
    x = big[:, ::2, 1:11, ::2]                      # [3, 8, 10, 10], strided in every dimension
    wbig = torch.randn(12, 8, 3, 6, generator=g).cuda() * 0.1
    w = wbig[::2, :, :, ::2]                        # [6, 8, 3, 3]
    bias = torch.randn(1, generator=g).cuda().expand(6)   # stride 0
    q_scale = torch.tensor([127.0 / x.abs().max().item(), 127.0 / w.abs().max().item()]).cuda()
    q_mode = torch.tensor([1], dtype=torch.int32).cuda()
    args = ([1, 1], [1, 1], [1, 1], 1, q_scale, q_mode)
    y = torch.ops.torch_mlu.conv2d(x, w, bias, *args)
    y_ref = torch.ops.torch_mlu.conv2d(x.contiguous(), w.contiguous(), bias.contiguous(), *args)
    assert torch.equal(y, y_ref)
    y_cl = torch.ops.torch_mlu.conv2d(x.contiguous(memory_format=torch.channels_last), w.contiguous(), bias.contiguous(), *args)
    assert torch.equal(y_cl, y_ref)
    xl = torch.randn(40, 7, generator=g).cuda().t()          # [7, 40], column-major
    wl = torch.randn(80, 5, generator=g).cuda().t()[:, ::2]  # [5, 40]
    qs = torch.tensor([127.0 / xl.abs().max().item(), 127.0 / wl.abs().max().item()]).cuda()
    yl = torch.ops.torch_mlu.linear(xl, wl, bias[:5], qs, q_mode)
    assert torch.equal(yl, torch.ops.torch_mlu.linear(xl.contiguous(), wl.contiguous(), bias[:5].contiguous(), qs, q_mode))
    # host-resident q-params are accepted like device-resident ones (the reference copies them to the host itself)
    assert torch.equal(torch.ops.torch_mlu.linear(xl, wl, bias[:5], qs.cpu(), q_mode.cpu()), yl)
    qq = torch.ops.torch_mlu.quantize(x, 8, -4)
    assert torch.equal(qq, torch.ops.torch_mlu.quantize(x.contiguous(), 8, -4))


def test_ops_from_several_threads():
    """the prepared-weight cache is shared by every thread of the process: four threads, each on a stream of its
    own, run one shared and one private layer over and over; every result equals the single-threaded one"""
    import threading
    note("threads")
    g = torch.Generator().manual_seed(33)
    shared_w = (torch.randn(32, 16, 3, 3, generator=g) * 0.1).cuda()
    shared_b = torch.randn(32, generator=g).cuda()
    q_mode = torch.tensor([3], dtype=torch.int32).cuda()

    def qscale(x, w):
        s_c = 127.0 / w.reshape(w.shape[0], -1).abs().max(1)[0]
        return torch.cat([torch.tensor([127.0 / x.abs().max().item(), 0.0], device="cuda"), s_c.cuda()])
    jobs = []
    for t in range(4):
        x = torch.randn(2, 16, 20, 20, generator=g).cuda()
        w = (torch.randn(24, 16, 3, 3, generator=g) * 0.1).cuda()
        b = torch.randn(24, generator=g).cuda()
        jobs.append((x, w, b, qscale(x, shared_w), qscale(x, w)))
    conv = torch.ops.torch_mlu.conv2d
    want = [(conv(x, shared_w, shared_b, [1, 1], [1, 1], [1, 1], 1, qs_s, q_mode),
             conv(x, w, b, [1, 1], [2, 2], [1, 1], 1, qs_p, q_mode)) for x, w, b, qs_s, qs_p in jobs]
    torch.cuda.synchronize()
    errors = []

    def work(t):
        x, w, b, qs_s, qs_p = jobs[t]
        try:
            with torch.cuda.stream(torch.cuda.Stream()):
                for i in range(25):
                    a = conv(x, shared_w, shared_b, [1, 1], [1, 1], [1, 1], 1, qs_s, q_mode)
                    c = conv(x, w, b, [1, 1], [2, 2], [1, 1], 1, qs_p, q_mode)
                    torch.cuda.current_stream().synchronize()
                    if not (torch.equal(a, want[t][0]) and torch.equal(c, want[t][1])):
                        errors.append((t, i))
        except Exception as exc:  # noqa: BLE001
            errors.append((t, repr(exc)))
    threads = [threading.Thread(target=work, args=(t,)) for t in range(4)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors


def test_first_use_of_a_weight_from_several_streams():
    """the cache entry of a weight is created by whichever thread comes first, on its stream; the others wait for
    that stream's quantization kernels before they read the entry"""
    import threading
    note("first use from several streams")
    g = torch.Generator().manual_seed(35)
    conv = torch.ops.torch_mlu.conv2d
    q_mode = torch.tensor([3], dtype=torch.int32).cuda()
    for rep in range(6):
        w = (torch.randn(512, 256, 3, 3, generator=g) * 0.05).cuda()   # a fresh tensor: nothing cached for it
        b = torch.randn(512, generator=g).cuda()
        x = torch.randn(1, 256, 6, 6, generator=g).cuda()
        s_c = 127.0 / w.reshape(512, -1).abs().max(1)[0]
        qs = torch.cat([torch.tensor([127.0 / x.abs().max().item(), 0.0], device="cuda"), s_c])
        torch.cuda.synchronize()
        outs, errors = [None] * 4, []
        gate = threading.Barrier(4)

        def work(t):
            try:
                with torch.cuda.stream(torch.cuda.Stream()):
                    gate.wait()
                    outs[t] = conv(x, w, b, [1, 1], [1, 1], [1, 1], 1, qs, q_mode)
                    torch.cuda.current_stream().synchronize()
            except Exception as exc:  # noqa: BLE001
                errors.append(repr(exc))
        threads = [threading.Thread(target=work, args=(t,)) for t in range(4)]
        for th in threads:
            th.start()
        for th in threads:
            th.join()
        assert not errors, errors
        torch.ops.torch_mlu.clear_weight_cache()
        want = conv(x, w, b, [1, 1], [1, 1], [1, 1], 1, qs, q_mode)
        for t in range(4):
            assert torch.equal(outs[t], want), (rep, t)


def test_half_q_scale_that_half_cannot_hold_is_refused():
    """an int16 per-channel scale 32767 / absmax is inf in half for absmax < 0.5: the op says so instead of
    deriving positions from inf (the module keeps such a q_scale in fp32 under .half())"""
    note("half q_scale overflow")
    torch.manual_seed(5)
    x = torch.randn(2, 16, 8, 8).half().cuda()
    w = (torch.randn(16, 16, 3, 3) * 0.05).half().cuda()
    b = torch.zeros(16).half().cuda()
    s_c = 32767.0 / w.float().reshape(16, -1).abs().max(1)[0]
    q_scale = torch.cat([torch.tensor([32767.0 / 4.0, 0.0], device="cuda"), s_c]).half()
    assert torch.isinf(q_scale).any()
    with pytest.raises(RuntimeError, match="half"):
        torch.ops.torch_mlu.conv2d(x, w, b, [1, 1], [1, 1], [1, 1], 1, q_scale, torch.tensor([4], dtype=torch.int32))
    # weights of magnitude >= 0.5: every int16 scale fits half; int16 parameters are still derived in fp32, from
    # the values the half tensor holds (half has neither 32767 nor the integers above 2048)
    w2 = (torch.randn(16, 16, 3, 3) * 0.5).half().cuda()
    s2 = torch.cat([torch.tensor([32767.0 / 4.0, 0.0], device="cuda"), 32767.0 / w2.float().reshape(16, -1).abs().max(1)[0]]).half()
    assert torch.isfinite(s2).all()
    got = torch.ops.torch_mlu.conv2d(x, w2, b, [1, 1], [1, 1], [1, 1], 1, s2, torch.tensor([4], dtype=torch.int32))
    ref = oops.conv2d(x.cpu().numpy(), w2.float().cpu().numpy(), b.float().cpu().numpy(), (1, 1), (1, 1), (1, 1), 1,
                      s2.float().cpu().numpy(), [4])
    assert same_bits(ref["y"], got.cpu().numpy())
