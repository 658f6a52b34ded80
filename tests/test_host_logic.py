"""CPU-side tests: the C ABI library loads and exports what the header declares, the host
q-param math agrees with the oracle, and the Python quantization tool packs q-params the way the
reference does.  No kernel is launched here."""
import ctypes
import math
import os
import re

import numpy as np
import pytest
import torch
import torch.nn as nn

import oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
rng = np.random.default_rng(99)


@pytest.fixture(scope="module")
def lib():
    from catch_amd import _native
    return _native.kernel_lib()


def test_library_exports_every_declared_symbol(lib):
    from catch_amd import _native
    header = open(os.path.join(ROOT, "include", "catchq.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(catchq_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 17
    assert declared == set(_native.SIGNATURES), declared ^ set(_native.SIGNATURES)
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.catchq_version() >= 100
    assert lib.catchq_status_string(3) == b"bitwidth not support"
    assert lib.catchq_status_string(2) == b"quantify only support input float/half"


def test_launch_sharing_hint_is_per_thread():
    """the planning hint lives in the calling thread (the kernel library takes it per call and keeps nothing):
    the op returns the previous value, rejects counts below one, and another thread sees its own default
    (results never depend on it: the GPU suite runs graphs recorded with 1, 2, 3 and 4)"""
    import threading
    import catch_amd  # noqa: F401
    op = torch.ops.torch_mlu.set_launch_sharing
    assert op(1) >= 1
    assert op(4) == 1
    assert op(2) == 4
    for bad in (0, -3):
        with pytest.raises(Exception):
            op(bad)
    seen = []
    th = threading.Thread(target=lambda: seen.append((op(3), op(1))))
    th.start()
    th.join()
    assert seen == [(1, 3)]      # the other thread started from the default and changed only its own value
    assert op(1) == 2            # this thread's value survived the rejected calls and the other thread


def test_torch_ops_are_registered():
    import catch_amd  # noqa: F401
    for name in ("conv2d", "linear", "quantize", "quantize_per_channel", "quantize_param", "mm_q", "qconv2d",
                 "qlinear", "dequantize"):
        assert hasattr(torch.ops.torch_mlu, name)
    schema = str(torch.ops.torch_mlu.conv2d.default._schema)
    assert schema.startswith("torch_mlu::conv2d(Tensor input, Tensor weight, Tensor bias, int[] padding, "
                             "int[] stride, int[] dilation, int groups, Tensor q_scale, Tensor q_mode) -> Tensor")
    assert str(torch.ops.torch_mlu.linear.default._schema).startswith(
        "torch_mlu::linear(Tensor input, Tensor weight, Tensor bias, Tensor q_scale, Tensor q_mode) -> Tensor")


def test_host_positions_match_oracle(lib):
    for bw in (8, 16):
        for s in np.exp(rng.uniform(-12, 14, 3000)).astype(np.float32):
            p = ctypes.c_int()
            assert lib.catchq_pos_from_scale(bw, float(s), ctypes.byref(p)) == 0
            assert p.value == orc.pos_from_scale(bw, s)
            f, sf = ctypes.c_float(), ctypes.c_float()
            assert lib.catchq_quant_params(bw, float(s), ctypes.byref(p), ctypes.byref(f), ctypes.byref(sf)) == 0
            op, of, osf = orc.quant_params(bw, s)
            assert (p.value, np.float32(f.value), np.float32(sf.value)) == (op, of, osf)
    p = ctypes.c_int()
    assert lib.catchq_pos_from_scale(12, 1.0, ctypes.byref(p)) == 3
    assert lib.catchq_pos_from_scale(8, 0.0, ctypes.byref(p)) == 1
    assert lib.catchq_pos_from_scale(8, float("inf"), ctypes.byref(p)) == 1


def test_host_per_channel_params_match_oracle_and_fixture(lib):
    def run(bw, s):
        s = np.ascontiguousarray(s, np.float32)
        ns, sf = np.empty_like(s), np.empty_like(s)
        p = ctypes.c_int()
        st = lib.catchq_per_channel_params(bw, s.ctypes.data, s.size, ctypes.byref(p), ns.ctypes.data, sf.ctypes.data)
        assert st == 0
        return p.value, ns, sf
    for bw in (8, 16):
        for co in (1, 3, 64, 1000):
            s = np.exp(rng.uniform(-2, 9, co)).astype(np.float32)
            p, ns, sf = run(bw, s)
            op, ons, osf = orc.per_channel_params(bw, s)
            assert p == op and np.array_equal(ns, ons) and np.array_equal(sf, osf)
    # the reference's fixture again, through the shipped code this time
    for line in open(os.path.join(ROOT, "tests", "golden", "inception_v3_qparams.txt")):
        name, rest = line.split(" position: ")
        pos, sc = rest.split(" scale: ")
        sc = np.array(sc.split(), dtype=np.float32)
        if sc.size > 1:
            p, ns, _ = run(8, (sc.astype(np.float64) * 2.0 ** (-int(pos))).astype(np.float32))
            assert p == int(pos), name
            np.testing.assert_allclose(ns, sc, rtol=2e-6)


def test_conv_out_size(lib):
    for (n, k, p, s, d) in [(224, 7, 3, 2, 1), (56, 3, 1, 1, 1), (24, 3, 3, 3, 1), (13, 3, 2, 1, 2), (5, 5, 0, 1, 1)]:
        want = torch.nn.functional.conv2d(torch.zeros(1, 1, n, n), torch.zeros(1, 1, k, k), None, s, p, d).shape[-1]
        assert lib.catchq_conv_out_size(n, k, p, s, d) == want == orc.conv_out_size(n, k, p, s, d)


def test_routes(lib):
    from catch_amd._native import ConvDesc
    def route(ci, co, k, groups, bits=(8, 8)):
        d = ConvDesc(1, 16, 16, ci, co, k, k, 0, 0, 1, 1, 1, 1, groups)
        return lib.catchq_conv2d_route(bits[0], bits[1], ctypes.byref(d)).decode()
    assert route(64, 64, 3, 1) == "mfma"
    assert route(3, 64, 7, 1) == "direct"
    assert route(4, 64, 7, 1) == "mfma"
    assert route(32, 32, 3, 32) == "depthwise"
    assert route(4, 16, 3, 2) == "direct"
    assert route(64, 64, 3, 1, (16, 16)) == "mfma_a16w16"
    assert route(4, 32, 3, 1, (16, 16)) == "direct"
    assert route(64, 64, 3, 1, (16, 8)) == "mfma_a16"
    assert route(8, 32, 3, 1, (16, 8)) == "mfma_a16"
    assert route(4, 32, 3, 1, (16, 8)) == "direct"
    assert route(64, 64, 30, 1) == "invalid"  # kernel larger than the image
    assert lib.catchq_gemm_route(8, 8, 4096, 3072, 768) == b"mfma"
    assert lib.catchq_gemm_route(8, 8, 10, 25, 10) == b"direct"
    assert lib.catchq_gemm_route(16, 8, 4096, 3072, 768) == b"mfma_a16"
    assert lib.catchq_gemm_route(16, 16, 4096, 3072, 768) == b"mfma_a16w16"
    assert lib.catchq_gemm_route(16, 16, 40, 30, 70000) == b"direct"  # K beyond what int32 digit sums hold


# ------------------------------------------------------------------ the Python tool (A1/A2/A15)
def _tool():
    import catch_amd  # noqa: F401
    from catch_amd.core.mlu_quantize import quantize_dynamic_mlu
    return quantize_dynamic_mlu


def test_observer_scale_rules():
    from catch_amd.core.quantized.observer import MLUMinMaxObserver, MLUPerChannelMinMaxObserver
    o = MLUMinMaxObserver(dtype="int8", qscheme={"iteration": 3, "use_avg": False, "data_scale": 1.0})
    o(torch.tensor([-2.0, 1.0]))
    o(torch.tensor([-1.0, 3.0]))
    o.calculate_qparams()
    assert (o.min_val, o.max_val) == (-2.0, 3.0) and o.scale == 127.0 / 3.0 == orc.calib_scale(8, -2.0, 3.0)
    o(torch.tensor([0.0, 1.0]))
    o(torch.tensor([-100.0, 100.0]))  # past `iteration`: ignored
    assert (o.min_val, o.max_val) == (-2.0, 3.0)
    a = MLUMinMaxObserver(dtype="int16", qscheme={"iteration": 4, "use_avg": True, "data_scale": 2.0})
    a(torch.tensor([-1.0, 1.0]))
    a(torch.tensor([-2.0, 4.0]))
    # running mean weighted by the call counter, which has already advanced (observer.py:149-162)
    assert a.max_val == (2.0 * 2 + 8.0) / 3 and a.min_val == (-2.0 * 2 - 4.0) / 3
    a.calculate_qparams()
    assert a.scale == 32767.0 / max(a.max_val, -a.min_val)
    z = MLUMinMaxObserver()
    z(torch.zeros(4))
    z.calculate_qparams()
    assert z.scale == 1.0
    pc = MLUPerChannelMinMaxObserver(dtype="int8")
    w = torch.tensor([[[1.0, -3.0]], [[0.5, 0.25]], [[0.0, 0.0]]])
    pc(w)
    pc.calculate_qparams()
    assert pc.scales == [127.0 / 3.0, 127.0 / 0.5, 1.0]


@pytest.mark.parametrize("bw,per_channel", [("int8", False), ("int8", True), ("int16", False), ("int16", True)])
def test_state_dict_packing(bw, per_channel):
    quantize_dynamic_mlu = _tool()
    torch.manual_seed(0)
    model = nn.Sequential(nn.Conv2d(3, 8, 3, bias=False), nn.ReLU(), nn.Flatten(), nn.Linear(8 * 6 * 6, 5)).eval()
    x = torch.randn(2, 3, 8, 8)
    calib = quantize_dynamic_mlu(model, {"per_channel": per_channel, "firstconv": False}, dtype=bw, gen_quant=True)
    out = calib(x)
    assert torch.equal(out, model(x))  # calibration is the float model
    sd = calib.state_dict()
    qmax = 127.0 if bw == "int8" else 32767.0
    s_in = qmax / x.abs().max().item()
    assert sd["0.scale"][0].item() == pytest.approx(s_in, rel=1e-6)
    assert sd["0.quantized_mode"].tolist() == [1 if bw == "int8" else 2]
    w = model[0].weight.detach()
    if per_channel:
        assert sd["0.scale"][1].item() == 0.0 and sd["0.quantized_by_channel"].tolist() == [1]
        np.testing.assert_allclose(sd["0.scale_weight_per_channel"].numpy(),
                                   qmax / w.reshape(8, -1).abs().max(1)[0].numpy(), rtol=1e-6)
    else:
        assert "0.quantized_by_channel" not in sd
        assert sd["0.scale"][1].item() == pytest.approx(qmax / w.abs().max().item(), rel=1e-6)
    q = quantize_dynamic_mlu(model)
    q.load_state_dict(sd)
    conv, lin = q[0], q[3]
    assert conv.scale.dtype == torch.float32 and conv.quantized_mode.dtype == torch.int32
    assert conv.scale.numel() == (2 + 8 if per_channel else 2) and lin.scale.numel() == (2 + 5 if per_channel else 2)
    want_mode = {("int8", False): 1, ("int16", False): 2, ("int8", True): 3, ("int16", True): 4}[(bw, per_channel)]
    assert conv.quantized_mode.tolist() == [want_mode] == lin.quantized_mode.tolist()
    assert torch.equal(conv.bias, torch.zeros(8))  # a missing bias becomes zeros (conv.py:130-131)
    assert torch.equal(q(x), model(x))  # CPU tensors: float path


@pytest.mark.parametrize("nd", [1, 3])
def test_conv1d_conv3d_modules_calibrate_and_pack(nd):
    """nn.Conv1d / nn.Conv3d are swapped like nn.Conv2d (core/quantized/default_mappings.py:10-16 and
    core/quantized/modules/conv.py:258-380 in the reference)"""
    quantize_dynamic_mlu = _tool()
    torch.manual_seed(nd)
    conv = nn.Conv1d(4, 6, 3, 2, 1) if nd == 1 else nn.Conv3d(4, 6, (1, 3, 3), 1, (0, 1, 1))
    model = nn.Sequential(conv).eval()
    x = torch.randn(2, 4, 11) if nd == 1 else torch.randn(2, 4, 3, 6, 6)
    calib = quantize_dynamic_mlu(model, {"per_channel": False, "firstconv": False}, dtype="int16", gen_quant=True)
    assert type(calib[0]).__name__ == "MLUConv%dd" % nd
    assert torch.equal(calib(x), model(x))
    sd = calib.state_dict()
    assert sd["0.scale"][0].item() == pytest.approx(32767.0 / x.abs().max().item(), rel=1e-6)
    assert sd["0.scale"][1].item() == pytest.approx(32767.0 / conv.weight.abs().max().item(), rel=1e-6)
    assert sd["0.quantized_mode"].tolist() == [2]
    q = quantize_dynamic_mlu(model)
    q.load_state_dict(sd)
    assert q[0]._get_name() == "MLUConv%dd" % nd and q[0].scale.numel() == 2
    assert torch.equal(q(x), model(x))  # CPU tensors: float path
    if nd == 3:
        with pytest.raises(AssertionError, match="per_channel"):
            quantize_dynamic_mlu(model, {"per_channel": True, "firstconv": False}, dtype="int8", gen_quant=True)


def test_first_conv_mean_std():
    quantize_dynamic_mlu = _tool()
    model = nn.Sequential(nn.Conv2d(3, 4, 3)).eval()
    spec = {"firstconv": True, "mean": [0.485, 0.456, 0.406], "std": [0.229, 0.224, 0.225], "per_channel": False}
    calib = quantize_dynamic_mlu(model, spec, dtype="int8", gen_quant=True)
    calib(torch.randn(1, 3, 8, 8))
    sd = calib.state_dict()
    np.testing.assert_allclose(sd["0.input_mean"].flatten().numpy(), np.array(spec["mean"]) * 255, rtol=1e-6)
    np.testing.assert_allclose(sd["0.input_std"].flatten().numpy(), np.array(spec["std"]) * 255, rtol=1e-6)
    q = quantize_dynamic_mlu(model)
    q.load_state_dict(sd)
    assert q[0].input_mean.shape == (1, 3, 1, 1)


def test_missing_native_library_is_loud(tmp_path, monkeypatch):
    from catch_amd import _native
    monkeypatch.setattr(_native, "_lib", None)
    monkeypatch.setattr(_native, "KERNEL_LIB", str(tmp_path / "nope.so"))
    with pytest.raises(ImportError, match="catch_amd/build.py"):
        _native.kernel_lib()


def test_lrn_and_norm_observers():
    """observer.py:172-199 and :252-294 in the reference: the LRN observer's scale describes the squared range;
    the norm observer keeps two ranges, of the max-normalised squares and of the channel norms"""
    from catch_amd.core.quantized import observer as obs
    x = torch.tensor([[[[1.0, 3.0]], [[2.0, 0.5]]]])  # [1, 2, 1, 2], non-negative like a post-ReLU tensor
    lrn = obs.mlu_lrn_observer("int8", {"iteration": 2})()
    lrn(x)
    lrn(x * 0.5)
    lrn(x * 100)  # beyond `iteration`: ignored
    lrn.calculate_qparams()
    assert (lrn.min_val, lrn.max_val) == (0.25, 3.0)
    assert lrn.scale == 127.0 / 9.0
    norm = obs.mlu_norm_observer("int16", {"iteration": 1})()
    norm(x)
    norm.calculate_qparams()
    sq = (x / 3.0) ** 2
    nr = sq.sum(1).sqrt() + 1e-10
    assert norm.boundary_1 == [sq.min().item(), sq.max().item()] and norm.boundary_2 == [nr.min().item(), nr.max().item()]
    assert norm.scale == [32767.0 / sq.max().item(), 32767.0 / nr.max().item()]


def test_per_channel_params_in_half_follow_the_tensor_ops(lib):
    """A .half() model derives the per-channel parameters with half tensors (quantify.cpp:64-98 in the dtype of
    scale_data).  The shipped host routine rounds every step to binary16 by hand; torch's CPU half kernels,
    applied expression by expression (oracle/ref_order.py), are the independent statement of the same chain."""
    from oracle import ref_order
    r = np.random.default_rng(5)
    for bw in (8, 16):
        qmax = 127.0 if bw == 8 else 32767.0
        for co in (1, 7, 64, 513):
            absmax = np.exp(r.uniform(np.log(0.6 if bw == 16 else 0.003), np.log(40.0), co))
            s = torch.from_numpy((qmax / absmax).astype(np.float32)).half()
            assert torch.isfinite(s).all()
            sb = s.numpy().view(np.uint16).copy()
            ns, sf = np.empty_like(sb), np.empty_like(sb)
            p = ctypes.c_int()
            assert lib.catchq_per_channel_params_f16(bw, sb.ctypes.data, co, ctypes.byref(p), ns.ctypes.data,
                                                     sf.ctypes.data) == 0
            w = torch.zeros(co, 2).half()
            _, want_pos, want_ns = ref_order.quantify_per_channel(w, s, bw)
            assert p.value == int(want_pos.float()[0])
            assert np.array_equal(ns.view(np.float16), want_ns.numpy())
    # a scale that half cannot hold is refused, not turned into garbage
    bad = np.array([np.float16(np.inf)]).view(np.uint16)
    out = np.empty(1, np.uint16)
    p = ctypes.c_int()
    assert lib.catchq_per_channel_params_f16(16, bad.ctypes.data, 1, ctypes.byref(p), out.ctypes.data, out.ctypes.data) == 1
