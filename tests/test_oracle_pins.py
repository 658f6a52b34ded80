"""Pins the CPU oracle against facts that do not come from the oracle itself:
the reference's own fixture, library routines (torch/numpy) in the special cases
where they compute the same thing, closed forms and brute force."""
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle as orc
from oracle import ops as oops

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
rng = np.random.default_rng(1234)


# ---------------------------------------------------------------- fp16 <-> fp32
def test_f16_to_f32_exhaustive():
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([orc.f16_to_f32(int(v)) for v in h], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(nan, np.isnan(got))  # NaN payloads are not part of the contract
    assert np.array_equal(want.view(np.uint32)[~nan], got.view(np.uint32)[~nan])


def test_f32_to_f16_ties_and_random():
    # every half value, the midpoint to its successor, and one fp32 ulp around the midpoint
    h = np.arange(0, 0x7c00, dtype=np.uint16)
    lo = h.view(np.float16).astype(np.float64)
    hi = (h + 1).view(np.float16).astype(np.float64)
    mid = ((lo + hi) / 2).astype(np.float32)
    cands = np.concatenate([mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf)),
                            -mid, rng.standard_normal(20000).astype(np.float32) * 1000,
                            np.array([0.0, -0.0, np.inf, -np.inf, 65504, 65519.99, 65520, 1e-8, 2.0 ** -25,
                                      2.0 ** -24], dtype=np.float32)])
    want = cands.astype(np.float16).view(np.uint16)
    got = np.array([orc.f32_to_f16(v) for v in cands], dtype=np.uint16)
    assert np.array_equal(want, got)


# ---------------------------------------------------------------- positions (A3/A4)
def _exact_pos(bw, scale):
    qmax = 127 if bw == 8 else 32767
    absmax = np.float32(qmax) / np.float32(scale)
    return math.frexp(float(absmax))[1] - 1 - (bw - 2), float(absmax)


def test_pos_from_scale_known_answers():
    # absmax = 4 -> floor(log2 4) = 2 -> 2 - 6 ; absmax = 1 -> -6 ; absmax=0.4 -> -2-6
    assert orc.pos_from_scale(8, 127.0 / 4.0) == -4
    assert orc.pos_from_scale(8, 127.0) == -6
    assert orc.pos_from_scale(8, 127.0 / 0.4) == -8
    assert orc.pos_from_scale(16, 32767.0 / 3.0) == 1 - 14
    assert orc.pos_from_scale(16, 32767.0 / 100.0) == 6 - 14


def test_pos_from_scale_bruteforce_against_exponent():
    for bw in (8, 16):
        for s in np.exp(rng.uniform(-12, 12, 4000)).astype(np.float32):
            want, absmax = _exact_pos(bw, s)
            m = math.frexp(absmax)[0]  # in [0.5,1)
            got = orc.pos_from_scale(bw, s)
            if 0.5 + 1e-5 < m < 1 - 1e-5:
                assert got == want
            else:  # float log near an exact power of two may fall either side
                assert abs(got - want) <= 1


def test_quant_params_closed_form():
    for bw in (8, 16):
        qmax = 127 if bw == 8 else 32767
        for s in np.exp(rng.uniform(-10, 10, 2000)).astype(np.float32):
            pos, frac, sf = orc.quant_params(bw, s)
            assert pos == orc.pos_from_scale(bw, s)
            # scale_ = 2^pos * qmax / absmax lies in (qmax/2^(n-1), qmax/2^(n-2)]   (utils.cpp:97-100)
            assert qmax / 2.0 ** (bw - 1) - 1e-5 <= frac <= qmax / 2.0 ** (bw - 2) + 1e-5
            absmax = qmax / float(s)
            assert math.isclose(frac, 2.0 ** pos * qmax / absmax, rel_tol=1e-5)
            # scale_factor = absmax / qmax = 1/s
            assert math.isclose(sf * float(s), 1.0, rel_tol=1e-5)


def test_calib_scale():
    assert orc.calib_scale(8, -2.0, 1.0) == 127.0 / 2.0
    assert orc.calib_scale(16, -1.0, 4.0) == 32767.0 / 4.0
    assert orc.calib_scale(8, 0.0, 0.0) == 1.0
    assert orc.calib_scale(8, float("nan"), 1.0) == 1.0


# ---------------------------------------------------------------- per-channel params (A7)
def _fixture_rows():
    rows = []
    for line in open(os.path.join(GOLDEN, "inception_v3_qparams.txt")):
        name, rest = line.split(" position: ")
        pos, sc = rest.split(" scale: ")
        sc = np.array(sc.split(), dtype=np.float32)
        rows.append((name, int(pos), sc))
    return rows


def test_per_channel_params_reference_fixture():
    """torch_mlu/csrc/test/data/test.txt holds, per Inception-v3 conv weight, the shared
    position and the per-channel scales the reference's quantizer produced.  Feeding the
    calibration scales they imply (s_c = new_scale_c * 2^-position) back through the
    derivation must reproduce them; 43 of the 99 rows are exact half-way cases of
    round((max+min)/2) and only round-half-to-even reproduces all of them."""
    rows = [r for r in _fixture_rows() if r[2].size > 1]
    assert len(rows) == 99
    halfway = 0
    for name, pos, sc in rows:
        s = (sc.astype(np.float64) * 2.0 ** (-pos)).astype(np.float32)
        new_pos, new_scale, sf = orc.per_channel_params(8, s)
        assert new_pos == pos, name
        np.testing.assert_allclose(new_scale, sc, rtol=2e-6, err_msg=name)
        np.testing.assert_allclose(sf, 1.0 / s.astype(np.float64), rtol=2e-6, err_msg=name)
        pc = np.floor(np.log2(127.0 / s.astype(np.float64))) - 6
        if (pc.max() + pc.min()) % 2 != 0:
            halfway += 1
            # the two other common rounding rules disagree with the fixture on some rows
    assert halfway == 43
    up = sum(1 for _, pos, sc in rows if _np_round_rule(sc, pos, "half_up") != pos)
    away = sum(1 for _, pos, sc in rows if _np_round_rule(sc, pos, "half_away") != pos)
    assert up > 0 and away > 0


def _np_round_rule(sc, pos, rule):
    s = sc.astype(np.float64) * 2.0 ** (-pos)
    pc = np.floor(np.log2(127.0 / s)) - 6
    v = (pc.max() + pc.min()) / 2
    if rule == "half_up":
        return int(math.floor(v + 0.5))
    return int(math.copysign(math.floor(abs(v) + 0.5), v))


def test_per_channel_params_invariants():
    for bw in (8, 16):
        qmax = 127.0 if bw == 8 else 32767.0
        s = np.exp(rng.uniform(-3, 9, 300)).astype(np.float32)
        new_pos, new_scale, sf = orc.per_channel_params(bw, s)
        pos_c = np.array([_exact_pos(bw, v)[0] for v in s])
        scale_c = new_scale.astype(np.float64) * 2.0 ** (pos_c - new_pos)
        lo, hi = qmax / 2.0 ** (bw - 1), qmax / 2.0 ** (bw - 2)
        assert np.all(scale_c >= lo - 1e-5) and np.all(scale_c <= hi + 1e-5)
        np.testing.assert_allclose(sf.astype(np.float64) * s, 1.0, rtol=3e-6)
        assert new_pos == int(np.rint((pos_c.max() + pos_c.min()) / 2))
        # one channel: shared position is that channel's own position
        p1, ns1, _ = orc.per_channel_params(bw, s[:1])
        assert p1 == pos_c[0] and lo - 1e-5 <= ns1[0] <= hi + 1e-5
        np.testing.assert_allclose(ns1[0], 2.0 ** p1 * qmax / (qmax / float(s[0])), rtol=3e-6)


# ---------------------------------------------------------------- quantize (A5)
@pytest.mark.parametrize("bw", [8, 16, 31])
def test_quantize_pos0_is_torch_round_clamp(bw):
    qmin, qmax = {8: (-128, 127), 16: (-32768, 32767), 31: (-2 ** 30, 2 ** 30 - 1)}[bw]
    x = np.concatenate([rng.standard_normal(50000) * 100, rng.standard_normal(5000) * 1e5,
                        np.arange(-300, 300) + 0.5, [0.0, -0.0, 1e30, -1e30, np.inf, -np.inf]]).astype(np.float32)
    want = torch.round(torch.from_numpy(x)).clamp(qmin, qmax).to(torch.int64).numpy()
    got = orc.quantize(x, bw, 0).astype(np.int64)
    assert np.array_equal(want, got)


@pytest.mark.parametrize("bw", [8, 16])
@pytest.mark.parametrize("pos", [-12, -7, -3, 0, 2, 5])
def test_quantize_position_exact_vs_float64(bw, pos):
    qmin, qmax = (-128, 127) if bw == 8 else (-32768, 32767)
    k = np.arange(-400, 400)
    ties = ((k + 0.5) * 2.0 ** pos).astype(np.float32)  # exactly representable half-way points
    x = np.concatenate([ties, np.nextafter(ties, np.float32(np.inf)), np.nextafter(ties, np.float32(-np.inf)),
                        (rng.standard_normal(40000) * 2.0 ** (pos + 6)).astype(np.float32)])
    want = np.clip(np.rint(x.astype(np.float64) * 2.0 ** (-pos)), qmin, qmax).astype(np.int64)
    got = orc.quantize(x, bw, pos).astype(np.int64)
    assert np.array_equal(want, got)
    # half-to-even on the ties specifically: results are all even
    t = orc.quantize(ties, 16, pos).astype(np.int64)
    assert np.all(t % 2 == 0)


def test_quantize_fp16_exhaustive():
    h = np.arange(65536, dtype=np.uint16).view(np.float16)
    for bw, pos in ((8, -4), (16, -9), (8, 0), (16, 3)):
        qmin, qmax = (-128, 127) if bw == 8 else (-32768, 32767)
        f = h.astype(np.float64)
        want = np.where(np.isnan(f), 0, np.clip(np.rint(np.nan_to_num(f, nan=0.0) * 2.0 ** (-pos)), qmin, qmax))
        got = orc.quantize(h, bw, pos)
        assert np.array_equal(want.astype(np.int64), got.astype(np.int64))


def test_quantize_fractional_scale_and_nan():
    x = (rng.standard_normal(30000) * 3).astype(np.float32)
    s = np.float32(1.3721)
    want = np.clip(np.rint((x * s).astype(np.float32).astype(np.float64) * 2.0 ** 5), -128, 127)
    assert np.array_equal(want.astype(np.int64), orc.quantize(x, 8, -5, s).astype(np.int64))
    assert orc.quantize(np.array([np.nan], np.float32), 8, -3)[0] == 0
    assert orc.quantize(np.zeros((0,), np.float32), 8, 0).size == 0


def test_quantize_nchw_to_nhwc_matches_plain():
    x = rng.standard_normal((2, 3, 5, 7)).astype(np.float32)
    q = orc.quantize_nchw_to_nhwc(x, 8, -5, 1.0, cpad=4)
    want = orc.quantize(np.transpose(x, (0, 2, 3, 1)), 8, -5)
    assert np.array_equal(q[..., :3], want) and np.all(q[..., 3] == 0)


@pytest.mark.parametrize("bw", [8, 16])
def test_quantize_per_channel_is_round_div_clamp(bw):
    """the reference spells the op chain out: clamp(round(input / scale_factor)) (quantify.cpp:100-105)"""
    qmin, qmax = (-128, 127) if bw == 8 else (-32768, 32767)
    w = (rng.standard_normal((17, 5, 3, 3)) * 0.05).astype(np.float32)
    s = (qmax / np.abs(w).reshape(17, -1).max(1)).astype(np.float32)
    _, _, sf = orc.per_channel_params(bw, s)
    want = torch.clamp(torch.round(torch.from_numpy(w) / torch.from_numpy(sf).reshape(-1, 1, 1, 1)), qmin, qmax)
    got = orc.quantize_per_channel(w, bw, sf)
    assert np.array_equal(want.numpy().astype(np.int64), got.astype(np.int64))
    assert np.abs(got.astype(np.int64)).max() >= qmax - 1  # the range is used


def test_dequantize():
    q = rng.integers(-128, 128, 1000).astype(np.int8)
    np.testing.assert_array_equal(orc.dequantize(q, -5), q.astype(np.float32) * np.float32(2.0 ** -5))
    q32 = rng.integers(-2 ** 20, 2 ** 20, 1000).astype(np.int32)
    np.testing.assert_array_equal(orc.dequantize(q32, -9, 1.5),
                                  (q32.astype(np.float32) * np.float32(2.0 ** -9)) / np.float32(1.5))


# ---------------------------------------------------------------- int contraction (A9/A12)
@pytest.mark.parametrize("bits", [(8, 8), (16, 8), (16, 16)])
def test_gemm_nt_vs_torch_int64(bits):
    lim = {8: 128, 16: 32768}
    a = rng.integers(-lim[bits[0]], lim[bits[0]], (37, 129)).astype(np.int8 if bits[0] == 8 else np.int16)
    b = rng.integers(-lim[bits[1]], lim[bits[1]], (23, 129)).astype(np.int8 if bits[1] == 8 else np.int16)
    want = torch.from_numpy(a.astype(np.int64)) @ torch.from_numpy(b.astype(np.int64)).T
    got, ovf = orc.gemm_nt(a, b)
    assert ovf == 0 or bits == (16, 16)
    assert np.array_equal(want.numpy(), got)


def test_gemm_overflow_is_counted():
    a = np.full((1, 600), 32767, np.int16)
    b = np.full((1, 600), 127, np.int8)
    acc, ovf = orc.gemm_nt(a, b)
    assert ovf == 1 and acc[0, 0] == 32767 * 127 * 600


CONV_CASES = [
    # N, Ci, H, W, Co, kh, kw, pad, stride, dil, groups
    (3, 64, 24, 24, 64, 3, 3, (3, 3), (3, 3), (1, 1), 1),  # the reference's qint grid (test_conv.py:104-131)
    (2, 4, 6, 6, 16, 3, 3, (0, 0), (1, 1), (1, 1), 2),     # its groups case (test_conv.py:83-100)
    (1, 3, 14, 14, 8, 2, 2, (0, 0), (1, 1), (1, 1), 1),
    (2, 6, 9, 11, 10, 3, 2, (1, 2), (2, 1), (2, 1), 2),
    (1, 8, 10, 10, 8, 3, 3, (1, 1), (2, 2), (1, 1), 8),    # depthwise
    (1, 5, 7, 7, 4, 1, 1, (0, 0), (1, 1), (1, 1), 1),
    (1, 16, 5, 5, 32, 5, 5, (2, 2), (1, 1), (1, 1), 1),
]


@pytest.mark.parametrize("case", CONV_CASES)
@pytest.mark.parametrize("xbits", [8, 16])
def test_conv2d_vs_torch_float64(case, xbits):
    n, ci, h, w, co, kh, kw, pad, stride, dil, g = case
    lim = 128 if xbits == 8 else 32768
    x = rng.integers(-lim, lim, (n, ci, h, w)).astype(np.int8 if xbits == 8 else np.int16)
    wt = rng.integers(-128, 128, (co, ci // g, kh, kw)).astype(np.int8)
    want = F.conv2d(torch.from_numpy(x.astype(np.float64)), torch.from_numpy(wt.astype(np.float64)), None,
                    stride, pad, dil, g).numpy().astype(np.int64)
    got, ovf = orc.conv2d_nhwc(np.transpose(x, (0, 2, 3, 1)), np.transpose(wt, (0, 2, 3, 1)), pad, stride, dil, g)
    assert ovf == 0
    assert np.array_equal(want, np.transpose(got, (0, 3, 1, 2)).astype(np.int64))
    assert got.shape[1] == orc.conv_out_size(h, kh, pad[0], stride[0], dil[0])


# ---------------------------------------------------------------- epilogue
def test_epilogue_identity_and_order():
    acc = rng.integers(-2 ** 26, 2 ** 26, (50, 12)).astype(np.int32)
    assert np.array_equal(orc.epilogue(acc, 0), acc.astype(np.float32))
    div = rng.uniform(0.5, 4, 12).astype(np.float32)
    bias = rng.standard_normal(12).astype(np.float32)
    res = rng.standard_normal((50, 12)).astype(np.float32)
    v = acc.astype(np.float32) * np.float32(2.0 ** -11)
    v = v / div
    v = v + bias
    v = v + res
    relu = np.where(v > 0, v, np.float32(0))
    assert np.array_equal(orc.epilogue(acc, -11, div, bias, res, 1), relu)
    assert np.array_equal(orc.epilogue(acc, -11, div, bias, res, 2), np.minimum(relu, np.float32(6)))
    assert np.array_equal(orc.epilogue(acc, -11, div, bias, res, 1, np.float16), relu.astype(np.float16))
    # no fused multiply-add between the scaling and the bias: exact because 2^e scaling is exact
    a1 = np.array([[2 ** 24 + 1]], np.int32)  # cvt rounds to 2^24, then exact scale, then add
    assert orc.epilogue(a1, -24, None, np.array([1.0], np.float32))[0, 0] == np.float32(2.0)


# ---------------------------------------------------------------- the reference's own acceptance metric
def _rel_rms(a, b):  # test/common_utils.py:514-522 (use_MSE)
    return math.sqrt(((a - b) ** 2).sum() / (a ** 2).sum())


def _calibrate(x, w, bw, per_channel):
    qmax = 127.0 if bw == 8 else 32767.0
    s_in = orc.calib_scale(bw, x.min(), x.max())
    if per_channel:
        wf = w.reshape(w.shape[0], -1)
        s_c = [orc.calib_scale(bw, lo, hi) for lo, hi in zip(wf.min(1), wf.max(1))]
        return np.array([s_in, 0.0] + s_c, np.float32), np.array([3 if bw == 8 else 4], np.int32)
    return np.array([s_in, orc.calib_scale(bw, w.min(), w.max())], np.float32), np.array([1 if bw == 8 else 2], np.int32)


@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("bw", [8, 16])
@pytest.mark.parametrize("per_channel", [True, False])
@pytest.mark.parametrize("half", [False, True])
def test_reference_conv_grid_rel_rms(bias, bw, per_channel, half):
    """test/magicmind/op_test/test_conv.py:103-156: N=3 Ci=Co=64 HW=24 K=3 pad=3 stride=3, <= 0.02 vs float"""
    g = torch.Generator().manual_seed(7)
    conv = torch.nn.Conv2d(64, 64, 3, 3, 3, 1, 1, bias)
    x = torch.randn(3, 64, 24, 24, generator=g)
    with torch.no_grad():
        want = conv(x).numpy()
    w = conv.weight.detach().numpy()
    b = conv.bias.detach().numpy() if bias else None
    q_scale, q_mode = _calibrate(x.numpy(), w, bw, per_channel)
    xin = x.numpy().astype(np.float16) if half else x.numpy()
    r = oops.conv2d(xin, w, b, (3, 3), (3, 3), (1, 1), 1, q_scale, q_mode)
    assert r["overflow"] == 0 or bw == 16  # int16 x int16 is defined on the exact (int64) sum
    assert r["y"].dtype == (np.float16 if half else np.float32)
    assert _rel_rms(want.astype(np.float64), r["y"].astype(np.float64)) <= 0.02


@pytest.mark.parametrize("ni,ci,co", [(1, 10, 25), (10, 50, 75), (20, 100, 125)])
@pytest.mark.parametrize("bw", [8, 16])
@pytest.mark.parametrize("per_channel", [True, False])
def test_reference_linear_grid_rel_rms(ni, ci, co, bw, per_channel):
    """test/magicmind/op_test/test_matmul.py:116-174, <= 0.02 vs float"""
    g = torch.Generator().manual_seed(ni + ci)
    lin = torch.nn.Linear(ci, co, True)
    x = torch.rand(ni, ci, generator=g)
    with torch.no_grad():
        want = lin(x).numpy()
    w, b = lin.weight.detach().numpy(), lin.bias.detach().numpy()
    q_scale, q_mode = _calibrate(x.numpy(), w, bw, per_channel)
    r = oops.linear(x.numpy(), w, b, q_scale, q_mode)
    assert (r["overflow"] == 0 or bw == 16) and r["y"].dtype == np.float32
    assert _rel_rms(want.astype(np.float64), r["y"].astype(np.float64)) <= 0.02


def test_dequantized_float_conv_agrees():
    """float conv of the dequantized integers == integer conv scaled by 2^(pos_x+pos_w)"""
    x = rng.standard_normal((1, 8, 9, 9)).astype(np.float32)
    w = (rng.standard_normal((6, 8, 3, 3)) * 0.1).astype(np.float32)
    q_scale, q_mode = _calibrate(x, w, 8, False)
    r = oops.conv2d(x, w, None, (1, 1), (1, 1), (1, 1), 1, q_scale, q_mode)
    xd = orc.dequantize(np.transpose(r["qx"], (0, 3, 1, 2)), r["pos_x"]).astype(np.float64)
    wd = orc.dequantize(np.transpose(r["qw"], (0, 3, 1, 2)), r["pos_w"]).astype(np.float64)
    want = F.conv2d(torch.from_numpy(xd), torch.from_numpy(wd), None, 1, 1).numpy()
    np.testing.assert_allclose(r["y"], want, rtol=1e-6, atol=1e-6)


# ---------------------------------------------------------------- 1-d and 3-d convolutions
@pytest.mark.parametrize("case", [
    # N, Ci, L, Co, k, pad, stride, dil, groups
    (2, 6, 33, 8, 3, 1, 1, 1, 1),
    (3, 8, 40, 12, 5, 2, 2, 2, 4),
    (1, 4, 9, 4, 1, 0, 1, 1, 1),
])
@pytest.mark.parametrize("per_channel", [False, True])
def test_conv1d_dequantized_float_conv_agrees(case, per_channel):
    """torch's float64 conv1d of the dequantized integers pins the oracle's 1-d composition"""
    n, ci, length, co, k, pad, stride, dil, g = case
    x = rng.standard_normal((n, ci, length)).astype(np.float32)
    w = (rng.standard_normal((co, ci // g, k)) * 0.1).astype(np.float32)
    q_scale, q_mode = _calibrate(x, w, 8, per_channel)
    r = oops.conv1d(x, w, None, (pad,), (stride,), (dil,), g, q_scale, q_mode)
    xq = torch.from_numpy(np.transpose(r["qx"][:, 0], (0, 2, 1)).astype(np.float64))
    wq = torch.from_numpy(np.transpose(r["qw"][:, 0], (0, 2, 1)).astype(np.float64))
    want_acc = F.conv1d(xq, wq, None, stride, pad, dil, g).numpy().astype(np.int64)
    assert np.array_equal(want_acc, np.transpose(r["acc"][:, 0], (0, 2, 1)))
    want = want_acc * 2.0 ** (r["pos_x"] + r["pos_w"])
    if per_channel:
        want = want / r["new_scale"].astype(np.float64)[None, :, None]
    np.testing.assert_allclose(r["y"], want, rtol=1e-6, atol=1e-6)
    assert _rel_rms(F.conv1d(torch.from_numpy(x), torch.from_numpy(w), None, stride, pad, dil, g).numpy(), r["y"]) <= 0.03


@pytest.mark.parametrize("case", [
    # N, Ci, D, H, W, Co, (kd,kh,kw), pad, stride, dil, groups
    (2, 4, 6, 8, 8, 8, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 1),
    (1, 6, 7, 9, 5, 4, (2, 3, 1), (1, 0, 1), (2, 1, 2), (2, 1, 1), 2),
    (2, 3, 5, 6, 6, 5, (1, 3, 3), (0, 1, 1), (1, 2, 2), (1, 1, 1), 1),   # kd == 1: depth folds into the batch
    (1, 8, 4, 5, 5, 8, (3, 1, 1), (0, 0, 0), (1, 1, 1), (1, 1, 1), 1),   # kh == kw == 1
])
@pytest.mark.parametrize("xbits", [8, 16])
def test_conv3d_vs_torch_float64(case, xbits):
    """the oracle's sum over depth taps against torch's float64 conv3d of the same integers"""
    n, ci, d, h, w, co, k, pad, stride, dil, g = case
    x = rng.standard_normal((n, ci, d, h, w)).astype(np.float32)
    wt = (rng.standard_normal((co, ci // g) + k) * 0.1).astype(np.float32)
    bias = rng.standard_normal(co).astype(np.float32)
    q_scale, q_mode = _calibrate(x, wt, xbits, False)
    r = oops.conv3d(x, wt, bias, pad, stride, dil, g, q_scale, q_mode)
    assert r["qx"].dtype == (np.int8 if xbits == 8 else np.int16)
    xq = torch.from_numpy(np.transpose(r["qx"], (0, 4, 1, 2, 3)).astype(np.float64))
    wq = torch.from_numpy(np.transpose(r["qw"], (0, 4, 1, 2, 3)).astype(np.float64))
    want_acc = F.conv3d(xq, wq, None, stride, pad, dil, g).numpy().astype(np.int64)
    assert np.array_equal(want_acc, np.transpose(r["acc"], (0, 4, 1, 2, 3)))
    want = want_acc * 2.0 ** (r["pos_x"] + r["pos_w"]) + bias.astype(np.float64)[None, :, None, None, None]
    np.testing.assert_allclose(r["y"], want, rtol=1e-6, atol=1e-6)
    ref = F.conv3d(torch.from_numpy(x), torch.from_numpy(wt), torch.from_numpy(bias), stride, pad, dil, g).numpy()
    assert _rel_rms(ref, r["y"]) <= 0.03


# ---------------------------------------------------------------- position + fractional scale per tensor / per axis
@pytest.mark.parametrize("per_axis", [False, True])
@pytest.mark.parametrize("bw", [8, 16])
def test_decode_fractional_is_the_exact_step_quantization(per_axis, bw):
    """decode_fractional restates setQuantizedParams / ...PerAxis (jit/utils/utils.cpp:81-167): what fixes it is
    that position and fractional scale together give a step of absmax / qmax -- the extreme element maps to
    +-qmax, every element is within half a step, and acc * 2^exp2 / div[c] is the real-valued product."""
    qmax = 127.0 if bw == 8 else 32767.0
    co = 6
    w = (rng.standard_normal((co, 3, 3, 5)) * np.exp(rng.uniform(-3, 3, (co, 1, 1, 1)))).astype(np.float32)
    x = (rng.standard_normal((2, 7, 7, 5)) * 3.7).astype(np.float32)
    s_in = np.float32(qmax / np.abs(x).max())
    if per_axis:
        s_c = (qmax / np.abs(w).reshape(co, -1).max(1)).astype(np.float32)
        q_scale, mode = np.concatenate(([s_in, 0.0], s_c)).astype(np.float32), (3 if bw == 8 else 4)
    else:
        s_c = np.full(co, qmax / np.abs(w).max(), np.float32)
        q_scale, mode = np.array([s_in, s_c[0]], np.float32), (1 if bw == 8 else 2)
    d = oops.decode_fractional(q_scale, [mode], co)
    assert d["bw"] == bw and d["pos_c"].size == (co if per_axis else 1)
    assert 1.0 <= d["scale_x"] < 2.0 + 1e-6 and ((1.0 <= d["scale_c"]) & (d["scale_c"] < 2.0 + 1e-6)).all()
    qx = orc.quantize(x, bw, d["pos_x"], d["scale_x"])
    qw = oops.quantize_weight_fractional(w, d)
    assert np.abs(qx).max() == qmax
    step_x = 1.0 / float(s_in)
    assert np.abs(qx * step_x - x).max() <= 0.5 * step_x * (1 + 1e-4)
    for c in range(co):
        step = 1.0 / float(s_c[c])
        if per_axis:
            assert np.abs(qw[c]).max() == qmax
        assert np.abs(qw[c] * step - w[c]).max() <= 0.5 * step * (1 + 1e-4)
        # dequantization constant: 2^exp2 / div[c] = step_x * step_c
        assert math.isclose(2.0 ** d["exp2"] / float(d["div"][c]), step_x * step, rel_tol=1e-5)
    if not per_axis:
        assert np.abs(qw).max() == qmax
    # against the float convolution: finer than the power-of-two quantization of the same tensors can be
    acc, _ = orc.conv2d_nhwc(qx, qw, (1, 1), (1, 1), (1, 1), 1)
    y = orc.epilogue(acc, d["exp2"], d["div"], None, None, 0, np.float32)
    ref = F.conv2d(torch.from_numpy(np.transpose(x, (0, 3, 1, 2)).astype(np.float64)),
                   torch.from_numpy(np.transpose(w, (0, 3, 1, 2)).astype(np.float64)), None, 1, 1).numpy()
    assert _rel_rms(np.transpose(ref, (0, 2, 3, 1)), y) <= (0.03 if bw == 8 else 2e-4)


# ---------------------------------------------------------------- position (+ scale) from a tensor's max-abs (A6)
@pytest.mark.parametrize("bw", [8, 16])
def test_quantize_param_position_is_the_exponent_and_scale_the_exact_quotient(bw):
    """What fixes position and scale without the vendor library: the position is the one of
    get_pos_from_scale_data (cnnl_util.cpp:337-347: floor(log2 absmax) - (n-2), here from frexp, which is
    exact where the float logarithm is not), and position + scale together map absmax onto qmax
    (setQuantizedParams, jit/utils/utils.cpp:97-100: scale = 2^pos * qmax / absmax), evaluated in exact
    rational arithmetic and rounded once to fp32."""
    from fractions import Fraction
    qmax = 127 if bw == 8 else 32767
    n = bw
    vals = np.concatenate([np.exp(rng.uniform(-30, 30, 3000)),
                           2.0 ** np.arange(-40, 41),                       # exact powers of two
                           np.nextafter(np.float32(2.0) ** np.arange(-20, 21, dtype=np.float32), np.float32(0)),
                           [1e-40, 1.4e-45, 3.0e-39, 3.4e38, 1.0, 127.0, 32767.0]]).astype(np.float32)
    for a in vals:
        pos, scale, off = orc.quantize_param(a, bw)
        m, e = math.frexp(float(a))          # a = m * 2^e, m in [0.5, 1)
        assert pos == e - 1 - (n - 2), a
        assert off == 0.0
        exact = Fraction(2) ** pos * qmax / Fraction(float(a))
        if exact > Fraction(3.4e38):
            continue                          # the quotient leaves fp32 (denormal absmax): no finite scale to pin
        want = np.float32(float(exact)) if exact < Fraction(2) ** 1000 else np.float32(np.inf)
        # float(Fraction) rounds once to double; the fp32 quotient of two fp32-exact numbers is the
        # correctly rounded result, which the double detour reproduces except on a double-rounding tie
        assert abs(float(scale) - float(exact)) <= float(np.spacing(np.float32(float(exact)))) / 2 * (1 + 1e-9), a
        # scale in (qmax / 2^(n-1), qmax / 2^(n-2)]: the tensor's extreme element lands on +-qmax exactly
        assert qmax / 2.0 ** (n - 1) * (1 - 1e-6) <= scale <= qmax / 2.0 ** (n - 2) * (1 + 1e-6)
        assert abs(int(orc.quantize(np.array([a, -a], np.float32), bw, pos, scale)[0])) == qmax
        # position alone (the eager quantizer's scale = 1) uses at least half of the range
        q = orc.quantize(np.array([a], np.float32), bw, pos)[0]
        assert 2 ** (n - 2) <= int(q) <= qmax


@pytest.mark.parametrize("bw", [8, 16])
def test_quantize_param_agrees_with_the_scale_route(bw):
    """absmax -> (position, scale) must be the same numbers the reference derives from the calibration
    scale qmax / absmax (orc_quant_params, pinned above), away from exact powers of two where the
    float logarithm of that route may fall either side."""
    qmax = 127.0 if bw == 8 else 32767.0
    for a in np.exp(rng.uniform(-8, 8, 2000)).astype(np.float32):
        if not 0.5 + 1e-4 < math.frexp(float(a))[0] < 1 - 1e-4:
            continue
        pos, scale, _ = orc.quantize_param(a, bw)
        p2, frac, _ = orc.quant_params(bw, np.float32(qmax) / a)
        assert pos == p2
        assert math.isclose(float(scale), float(frac), rel_tol=3e-7)


def test_quantize_param_degenerate_inputs():
    for bw in (8, 16):
        assert orc.quantize_param(0.0, bw) == (0, 1.0, 0.0)
        assert orc.quantize_param(np.inf, bw) == (0, 1.0, 0.0)
        assert orc.quantize_param(np.nan, bw) == (0, 1.0, 0.0)
    # smallest denormal: exponent -149
    assert orc.quantize_param(1.4e-45, 8)[0] == -149 - 6
    assert orc.absmax(np.array([1.0, -3.5, np.nan, 2.0], np.float32)) == 3.5   # NaN is skipped
    assert orc.absmax(np.zeros(0, np.float32)) == 0.0


# ---------------------------------------------------------------- pooling between the quantized ops
@pytest.mark.parametrize("k,stride,pad", [(2, 2, 0), (3, 2, 1), (3, 1, 1), (2, 1, 1), (5, 1, 2), (3, 3, 0), (4, 2, 2),
                                          (1, 1, 0), (13, 1, 6), (3, 2, 0)])
@pytest.mark.parametrize("hw", [(7, 9), (12, 12), (5, 6)])
def test_maxpool_vs_torch(k, stride, pad, hw):
    """F.max_pool2d (floor mode, -inf padding) over windows that hang over every border"""
    h, w = hw
    if h + 2 * pad < k or w + 2 * pad < k:
        pytest.skip("window larger than the padded image")
    x = rng.standard_normal((2, h, w, 5)).astype(np.float32)
    x[0, 0, 0, :] = 1e30       # corners and edges carry the extreme values
    x[1, -1, -1, :] = 1e30
    x[1, 0, -1, 2] = -1e30
    want = F.max_pool2d(torch.from_numpy(np.transpose(x, (0, 3, 1, 2))), k, stride, pad).numpy()
    got = orc.maxpool_nhwc(x, k, stride, pad)
    assert np.array_equal(np.transpose(want, (0, 2, 3, 1)), got)
    neg = -np.abs(x)            # all-negative input: a zero-valued padding would win, -inf never does
    want = F.max_pool2d(torch.from_numpy(np.transpose(neg, (0, 3, 1, 2))), k, stride, pad).numpy()
    assert np.array_equal(np.transpose(want, (0, 2, 3, 1)), orc.maxpool_nhwc(neg, k, stride, pad))


def test_global_avgpool_is_the_sequential_fp32_sum():
    """np.cumsum over fp32 is a sequential left-to-right sum by construction: its last element over the
    pixel axis, divided once by the pixel count, is the definition; a float64 mean bounds it; and an input
    built so that sequential, pairwise and reversed summation give three different fp32 results tells
    the order apart."""
    x = (rng.standard_normal((3, 7, 7, 11)) * 10).astype(np.float32)
    got = orc.global_avgpool_nhwc(x)
    flat = x.reshape(3, 49, 11)
    want = np.cumsum(flat, axis=1, dtype=np.float32)[:, -1, :] / np.float32(49)
    assert np.array_equal(want, got)
    mean64 = flat.astype(np.float64).mean(1)
    bound = 49 * 2.0 ** -24 * np.abs(flat).astype(np.float64).sum(1) / 49 + 2.0 ** -24 * np.abs(mean64)
    assert np.all(np.abs(got - mean64) <= bound)
    # 2^24, 1, 1, 1: left to right every +1 is a tie that rounds back to 2^24 -> 2^24; pairwise
    # (2^24 + 1) + (1 + 1) -> 2^24 + 2; right to left 1+1+1 = 3, + 2^24 -> 2^24 + 4 (tie to even)
    c = np.array([2.0 ** 24, 1, 1, 1], np.float32).reshape(1, 2, 2, 1)
    assert orc.global_avgpool_nhwc(c)[0, 0] == np.float32(2.0 ** 24) / np.float32(4)
    pair = (c[0, 0, 0, 0] + c[0, 0, 1, 0]) + (c[0, 1, 0, 0] + c[0, 1, 1, 0])
    rev = ((c[0, 1, 1, 0] + c[0, 1, 0, 0]) + c[0, 0, 1, 0]) + c[0, 0, 0, 0]
    assert pair == np.float32(2.0 ** 24 + 2) and rev == np.float32(2.0 ** 24 + 4)
    # one pixel, and the division is a true division (49 is not a power of two)
    one = rng.standard_normal((2, 1, 1, 4)).astype(np.float32)
    assert np.array_equal(orc.global_avgpool_nhwc(one), one.reshape(2, 4))
    t = np.full((1, 7, 7, 1), 0.1, np.float32)
    assert orc.global_avgpool_nhwc(t)[0, 0] == np.cumsum(t.reshape(-1), dtype=np.float32)[-1] / np.float32(49)


# ---------------------------------------------------------------- the reference's tensor-op order, dtype by dtype
@pytest.mark.parametrize("bw", [8, 16])
def test_tensor_op_restatement_equals_the_c_oracle_in_fp32(bw):
    """oracle/ref_order.py spells the per-channel branches out of torch tensor ops the way the reference does
    (quantify.cpp:55-114; quantify_conv_forward.cpp:107-131; linear.cpp:40-70).  With fp32 tensors it must give
    the numbers of the C restatement bit for bit -- two independent statements of the same lines."""
    from oracle import ref_order
    g = torch.Generator().manual_seed(3 + bw)
    qmax = 127.0 if bw == 8 else 32767.0
    x = torch.randn(3, 64, 24, 24, generator=g)
    w = torch.randn(64, 64, 3, 3, generator=g) * 0.04 * (torch.rand(64, 1, 1, 1, generator=g) * 4 + 0.1)
    b = torch.randn(64, generator=g)
    q_scale = torch.cat([torch.tensor([qmax / x.abs().max().item(), 0.0]), qmax / w.reshape(64, -1).abs().max(1)[0]]).float()
    mode = [3 if bw == 8 else 4]
    r = ref_order.conv2d_per_channel(x, w, b, (3, 3), (3, 3), (1, 1), 1, q_scale, mode)
    o = oops.conv2d(x.numpy(), w.numpy(), b.numpy(), (3, 3), (3, 3), (1, 1), 1, q_scale.numpy(), mode)
    assert r["new_pos"] == o["pos_w"] and np.array_equal(r["new_scale"].numpy(), o["new_scale"])
    assert np.array_equal(r["qw"], o["qw"]) and np.array_equal(r["qx"], o["qx"])
    assert np.array_equal(r["y"].numpy(), o["y"])
    xl, wl = torch.randn(20, 100, generator=g), torch.randn(125, 100, generator=g) * 0.1
    bl = torch.randn(125, generator=g)
    qs = torch.cat([torch.tensor([qmax / xl.abs().max().item(), 0.0]), qmax / wl.abs().max(1)[0]]).float()
    rl = ref_order.linear_per_channel(xl, wl, bl, qs, mode)
    ol = oops.linear(xl.numpy(), wl.numpy(), bl.numpy(), qs.numpy(), mode)
    assert np.array_equal(rl["qw"], ol["qw"]) and np.array_equal(rl["y"].numpy(), ol["y"])


def test_half_order_of_the_reference_what_it_changes():
    """A .half() model rounds to half after every tensor op.  Measured against the single-rounding fp32
    evaluation of the same half inputs: with the q-params kept in fp32 the integers are the same and the
    output moves by a few 1e-4 of its range; with the q-params in half as well, the weight quotient's
    rounding to half moves some weights by one step, which is quantization noise (1e-3 of the range)."""
    from oracle import ref_order
    g = torch.Generator().manual_seed(7)
    x = torch.randn(3, 64, 24, 24, generator=g)
    w = torch.randn(64, 64, 3, 3, generator=g) * 0.04
    b = torch.randn(64, generator=g)
    q_scale = torch.cat([torch.tensor([127.0 / x.abs().max().item(), 0.0]), 127.0 / w.reshape(64, -1).abs().max(1)[0]]).float()
    args = ((3, 3), (3, 3), (1, 1), 1)
    single = oops.conv2d(x.half().numpy(), w.half().numpy(), b.half().numpy(), *args, q_scale.numpy(), [3])
    span = float(single["y"].astype(np.float32).max() - single["y"].astype(np.float32).min())
    mixed = ref_order.conv2d_per_channel(x.half(), w.half(), b.half(), *args, q_scale, [3])
    assert mixed["y"].dtype == torch.float32            # half / float promotes (output / new_scale, :127)
    assert np.array_equal(mixed["qw"], single["qw"])
    assert np.abs(mixed["y"].numpy() - single["y"].astype(np.float32)).max() <= 1e-3 * span
    allhalf = ref_order.conv2d_per_channel(x.half(), w.half(), b.half(), *args, q_scale.half(), [3])
    assert allhalf["y"].dtype == torch.float16 and torch.isfinite(allhalf["y"]).all()
    moved = (allhalf["qw"] != single["qw"]).mean()
    assert 0.005 < moved < 0.10
    assert np.abs(allhalf["qw"].astype(np.int32) - single["qw"]).max() == 1
    assert _rel_rms(F.conv2d(x, w, b, 3, 3).numpy().astype(np.float64), allhalf["y"].float().numpy().astype(np.float64)) <= 0.02
    # int16: 32767 / absmax exceeds the largest half for absmax < 0.5 -> inf in the half q_scale
    assert torch.isinf((32767.0 / w.reshape(64, -1).abs().max(1)[0]).half()).all()
