"""GPU parity: every HIP kernel, called through the C ABI, against the CPU oracle on the same
seeded inputs.  Bit-exact for integer outputs; floating outputs are compared bit-exactly too
where the oracle fixes the operation order, and within 1e-3 of the output range otherwise."""
import sys

import numpy as np
import pytest
import torch

import oracle as orc
from oracle import ops as oops

pytestmark = pytest.mark.gpu

if torch.cuda.is_available():
    import cabi


def note(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def rng(seed):
    return np.random.default_rng(seed)


def same_bits(a, b):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    assert a.shape == b.shape and a.dtype == b.dtype
    return np.array_equal(a.view(np.uint8), b.view(np.uint8))


def assert_float_close(got, want, what=""):
    """max-abs <= 1e-3 * output range (the tolerance the target states for fp outputs)"""
    got, want = got.astype(np.float64), want.astype(np.float64)
    span = max(want.max() - want.min(), 1e-30) if want.size else 1.0
    err = np.abs(got - want).max() if want.size else 0.0
    assert err <= 1e-3 * span, "%s: max-abs %g > 1e-3 * range %g" % (what, err, span)


# ------------------------------------------------------------------------------ quantize
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("bw", [8, 16, 31])
@pytest.mark.parametrize("n", [0, 1, 3, 4, 1023, 4096 * 37 + 5])
def test_quantize_flat(dtype, bw, n):
    note("quantize_flat", dtype.__name__, bw, n)
    r = rng(n + bw)
    pos = -5 if bw == 8 else -11 if bw == 16 else -20
    x = (r.standard_normal(n) * 3).astype(dtype)
    if n > 600:
        k = np.arange(-300, 300)
        x[:600] = ((k + 0.5) * 2.0 ** pos).astype(dtype)  # exact ties
        x[600:606] = [np.inf, -np.inf, np.nan, 1e4, -1e4, 0.0]
    want = orc.quantize(x, bw, pos)
    got = cabi.quantize(cabi.dev(x), bw, pos).cpu().numpy()
    assert same_bits(want, got)


def test_quantize_fp16_exhaustive_and_scale():
    h = np.arange(65536, dtype=np.uint16).view(np.float16)
    for bw, pos, scale in ((8, -4, 1.0), (16, -9, 1.0), (8, 2, 1.0), (16, -3, 1.3721)):
        note("quantize_fp16_exhaustive", bw, pos, scale)
        want = orc.quantize(h, bw, pos, scale)
        got = cabi.quantize(cabi.dev(h), bw, pos, scale).cpu().numpy()
        assert same_bits(want, got)
    x = (rng(5).standard_normal(100003) * 2).astype(np.float32)
    assert same_bits(orc.quantize(x, 8, -6, 1.61803), cabi.quantize(cabi.dev(x), 8, -6, 1.61803).cpu().numpy())


def test_quantize_unaligned_and_devpos():
    x = (rng(6).standard_normal(50001) * 4).astype(np.float32)
    xd = cabi.dev(x)
    note("quantize unaligned")
    got = cabi.quantize(xd[1:], 8, -4).cpu().numpy()  # 4-byte aligned only -> scalar kernel
    assert same_bits(orc.quantize(x[1:], 8, -4), got)
    note("quantize devpos")
    pos = torch.tensor([-4], dtype=torch.int32, device="cuda")
    assert same_bits(orc.quantize(x, 16, -4), cabi.quantize_devpos(xd, 16, pos).cpu().numpy())
    sc = torch.tensor([1.25], dtype=torch.float32, device="cuda")
    assert same_bits(orc.quantize(x, 8, -4, 1.25), cabi.quantize_devpos(xd, 8, pos, sc).cpu().numpy())


@pytest.mark.parametrize("shape,cpad", [((2, 3, 17, 19), 4), ((1, 3, 224, 224), 4), ((2, 1, 9, 9), 4),
                                         ((2, 5, 7, 9), 8), ((2, 70, 5, 6), 70), ((1, 3, 8, 8), 3),
                                         ((1, 130, 9, 9), 144)])
@pytest.mark.parametrize("bw", [8, 16])
def test_quantize_nchw_to_nhwc(shape, cpad, bw):
    note("quantize_nchw_to_nhwc", shape, cpad, bw)
    x = rng(sum(shape)).standard_normal(shape).astype(np.float32)
    want = orc.quantize_nchw_to_nhwc(x, bw, -5, 1.0, cpad)
    got = cabi.quantize_nchw_to_nhwc(cabi.dev(x), bw, -5, 1.0, cpad).cpu().numpy()
    assert same_bits(want, got)
    if bw == 8:
        goth = cabi.quantize_nchw_to_nhwc(cabi.dev(x.astype(np.float16)), bw, -5, 1.0, cpad).cpu().numpy()
        assert same_bits(orc.quantize_nchw_to_nhwc(x.astype(np.float16).astype(np.float32), bw, -5, 1.0, cpad), goth)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("n", [1, 7, 100000, 4096 * 300 + 3, 4096 * 256 * 4 * 5 + 1029])
def test_quantize_param(dtype, n):
    note("quantize_param", dtype.__name__, n)
    x = (rng(n).standard_normal(n) * 2.5).astype(dtype)
    if n > 10:
        x[n // 2] = np.nan  # ignored by the reduction
    for bw in (8, 16):
        absmax, pos, scale, off = cabi.quantize_param(cabi.dev(x), bw)
        am = orc.absmax(x)
        p, s, o = orc.quantize_param(am, bw)
        assert absmax.item() == am and pos.item() == p and np.float32(scale.item()) == s and off.item() == 0.0
        assert am == np.nanmax(np.abs(x.astype(np.float32)))
    z = torch.zeros(100, device="cuda")
    absmax, pos, scale, _ = cabi.quantize_param(z, 8)
    assert (absmax.item(), pos.item(), scale.item()) == (0.0, 0, 1.0)
    if dtype is np.float32 and n == 7:
        # magnitudes at both ends of fp32 (denormals included) and exact powers of two
        for mag in (1.4e-45, 1e-40, 2.0 ** -126, 2.0 ** -20, 1.0, 2.0 ** 20, 3.0e38, np.inf):
            t = np.array([0.0, -mag, mag / 2], np.float32)
            for bw in (8, 16):
                absmax, pos, scale, _ = cabi.quantize_param(cabi.dev(t), bw)
                p, s, _ = orc.quantize_param(orc.absmax(t), bw)
                assert (pos.item(), np.float32(scale.item())) == (p, s), (mag, bw)


@pytest.mark.parametrize("bw", [8, 16])
@pytest.mark.parametrize("shape", [(64, 64, 3, 3), (7, 5), (130, 33, 1, 1)])
def test_quantize_per_channel(bw, shape):
    note("quantize_per_channel", bw, shape)
    r = rng(bw + len(shape))
    w = (r.standard_normal(shape) * 0.05 * r.uniform(0.2, 3, (shape[0],) + (1,) * (len(shape) - 1))).astype(np.float32)
    qmax = 127.0 if bw == 8 else 32767.0
    s = (qmax / np.abs(w).reshape(shape[0], -1).max(1)).astype(np.float32)
    new_pos, new_scale, sf = orc.per_channel_params(bw, s)
    got = cabi.quantize_per_channel(cabi.dev(w), bw, cabi.dev(sf)).cpu().numpy()
    assert same_bits(orc.quantize_per_channel(w, bw, sf), got)


def test_dequantize():
    r = rng(9)
    for bits, dtype in ((8, np.int8), (16, np.int16), (32, np.int32)):
        note("dequantize", bits)
        q = r.integers(-2 ** (bits - 2), 2 ** (bits - 2), 10007).astype(dtype)
        assert same_bits(orc.dequantize(q, -7), cabi.dequantize(cabi.dev(q), -7).cpu().numpy())
        assert same_bits(orc.dequantize(q, -7, 1.7), cabi.dequantize(cabi.dev(q), -7, 1.7).cpu().numpy())
        h = cabi.dequantize(cabi.dev(q), -7, 1.7, half=True).cpu().numpy()
        assert same_bits(orc.dequantize(q, -7, 1.7).astype(np.float16), h)


@pytest.mark.parametrize("bits,dtype", [(8, np.int8), (16, np.int16), (32, np.int32)])
def test_dequantize_vector_paths(bits, dtype):
    """sizes that run the unrolled vector body several times over plus a ragged tail; every integer of the narrow
    types; scales that take the reciprocal form of the division (ordinary), the true division (all-ones significand,
    extreme exponents) and none (1.0); an unaligned view (scalar body)"""
    note("dequantize vector", bits)
    r = rng(90 + bits)
    lim = 2 ** (bits - 1)
    n = 4096 * 256 * 3 + 11
    q = r.integers(-lim, lim, n).astype(dtype)
    if bits <= 16:
        q[:2 * lim] = np.arange(-lim, lim).astype(dtype)
    qd = cabi.dev(q)
    ones = np.frombuffer(np.uint32(0x3fffffff).tobytes(), np.float32)[0]  # 1.9999999: significand all ones
    for pos, scale in ((-7, 1.0), (3, 1.7), (-20, 0.37), (0, float(ones)), (-7, 3.0e-12), (5, 2.5e11), (-60, 1.25)):
        want = orc.dequantize(q, pos, scale)
        assert same_bits(want, cabi.dequantize(qd, pos, scale).cpu().numpy()), (pos, scale)
        got_h = cabi.dequantize(qd, pos, scale, half=True).cpu().numpy()
        with np.errstate(over="ignore"):
            assert same_bits(want.astype(np.float16), got_h), (pos, scale, "half")
    # views off 16-byte alignment take the scalar body
    assert same_bits(orc.dequantize(q[1:70001], -3, 1.7), cabi.dequantize(qd[1:70001], -3, 1.7).cpu().numpy())


# ------------------------------------------------------------------------------ GEMM
def _ints(r, shape, bits):
    lim = 2 ** (bits - 1)
    return r.integers(-lim, lim, shape).astype(np.int8 if bits == 8 else np.int16)


GEMM_SHAPES = [(1, 1, 16), (5, 7, 16), (128, 128, 64), (130, 70, 80), (257, 129, 1040), (64, 1000, 2048),
               # a handful of blocks, long K: 128-byte steps through a four-stage ring (K ending inside a step, ragged tiles)
               (100, 200, 1072), (33, 500, 4096), (7, 65, 1936),
               (300, 64, 48), (1, 10, 10), (20, 125, 100), (33, 17, 7),
               # many rows, short K, narrow N: the streaming kernel, one shape per (K steps, N fragments) class
               (5000, 96, 16), (4100, 16, 32), (8200, 144, 32), (4099, 24, 96), (6000, 64, 64), (4097, 160, 32),
               (4500, 100, 48), (9000, 128, 16), (4096, 36, 80), (5555, 64, 96)]


@pytest.mark.parametrize("m,n,k", GEMM_SHAPES)
def test_gemm_i8_acc_and_epilogue(m, n, k):
    note("gemm_i8", m, n, k, cabi.lib().catchq_gemm_route(8, 8, m, n, k))
    r = rng(m * 7 + n * 3 + k)
    a, b = _ints(r, (m, k), 8), _ints(r, (n, k), 8)
    div = r.uniform(0.6, 3.5, n).astype(np.float32)
    bias = r.standard_normal(n).astype(np.float32)
    acc, ovf = orc.gemm_nt(a, b)
    assert ovf == 0
    ad, bd = cabi.dev(a), cabi.dev(b)
    out = cabi.gemm_nt(ad, bd, exp2=-9, chan_div=cabi.dev(div), bias=cabi.dev(bias), act=1)
    assert same_bits(acc.astype(np.int32), out["acc"].cpu().numpy())
    assert same_bits(orc.epilogue(acc, -9, div, bias, None, 1), out["y"].cpu().numpy())
    # the same through the reciprocal form of the division
    out = cabi.gemm_nt(ad, bd, exp2=-9, chan_div=cabi.dev(div), bias=cabi.dev(bias), act=1,
                       chan_rcp=cabi.dev(np.float32(1) / div))
    assert same_bits(orc.epilogue(acc, -9, div, bias, None, 1), out["y"].cpu().numpy())
    out = cabi.gemm_nt(ad, bd, exp2=-9, bias=cabi.dev(bias), act=0, y_dtype=torch.float16, want_acc=False,
                       q_bw=8, q_pos=-2)
    y = orc.epilogue(acc, -9, None, bias, None, 0)
    assert same_bits(y.astype(np.float16), out["y"].cpu().numpy())
    assert same_bits(orc.quantize(y, 8, -2), out["q"].cpu().numpy())


@pytest.mark.parametrize("seed", range(8))
def test_gemm_random_sweep(seed):
    """15 random products per seed over all three operand widths, ragged in every dimension (rows up to 7000 so that
    the streaming kernel is drawn, K from 1), each with a random epilogue: bit-exact against the oracle."""
    r = rng(2000 + seed)
    for i in range(15):
        bits = [(8, 8), (8, 8), (16, 8), (16, 16)][int(r.integers(0, 4))]
        m = int(r.choice([r.integers(1, 70), r.integers(70, 700), r.integers(4000, 7000)]))
        n = int(r.choice([r.integers(1, 40), r.integers(40, 400), 16 * r.integers(1, 11)]))
        k = int(r.choice([r.integers(1, 100), r.integers(100, 900), 16 * r.integers(1, 7)]))
        a, b = _ints(r, (m, k), bits[0]), _ints(r, (n, k), bits[1])
        use_div, use_rcp, use_bias = r.random() < 0.6, r.random() < 0.7, r.random() < 0.7
        act = int(r.integers(0, 3))
        y_dtype = [None, torch.float32, torch.float32, torch.float16][int(r.integers(0, 4))]
        q_bw = int(r.choice([0, 8, 8, 16]))
        want_acc = bits != (16, 16) and r.random() < 0.3
        if y_dtype is None and not q_bw and not want_acc:
            y_dtype = torch.float32
        q_scale = 1.0 if r.random() < 0.5 else float(np.float32(r.uniform(1.0, 2.0)))
        exp2 = {(8, 8): -10, (16, 8): -18, (16, 16): -26}[bits] + int(r.integers(-2, 3))
        q_pos = int(r.integers(-5, 0)) if q_bw == 8 else int(r.integers(-12, -6))
        case = dict(seed=seed, i=i, mnk=(m, n, k), bits=bits, route=cabi.lib().catchq_gemm_route(bits[0], bits[1], m, n, k),
                    div=use_div, rcp=use_rcp, bias=use_bias, act=act, y=y_dtype, q_bw=q_bw, q_scale=q_scale, q_pos=q_pos,
                    exp2=exp2, acc=want_acc)
        note("gemm sweep", case)
        acc, ovf = orc.gemm_nt(a, b)
        div = r.uniform(0.6, 3.5, n).astype(np.float32) if use_div else None
        bias = r.standard_normal(n).astype(np.float32) if use_bias else None
        out = cabi.gemm_nt(cabi.dev(a), cabi.dev(b), exp2=exp2, chan_div=cabi.dev(div) if use_div else None,
                           bias=cabi.dev(bias) if use_bias else None, act=act, y_dtype=y_dtype, want_acc=want_acc,
                           q_bw=q_bw, q_pos=q_pos, q_scale=q_scale,
                           chan_rcp=cabi.dev(np.float32(1) / div) if use_div and use_rcp else None)
        torch.cuda.synchronize()
        y = orc.epilogue(acc, exp2, div, bias, None, act)
        if want_acc:
            assert ovf == 0 and same_bits(acc.astype(np.int32), out["acc"].cpu().numpy()), case
        if y_dtype is not None:
            want = y.astype(np.float16) if y_dtype == torch.float16 else y
            assert same_bits(want, out["y"].cpu().numpy()), case
        if q_bw:
            assert same_bits(orc.quantize(y, q_bw, q_pos, q_scale), out["q"].cpu().numpy()), case


def test_division_by_reciprocal_is_exact():
    """v/d evaluated as q=v*r, e=fma(-q,d,v), fma(e,r,q) with r = RN(1/d) must equal IEEE division bit
    for bit: adversarial divisor significands x a wide set of dividends x several exponents."""
    r = rng(77)
    n = 256
    mant = np.concatenate([[0, 1, 2, 3, 0x7ffffe, 0x7ffffd, 0x400000, 0x400001, 0x3fffff, 0x2aaaaa, 0x555555, 0x6db6db,
                            0x7ff000, 0x000fff], r.integers(0, 0x7fffff, n - 14)]).astype(np.uint32)
    expo = r.integers(125, 130, n).astype(np.uint32)  # divisors in [0.25, 8)
    div = ((expo << 23) | mant).view(np.float32)
    rcp = (np.float32(1) / div).astype(np.float32)
    for k, m in ((16, 4096), (64, 2048), (1024, 512)):
        a, b = _ints(r, (m, k), 8), _ints(r, (n, k), 8)
        if k == 16:
            a[:, 4:] = 0  # small sums: every short bit pattern shows up
        acc, _ = orc.gemm_nt(a, b)
        for exp2 in (-13, 0, 7, -64, 64):
            note("div by rcp", k, m, exp2)
            out = cabi.gemm_nt(cabi.dev(a), cabi.dev(b), exp2=exp2, chan_div=cabi.dev(div), chan_rcp=cabi.dev(rcp),
                               want_acc=False)
            assert same_bits(orc.epilogue(acc, exp2, div), out["y"].cpu().numpy())
    # outside the exponent window the kernels divide even when reciprocals are supplied
    out = cabi.gemm_nt(cabi.dev(a), cabi.dev(b), exp2=-90, chan_div=cabi.dev(div), chan_rcp=cabi.dev(rcp * 0))
    assert same_bits(orc.epilogue(acc, -90, div), out["y"].cpu().numpy())


@pytest.mark.parametrize("bits", [(16, 8), (16, 16)])
@pytest.mark.parametrize("m,n,k", [(20, 125, 100), (64, 64, 128), (3, 5, 600), (200, 96, 72), (130, 260, 520),
                                   (1, 4, 8), (77, 64, 1024)])
def test_gemm_wide(bits, m, n, k):
    note("gemm_wide", bits, m, n, k, cabi.lib().catchq_gemm_route(bits[0], bits[1], m, n, k))
    r = rng(k + bits[1])
    a, b = _ints(r, (m, k), bits[0]), _ints(r, (n, k), bits[1])
    bias = r.standard_normal(n).astype(np.float32)
    acc, ovf = orc.gemm_nt(a, b)
    out = cabi.gemm_nt(cabi.dev(a), cabi.dev(b), exp2=-20, bias=cabi.dev(bias), want_acc=(bits == (16, 8)))
    if bits == (16, 8):
        assert ovf == 0
        assert same_bits(acc.astype(np.int32), out["acc"].cpu().numpy())
    assert same_bits(orc.epilogue(acc, -20, None, bias), out["y"].cpu().numpy())


@pytest.mark.parametrize("m,n,k", [(64, 64, 64), (200, 130, 72), (1, 1, 8), (96, 75, 1024), (3 * 10 * 10, 64, 576), (500, 300, 8200)])
def test_gemm_a16w16_extreme_digits(m, n, k):
    """int16 x int16 on the matrix cores (four int8 digit products, digit sums of rows and columns, 64-bit
    combination): every digit pattern that could break the split -- -32768, 32767, -1, 0, +-128, 255, 256, all
    low bytes 0x80, all high bytes 0x80 -- on both operands, the exact int64 sums through a power-of-two
    epilogue that loses nothing (|sum| < 2^24 is not required: the comparison is with the oracle's float of the
    same integer), and K not a multiple of the 64-element step."""
    assert cabi.lib().catchq_gemm_route(16, 16, m, n, k) == b"mfma_a16w16"
    note("gemm_a16w16", m, n, k)
    r = rng(m * 7 + n + k)
    a, b = _ints(r, (m, k), 16), _ints(r, (n, k), 16)
    ext = np.array([-32768, 32767, -1, 0, 128, -128, 255, 256, -129, 127, -32641, 32640], np.int16)
    a[0, :min(k, 12)] = ext[:min(k, 12)]
    b[0, :min(k, 12)] = ext[::-1][:min(k, 12)]
    if m > 2 and n > 2:
        a[1] = -32768; b[1] = -32768          # the largest product everywhere: 2^30 * K
        a[2] = 32767; b[2] = -32768
        a[m - 1] = 0x0080 - 0 if k else 0     # low byte 0x80, high byte 0
        b[n - 1] = -128                        # 0xff80
    acc, _ = orc.gemm_nt(a, b)
    assert acc.dtype == np.int64 and (m < 3 or n < 3 or acc[1, 1] == k * 2 ** 30)
    bias = r.standard_normal(n).astype(np.float32)
    out = cabi.gemm_nt(cabi.dev(a), cabi.dev(b), exp2=-30, bias=cabi.dev(bias), want_acc=False)
    assert same_bits(orc.epilogue(acc, -30, None, bias), out["y"].cpu().numpy())
    # small values: the sums stay below 2^24, the fp32 output with exp2 = 0 and no bias is the integer itself
    a2, b2 = (a // 4096).astype(np.int16), (b // 4096).astype(np.int16)
    acc2, _ = orc.gemm_nt(a2, b2)
    if np.abs(acc2).max() < 2 ** 24:
        y2 = cabi.gemm_nt(cabi.dev(a2), cabi.dev(b2), want_acc=False)["y"].cpu().numpy()
        assert np.array_equal(y2.astype(np.int64), acc2)


@pytest.mark.parametrize("m,n,k", [(16384, 1024, 1024), (8192, 768, 320), (4096, 768, 256), (4096, 3072, 768)])
def test_gemm_a16_tiles(m, n, k):
    """int16 x int8 on the matrix cores (the first shape takes the wide 128x256 tile), with the extreme digits
    (-32768, 32767, -1, 0, 255, 256) planted; sampled rows against the oracle, all rows by linearity."""
    note("gemm_a16", m, n, k, cabi.lib().catchq_gemm_route(16, 8, m, n, k))
    r = rng(m + k)
    a, b = (_ints(r, (m, k), 16) // 8).astype(np.int16), _ints(r, (n, k), 8)
    a[5, :6] = (-32768, 32767, -1, 0, 255, 256)
    a[m - 1, -6:] = (32767, -32768, 128, -128, 127, -129)
    out = cabi.gemm_nt(cabi.dev(a), cabi.dev(b), y_dtype=None)
    acc = out["acc"].cpu().numpy()
    rows = np.concatenate([r.integers(0, m, 96), [0, 5, m - 1]])
    want, ovf = orc.gemm_nt(a[rows], b)
    assert ovf == 0 and np.array_equal(want.astype(np.int32), acc[rows])
    # (a_hi*256 + a_lo) B^T = 256 * a_hi B^T + a_lo B^T, both halves through the int8 kernel
    a_hi, a_lo = (a >> 8).astype(np.int8), ((a & 255) - 128).astype(np.int8)
    hi = cabi.gemm_nt(cabi.dev(a_hi), cabi.dev(b), y_dtype=None)["acc"]
    lo = cabi.gemm_nt(cabi.dev(a_lo), cabi.dev(b), y_dtype=None)["acc"]
    bsum = torch.from_numpy(b.astype(np.int32).sum(1)).cuda()
    assert torch.equal(hi * 256 + lo + 128 * bsum[None, :], out["acc"])


@pytest.mark.parametrize("m,n,k", [(4997, 2100, 512), (2500, 1100, 1024), (9001, 600, 256), (6000, 4100, 128)])
def test_gemm_banded_tile_order(m, n, k):
    """grids that are large in both directions walk their tiles in bands of eight row tiles; ragged last band,
    ragged last row and column tiles: rows sampled from every band against the oracle, and every row of C
    against the sum over K halves (two launches whose grids walk the same way)"""
    note("gemm_banded", m, n, k)
    r = rng(m + n + k)
    a, b = _ints(r, (m, k), 8), _ints(r, (n, k), 8)
    acc = cabi.gemm_nt(cabi.dev(a), cabi.dev(b), y_dtype=None)["acc"]
    rows = np.unique(np.concatenate([np.arange(0, m, 97), [m - 1, m - 2, 63, 64, 255, 256, 2047, 2048]]))
    rows = rows[rows < m]
    want, ovf = orc.gemm_nt(a[rows], b)
    assert ovf == 0 and np.array_equal(want.astype(np.int32), acc.cpu().numpy()[rows])
    h = k // 2
    s = cabi.gemm_nt(cabi.dev(a[:, :h]), cabi.dev(b[:, :h]), y_dtype=None)["acc"] + \
        cabi.gemm_nt(cabi.dev(a[:, h:]), cabi.dev(b[:, h:]), y_dtype=None)["acc"]
    assert torch.equal(s, acc)


def test_gemm_full_size_properties():
    """Config-2 sizes: too big for the oracle in seconds, so check what the integers must satisfy:
    rows of A that are copies give equal rows of C, and a sampled set of entries equals the
    oracle's dot products."""
    for (m, n, k) in ((4096, 3072, 768), (4096, 768, 3072)):
        note("gemm_full", m, n, k)
        r = rng(k)
        a, b = _ints(r, (m, k), 8), _ints(r, (n, k), 8)
        a[1234] = a[17]
        out = cabi.gemm_nt(cabi.dev(a), cabi.dev(b), y_dtype=None)
        acc = out["acc"].cpu().numpy()
        assert np.array_equal(acc[1234], acc[17])
        rows = r.integers(0, m, 64)
        want, _ = orc.gemm_nt(a[rows], b)
        assert np.array_equal(want.astype(np.int32), acc[rows])
        # linearity in A: (a1 + a2) B^T = a1 B^T + a2 B^T with halves that cannot overflow int8
        a1, a2 = (a // 2).astype(np.int8), (a - a // 2).astype(np.int8)
        s = cabi.gemm_nt(cabi.dev(a1), cabi.dev(b), y_dtype=None)["acc"] + \
            cabi.gemm_nt(cabi.dev(a2), cabi.dev(b), y_dtype=None)["acc"]
        assert torch.equal(s, out["acc"])


# ------------------------------------------------------------------------------ conv
CONV_CASES = [
    # N, Ci, H, W, Co, kh, kw, pad, stride, dil, groups
    (3, 64, 24, 24, 64, 3, 3, (3, 3), (3, 3), (1, 1), 1),      # reference qint grid
    (2, 4, 6, 6, 16, 3, 3, (0, 0), (1, 1), (1, 1), 2),         # reference groups case
    (1, 3, 14, 14, 8, 2, 2, (0, 0), (1, 1), (1, 1), 1),
    (2, 6, 9, 11, 10, 3, 2, (1, 2), (2, 1), (2, 1), 2),
    (2, 16, 9, 11, 24, 3, 3, (1, 1), (1, 1), (1, 1), 1),       # MFMA, K=144 (tail step)
    (2, 64, 14, 14, 128, 1, 1, (0, 0), (1, 1), (1, 1), 1),     # 1x1
    (2, 64, 15, 15, 160, 1, 1, (0, 0), (2, 2), (1, 1), 1),     # 1x1 stride 2 (downsample)
    (2, 32, 13, 13, 64, 3, 3, (1, 1), (2, 2), (1, 1), 1),      # 3x3 stride 2
    (1, 48, 10, 12, 40, 3, 3, (2, 2), (1, 1), (2, 2), 1),      # dilation
    (1, 128, 7, 7, 256, 3, 3, (1, 1), (1, 1), (1, 1), 1),
    (2, 128, 9, 9, 96, 3, 3, (1, 1), (2, 2), (1, 1), 1),       # few blocks, K = 1152: the wide ring with the im2col loader
    (1, 16, 5, 5, 32, 5, 5, (2, 2), (1, 1), (1, 1), 1),
    (1, 80, 8, 8, 16, 7, 1, (3, 0), (1, 1), (1, 1), 1),        # asymmetric kernel
    (2, 4, 30, 30, 64, 7, 7, (3, 3), (2, 2), (1, 1), 1),       # 4-channel input, 7x7 s2 (network stem)
    (1, 4, 9, 13, 24, 3, 3, (1, 1), (1, 1), (1, 1), 1),        # 4-channel input, 3x3
    (2, 4, 11, 10, 40, 5, 2, (2, 0), (1, 1), (2, 1), 1),       # 4-channel input, 5x2, vertical dilation
    (1, 4, 6, 6, 8, 1, 1, (0, 0), (1, 1), (1, 1), 1),          # 4-channel input, 1x1
    (2, 4, 36, 37, 64, 7, 8, (0, 0), (2, 2), (1, 1), 1),       # 4-channel framed input, rows of 8 taps (stem form)
    (1, 4, 12, 20, 24, 3, 4, (1, 0), (1, 1), (1, 1), 1),       # 4-channel, rows of 4 taps, vertical padding only
    (2, 4, 9, 33, 40, 5, 12, (2, 0), (1, 3), (2, 1), 1),       # 4-channel, rows of 12 taps, stride 3, vertical dilation
    (2, 4, 100, 101, 64, 7, 8, (0, 0), (2, 2), (1, 1), 1),     # framed stem, 4512 pixels: streaming stem kernel, 7 steps
    (3, 4, 90, 91, 32, 3, 4, (0, 0), (2, 2), (1, 1), 1),       # framed 3x3 stem (rows of 4 taps, two rows per K step)
    (1, 4, 70, 72, 40, 4, 4, (0, 0), (1, 1), (2, 1), 1),       # even filter height, stride 1, vertical dilation, Co = 40
    (1, 64, 9, 9, 72, 1, 1, (0, 0), (1, 1), (1, 1), 1),        # Co % 64 != 0
    (1, 32, 5, 5, 30, 3, 3, (1, 1), (1, 1), (1, 1), 1),        # Co % 4 != 0 -> scalar epilogue
    (2, 32, 12, 12, 32, 3, 3, (1, 1), (1, 1), (1, 1), 32),     # depthwise s1
    (2, 96, 15, 15, 96, 3, 3, (1, 1), (2, 2), (1, 1), 96),     # depthwise s2
    (1, 8, 10, 10, 8, 3, 3, (1, 1), (2, 2), (1, 1), 8),        # depthwise, few channels
    (1, 36, 40, 40, 36, 5, 5, (2, 2), (1, 1), (1, 1), 36),     # depthwise 5x5, several strips
    (1, 6, 7, 7, 6, 3, 3, (1, 1), (1, 1), (1, 1), 6),          # depthwise C%4 != 0 -> direct
    (1, 16, 9, 7, 16, 3, 3, (0, 0), (1, 1), (1, 1), 16),       # depthwise, no padding, ragged 2x4 windows
    (2, 24, 11, 13, 24, 3, 3, (1, 1), (2, 2), (1, 1), 24),     # depthwise s2, odd extents
    (1, 320, 7, 7, 320, 3, 3, (1, 1), (1, 1), (1, 1), 320),    # depthwise, many channels, tiny image
    (1, 16, 9, 9, 16, 3, 3, (2, 2), (1, 1), (2, 2), 16),       # depthwise dilated -> strip kernel
    (2, 32, 50, 50, 16, 1, 1, (0, 0), (1, 1), (1, 1), 1),      # pointwise, 5000 pixels: streaming kernel
    (1, 16, 70, 71, 96, 1, 1, (0, 0), (1, 1), (1, 1), 1),      # pointwise expand, K = 16
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_i8_acc_and_epilogue(case):
    n, ci, h, w, co, kh, kw, pad, stride, dil, g = case
    route = cabi.conv_route(8, 8, (n, h, w, ci), (co, kh, kw, ci // g), pad, stride, dil, g)
    note("conv_i8", case, route)
    r = rng(sum(case[:7]))
    x, wt = _ints(r, (n, h, w, ci), 8), _ints(r, (co, kh, kw, ci // g), 8)
    acc, ovf = orc.conv2d_nhwc(x, wt, pad, stride, dil, g)
    assert ovf == 0
    div = r.uniform(0.6, 3.5, co).astype(np.float32)
    bias = r.standard_normal(co).astype(np.float32)
    resid = r.standard_normal(acc.shape).astype(np.float32)
    xd, wd = cabi.dev(x), cabi.dev(wt)
    out = cabi.conv2d_nhwc(xd, wd, pad, stride, dil, g, exp2=-10, chan_div=cabi.dev(div), bias=cabi.dev(bias),
                           resid=cabi.dev(resid), act=1, q_bw=8, q_pos=-3, chan_rcp=cabi.dev(np.float32(1) / div))
    assert same_bits(acc.astype(np.int32), out["acc"].cpu().numpy())
    y = orc.epilogue(acc, -10, div, bias, resid, 1)
    assert same_bits(y, out["y"].cpu().numpy())
    assert same_bits(orc.quantize(y, 8, -3), out["q"].cpu().numpy())
    out = cabi.conv2d_nhwc(xd, wd, pad, stride, dil, g, exp2=-10, act=2, y_dtype=torch.float16, want_acc=False)
    assert same_bits(orc.epilogue(acc, -10, None, None, None, 2, np.float16), out["y"].cpu().numpy())


GROUPED_CASES = [
    # N, Ci, H, W, Co, k, pad, stride, dil, groups, route
    (2, 64, 14, 14, 64, 3, 1, 1, 1, 2, "mfma_grouped"),      # two groups of 32 -> 32
    (1, 64, 9, 11, 80, 3, 1, 2, 1, 4, "mfma_grouped"),       # 16 -> 20 channels per group, stride 2, ragged tiles
    (2, 256, 14, 14, 256, 3, 1, 1, 1, 8, "mfma_grouped"),    # a wide-group bottleneck: 32 -> 32 per group
    (1, 128, 20, 20, 64, 1, 0, 1, 1, 2, "mfma_grouped"),     # grouped pointwise
    (1, 96, 12, 12, 96, 3, 2, 1, 2, 3, "mfma_grouped"),      # dilation 2, three groups of 32
    (3, 512, 7, 7, 1024, 3, 1, 1, 1, 32, "mfma_grouped"),    # 32 groups of 16 -> 32 (cardinality 32)
    (1, 128, 8, 8, 128, 3, 1, 1, 1, 32, "direct"),           # 4 channels per group: not a whole K chunk
    (1, 64, 8, 8, 36, 3, 1, 1, 1, 2, "direct"),              # 18 outputs per group: not a multiple of 4
]


@pytest.mark.parametrize("case", GROUPED_CASES)
def test_conv_grouped(case):
    """grouped (not depthwise) int8 convolutions: groups whose channels fill whole 16-byte K chunks run as one
    implicit GEMM per group on the matrix cores, the rest on the direct kernel; int32 sums, the generic epilogue with
    every per-channel vector and a residual, and the ReLU -> int8 instance, all against the oracle"""
    n, ci, h, w, co, k, pad, stride, dil, g, route = case
    note("conv_grouped", case)
    assert cabi.conv_route(8, 8, (n, h, w, ci), (co, k, k, ci // g), (pad, pad), (stride, stride), (dil, dil), g) == route
    r = rng(sum(case[:10]))
    x, wt = _ints(r, (n, h, w, ci), 8), _ints(r, (co, k, k, ci // g), 8)
    acc, ovf = orc.conv2d_nhwc(x, wt, (pad, pad), (stride, stride), (dil, dil), g)
    assert ovf == 0
    div = r.uniform(0.6, 3.5, co).astype(np.float32)
    bias = r.standard_normal(co).astype(np.float32)
    resid = r.standard_normal(acc.shape).astype(np.float32)
    xd, wd = cabi.dev(x), cabi.dev(wt)
    args = ((pad, pad), (stride, stride), (dil, dil), g)
    out = cabi.conv2d_nhwc(xd, wd, *args, exp2=-10, chan_div=cabi.dev(div), bias=cabi.dev(bias), resid=cabi.dev(resid), act=1,
                           q_bw=8, q_pos=-3, chan_rcp=cabi.dev(np.float32(1) / div))
    assert same_bits(acc.astype(np.int32), out["acc"].cpu().numpy())
    y = orc.epilogue(acc, -10, div, bias, resid, 1)
    assert same_bits(y, out["y"].cpu().numpy())
    assert same_bits(orc.quantize(y, 8, -3), out["q"].cpu().numpy())
    q = cabi.conv2d_nhwc(xd, wd, *args, exp2=-10, chan_div=cabi.dev(div), chan_rcp=cabi.dev(np.float32(1) / div),
                         bias=cabi.dev(bias), act=1, y_dtype=None, want_acc=False, q_bw=8, q_pos=-3)["q"]
    assert same_bits(orc.quantize(orc.epilogue(acc, -10, div, bias, None, 1), 8, -3), q.cpu().numpy())
    h16 = cabi.conv2d_nhwc(xd, wd, *args, exp2=-10, bias=cabi.dev(bias), act=2, y_dtype=torch.float16, want_acc=False)["y"]
    assert same_bits(orc.epilogue(acc, -10, None, bias, None, 2, np.float16), h16.cpu().numpy())


@pytest.mark.parametrize("case", [CONV_CASES[4], CONV_CASES[17], CONV_CASES[18], CONV_CASES[3]])
@pytest.mark.parametrize("after", [False, True])
def test_conv_leaky_relu_and_residual_order(case, after):
    """leaky ReLU (v > 0 ? v : v*slope) and the residual added before / after the activation, on the
    vector epilogue (matrix cores, depthwise) and the scalar one (direct kernel, Co % 4 != 0)."""
    n, ci, h, w, co, kh, kw, pad, stride, dil, g = case
    note("conv_leaky", case, after)
    r = rng(sum(case[:7]) + 99)
    x, wt = _ints(r, (n, h, w, ci), 8), _ints(r, (co, kh, kw, ci // g), 8)
    acc, _ = orc.conv2d_nhwc(x, wt, pad, stride, dil, g)
    bias = r.standard_normal(co).astype(np.float32)
    resid = r.standard_normal(acc.shape).astype(np.float32)
    for act in (3, 1):
        out = cabi.conv2d_nhwc(cabi.dev(x), cabi.dev(wt), pad, stride, dil, g, exp2=-11, bias=cabi.dev(bias),
                               resid=cabi.dev(resid), act=act, q_bw=16, q_pos=-9, want_acc=False, act_slope=0.1,
                               resid_after_act=after)
        y = orc.epilogue(acc, -11, None, bias, resid, act, act_slope=0.1, resid_after_act=after)
        assert same_bits(y, out["y"].cpu().numpy())
        assert same_bits(orc.quantize(y, 16, -9), out["q"].cpu().numpy())


@pytest.mark.parametrize("bits", [(16, 8), (16, 16)])
@pytest.mark.parametrize("case", [CONV_CASES[i] for i in (0, 1, 4, 5, 6, 7, 8, 9, 10, 11, 12, 16, 17)] + [
    (2, 8, 13, 13, 32, 3, 3, (1, 1), (1, 1), (1, 1), 1),        # 8 channels: K = 72, ragged last K step
    (1, 24, 9, 9, 255, 1, 1, (0, 0), (1, 1), (1, 1), 1),        # detection head: 255 outputs
    (2, 256, 12, 12, 320, 3, 3, (1, 1), (1, 1), (1, 1), 1),     # wider tile
    (2, 8, 70, 71, 32, 3, 4, (0, 0), (1, 1), (1, 1), 1),        # framed 8-channel first layer: streaming kernel
    (1, 8, 100, 101, 40, 3, 4, (0, 0), (2, 2), (2, 1), 1),      # the same, stride 2, vertical dilation, 40 channels
])
def test_conv_wide(bits, case):
    n, ci, h, w, co, kh, kw, pad, stride, dil, g = case
    note("conv_wide", bits, case, cabi.conv_route(bits[0], bits[1], (n, h, w, ci), (co, kh, kw, ci // g), pad, stride, dil, g))
    r = rng(sum(case[:7]) + bits[1])
    x, wt = _ints(r, (n, h, w, ci), bits[0]), _ints(r, (co, kh, kw, ci // g), bits[1])
    acc, ovf = orc.conv2d_nhwc(x, wt, pad, stride, dil, g)
    bias = r.standard_normal(co).astype(np.float32)
    out = cabi.conv2d_nhwc(cabi.dev(x), cabi.dev(wt), pad, stride, dil, g, exp2=-22, bias=cabi.dev(bias),
                           want_acc=(bits == (16, 8)))
    if bits == (16, 8):
        assert ovf == 0 and same_bits(acc.astype(np.int32), out["acc"].cpu().numpy())
    assert same_bits(orc.epilogue(acc, -22, None, bias), out["y"].cpu().numpy())


@pytest.mark.parametrize("n,h,w,ci,co,stride", [
    (2, 56, 56, 64, 64, 1),      # bands of 4 rows of one image, 7 sub-tiles
    (2, 28, 28, 128, 128, 1),    # bands of 7 rows
    (3, 14, 14, 256, 256, 1),    # one whole image per tile
    (5, 7, 7, 512, 512, 1),      # two whole images per tile, odd batch: the last tile is half empty
    (7, 7, 7, 64, 32, 1),        # five images per tile, one 32-channel block
    (1, 10, 12, 64, 100, 1),     # ragged channel block (100 = 3 * 32 + 4); room for two images, one present
    (2, 9, 31, 128, 68, 1),      # odd width: a row is not a multiple of 32 pixels; bands of 3 rows
    (1, 33, 17, 64, 64, 1),      # bands of 11 rows, 187 pixels
    (2, 4, 4, 256, 64, 1),       # tiny images: 15 per tile
    (1, 1, 1, 64, 64, 1),        # a single pixel
    (1, 60, 120, 64, 64, 1),     # a band is two rows of 120 pixels
    (1, 6, 254, 64, 32, 1),      # the widest row this route takes: one row per tile
    (1, 26, 26, 512, 64, 1),     # the patch of a deep layer limits the band: 7, 7, 7 and 5 rows
    (1, 52, 52, 256, 32, 1),     # 13 bands of 4 rows
    (2, 13, 40, 64, 32, 1),      # bands of 5, 5 and 3 rows
    (2, 56, 56, 128, 128, 2),    # stride 2: 28 x 28 outputs, bands of 7 rows over 15 input rows
    (3, 28, 28, 256, 256, 2),    # 14 x 14 outputs in two bands
    (3, 14, 14, 512, 512, 2),    # 7 x 7 outputs: one image per tile, two sub-tiles
    (2, 15, 13, 128, 36, 2),     # odd input sides: 8 x 7 outputs, the last input row and column are used
    (5, 6, 6, 256, 32, 2),       # 3 x 3 outputs, several images per tile
    (1, 30, 50, 128, 64, 2),     # 15 x 25 outputs: bands of 8 and 7 rows
])
def test_conv3x3_patch_resident(n, h, w, ci, co, stride):
    """3x3 / padding 1 layers (stride 1 or 2) whose input patch stays in LDS for all nine taps: int32 sums and the
    generic epilogue against the oracle, then the ReLU -> int8 instance the classifier layers use"""
    note("conv3x3 patch-resident", n, h, w, ci, co, stride)
    r = rng(n * 1000 + h * 10 + ci + co + stride)
    x, wt = _ints(r, (n, h, w, ci), 8), _ints(r, (co, 3, 3, ci), 8)
    x[0, 0, 0, :] = -128          # corners and edges carry the extremes: the padding must contribute nothing
    x[-1, -1, -1, :] = 127
    wt[0] = -128
    st = (stride, stride)
    acc, ovf = orc.conv2d_nhwc(x, wt, (1, 1), st, (1, 1), 1)
    assert ovf == 0
    bias = r.standard_normal(co).astype(np.float32)
    div = r.uniform(0.5, 2.0, co).astype(np.float32)
    out = cabi.conv2d_nhwc(cabi.dev(x), cabi.dev(wt), (1, 1), st, exp2=-14, chan_div=cabi.dev(div), bias=cabi.dev(bias))
    assert same_bits(acc.astype(np.int32), out["acc"].cpu().numpy())
    assert same_bits(orc.epilogue(acc, -14, div, bias), out["y"].cpu().numpy())
    rcp = (np.float32(1.0) / div).astype(np.float32)
    q = cabi.conv2d_nhwc(cabi.dev(x), cabi.dev(wt), (1, 1), st, exp2=-14, chan_div=cabi.dev(div), chan_rcp=cabi.dev(rcp),
                         bias=cabi.dev(bias), act=1, y_dtype=None, want_acc=False, q_bw=8, q_pos=-3)["q"]
    want = orc.quantize(orc.epilogue(acc, -14, div, bias, None, 1), 8, -3)
    assert same_bits(want, q.cpu().numpy())


@pytest.mark.parametrize("n,h,w,ci,co", [
    (2, 52, 52, 128, 256),    # Darknet-53's widest 3x3 family
    (1, 104, 104, 64, 128),
    (1, 60, 208, 32, 64),     # K = 288
    (2, 26, 26, 256, 512),
    (3, 13, 13, 128, 100),    # ragged channel block
    (5, 7, 7, 64, 32),        # odd batch of small images
    (2, 9, 31, 32, 68),       # odd width, Co % 32 != 0
    (1, 1, 1, 64, 64),        # a single pixel
    (1, 6, 254, 32, 32),      # long rows
])
def test_conv3x3_int16_detector_epilogues(n, h, w, ci, co):
    """3x3 / stride 1 / padding 1 layers of int16 activations x int8 weights at the detector's shapes: int32 sums
    and the generic epilogue against the oracle (extreme digits in both operands and at the image corners), then the
    detector's epilogue instances: leaky ReLU -> int16, with the residual behind the activation, with and without fp32"""
    note("conv3x3 int16", n, h, w, ci, co)
    r = rng(n * 1000 + h * 10 + ci + co)
    # values of a few thousand: the int32 sums of 9 * ci products stay exact
    x = (_ints(r, (n, h, w, ci), 16) // (16 if ci <= 64 else 32)).astype(np.int16)
    wt = _ints(r, (co, 3, 3, ci), 8)
    ext = np.array([-1, 0, 127, 128, 255, 256, -128, -129, -256, -257, 1023, -1024], np.int16)
    x[0, 0, 0, :ext.size] = ext          # every digit pattern at a corner: the padding must contribute nothing
    x[-1, -1, -1, :ext.size] = ext[::-1]
    wt[0, :, :, 0] = -128
    wt[-1, :, :, -1] = 127
    acc, ovf = orc.conv2d_nhwc(x, wt, (1, 1), (1, 1), (1, 1), 1)
    assert ovf == 0
    xd, wd = cabi.dev(x), cabi.dev(wt)
    assert cabi.conv_route(16, 8, (n, h, w, ci), (co, 3, 3, ci), (1, 1), (1, 1), (1, 1), 1) == "mfma_a16"
    bias = r.standard_normal(co).astype(np.float32)
    div = r.uniform(0.5, 2.0, co).astype(np.float32)
    out = cabi.conv2d_nhwc(xd, wd, (1, 1), (1, 1), exp2=-20, chan_div=cabi.dev(div), bias=cabi.dev(bias))
    assert same_bits(acc.astype(np.int32), out["acc"].cpu().numpy())
    assert same_bits(orc.epilogue(acc, -20, div, bias), out["y"].cpu().numpy())
    resid = r.standard_normal(acc.shape).astype(np.float32)
    for with_resid, want_y in ((False, False), (True, False), (True, True)):
        if co % 4:
            break  # the instances are vector epilogues
        o = cabi.conv2d_nhwc(xd, wd, (1, 1), (1, 1), exp2=-20, bias=cabi.dev(bias), resid=cabi.dev(resid) if with_resid else None,
                             act=3, y_dtype=torch.float32 if want_y else None, want_acc=False, q_bw=16, q_pos=-9,
                             act_slope=0.1, resid_after_act=True)
        y = orc.epilogue(acc, -20, None, bias, resid if with_resid else None, 3, act_slope=0.1, resid_after_act=True)
        assert same_bits(orc.quantize(y, 16, -9), o["q"].cpu().numpy()), (with_resid, want_y)
        if want_y:
            assert same_bits(y, o["y"].cpu().numpy())


@pytest.mark.parametrize("bits", [(8, 8), (16, 8), (16, 16)])
@pytest.mark.parametrize("case", [CONV_CASES[i] for i in (0, 1, 3, 4, 7, 12, 18)])
def test_quantize_conv2d_device_positions(bits, case):
    """float operands quantized on the fly with positions read from device memory
    (cnnlQuantizeConvolutionForward's contract): equal to quantize -> integer conv -> dequant + bias."""
    n, ci, h, w, co, kh, kw, pad, stride, dil, g = case
    note("quantize_conv2d", bits, case)
    r = rng(sum(case[:7]) + bits[0])
    x = (r.standard_normal((n, h, w, ci)) * 3).astype(np.float32)
    wt = (r.standard_normal((co, kh, kw, ci // g)) * 0.3).astype(np.float32)
    bias = r.standard_normal(co).astype(np.float32)
    pos_x, pos_w = (-4, -8) if bits[0] == 8 else (-11, -8 if bits[1] == 8 else -15)
    qx, qw = orc.quantize(x, bits[0], pos_x), orc.quantize(wt, bits[1], pos_w)
    acc, _ = orc.conv2d_nhwc(qx, qw, pad, stride, dil, g)
    want = orc.epilogue(acc, pos_x + pos_w, None, bias)
    px = torch.tensor([pos_x], dtype=torch.int32, device="cuda")
    pw = torch.tensor([pos_w], dtype=torch.int32, device="cuda")
    got = cabi.quantize_conv2d(cabi.dev(x), px, cabi.dev(wt), pw, bits[0], bits[1], pad, stride, dil, g, cabi.dev(bias))
    assert same_bits(want, got.cpu().numpy())
    # half tensors in, half out (one rounding at the end)
    xh, wh = x.astype(np.float16), wt.astype(np.float16)
    acc, _ = orc.conv2d_nhwc(orc.quantize(xh, bits[0], pos_x), orc.quantize(wh, bits[1], pos_w), pad, stride, dil, g)
    want = orc.epilogue(acc, pos_x + pos_w, None, bias, None, 0, np.float16)
    got = cabi.quantize_conv2d(cabi.dev(xh), px, cabi.dev(wh), pw, bits[0], bits[1], pad, stride, dil, g, cabi.dev(bias))
    assert same_bits(want, got.cpu().numpy())


# (per-channel divisor with reciprocals, residual: 0 none / 1 before / 2 after the activation, activation, fp output, q bits):
# one row per specialised epilogue instance of the kernels (these skip the run-time branches of the generic one)
EPILOGUE_ROWS = [
    (True, 0, 1, None, 8), (True, 1, 1, torch.float32, 8), (True, 0, 0, torch.float32, 0), (True, 1, 1, torch.float32, 0),
    (True, 0, 1, torch.float16, 0), (True, 0, 2, None, 8), (True, 1, 1, None, 8), (True, 0, 0, None, 8),
    (True, 0, 0, torch.float32, 8), (True, 1, 0, None, 8), (True, 1, 0, torch.float32, 8), (False, 0, 3, None, 16),
    (False, 0, 3, torch.float32, 16), (False, 2, 3, None, 16), (False, 2, 3, torch.float32, 16),
]
EPILOGUE_SHAPES = [
    # N, Ci, H, W, Co, k, pad, x bits
    (2, 128, 10, 10, 64, 1, 0, 8),     # LDS-ring kernel, 64x64 tiles
    (1, 64, 24, 24, 256, 1, 0, 8),     # 64x128 tiles when a residual is added
    (1, 32, 70, 70, 16, 1, 0, 8),      # streaming pointwise kernel
    (1, 32, 12, 12, 64, 3, 1, 16),     # int16 activations
    (1, 16, 20, 20, 16, 3, 1, 8),      # depthwise (groups = 16)
]


@pytest.mark.parametrize("q_scale", [1.0, 1.3720703125, 1.9999998807907104])
@pytest.mark.parametrize("shape", EPILOGUE_SHAPES)
def test_specialised_epilogues(shape, q_scale):
    """every epilogue instance the kernels are compiled with, with a unit requantization scale (the eager ops'
    power-of-two steps) and with fractional ones"""
    n, ci, h, w, co, k, pad, xbits = shape
    g = ci if (k == 3 and ci == co == 16) else 1
    note("specialised epilogues", shape, q_scale)
    r = rng(sum(shape))
    x, wt = _ints(r, (n, h, w, ci), xbits), _ints(r, (co, k, k, ci // g), 8)
    acc, ovf = orc.conv2d_nhwc(x, wt, (pad, pad), (1, 1), (1, 1), g)
    assert ovf == 0
    div = r.uniform(0.6, 3.5, co).astype(np.float32)
    bias = r.standard_normal(co).astype(np.float32)
    resid = r.standard_normal(acc.shape).astype(np.float32)
    xd, wd = cabi.dev(x), cabi.dev(wt)
    exp2 = -10 if xbits == 8 else -18
    for per_channel, res_mode, act, y_dtype, q_bw in EPILOGUE_ROWS:
        out = cabi.conv2d_nhwc(xd, wd, (pad, pad), (1, 1), (1, 1), g, exp2=exp2,
                               chan_div=cabi.dev(div) if per_channel else None, bias=cabi.dev(bias),
                               resid=cabi.dev(resid) if res_mode else None, act=act, y_dtype=y_dtype, want_acc=False,
                               q_bw=q_bw, q_pos=-3 if q_bw == 8 else -10, q_scale=q_scale,
                               chan_rcp=cabi.dev(np.float32(1) / div) if per_channel else None, act_slope=0.1,
                               resid_after_act=res_mode == 2)
        y = orc.epilogue(acc, exp2, div if per_channel else None, bias, resid if res_mode else None, act,
                         act_slope=0.1, resid_after_act=res_mode == 2)
        row = (per_channel, res_mode, act, y_dtype, q_bw)
        if y_dtype is not None:
            want = y.astype(np.float16) if y_dtype == torch.float16 else y
            assert same_bits(want, out["y"].cpu().numpy()), row
        if q_bw:
            assert same_bits(orc.quantize(y, q_bw, -3 if q_bw == 8 else -10, q_scale), out["q"].cpu().numpy()), row


def test_conv_streamed_output_and_residual():
    """an fp32 output of 64 MiB: the library writes it, and reads a residual of that size, with non-temporal hints
    (a different store / load instruction in every epilogue); results must not depend on that"""
    n, h, w, ci, co = 8, 128, 128, 16, 128
    assert n * h * w * co * 4 >= 64 << 20
    note("streamed output", (n, h, w, ci, co))
    r = rng(77)
    x, wt = _ints(r, (n, h, w, ci), 8), _ints(r, (co, 1, 1, ci), 8)
    acc, _ = orc.conv2d_nhwc(x, wt, (0, 0), (1, 1), (1, 1), 1)
    div = r.uniform(0.6, 3.5, co).astype(np.float32)
    bias = r.standard_normal(co).astype(np.float32)
    resid = r.standard_normal(acc.shape).astype(np.float32)
    for per_channel, use_res, act, y_dtype, q_bw in ((True, True, 1, torch.float32, 8), (True, False, 0, torch.float32, 0),
                                                     (False, True, 3, torch.float32, 16), (True, True, 2, torch.float32, 0)):
        out = cabi.conv2d_nhwc(cabi.dev(x), cabi.dev(wt), exp2=-9, chan_div=cabi.dev(div) if per_channel else None,
                               bias=cabi.dev(bias), resid=cabi.dev(resid) if use_res else None, act=act, y_dtype=y_dtype,
                               want_acc=False, q_bw=q_bw, q_pos=-3 if q_bw == 8 else -10,
                               chan_rcp=cabi.dev(np.float32(1) / div) if per_channel else None, act_slope=0.1)
        y = orc.epilogue(acc, -9, div if per_channel else None, bias, resid if use_res else None, act, act_slope=0.1)
        assert same_bits(y, out["y"].cpu().numpy()), (per_channel, use_res, act)
        if q_bw:
            assert same_bits(orc.quantize(y, q_bw, -3 if q_bw == 8 else -10), out["q"].cpu().numpy())
    # the LDS-ring kernel (K = 128) and the two-branch kernel at the same output size
    x2, w2 = _ints(r, (n, h, w, 128), 8), _ints(r, (co, 1, 1, 128), 8)
    acc2, _ = orc.conv2d_nhwc(x2, w2, (0, 0), (1, 1), (1, 1), 1)
    assert cabi.conv_route(8, 8, x2.shape, w2.shape) == "mfma"
    out = cabi.conv2d_nhwc(cabi.dev(x2), cabi.dev(w2), exp2=-12, chan_div=cabi.dev(div), bias=cabi.dev(bias),
                           resid=cabi.dev(resid), act=1, want_acc=False, q_bw=8, q_pos=-3,
                           chan_rcp=cabi.dev(np.float32(1) / div))
    y2 = orc.epilogue(acc2, -12, div, bias, resid, 1)
    assert same_bits(y2, out["y"].cpu().numpy()) and same_bits(orc.quantize(y2, 8, -3), out["q"].cpu().numpy())
    sdiv = r.uniform(0.6, 3.5, co).astype(np.float32)
    out, ws = cabi.conv2d_shortcut_nhwc(cabi.dev(x2), cabi.dev(w2), cabi.dev(x), cabi.dev(wt), 1, -9, cabi.dev(sdiv), cabi.dev(bias),
                                        cabi.dev(np.float32(1) / sdiv), exp2=-12, chan_div=cabi.dev(div), bias=cabi.dev(bias),
                                        act=1, q_bw=8, q_pos=-3, chan_rcp=cabi.dev(np.float32(1) / div))
    assert ws == 0  # served by the two-branch kernel
    y3 = orc.epilogue(acc2, -12, div, bias, orc.epilogue(acc, -9, sdiv, bias, None, 0), 1)
    assert same_bits(y3, out["y"].cpu().numpy()) and same_bits(orc.quantize(y3, 8, -3), out["q"].cpu().numpy())
    # the same through the GEMM entry point
    a, b = x.reshape(-1, ci), wt.reshape(co, ci)
    out = cabi.gemm_nt(cabi.dev(a), cabi.dev(b), exp2=-9, chan_div=cabi.dev(div), bias=cabi.dev(bias), act=1,
                       want_acc=False, chan_rcp=cabi.dev(np.float32(1) / div))
    assert same_bits(orc.epilogue(acc.reshape(-1, co), -9, div, bias, None, 1), out["y"].cpu().numpy())


def _random_conv_case(r):
    """a convolution problem drawn so that every kernel family turns up: few / odd / multiple-of-16 channel
    counts, depthwise and grouped, 1x1 to 7x7 filters, strides, dilations, padding"""
    kh, kw = (int(v) for v in r.choice([1, 1, 2, 3, 3, 5, 7], 2))
    if r.random() < 0.6:
        kw = kh
    dil = (int(r.choice([1, 1, 1, 2])), int(r.choice([1, 1, 1, 2])))
    stride = (int(r.choice([1, 1, 2, 3])), int(r.choice([1, 1, 2, 3])))
    pad = (int(r.integers(0, kh // 2 + 2)), int(r.integers(0, kw // 2 + 2)))
    h = int(r.integers(max(1, dil[0] * (kh - 1) + 1 - 2 * pad[0]), 40))
    w = int(r.integers(max(1, dil[1] * (kw - 1) + 1 - 2 * pad[1]), 40))
    kind = r.choice(["dense", "dense", "dense", "depthwise", "grouped", "pointwise_long"])
    ci = int(r.choice([1, 3, 4, 8, 16, 16, 24, 32, 32, 48, 64, 96, 130, 256]))
    co = int(r.choice([1, 4, 5, 8, 16, 24, 32, 36, 64, 64, 100, 128, 160, 255]))
    g = 1
    if kind == "depthwise":
        ci = co = g = int(r.choice([4, 6, 8, 16, 24, 32, 96]))
    elif kind == "grouped":
        g = int(r.choice([2, 4]))
        ci, co = g * int(r.choice([1, 3, 4, 8])), g * int(r.choice([1, 2, 4, 6]))
    elif kind == "pointwise_long":  # many pixels, short K: the streaming kernels' territory
        kh = kw = 1
        pad, dil = (0, 0), (1, 1)
        h, w = int(r.integers(40, 90)), int(r.integers(40, 90))
        ci, co = int(r.choice([16, 32, 48, 64, 96])), int(r.choice([16, 24, 32, 64, 96, 144, 160]))
    n = int(r.integers(1, 4))
    bits = [(8, 8), (8, 8), (16, 8), (16, 16)][int(r.integers(0, 4))]
    return n, ci, h, w, co, kh, kw, pad, stride, dil, g, bits


@pytest.mark.parametrize("seed", range(12))
def test_conv_random_sweep(seed):
    """20 random problems per seed, each with a random epilogue (divisor in reciprocal or true-division form, bias,
    residual before / after the activation, all four activations, fp32 / fp16 / no float output, int8 / int16 / no
    requantization at unit and fractional scale, integer sums): everything bit-exact against the oracle."""
    r = rng(1000 + seed)
    for i in range(20):
        n, ci, h, w, co, kh, kw, pad, stride, dil, g, bits = _random_conv_case(r)
        route = cabi.conv_route(bits[0], bits[1], (n, h, w, ci), (co, kh, kw, ci // g), pad, stride, dil, g)
        x, wt = _ints(r, (n, h, w, ci), bits[0]), _ints(r, (co, kh, kw, ci // g), bits[1])
        use_div, use_rcp = r.random() < 0.6, r.random() < 0.7
        use_bias, res_mode = r.random() < 0.7, int(r.choice([0, 0, 1, 2]))
        act = int(r.integers(0, 4))
        y_dtype = [None, torch.float32, torch.float32, torch.float16][int(r.integers(0, 4))]
        q_bw = int(r.choice([0, 8, 8, 16]))
        want_acc = bits != (16, 16) and r.random() < 0.3
        if y_dtype is None and not q_bw and not want_acc:
            y_dtype = torch.float32
        q_scale = 1.0 if r.random() < 0.5 else float(np.float32(r.uniform(1.0, 2.0)))
        exp2 = {(8, 8): -10, (16, 8): -18, (16, 16): -26}[bits] + int(r.integers(-2, 3))
        q_pos = int(r.integers(-5, 0)) if q_bw == 8 else int(r.integers(-12, -6))
        case = dict(seed=seed, i=i, shape=(n, ci, h, w, co, kh, kw), pad=pad, stride=stride, dil=dil, groups=g, bits=bits,
                    route=route, div=use_div, rcp=use_rcp, bias=use_bias, res=res_mode, act=act, y=y_dtype, q_bw=q_bw,
                    q_scale=q_scale, q_pos=q_pos, exp2=exp2, acc=want_acc)
        note("sweep", case)
        acc, ovf = orc.conv2d_nhwc(x, wt, pad, stride, dil, g)
        assert acc.size > 0
        div = r.uniform(0.6, 3.5, co).astype(np.float32) if use_div else None
        bias = r.standard_normal(co).astype(np.float32) if use_bias else None
        resid = r.standard_normal(acc.shape).astype(np.float32) if res_mode else None
        out = cabi.conv2d_nhwc(cabi.dev(x), cabi.dev(wt), pad, stride, dil, g, exp2=exp2,
                               chan_div=cabi.dev(div) if use_div else None, bias=cabi.dev(bias) if use_bias else None,
                               resid=cabi.dev(resid) if res_mode else None, act=act, y_dtype=y_dtype, want_acc=want_acc,
                               q_bw=q_bw, q_pos=q_pos, q_scale=q_scale,
                               chan_rcp=cabi.dev(np.float32(1) / div) if use_div and use_rcp else None, act_slope=0.1,
                               resid_after_act=res_mode == 2)
        torch.cuda.synchronize()
        y = orc.epilogue(acc, exp2, div, bias, resid, act, act_slope=0.1, resid_after_act=res_mode == 2)
        if want_acc:
            assert ovf == 0 and same_bits(acc.astype(np.int32), out["acc"].cpu().numpy()), case
        if y_dtype is not None:
            want = y.astype(np.float16) if y_dtype == torch.float16 else y
            assert same_bits(want, out["y"].cpu().numpy()), case
        if q_bw:
            assert same_bits(orc.quantize(y, q_bw, q_pos, q_scale), out["q"].cpu().numpy()), case


@pytest.mark.parametrize("shape", [EPILOGUE_SHAPES[0], EPILOGUE_SHAPES[2], EPILOGUE_SHAPES[4]])
@pytest.mark.parametrize("act", [1, 2])
def test_relu_folded_into_requantization_handles_non_finite_values(shape, act):
    """ReLU / ReLU6 -> int8 only: the kernels fold the activation into the quantizer's clamp.  NaN, +inf and -inf
    (here from the bias) must still come out as ReLU then quantize make them: 0, the saturation value, 0; and a
    requantization position at which the ReLU6 bound, not the int8 range, is the smaller clamp"""
    n, ci, h, w, co, k, pad, xbits = shape
    g = ci if (k == 3 and ci == co == 16) else 1
    note("folded relu", shape, act)
    r = rng(sum(shape) + act)
    x, wt = _ints(r, (n, h, w, ci), xbits), _ints(r, (co, k, k, ci // g), 8)
    acc, _ = orc.conv2d_nhwc(x, wt, (pad, pad), (1, 1), (1, 1), g)
    div = r.uniform(0.6, 3.5, co).astype(np.float32)
    bias = r.standard_normal(co).astype(np.float32)
    bias[0], bias[1], bias[2] = np.nan, np.inf, -np.inf
    resid = r.standard_normal(acc.shape).astype(np.float32)
    for q_pos, exp2, with_res, q_scale in ((-3, -10, False, 1.0), (-6, -10, False, 1.0), (-4, -9, True, 1.0),
                                           (-3, -10, False, 1.37), (-4, -10, True, 1.77), (-5, -10, False, 1.12)):
        out = cabi.conv2d_nhwc(cabi.dev(x), cabi.dev(wt), (pad, pad), (1, 1), (1, 1), g, exp2=exp2, chan_div=cabi.dev(div),
                               bias=cabi.dev(bias), resid=cabi.dev(resid) if with_res else None, act=act, y_dtype=None,
                               want_acc=False, q_bw=8, q_pos=q_pos, q_scale=q_scale,
                               chan_rcp=cabi.dev(np.float32(1) / div))
        y = orc.epilogue(acc, exp2, div, bias, resid if with_res else None, act)
        want = orc.quantize(y, 8, q_pos, q_scale)
        got = out["q"].cpu().numpy()
        assert same_bits(want, got), (q_pos, exp2, with_res, q_scale)
        assert not got[..., 0].any() and not got[..., 2].any()
        six = np.rint(np.float32(6) * np.float32(q_scale) * np.float32(2.0 ** -q_pos))
        assert (got[..., 1] == min(127, int(six) if act == 2 else 127)).all()


SHORTCUT_CASES = [
    # N, H, W, Ci, Co, k, pad, stride (main conv);  Hs, Ws, Cs, shortcut stride;  x bits, expected workspace use
    (2, 14, 14, 64, 256, 1, 0, 1, 14, 14, 64, 1, 8, False),     # first block of a bottleneck stage: both 1x1 s1
    (2, 7, 7, 128, 512, 1, 0, 1, 14, 14, 256, 2, 8, False),     # later stages: shortcut reads every other pixel
    (3, 9, 11, 32, 64, 3, 1, 1, 9, 11, 16, 1, 8, False),        # basic block: 3x3 main convolution, ragged extents
    (1, 16, 16, 64, 128, 3, 1, 2, 16, 16, 48, 2, 8, False),     # main convolution strided as well
    (2, 40, 40, 256, 1024, 1, 0, 1, 80, 80, 512, 2, 8, False),  # long K on both branches, many tiles
    (2, 20, 21, 64, 128, 1, 0, 1, 20, 21, 64, 1, 8, False),     # short K, Co >= 128: 64x128 tiles
    (2, 6, 6, 32, 36, 1, 0, 1, 6, 6, 16, 1, 8, False),          # Co % 32 != 0
    (2, 6, 6, 24, 32, 1, 0, 1, 6, 6, 16, 1, 8, True),           # Ci % 16 != 0: two launches through the workspace
    (2, 6, 6, 32, 30, 1, 0, 1, 6, 6, 16, 1, 8, True),           # Co % 4 != 0
    (1, 8, 8, 32, 32, 3, 1, 1, 8, 8, 16, 1, 16, True),          # int16 activations
]


@pytest.mark.parametrize("case", SHORTCUT_CASES)
def test_conv_with_projection_shortcut(case):
    """catchq_conv2d_shortcut_nhwc against the oracle's two convolutions in sequence: shortcut (dequant + bias,
    fp32) -> main convolution with that tensor as its residual, ReLU, fp32 and requantized outputs."""
    n, h, w, ci, co, k, pad, stride, hs, ws_, cs, ss, xbits, uses_ws = case
    note("conv_shortcut", case)
    r = rng(sum(case[:12]))
    x, wt = _ints(r, (n, h, w, ci), xbits), _ints(r, (co, k, k, ci), 8)
    sx, sw = _ints(r, (n, hs, ws_, cs), xbits), _ints(r, (co, 1, 1, cs), 8)
    acc, ovf = orc.conv2d_nhwc(x, wt, (pad, pad), (stride, stride), (1, 1), 1)
    acc_s, ovf_s = orc.conv2d_nhwc(sx, sw, (0, 0), (ss, ss), (1, 1), 1)
    assert ovf == 0 and ovf_s == 0 and acc.shape == acc_s.shape
    div, div_s = r.uniform(0.6, 3.5, co).astype(np.float32), r.uniform(0.6, 3.5, co).astype(np.float32)
    bias, bias_s = r.standard_normal(co).astype(np.float32), r.standard_normal(co).astype(np.float32)
    e_main, e_sc = (-10, -12) if xbits == 8 else (-18, -20)
    y_s = orc.epilogue(acc_s, e_sc, div_s, bias_s, None, 0)
    xd, wd, sxd, swd = cabi.dev(x), cabi.dev(wt), cabi.dev(sx), cabi.dev(sw)
    for act, after, with_rcp in ((1, False, True), (1, False, False), (3, True, True), (0, False, True)):
        out, ws_bytes = cabi.conv2d_shortcut_nhwc(
            xd, wd, sxd, swd, ss, e_sc, cabi.dev(div_s), cabi.dev(bias_s), cabi.dev(np.float32(1) / div_s) if with_rcp else None,
            (pad, pad), (stride, stride), (1, 1), exp2=e_main, chan_div=cabi.dev(div), bias=cabi.dev(bias), act=act,
            q_bw=8, q_pos=-3, chan_rcp=cabi.dev(np.float32(1) / div) if with_rcp else None, act_slope=0.1,
            resid_after_act=after)
        assert (ws_bytes > 0) == uses_ws
        y = orc.epilogue(acc, e_main, div, bias, y_s, act, act_slope=0.1, resid_after_act=after)
        assert same_bits(y, out["y"].cpu().numpy()), (act, after, with_rcp)
        assert same_bits(orc.quantize(y, 8, -3), out["q"].cpu().numpy()), (act, after, with_rcp)
    # no divisors, no biases, fp16 output only
    out, _ = cabi.conv2d_shortcut_nhwc(xd, wd, sxd, swd, ss, e_sc, padding=(pad, pad), stride=(stride, stride),
                                       exp2=e_main, act=2, y_dtype=torch.float16)
    y = orc.epilogue(acc, e_main, None, None, orc.epilogue(acc_s, e_sc, None, None, None, 0), 2, np.float16)
    assert same_bits(y, out["y"].cpu().numpy())


HEAD_CASES = [
    # N, H, W, K1 (head input channels), Cm, Co, fused in one launch?
    (3, 56, 56, 256, 64, 64, True),    # ResNet-50 stage 1, blocks 2 and 3: bands of 4 rows, 11 head sub-tiles
    (2, 56, 56, 64, 64, 64, True),     # its first block: one K step pair in the head
    (2, 30, 20, 256, 64, 64, True),    # bands of unequal height (the last one shorter), W not a multiple of 4
    (5, 17, 33, 64, 64, 64, True),     # odd sizes: ragged sub-tiles in both phases
    (2, 14, 14, 256, 64, 64, True),    # one band per image: both halo rows lie outside the image
    (2, 7, 7, 256, 64, 64, False),     # small images go several to a tile: two launches
    (1, 28, 28, 512, 128, 128, False), # other channel counts: two launches
    (2, 12, 12, 64, 64, 96, False),
]


@pytest.mark.parametrize("case", HEAD_CASES)
def test_conv1x1_then_conv3x3(case):
    """catchq_conv1x1_conv3x3_nhwc against the oracle's two convolutions in sequence: 1x1 (dequant + bias, ReLU,
    requantized to int8) then 3x3 with padding 1 (the zeros of the padding are zeros of the requantized tensor);
    int8 and fp32 outputs of the second convolution, bit for bit, with and without planning for a shared device."""
    n, h, w, k1, cm, co, fused = case
    note("conv1x1_conv3x3", case)
    r = rng(sum(case[:6]))
    x, w1, w2 = _ints(r, (n, h, w, k1), 8), _ints(r, (cm, 1, 1, k1), 8), _ints(r, (co, 3, 3, cm), 8)
    x[0, 0, :, :] = 127  # the first image row at full scale: what the halo above it must not leak into
    x[-1, -1, :, :] = -128
    div1, bias1 = r.uniform(0.6, 3.5, cm).astype(np.float32), r.standard_normal(cm).astype(np.float32) * 4
    div2, bias2 = r.uniform(0.6, 3.5, co).astype(np.float32), r.standard_normal(co).astype(np.float32)
    e1, qp1, e2 = {64: -10, 256: -11, 512: -12}[k1], -2, -8
    acc1, ovf1 = orc.conv2d_nhwc(x, w1, (0, 0), (1, 1), (1, 1), 1)
    q1 = orc.quantize(orc.epilogue(acc1, e1, div1, bias1, None, 1), 8, qp1)
    assert ovf1 == 0 and 0 < (q1 == 127).mean() < 0.2 and (q1 == 0).mean() < 0.8  # saturation and ReLU both occur
    acc2, ovf2 = orc.conv2d_nhwc(q1, w2, (1, 1), (1, 1), (1, 1), 1)
    assert ovf2 == 0
    xd, w1d, w2d = cabi.dev(x), cabi.dev(w1.reshape(cm, k1)), cabi.dev(w2)
    d1, r1, b1 = cabi.dev(div1), cabi.dev(np.float32(1) / div1), cabi.dev(bias1)
    for act, want_y, sharing in ((1, False, 0), (1, False, 2), (0, True, 0), (2, True, 2)):
        out, ws_bytes = cabi.conv1x1_conv3x3_nhwc(xd, w1d, e1, d1, r1, b1, qp1, w2d, exp2=e2, chan_div=cabi.dev(div2),
                                                  bias=cabi.dev(bias2), act=act, y_dtype=torch.float32 if want_y else None,
                                                  q_bw=8, q_pos=-1, chan_rcp=cabi.dev(np.float32(1) / div2), sharing=sharing)
        assert (ws_bytes == 0) == fused, ws_bytes
        y = orc.epilogue(acc2, e2, div2, bias2, None, act)
        assert same_bits(orc.quantize(y, 8, -1), out["q"].cpu().numpy()), (act, want_y, sharing)
        if want_y:
            assert same_bits(y, out["y"].cpu().numpy()), (act, want_y, sharing)


IRB_CASES = [
    # N, H, W, Ci, hidden, Co, stride, shortcut?, fused in one launch?
    (3, 14, 14, 64, 384, 64, 1, True, True),     # MobileNetV2 at 14 x 14: two bands of 7 rows, two chunks of hidden channels
    (2, 14, 14, 64, 384, 96, 1, False, True),    # three column tiles on two wave columns
    (2, 14, 14, 96, 576, 96, 1, True, True),     # three K steps in the expansion, three chunks
    (2, 14, 14, 96, 576, 160, 2, False, True),   # stride 2: 7 x 7 out of a 15-row patch
    (2, 7, 7, 160, 960, 160, 1, True, True),     # whole 7 x 7 images, five chunks
    (1, 7, 7, 160, 960, 320, 1, False, True),    # ten column tiles: three per wave
    (2, 28, 28, 32, 192, 32, 1, True, True),     # one chunk, bands of 28 x 28 images
    (2, 28, 28, 32, 192, 64, 2, False, True),    # stride 2 from 28 x 28: bands of two output rows
    (2, 12, 20, 32, 192, 32, 1, True, True),     # W not a multiple of 4: ragged stencil groups
    (1, 9, 11, 64, 192, 64, 2, False, True),     # odd sizes with stride 2
    (2, 10, 10, 16, 96, 32, 1, False, False),    # channel counts outside the fused kernel: three launches
    (1, 6, 6, 32, 192, 24, 1, False, False),
]


@pytest.mark.parametrize("case", IRB_CASES)
def test_inverted_residual_block(case):
    """catchq_inverted_residual_nhwc against the oracle's three convolutions in sequence: 1x1 expansion and 3x3 depthwise
    convolution (padding 1), each dequantized, biased, sent through ReLU6 and requantized to int8, then the 1x1 projection
    with its own epilogue (no activation, optional fp32 shortcut); int8 and fp32 outputs, bit for bit."""
    n, h, w, ci, hid, co, stride, shortcut, fused = case
    note("inverted_residual", case)
    r = rng(sum(case[:7]))
    x, w1 = _ints(r, (n, h, w, ci), 8), _ints(r, (hid, 1, 1, ci), 8)
    wd, w3 = _ints(r, (hid, 3, 3, 1), 8), _ints(r, (co, 1, 1, hid), 8)
    x[0, 0, :, :] = 127  # full-scale border rows: what the zero padding of the hidden tensor must not be replaced by
    x[-1, -1, :, :] = -128

    def consts(c, spread):
        return r.uniform(0.6, 3.5, c).astype(np.float32), (r.standard_normal(c) * spread).astype(np.float32)

    (div1, bias1), (div2, bias2), (div3, bias3) = consts(hid, 1.5), consts(hid, 1.5), consts(co, 1.0)
    e1 = -12 - int(np.log2(ci / 32) / 2 + 0.5)
    e2, e3, qp1, qp2, qp3 = -11, -10, -4, -4, -1
    acc1, ovf1 = orc.conv2d_nhwc(x, w1, (0, 0), (1, 1), (1, 1), 1)
    q1 = orc.quantize(orc.epilogue(acc1, e1, div1, bias1, None, 2), 8, qp1)
    assert ovf1 == 0 and 0.02 < (q1 == 96).mean() < 0.5 and (q1 == 0).mean() < 0.8  # ReLU6's 6 and ReLU's 0 both occur
    acc2, ovf2 = orc.conv2d_nhwc(q1, wd, (1, 1), (stride, stride), (1, 1), hid)
    q2 = orc.quantize(orc.epilogue(acc2, e2, div2, bias2, None, 2), 8, qp2)
    assert ovf2 == 0 and 0.005 < (q2 == 96).mean() < 0.6 and (q2 == 0).mean() < 0.8
    acc3, ovf3 = orc.conv2d_nhwc(q2, w3, (0, 0), (1, 1), (1, 1), 1)
    assert ovf3 == 0
    resid = (r.standard_normal(acc3.shape) * 8).astype(np.float32) if shortcut else None
    y = orc.epilogue(acc3, e3, div3, bias3, resid, 0)
    q = orc.quantize(y, 8, qp3)
    assert 0 < (np.abs(q.astype(np.int32)) >= 127).mean() < 0.4

    dv = cabi.dev
    st1 = dict(w=dv(w1.reshape(hid, ci)), exp2=e1, chan_div=dv(div1), chan_rcp=dv(np.float32(1) / div1), bias=dv(bias1),
               act=2, q_pos=qp1)
    st2 = dict(w=dv(wd.reshape(hid, 3, 3)), exp2=e2, chan_div=dv(div2), chan_rcp=dv(np.float32(1) / div2), bias=dv(bias2),
               act=2, q_pos=qp2)
    xd, w3d, d3, r3, b3 = dv(x), dv(w3.reshape(co, hid)), dv(div3), dv(np.float32(1) / div3), dv(bias3)
    rd = dv(resid) if shortcut else None
    for want_y, sharing in ((False, 0), (True, 2)):
        out, ws_bytes = cabi.inverted_residual_nhwc(xd, st1, st2, w3d, stride=stride, exp2=e3, chan_div=d3, bias=b3, resid=rd,
                                                    act=0, y_dtype=torch.float32 if want_y else None, q_bw=8, q_pos=qp3,
                                                    chan_rcp=r3, sharing=sharing)
        assert (ws_bytes == 0) == fused, ws_bytes
        assert same_bits(q, out["q"].cpu().numpy()), (want_y, sharing)
        if want_y:
            assert same_bits(y, out["y"].cpu().numpy()), (want_y, sharing)


FIRST_LAYER_CASES = [
    # N, C, H, W, Co, k, stride, pad, pool (k, stride, pad), activation, planning hint, fused in one launch?
    (2, 3, 64, 64, 64, 7, 2, 3, (3, 2, 1), 1, 0, True),       # few images: bands of one pooled row
    (32, 3, 64, 64, 64, 7, 2, 3, (3, 2, 1), 1, 4, True),      # bands of two pooled rows
    (48, 3, 52, 52, 64, 7, 2, 3, (3, 2, 1), 1, 0, True),      # bands of three pooled rows, the last band one row
    (96, 3, 44, 44, 64, 7, 2, 3, (3, 2, 1), 2, 2, True),      # bands of six pooled rows, the last band five
    (32, 3, 224, 224, 64, 7, 2, 3, (3, 2, 1), 1, 2, True),    # the ImageNet shape: seven pooled rows per block of sixteen waves
    (2, 3, 50, 36, 64, 7, 2, 3, (3, 2, 1), 2, 8, True),       # odd convolution height: the last window is cut by the image
    (3, 1, 32, 40, 32, 7, 2, 3, (3, 2, 1), 1, 0, True),       # one input channel, 32 output channels
    (1, 2, 40, 32, 128, 7, 2, 3, (3, 2, 1), 2, 0, True),      # 128 output channels: four channel groups
    (2, 3, 30, 30, 64, 7, 2, 3, (3, 2, 1), 1, 0, False),      # width not a multiple of 4: three launches
    (1, 4, 32, 32, 64, 7, 2, 3, (3, 2, 1), 1, 0, False),      # four input channels
    (2, 3, 24, 24, 32, 3, 1, 1, (2, 2, 0), 2, 0, False),      # another filter and window
]


@pytest.mark.parametrize("case", FIRST_LAYER_CASES)
def test_first_layers(case):
    """catchq_first_layers_nchw against the oracle's quantizer, convolution, epilogue + requantization and max pooling in
    sequence, bit for bit; full-scale pixels on the image's border show a wrong frame or a wrong window."""
    n, c, h, w, co, k, stride, pad, pool, act, sharing, fused = case
    note("first_layers", case)
    r = rng(n + c + h + w + co + k)
    x = (r.standard_normal((n, c, h, w)) * 1.5).astype(np.float32)
    x[:, :, 0, :] = 5.0
    x[:, :, -1, :] = -5.0
    x[:, :, :, 0] = 4.5
    x[:, :, :, -1] = -4.5
    x_pos, x_scale = -5, 1.0 if n % 2 else 0.9371
    wt = _ints(r, (co, k, k, 4), 8)
    wt[..., c:] = 0
    div = r.uniform(0.6, 3.5, co).astype(np.float32)
    bias = (r.standard_normal(co) * 2.0).astype(np.float32)
    e1 = -11 - int(np.log2(k * k * c / 49.0) / 2 + 0.5)
    qp = -3
    qx = orc.quantize_nchw_to_nhwc(x, 8, x_pos, x_scale, cpad=4)
    assert 0 < (np.abs(qx.astype(np.int32)) >= 127).mean() < 0.2
    acc, ovf = orc.conv2d_nhwc(qx, wt, (pad, pad), (stride, stride), (1, 1), 1)
    assert ovf == 0
    q1 = orc.quantize(orc.epilogue(acc, e1, div, bias, None, act), 8, qp)
    assert 0.005 < (q1 == (48 if act == 2 else 127)).mean() < 0.6 and 0.1 < (q1 == 0).mean() < 0.8
    want = orc.maxpool_nhwc(q1.astype(np.float32), *pool).astype(np.int8)  # the oracle pools floats; int8 values survive the trip

    kw4 = (k + 3) // 4 * 4
    wdev = np.zeros((co, k, kw4, 4), np.int8)
    wdev[:, :, :k] = wt
    dv = cabi.dev
    conv = dict(w=dv(wdev), exp2=e1, chan_div=dv(div), chan_rcp=dv(np.float32(1) / div), bias=dv(bias), act=act, q_pos=qp)
    got, ws_bytes = cabi.first_layers_nchw(dv(x), x_pos, conv, k, stride, pad, pool, x_scale, sharing)
    assert (ws_bytes == 0) == fused, ws_bytes
    assert same_bits(want, got.cpu().numpy())


CONV_AVGPOOL_CASES = [
    # N, H, W, Ci, Co, residual?, activation, fused in one launch?
    (32, 7, 7, 512, 2048, True, 1, True),     # ResNet-50's last block: eight waves per block
    (3, 7, 7, 512, 2048, True, 1, True),      # few images: four waves per block
    (5, 7, 7, 320, 1280, False, 2, True),     # MobileNetV2's last convolution: ReLU6, rows of 20 pieces (swizzle over 4)
    (2, 8, 8, 64, 96, False, 0, True),        # 64 pixels: both pixel groups full; three channel groups on four waves
    (4, 5, 6, 96, 32, True, 2, True),         # 30 pixels: one pixel group; rows of 6 pieces (swizzle over 2)
    (2, 1, 1, 32, 64, False, 1, True),        # a single pixel
    (2, 3, 3, 2048, 64, False, 1, True),      # long K: four passes through LDS
    (2, 9, 9, 64, 64, False, 1, False),       # 81 pixels: two launches
    (2, 4, 4, 48, 64, True, 1, False),        # Ci % 32 != 0
    (1, 8, 8, 4096, 32, False, 1, True),      # 64 pixels x 4096 channels: eight passes of 512 bytes through LDS
    (300, 2, 2, 512, 64, True, 1, True),      # more blocks than compute units: passes of 256 bytes, two blocks a unit
    (130, 3, 3, 320, 512, False, 2, True),    # the same with rows of 10 pieces (passes of 160 bytes)
]


@pytest.mark.parametrize("case", CONV_AVGPOOL_CASES)
def test_conv1x1_global_avgpool(case):
    """catchq_conv1x1_avgpool_nhwc against the oracle's convolution, epilogue (dequantization, bias, fp32 residual,
    activation), ordered global average and quantizer, bit for bit, with and without the fp32 mean / the int8 form."""
    n, h, w, ci, co, shortcut, act, fused = case
    note("conv1x1_avgpool", case)
    r = rng(sum(case[:5]))
    x, wt = _ints(r, (n, h, w, ci), 8), _ints(r, (co, 1, 1, ci), 8)
    div = r.uniform(0.6, 3.5, co).astype(np.float32)
    bias = (r.standard_normal(co) * 1.5).astype(np.float32)
    e1 = -11 - int(np.log2(ci / 32) / 2 + 0.5)
    acc, ovf = orc.conv2d_nhwc(x, wt, (0, 0), (1, 1), (1, 1), 1)
    assert ovf == 0
    resid = (r.standard_normal(acc.shape) * 4).astype(np.float32) if shortcut else None
    y = orc.epilogue(acc, e1, div, bias, resid, act)
    assert (act == 0 or 0.1 < (y == 0).mean() < 0.9) and (act != 2 or 0.02 < (y == 6).mean() < 0.9)
    mean = orc.global_avgpool_nhwc(y)
    qp = -4 if act != 2 else -3
    q8 = orc.quantize(mean, 8, qp, 0.93)
    assert len(np.unique(q8)) > 8
    dv = cabi.dev
    xd, wd, dd, rd, bd = dv(x), dv(wt.reshape(co, ci)), dv(div), dv(np.float32(1) / div), dv(bias)
    sd = dv(resid) if shortcut else None
    for want_mean, q_bw in ((True, 8), (False, 8), (True, 0), (True, 16)):
        out, ws_bytes = cabi.conv1x1_avgpool_nhwc(xd, wd, exp2=e1, chan_div=dd, bias=bd, resid=sd, act=act, chan_rcp=rd,
                                                  want_mean=want_mean, q_bw=q_bw, q_pos=qp if q_bw == 8 else qp - 8, q_scale=0.93)
        assert (ws_bytes == 0) == fused, ws_bytes
        if want_mean:
            assert same_bits(mean, out["mean"].cpu().numpy()), (want_mean, q_bw)
        if q_bw == 8:
            assert same_bits(q8, out["q"].cpu().numpy()), (want_mean, q_bw)
        if q_bw == 16:
            assert same_bits(orc.quantize(mean, 16, qp - 8, 0.93), out["q"].cpu().numpy()), (want_mean, q_bw)


@pytest.mark.parametrize("seed", range(2))
def test_first_layers_and_pooled_convolution_random_sweep(seed):
    """random shapes inside the one-launch kernels' domains: 30 convolutions with the average pooling inside (1 to 64
    pixels, 32 to 256 input and up to 352 output channels, one to 70 images, every activation, with and without
    residual) and 20 first-layer stacks (one to three input channels, heights 7 to 69, widths 8 to 68, 32 / 64 / 128 output
    channels, with and without a fractional input scale), bit-exact against the oracle, none through the workspace."""
    r = rng(4100 + seed)
    dv = cabi.dev
    for it in range(30):
        n = int(r.choice([1, 2, 3, 5, 9, 33, 70]))
        h, w = int(r.integers(1, 9)), int(r.integers(1, 9))
        ci, co = 32 * int(r.integers(1, 9)), 32 * int(r.integers(1, 12))
        if n >= 33:
            ci, co = min(ci, 128), min(co, 128)
        act, use_res = int(r.integers(0, 3)), bool(r.integers(0, 2))
        case = ("conv1x1_avgpool sweep", seed, it, n, h, w, ci, co, act, use_res)
        note(*case)
        x, wt = _ints(r, (n, h, w, ci), 8), _ints(r, (co, 1, 1, ci), 8)
        div = r.uniform(0.6, 3.5, co).astype(np.float32)
        bias = (r.standard_normal(co) * 1.5).astype(np.float32)
        e1 = -11 - int(np.log2(ci / 32) / 2 + 0.5)
        acc, ovf = orc.conv2d_nhwc(x, wt, (0, 0), (1, 1), (1, 1), 1)
        assert ovf == 0
        resid = (r.standard_normal(acc.shape) * 4).astype(np.float32) if use_res else None
        mean = orc.global_avgpool_nhwc(orc.epilogue(acc, e1, div, bias, resid, act))
        out, ws_bytes = cabi.conv1x1_avgpool_nhwc(dv(x), dv(wt.reshape(co, ci)), exp2=e1, chan_div=dv(div), bias=dv(bias),
                                                  resid=dv(resid) if use_res else None, act=act,
                                                  chan_rcp=dv(np.float32(1) / div), want_mean=True, q_bw=8, q_pos=-4)
        assert ws_bytes == 0, case
        assert same_bits(mean, out["mean"].cpu().numpy()), case
        assert same_bits(orc.quantize(mean, 8, -4), out["q"].cpu().numpy()), case
    for it in range(20):
        n, c = int(r.choice([1, 2, 3, 7, 20, 40])), int(r.integers(1, 4))
        h, w, co = int(r.integers(7, 70)), 4 * int(r.integers(2, 18)), int(r.choice([32, 64, 128]))
        if n >= 20:
            h, w = min(h, 40), min(w, 40)
        act = int(r.integers(1, 3))
        x_scale = float(np.float32(r.uniform(0.8, 1.2))) if r.integers(0, 2) else 1.0
        case = ("first_layers sweep", seed, it, n, c, h, w, co, act, x_scale)
        note(*case)
        x = (r.standard_normal((n, c, h, w)) * 1.5).astype(np.float32)
        wt = _ints(r, (co, 7, 7, 4), 8)
        wt[..., c:] = 0
        div = r.uniform(0.6, 3.5, co).astype(np.float32)
        bias = (r.standard_normal(co) * 2.0).astype(np.float32)
        e1 = -11 - int(np.log2(c) / 2 + 0.5)
        qx = orc.quantize_nchw_to_nhwc(x, 8, -5, x_scale, cpad=4)
        acc, ovf = orc.conv2d_nhwc(qx, wt, (3, 3), (2, 2), (1, 1), 1)
        assert ovf == 0
        q1 = orc.quantize(orc.epilogue(acc, e1, div, bias, None, act), 8, -3)
        want = orc.maxpool_nhwc(q1.astype(np.float32), 3, 2, 1).astype(np.int8)
        wdev = np.zeros((co, 7, 8, 4), np.int8)
        wdev[:, :, :7] = wt
        conv = dict(w=dv(wdev), exp2=e1, chan_div=dv(div), chan_rcp=dv(np.float32(1) / div), bias=dv(bias), act=act, q_pos=-3)
        got, ws_bytes = cabi.first_layers_nchw(dv(x), -5, conv, 7, 2, 3, (3, 2, 1), x_scale, 0)
        assert ws_bytes == 0, case
        assert same_bits(want, got.cpu().numpy()), case


CHAIN_CASES = [
    # N, Ho, Wo, Co, shortcut (Cs, stride), main channel counts (one per block)
    (2, 14, 14, 256, (64, 1), (64,)),                  # first block of stage 1: shortcut + one block
    (2, 14, 14, 256, (64, 1), (64, 64, 64)),           # all of stage 1
    (2, 7, 7, 512, (256, 2), (128, 128, 128, 128)),    # stage 2: strided shortcut, two K steps per block
    (3, 5, 7, 1024, (512, 2), (256, 256)),             # ragged pixel count, eight K steps in the shortcut
    (1, 9, 9, 64, (128, 1), (64, 192)),                # Co < 128: 64x64 tiles; unequal K
    (2, 6, 6, 132, (64, 1), (64, 64)),                 # Co % 128 != 0: a ragged column tile
    (1, 3, 3, 2048, (1024, 2), (512, 512, 512)),       # stage 4: long K, few pixels
    (2, 8, 8, 128, (64, 1), (64,) * 7),                # the most links the entry point takes
]


@pytest.mark.parametrize("case", CHAIN_CASES)
def test_residual_chain(case):
    """catchq_conv1x1_chain_nhwc against the oracle's block-by-block evaluation: shortcut (dequant + bias, fp32),
    then every block's last convolution with the running fp32 tensor as its residual and ReLU; fp32 and int8
    outputs of the last block, bit for bit, and of every prefix of the chain."""
    n, ho, wo, co, (cs, ss), mains = case
    note("residual_chain", case)
    r = rng(n + ho + wo + co + cs + sum(mains))
    links, run = [], None
    for i, ci in enumerate((cs,) + tuple(mains)):
        stride = ss if i == 0 else 1
        h, w = (ho - 1) * stride + 1 + (stride - 1) * (i % 2), (wo - 1) * stride + 1
        x, wt = _ints(r, (n, h, w, ci), 8), _ints(r, (co, 1, 1, ci), 8)
        acc, ovf = orc.conv2d_nhwc(x, wt, (0, 0), (stride, stride), (1, 1), 1)
        assert ovf == 0 and acc.shape == (n, ho, wo, co)
        div, bias = r.uniform(0.6, 3.5, co).astype(np.float32), r.standard_normal(co).astype(np.float32)
        exp2 = -10 - (i % 3) - (3 if ci > 256 else 0)
        run = orc.epilogue(acc, exp2, div, bias, run, 0 if i == 0 else 1)
        links.append(dict(x=cabi.dev(x), w=cabi.dev(wt.reshape(co, ci)), stride=stride, exp2=exp2, chan_div=cabi.dev(div),
                          chan_rcp=cabi.dev(np.float32(1) / div), bias=cabi.dev(bias)))
        if i == 0:
            continue
        out = cabi.conv1x1_chain_nhwc(links, q_pos=-3)
        assert same_bits(run, out["y"].cpu().numpy()), i
        assert same_bits(orc.quantize(run, 8, -3), out["q"].cpu().numpy()), i
    q_only = cabi.conv1x1_chain_nhwc(links, want_y=False, q_pos=-2)
    assert q_only["y"] is None and same_bits(orc.quantize(run, 8, -2), q_only["q"].cpu().numpy())
    y_only = cabi.conv1x1_chain_nhwc(links, want_q=False)
    assert y_only["q"] is None and same_bits(run, y_only["y"].cpu().numpy())


def test_residual_chain_argument_checks():
    note("residual_chain errors")
    x = torch.zeros((1, 8, 8, 64), dtype=torch.int8, device="cuda")
    w = torch.zeros((64, 64), dtype=torch.int8, device="cuda")
    v = torch.ones(64, device="cuda")
    ok = dict(x=x, w=w, stride=1, exp2=0, chan_div=v, chan_rcp=v, bias=v)
    with pytest.raises(Exception):  # a single link is an ordinary convolution
        cabi.conv1x1_chain_nhwc([ok])
    with pytest.raises(Exception):  # grids differ: 4x4 against 8x8
        cabi.conv1x1_chain_nhwc([ok, dict(ok, stride=2)])
    with pytest.raises(Exception):  # no reciprocals
        cabi.conv1x1_chain_nhwc([ok, dict(ok, chan_rcp=None)])
    x48 = torch.zeros((1, 8, 8, 48), dtype=torch.int8, device="cuda")
    with pytest.raises(Exception):  # channels not a multiple of 64
        cabi.conv1x1_chain_nhwc([ok, dict(ok, x=x48, w=torch.zeros((64, 48), dtype=torch.int8, device="cuda"))])


def test_conv_shortcut_argument_checks():
    note("conv_shortcut errors")
    x = torch.zeros((1, 8, 8, 16), dtype=torch.int8, device="cuda")
    w = torch.zeros((16, 1, 1, 16), dtype=torch.int8, device="cuda")
    with pytest.raises(Exception):  # shortcut grid 4x4 != main grid 8x8
        cabi.conv2d_shortcut_nhwc(x, w, x, w, 2, 0)
    with pytest.raises(Exception):  # non-positive stride
        cabi.conv2d_shortcut_nhwc(x, w, x, w, 0, 0)


def test_quantize_into_frame():
    """NCHW float -> NHWC int8/int16 inside a zero frame equals the plain transposing quantizer placed by hand."""
    note("quantize frame")
    r = rng(77)
    x = (r.standard_normal((2, 3, 9, 11)) * 40).astype(np.float32)
    for bits, cpad in ((8, 4), (8, 8), (16, 8)):
        want = np.zeros((2, 9 + 5, 11 + 7, cpad), np.int8 if bits == 8 else np.int16)
        want[:, 2:11, 3:14, :3] = orc.quantize(np.transpose(x, (0, 2, 3, 1)), bits, -1)
        got = torch.ops.torch_mlu.quantize_nhwc_frame(cabi.dev(x), bits, -1, cpad, 14, 18, 2, 3)
        assert np.array_equal(want, got.cpu().numpy())


@pytest.mark.parametrize("shape,frame", [((3, 3, 10, 12), (2, 3, 1, 4)), ((2, 3, 33, 224), (3, 3, 3, 4)),
                                         ((5, 1, 7, 260), (0, 1, 2, 0)), ((1, 2, 3, 4), (1, 0, 0, 70)),
                                         ((2, 3, 224, 224), (3, 3, 3, 4))])
def test_quantize_into_frame_vector_path(shape, frame):
    """widths that are multiples of 4 (fp32 -> int8, 4 channels per pixel) take the kernel that moves 4 pixels per
    lane: rows of more than 64 groups, odd numbers of rows, frames with no border on a side, a border wider than a
    wave, 1 to 3 channels; the output buffer is pre-filled so that an unwritten border pixel shows"""
    note("quantize frame vector", shape, frame)
    n, c, h, w = shape
    top, left, bottom, right = frame
    r = rng(sum(shape) + sum(frame))
    x = (r.standard_normal(shape) * 50).astype(np.float32)
    x[0, 0, 0, :4] = (np.nan, np.inf, -np.inf, 0.5)
    oh, ow = h + top + bottom, w + left + right
    want = np.zeros((n, oh, ow, 4), np.int8)
    want[:, top:top + h, left:left + w, :c] = orc.quantize(np.transpose(x, (0, 2, 3, 1)), 8, -1)
    q = torch.full((n, oh, ow, 4), 77, dtype=torch.int8, device="cuda")
    cabi.check(cabi.lib().catchq_quantize_nchw_to_nhwc_frame(cabi.ptr(cabi.dev(x)), cabi.F32, cabi.ptr(q), 8, n, c, h, w, 4,
                                                             oh, ow, top, left, -1, 1.0, cabi.stream()))
    assert np.array_equal(want, q.cpu().numpy())


def test_error_statuses():
    note("error statuses")
    x = torch.zeros(16, device="cuda")
    q = torch.zeros(16, dtype=torch.int8, device="cuda")
    L = cabi.lib()
    assert L.catchq_quantize(cabi.ptr(x), 0, cabi.ptr(q), 7, 16, 0, 1.0, cabi.stream()) == 3  # bitwidth
    assert L.catchq_quantize(cabi.ptr(x), 5, cabi.ptr(q), 8, 16, 0, 1.0, cabi.stream()) == 2  # dtype
    assert L.catchq_quantize(None, 0, cabi.ptr(q), 8, 16, 0, 1.0, cabi.stream()) == 1          # null
    assert L.catchq_quantize(None, 0, None, 8, 0, 0, 1.0, cabi.stream()) == 0                  # empty is fine
    with pytest.raises(Exception):
        cabi.conv2d_nhwc(torch.zeros((1, 2, 2, 4), dtype=torch.int8, device="cuda"),
                         torch.zeros((4, 3, 3, 4), dtype=torch.int8, device="cuda"))  # output extent <= 0


# ------------------------------------------------------------------------------ operands of 2 GiB and more
def _sample_rows(total, block, r):
    """row blocks at the start, around the 2^31-byte marks and at the end"""
    starts = {0, total - block}
    for frac in (0.25, 0.5, 0.75):
        starts.add(int(total * frac) // 32 * 32)
    starts.update(int(v) for v in r.integers(0, total - block, 3))
    return sorted(starts)


def test_quantize_more_than_2g_elements():
    """2^31 + 37 elements: indices beyond 32 bits in the streaming quantizer (fp16 in, int8 out)"""
    n = 2 ** 31 + 37
    note("quantize", n)
    x = torch.empty(n, dtype=torch.float16, device="cuda")
    x.normal_(0.0, 3.0)
    q = cabi.quantize(x, 8, -4)
    torch.cuda.synchronize()
    r = rng(5)
    for s in _sample_rows(n, 4096, r) + [n - 4096 - 37, n - 64]:
        e = min(s + 4096, n)
        assert same_bits(orc.quantize(x[s:e].cpu().numpy(), 8, -4), q[s:e].cpu().numpy()), s
    del x, q
    torch.cuda.empty_cache()


@pytest.mark.parametrize("m,n,k", [(2 ** 25, 16, 64),      # A operand of exactly 2 GiB: beyond the 32-bit buffer offsets
                                   (2 ** 25 + 40, 160, 16),  # 5.4 G output elements: element indices beyond 32 bits
                                   (2 ** 22 + 3, 64, 512)])  # 2 GiB A operand with long K: the LDS ring is not eligible
def test_gemm_operands_beyond_32_bit_offsets(m, n, k):
    route = cabi.lib().catchq_gemm_route(8, 8, m, n, k)
    note("gemm beyond 32 bits", m, n, k, route)
    a = torch.randint(-128, 128, (m, k), dtype=torch.int8, device="cuda")
    b = torch.randint(-128, 128, (n, k), dtype=torch.int8, device="cuda")
    r = rng(m % 1000 + n + k)
    div = r.uniform(0.6, 3.5, n).astype(np.float32)
    bias = r.standard_normal(n).astype(np.float32)
    out = cabi.gemm_nt(a, b, exp2=-8, chan_div=cabi.dev(div), bias=cabi.dev(bias), act=1, y_dtype=None, want_acc=False,
                       q_bw=8, q_pos=-2, chan_rcp=cabi.dev(np.float32(1) / div))
    torch.cuda.synchronize()
    bh = b.cpu().numpy()
    for s in _sample_rows(m, 256, r):  # the rows of a product are independent: check blocks of them
        acc, _ = orc.gemm_nt(a[s:s + 256].cpu().numpy(), bh)
        want = orc.quantize(orc.epilogue(acc, -8, div, bias, None, 1), 8, -2)
        assert same_bits(want, out["q"][s:s + 256].cpu().numpy()), (s, route)
    del a, out
    torch.cuda.empty_cache()


def test_conv_input_beyond_32_bit_offsets():
    """a 2.1 GB input image pair: the convolution takes the kernel with 64-bit addressing; horizontal bands of
    the output (which depend on their own input rows only) against the oracle"""
    n, h, w, ci, co = 2, 4100, 4096, 64, 16
    assert n * h * w * ci >= 2 ** 31
    note("conv beyond 32 bits", (n, h, w, ci, co), cabi.conv_route(8, 8, (n, h, w, ci), (co, 3, 3, ci), (1, 1)))
    x = torch.randint(-128, 128, (n, h, w, ci), dtype=torch.int8, device="cuda")
    r = rng(9)
    wt = _ints(r, (co, 3, 3, ci), 8)
    bias = r.standard_normal(co).astype(np.float32)
    out = cabi.conv2d_nhwc(x, cabi.dev(wt), (1, 1), (1, 1), (1, 1), 1, exp2=-12, bias=cabi.dev(bias), act=1, y_dtype=None,
                           want_acc=False, q_bw=8, q_pos=-1)
    torch.cuda.synchronize()
    for img, h0 in ((0, 0), (0, 2047), (1, 1), (1, 2050), (1, h - 6)):
        lo, hi = max(h0 - 1, 0), min(h0 + 7, h)          # input rows that output rows h0 .. h0+5 read
        band = x[img:img + 1, lo:hi].cpu().numpy()
        acc, _ = orc.conv2d_nhwc(band, wt, (1, 1), (1, 1), (1, 1), 1)  # its first / last rows see zero padding instead
        want = orc.quantize(orc.epilogue(acc, -12, None, bias, None, 1), 8, -1)
        first = 0 if lo == 0 else 1                        # of the band's output rows, the ones with true neighbours
        last = want.shape[1] if hi == h else want.shape[1] - 1
        got = out["q"][img:img + 1, lo + first:lo + last].cpu().numpy()
        assert same_bits(want[:, first:last], got), (img, h0)
    del x, out
    torch.cuda.empty_cache()
