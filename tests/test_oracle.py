"""Pins the CPU oracle (oracle/vpx_oracle.c) before anything is compared against it:
reference golden vectors, the reference's own compiled float16 (oracle/_ref, when built),
closed forms and fp64 brute force.  No GPU."""
import json
import math
import os
from fractions import Fraction

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "reference_goldens.json")) as f:
    GOLD = json.load(f)


def _bits(x):
    return np.asarray(x, dtype=np.float32).view(np.uint32)


def _interesting_f32(rng, n_random=2_000_000):
    """fp32 bit patterns that stress fp32->fp16 rounding: every exponent near the half range with
    mantissas on and around the round/tie boundaries, plus random bits."""
    exps = np.arange(0, 256, dtype=np.uint32)
    mant = []
    for low in (0x0000, 0x0001, 0x0fff, 0x1000, 0x1001, 0x1fff, 0x2000, 0x2001, 0x2fff, 0x3000, 0x3001):
        for hi in (0x000000, 0x7fc000, 0x7fe000, 0x400000, 0x002000, 0x7f8000, 0x555000 & ~0x3fff):
            mant.append((hi | low) & 0x7fffff)
    mant = np.unique(np.array(mant, dtype=np.uint32))
    grid = (exps[:, None] << 23 | mant[None, :]).ravel()
    # dense sweep of the subnormal-half range, exponents 102..113, coarse mantissa steps
    e = np.arange(100, 115, dtype=np.uint32)
    m = np.arange(0, 1 << 23, 509, dtype=np.uint32)
    dense = (e[:, None] << 23 | m[None, :]).ravel()
    rnd = rng.integers(0, 1 << 32, size=n_random, dtype=np.uint64).astype(np.uint32)
    pos = np.concatenate([grid, dense, rnd & 0x7fffffff])
    return np.concatenate([pos, pos | 0x80000000]).astype(np.uint32)


# ---------------------------------------------------------------------------------- fp16

def test_f16_reference_unit_test_vectors(orc):
    g = GOLD["float16_values"]
    for fbits, hbits in g["f32_bits_to_f16_bits"]:
        x = np.array([int(fbits, 16)], dtype=np.uint32).view(np.float32)
        assert int(orc.f32_to_f16(x)[0]) == int(hbits, 16), fbits
    for val, hbits in g["double_to_f16_bits"]:
        got = int(orc.f32_to_f16(np.array([np.float32(val)]))[0])
        assert got == int(hbits, 16), (val, hex(got))
    assert int(orc.f32_to_f16(np.array([np.inf], np.float32))[0]) == 0x7c00
    assert int(orc.f32_to_f16(np.array([-np.inf], np.float32))[0]) == 0xfc00
    for nan_bits in (0x7fc00000, 0x7f800001, 0xffc00000, 0x7fa00000):
        h = int(orc.f32_to_f16(np.array([nan_bits], np.uint32).view(np.float32))[0])
        assert (h & 0x7fff) > 0x7c00  # std::isnan(float16)


def test_f16_widening_all_values_vs_numpy(orc):
    h = np.arange(65536, dtype=np.uint16)
    got = orc.f16_to_f32(h)
    want = h.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
    assert np.all(np.isnan(got[nan]))
    # round trip through the narrowing is the identity on every non-NaN half
    back = orc.f32_to_f16(got)
    assert np.array_equal(back[~nan], h[~nan])


def test_f16_narrowing_vs_numpy_rne(orc):
    rng = np.random.default_rng(1)
    bits = _interesting_f32(rng)
    x = bits.view(np.float32)
    got = orc.f32_to_f16(x)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    nan = np.isnan(x)
    # The reference's constructor doubles |v| < 2^-15 whose mantissa is >= 0x7ff000 before rounding
    # (float16.cpp:74-107, the exponent bump of the first rounding leaks into the subnormal branch);
    # everywhere else it is plain IEEE round-to-nearest-even.  fp32 subnormal inputs give zero,
    # which is also what RNE gives.
    e = (bits >> 23) & 0xff
    quirk = (e >= 1) & (e <= 111) & ((bits & 0x7fffff) >= 0x7ff000)
    ok = ~nan & ~quirk
    assert np.array_equal(got[ok], want[ok])
    with np.errstate(over="ignore"):
        want2 = (x[quirk] * np.float32(2)).astype(np.float16).view(np.uint16)
    assert np.array_equal(got[quirk], want2)


def test_f16_matches_compiled_reference(orc):
    ref = orc.ref_lib()
    if ref is None:
        pytest.skip("oracle/_ref not built (reference checkout absent)")
    import ctypes as C
    rng = np.random.default_rng(2)
    bits = _interesting_f32(rng)
    x = np.ascontiguousarray(bits.view(np.float32))
    want = np.empty(x.size, dtype=np.uint16)
    ref.ref_f32_to_f16_array(x.ctypes.data_as(C.c_void_p), want.ctypes.data_as(C.c_void_p), C.c_size_t(x.size))
    got = orc.f32_to_f16(x)
    assert np.array_equal(got, want)  # bit-exact, NaN payloads included
    h = np.arange(65536, dtype=np.uint16)
    wf = np.empty(65536, dtype=np.float32)
    ref.ref_f16_to_f32_array(h.ctypes.data_as(C.c_void_p), wf.ctypes.data_as(C.c_void_p), C.c_size_t(65536))
    assert np.array_equal(orc.f16_to_f32(h).view(np.uint32), wf.view(np.uint32))
    # float16 operator+ of the reference against the oracle's eltwise add
    a = rng.integers(0, 65536, size=200000).astype(np.uint16)
    b = rng.integers(0, 65536, size=200000).astype(np.uint16)
    ws = np.empty(a.size, dtype=np.uint16)
    ref.ref_f16_add_array(a.ctypes.data_as(C.c_void_p), b.ctypes.data_as(C.c_void_p), ws.ctypes.data_as(C.c_void_p),
                          C.c_size_t(a.size))
    gs = orc.eltwise_f16("add", a, b)
    nan = (ws & 0x7fff) > 0x7c00
    assert np.array_equal(gs[~nan], ws[~nan])
    assert np.all((gs[nan] & 0x7fff) > 0x7c00)


# ---------------------------------------------------------------------------------- quantize / dequantize / FQ

def test_dequantize_golden(orc):
    g = GOLD["dequantize"]
    q = np.array(g["q"], dtype=np.int8)
    y = orc.dequantize(q, g["scale"], g["zero_point"], to_f16=False)
    np.testing.assert_allclose(y, np.array(g["expected"], np.float32), rtol=4e-7)  # EXPECT_FLOAT_EQ = 4 ulp


def test_quantize_golden(orc):
    g = GOLD["quantize"]
    x = np.array(g["x"], dtype=np.float32)
    q = orc.quantize(x, g["scale"], g["zero_point"], signed=True, qmin=g["qmin"], qmax=g["qmax"])
    assert q.tolist() == g["expected"]


def test_quantize_per_axis_golden(orc):
    g = GOLD["quantize_per_axis"]
    x = np.array([g["x_row"], g["x_row"]], dtype=np.float32)
    q = orc.quantize(x, g["scales"], g["zero_points"], signed=True, qmin=g["qmin"], qmax=g["qmax"], axis=0)
    assert q.tolist() == g["expected"]


def test_dequantize_quantize_round_trip(orc):
    g = GOLD["dequantize_quantize_roundtrip"]
    q = np.array(g["q"], dtype=np.int8)
    x = orc.dequantize(q, g["scale"], g["zero_point"], to_f16=False)
    back = orc.quantize(x, g["scale"], g["zero_point"], signed=True, qmin=g["qmin"], qmax=g["qmax"])
    assert back.tolist() == g["q"]
    # full storage range, several types
    for signed, zp, scale in ((True, 0, 0.05), (True, -21, 0.003), (False, 128, 0.02), (False, 3, 1.0 / 255)):
        allq = np.arange(-128, 128, dtype=np.int8) if signed else np.arange(0, 256, dtype=np.uint8)
        x = orc.dequantize(allq, scale, zp, to_f16=False)
        assert np.array_equal(orc.quantize(x, scale, zp, signed=signed), allq)


def test_fake_quantize_properties(orc):
    L = orc.lib()
    # exact tie: x = 0 with limits +-4 and 256 levels sits at 127.5 -> rounds away from zero to level 128
    want = np.float32(128.0) / np.float32(255.0) * np.float32(8.0) + np.float32(-4.0)
    assert L.orc_fake_quantize(0.0, -4.0, 4.0, -4.0, 4.0, 256.0) == pytest.approx(float(want), abs=0)
    assert L.orc_fake_quantize(-4.0, -4.0, 4.0, -1.0, 1.0, 256.0) == -1.0   # x <= in_lo
    assert L.orc_fake_quantize(4.0001, -4.0, 4.0, -1.0, 1.0, 256.0) == 1.0  # x > in_hi
    assert L.orc_fake_quantize(4.0, -4.0, 4.0, -1.0, 1.0, 256.0) == 1.0     # top level
    rng = np.random.default_rng(3)
    x = np.clip(rng.normal(0, 1.5, 20000), -6, 6).astype(np.float32)
    xh = orc.f32_to_f16(x)
    lim = lambda v: orc.f32_to_f16(np.array([v], np.float32)).reshape(1)
    y = orc.fake_quantize_f16(xh, lim(-4), lim(4), lim(-4), lim(4), 256)
    yf = orc.f16_to_f32(y).astype(np.float64)
    # outputs lie on the 256-level grid (after fp16 rounding), are monotone in x and idempotent
    k = np.round((yf + 4.0) / 8.0 * 255.0)
    grid = orc.f16_to_f32(orc.f32_to_f16((k / 255.0 * 8.0 - 4.0).astype(np.float32)))
    assert np.max(np.abs(grid - yf)) <= 2 ** -8  # within one fp16 ulp at |y| < 4
    order = np.argsort(orc.f16_to_f32(xh), kind="stable")
    assert np.all(np.diff(yf[order]) >= 0)
    y2 = orc.fake_quantize_f16(y, lim(-4), lim(4), lim(-4), lim(4), 256)
    assert np.max(np.abs(orc.f16_to_f32(y2) - orc.f16_to_f32(y))) <= 2 ** -8
    # per-channel limits broadcast like numpy
    xc = orc.f32_to_f16(rng.normal(0, 2, (2, 3, 4, 5)).astype(np.float32))
    lo = orc.f32_to_f16(np.array([-1, -2, -3], np.float32)).reshape(1, 3, 1, 1)
    hi = orc.f32_to_f16(np.array([1, 2, 3], np.float32)).reshape(1, 3, 1, 1)
    yc = orc.fake_quantize_f16(xc, lo, hi, lo, hi, 16)
    for c in range(3):
        yc_c = orc.fake_quantize_f16(xc[:, c], lo[:, c].reshape(1), hi[:, c].reshape(1), lo[:, c].reshape(1),
                                     hi[:, c].reshape(1), 16)
        assert np.array_equal(yc[:, c], yc_c)


# ---------------------------------------------------------------------------------- softmax / MVN

def test_softmax_closed_forms(orc):
    rng = np.random.default_rng(4)
    x = rng.normal(0, 3, (7, 33, 19)).astype(np.float32)
    for axis in (0, 1, 2):
        y = orc.softmax_f32(x, axis)
        np.testing.assert_allclose(y.sum(axis=axis), 1.0, rtol=2e-6)
        # fp64 brute force
        xd = x.astype(np.float64)
        e = np.exp(xd - xd.max(axis=axis, keepdims=True))
        np.testing.assert_allclose(y, e / e.sum(axis=axis, keepdims=True), rtol=3e-6, atol=1e-30)
        # shift invariance
        y2 = orc.softmax_f32(x + np.float32(5.0), axis)
        np.testing.assert_allclose(y2, y, rtol=2e-5)
    # all-equal row -> 1/n exactly representable for n = 512
    eq = orc.softmax_f16(orc.f32_to_f16(np.full((3, 512), 1.25, np.float32)), 1)
    assert np.all(eq == orc.f32_to_f16(np.array([1.0 / 512], np.float32))[0])
    # masked entries (-60000) come out as exact zeros, the rest renormalises
    xm = rng.normal(0, 3, (4, 512)).astype(np.float32)
    mask = rng.random((4, 512)) < 0.05
    xm[mask] = -60000.0
    ym = orc.softmax_f16(orc.f32_to_f16(xm), 1)
    assert np.all(ym[mask] == 0)
    np.testing.assert_allclose(orc.f16_to_f32(ym).sum(axis=1), 1.0, atol=2e-3)
    # padding: trailing entries ignored and zeroed
    yp = orc.softmax_f32(x, 2, pad=4)
    assert np.all(yp[..., -4:] == 0)
    np.testing.assert_allclose(yp[..., :-4], orc.softmax_f32(np.ascontiguousarray(x[..., :-4]), 2), rtol=1e-6)


def test_mvn_closed_forms(orc):
    rng = np.random.default_rng(5)
    x = (rng.uniform(-8, 8, (2, 6, 5, 7)) + rng.normal(0, 2, (1, 6, 1, 1))).astype(np.float32)
    xh = orc.f32_to_f16(x)
    xd = orc.f16_to_f32(xh).astype(np.float64)
    for across in (True, False):
        for nv in (True, False):
            y = orc.f16_to_f32(orc.mvn_f16(xh, across, nv, 1e-9)).astype(np.float64)
            ax = (1, 2, 3) if across else (2, 3)
            mean = xd.mean(axis=ax, keepdims=True)
            var = ((xd - mean) ** 2).mean(axis=ax, keepdims=True)
            want = (xd - mean) / np.sqrt(var + 1e-9) if nv else xd - mean
            np.testing.assert_allclose(y, want, rtol=1e-3, atol=2e-3)
            assert np.max(np.abs(y.mean(axis=ax))) < 2e-3
            if nv:
                np.testing.assert_allclose(y.var(axis=ax), 1.0, rtol=5e-3)
    # constant input -> zeros (eps keeps the division finite)
    c = orc.f32_to_f16(np.full((1, 2, 3, 4), 3.5, np.float32))
    assert np.all(orc.mvn_f16(c, True, True, 1e-9) == 0)
    # NHWC memory layout gives the same numbers as NCHW on the transposed tensor
    xn = np.ascontiguousarray(xh.transpose(0, 2, 3, 1))
    for across in (True, False):
        y1 = orc.mvn_f16(xh, across, True, 1e-9)
        y2 = orc.mvn_f16(xn, across, True, 1e-9, layout="NHWC")
        assert np.array_equal(y2, np.ascontiguousarray(y1.transpose(0, 2, 3, 1)))


# ---------------------------------------------------------------------------------- integer path

def test_approximate_goldens(orc):
    for c in GOLD["approximate"]["cases"]:
        m, s, p = orc.approximate(c["bits"], c["target"])
        assert (m, s, p) == (c["mult"], c["shift"], 0), c
    # multiplier range and reconstruction error of the 15-bit form
    rng = np.random.default_rng(6)
    for t in np.exp(rng.uniform(np.log(1e-9), np.log(100.0), 300)):
        m, s, p = orc.approximate(15, float(t))
        assert 2 ** 14 <= m < 2 ** 15 and p == 0
        assert 0 <= t - m * 2.0 ** -s < t * 2.0 ** -14


def test_weight_table_word(orc):
    import ctypes as C
    L = orc.lib()
    for mult, shift in ((16384, 20), (32767, 24), (-19219, 31), (1, 0), (-32768, 63)):
        w = orc.wt_pack_scale(shift, mult)
        assert w == np.int32(np.uint32(((mult & 0xffff) << 16) | (shift << 8)))
        m, s = C.c_int32(), C.c_int32()
        L.orc_wt_unpack_scale(C.c_int32(w), C.byref(m), C.byref(s))
        assert (m.value, s.value) == (mult, shift)


def _rne_shift_exact(t, s):
    """round_half_even(t / 2^s) with Python integers and fractions."""
    from fractions import Fraction
    if s <= 0:
        return t
    fr = Fraction(t, 1 << s)
    fl = math.floor(fr)
    rem = fr - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        fl += 1
    return fl


def test_ppe_requant_properties(orc):
    rng = np.random.default_rng(7)
    noop = orc.ppe(1, 0, 0, -(2 ** 31), 2 ** 31 - 1)
    # zero shift, unit multiplier: identity (plus bias)
    for acc in (-5, 0, 7, 2 ** 30, -(2 ** 30)):
        assert orc.ppe_requant(acc, 3, 1, 0, noop) == acc + 3
    # ties go to even, on both signs
    for acc, want in ((1, 0), (3, 2), (5, 2), (7, 4), (-1, 0), (-3, -2), (-5, -2), (6, 3), (-6, -3)):
        assert orc.ppe_requant(acc, 0, 1, 1, noop) == want, acc
    # exact-arithmetic cross-check, including LeakyReLU parameters and big shifts
    lrelu = orc.ppe(1638, 14, 3, -128, 127)
    for _ in range(3000):
        acc = int(rng.integers(-2 ** 31, 2 ** 31))
        bias = int(rng.integers(-2 ** 15, 2 ** 15))
        mult = int(rng.integers(2 ** 14, 2 ** 15))
        shift = int(rng.integers(0, 50))
        for p, pm, ps, zp, lo, hi in ((noop, 1, 0, 0, -(2 ** 31), 2 ** 31 - 1), (lrelu, 1638, 14, 3, -128, 127)):
            biased = (acc + bias + 2 ** 31) % 2 ** 32 - 2 ** 31
            t = biased * mult
            s = shift
            if t < 0:
                t *= pm
                s += ps
            want = min(max(_rne_shift_exact(t, s) + zp, lo), hi)
            assert orc.ppe_requant(acc, bias, mult, shift, p) == want
    # monotone in acc for a positive multiplier; clamp saturates; relu (prelu_mult 0) zeroes negatives
    accs = np.sort(rng.integers(-10 ** 6, 10 ** 6, 500))
    outs = [orc.ppe_requant(int(a), 0, 20000, 22, lrelu) for a in accs]
    assert all(b >= a for a, b in zip(outs, outs[1:]))
    assert orc.ppe_requant(2 ** 30, 0, 32767, 0, orc.ppe(1, 0, 0, 0, 255)) == 255
    relu = orc.ppe(0, 0, 0, -128, 127)
    assert orc.ppe_requant(-123456, 0, 20000, 10, relu) == 0
    # LeakyReLU slope is 1638/16384 of the positive slope
    wide = orc.ppe(1638, 14, 3, -2 ** 31, 2 ** 31 - 1)
    pos = orc.ppe_requant(10 ** 6, 0, 16384, 14, wide) - 3
    neg = orc.ppe_requant(-10 ** 6, 0, 16384, 14, wide) - 3
    assert abs(neg / pos + 1638 / 16384) < 1e-5


def _f16_bits_of_fixed(fx):
    """fx * 2^-15 narrowed to fp16 by numpy: the value is exact in a double, so this is one round-to-nearest-even."""
    with np.errstate(over="ignore"):
        return int(np.array([fx / 32768.0], dtype=np.float64).astype(np.float16).view(np.uint16)[0])


def test_ppe_requant_f16_fixed_point_conversion(orc):
    """acc with multiplier 1 and shift 15 is the s17.15 number itself: the conversion alone, against numpy."""
    none = orc.ppe(1, 0, 0, -(2 ** 31), 2 ** 31 - 1)
    rng = np.random.default_rng(17)
    cases = list(range(-70000, 70001, 1))
    # every 11-bit significand boundary: ties and their neighbours at each magnitude, both signs
    for top in range(11, 31):
        step = 1 << (top - 10)
        for q in (1 << 10, (1 << 10) + 1, (1 << 11) - 2, (1 << 11) - 1):
            base = q * step
            for d in (-1, 0, 1, step // 2 - 1, step // 2, step // 2 + 1, step - 1):
                cases += [base + d, -(base + d)]
    cases += [2 ** 31 - 1, -(2 ** 31), 65519 * 32768 + 16384, 65520 * 32768, 65504 * 32768, 1, -1, 2, 3, 0]
    cases += [int(v) for v in rng.integers(-2 ** 31, 2 ** 31, 20000)]
    for fx in cases:
        if not -(2 ** 31) <= fx < 2 ** 31:
            continue
        assert orc.ppe_requant_f16(fx, 0, 1, 15, none) == _f16_bits_of_fixed(fx), fx
    assert orc.ppe_requant_f16(1, 0, 1, 15, none) == 0x0200          # 2^-15 is a subnormal half
    assert orc.ppe_requant_f16(65520 * 32768, 0, 1, 15, none) == 0x7c00  # rounds to infinity
    assert orc.ppe_requant_f16(-32768, 0, 1, 15, none) == 0xbc00      # -1.0


def test_ppe_requant_f16_against_exact_arithmetic(orc):
    """Whole pipeline against exact rationals: scale, PReLU on negatives, one rounding to 15 fractional bits,
    saturation to 32 bits, narrowing, packed fp16 clamp."""
    rng = np.random.default_rng(18)
    none = orc.ppe(1, 0, 0, -(2 ** 31), 2 ** 31 - 1)
    lrelu = orc.ppe(1638, 14, 0, -(2 ** 31), 2 ** 31 - 1)
    relu = orc.ppe(0, 0, 0, -(2 ** 31), 2 ** 31 - 1)
    clamp = orc.ppe(0, 0, 0, -(2 ** 31), orc.pack_clamp_f16(20.0, 300.0))
    # the packed word of the reference's own test (ppe_factory_tests.cpp:781-791 unpacks it to 20.0 and 300.0)
    packed = orc.pack_clamp_f16(20.0, 300.0) & 0xffffffff
    assert (packed >> 16, packed & 0xffff) == (0x4d00, 0x5cb0)
    for it in range(6000):
        acc = int(rng.integers(-2 ** 31, 2 ** 31)) if it % 3 else int(rng.integers(-2 ** 16, 2 ** 16))
        bias = int(rng.integers(-2 ** 15, 2 ** 15))
        mult = int(rng.integers(2 ** 14, 2 ** 15)) * (1 if it % 7 else -1)
        shift = int(rng.integers(0, 50))
        for p, pm, ps in ((none, 1, 0), (lrelu, 1638, 14), (relu, 0, 0), (clamp, 0, 0)):
            biased = (acc + bias + 2 ** 31) % 2 ** 32 - 2 ** 31
            t = biased * mult
            s = shift
            if t < 0:
                t *= pm
                s += ps
            fx = Fraction(t * 2 ** 15, 2 ** s)
            fl = math.floor(fx)
            rem = fx - fl
            if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
                fl += 1
            fl = min(max(fl, -(2 ** 31)), 2 ** 31 - 1)
            want = _f16_bits_of_fixed(fl)
            if p is clamp:
                v = float(np.array([want], dtype=np.uint16).view(np.float16)[0])
                want = 0x4d00 if v < 20.0 else (0x5cb0 if v > 300.0 else want)
            assert orc.ppe_requant_f16(acc, bias, mult, shift, p) == want, (acc, bias, mult, shift, pm, ps)
    # the value is (acc + bias) * mult * 2^-shift: scale 0.5 (16384 / 2^15) of 6 is 3.0
    assert orc.ppe_requant_f16(6, 0, 16384, 15, none) == 0x4200
    # LeakyReLU 0.1 = 1638 / 2^14 on a negative value: -1000 * 0.5 * 0.0999755859375 = -49.98779296875 -> fp16
    assert orc.ppe_requant_f16(-1000, 0, 16384, 15, lrelu) == int(np.array([-49.98779296875]).astype(np.float16).view(np.uint16)[0])


def test_nce_matmul_f16_output_uses_the_fixed_point_path(orc):
    rng = np.random.default_rng(19)
    A = rng.integers(0, 256, (5, 48), dtype=np.uint8)
    B = rng.integers(-127, 128, (7, 48)).astype(np.int8)
    mults, shifts = rng.integers(2 ** 14, 2 ** 15, 7), rng.integers(14, 26, 7)
    bias = rng.integers(-2 ** 12, 2 ** 12, 7).astype(np.int32)
    wt = orc.make_weights_table(mults, shifts, bias, 48)
    p = orc.ppe(1638, 14, 0, -(2 ** 31), 2 ** 31 - 1)
    out, acc = orc.nce_matmul(A, B, wt, p, zp_a=128, want_acc=True, out_f16=True)
    assert out.dtype == np.uint16 and out.shape == (5, 7)
    ref_acc = (A.astype(np.int64) - 128) @ B.astype(np.int64).T
    assert np.array_equal(acc, ref_acc)
    for m in range(5):
        for n in range(7):
            assert out[m, n] == orc.ppe_requant_f16(int(acc[m, n]), int(bias[n]), int(mults[n]), int(shifts[n]), p)


def test_nce_conv_against_brute_force(orc):
    import torch
    rng = np.random.default_rng(8)
    N, H, W, IC, OC, KY, KX = 2, 7, 6, 16, 5, 3, 3
    inp = rng.integers(0, 256, (N, H, W, IC), dtype=np.uint8)
    w = rng.integers(-127, 128, (OC, KY, KX, IC)).astype(np.int8)
    mults = rng.integers(2 ** 14, 2 ** 15, OC)
    shifts = rng.integers(12, 16, OC)
    bias = rng.integers(-2 ** 15, 2 ** 15, OC).astype(np.int32)
    wt = orc.make_weights_table(mults, shifts, bias, KY * KX * IC)
    p = orc.ppe(1, 0, 0, 0, 255)
    for strides, pads in (((1, 1), (1, 1, 1, 1)), ((2, 2), (0, 1, 1, 0)), ((1, 2), (0, 0, 0, 0))):
        out, acc = orc.nce_conv(inp, w, wt, p, zp_in=128, strides=strides, pads=pads, want_acc=True)
        # independent integer reference: zero padding in the real domain == padding (in - zp) with 0
        xi = torch.from_numpy(inp.astype(np.int64) - 128).permute(0, 3, 1, 2)
        xi = torch.nn.functional.pad(xi, (pads[1], pads[3], pads[0], pads[2]))
        wi = torch.from_numpy(w.astype(np.int64)).permute(0, 3, 1, 2)
        ref = torch.nn.functional.conv2d(xi.double(), wi.double(), stride=strides).permute(0, 2, 3, 1).numpy()
        assert np.array_equal(acc.astype(np.float64), ref)
        want = np.empty_like(out)
        for idx in np.ndindex(*acc.shape):
            oc = idx[3]
            want[idx] = orc.ppe_requant(int(acc[idx]), int(bias[oc]), int(mults[oc]), int(shifts[oc]), p)
        assert np.array_equal(out, want)
    # matmul form with an asymmetric activation zero point
    A = rng.integers(-128, 128, (9, 32)).astype(np.int8)
    B = rng.integers(-127, 128, (11, 32)).astype(np.int8)
    wt2 = orc.make_weights_table([20000] * 11, [10] * 11, [0] * 11, 32)
    out, acc = orc.nce_matmul(A, B, wt2, orc.ppe(1638, 14, 0, -128, 127), zp_a=3, want_acc=True)
    assert np.array_equal(acc, (A.astype(np.int64) - 3) @ B.astype(np.int64).T)
    # row-range evaluation equals the full evaluation on those rows
    part = orc.nce_matmul(A, B, wt2, orc.ppe(1638, 14, 0, -128, 127), zp_a=3, rows=(2, 4))
    assert np.array_equal(part[2:6], out[2:6])


def test_nce_operands_as_views_of_larger_tensors(orc):
    """Strided operands: the result on views equals the dense result on packed copies, and nothing outside the
    output view is written."""
    rng = np.random.default_rng(9)
    N, H, W, IC, OC, KY, KX = 2, 7, 6, 16, 5, 3, 3
    parent = rng.integers(0, 256, (N, H + 3, W + 4, IC + 7), dtype=np.uint8)
    inp = parent[:, 2:2 + H, 1:1 + W, 3:3 + IC]
    w = rng.integers(-127, 128, (OC, KY, KX, IC)).astype(np.int8)
    wt = orc.make_weights_table(rng.integers(2 ** 14, 2 ** 15, OC), rng.integers(12, 16, OC), rng.integers(-2 ** 15, 2 ** 15, OC).astype(np.int32),
                                KY * KX * IC)
    p = orc.ppe(1638, 14, 2, 0, 255)
    for out_f16 in (False, True):
        dense = orc.nce_conv(np.ascontiguousarray(inp), w, wt, p, zp_in=128, strides=(2, 1), pads=(1, 1, 0, 1), out_f16=out_f16)
        oparent = np.full((N, dense.shape[1] + 2, dense.shape[2] + 3, OC + 9), 99, dtype=dense.dtype)
        oview = oparent[:, 1:1 + dense.shape[1], 2:2 + dense.shape[2], 4:4 + OC]
        got = orc.nce_conv(inp, w, wt, p, zp_in=128, strides=(2, 1), pads=(1, 1, 0, 1), out_f16=out_f16, out=oview)
        assert got is oview and np.array_equal(oview, dense)
        mask = np.ones(oparent.shape, bool)
        mask[:, 1:1 + dense.shape[1], 2:2 + dense.shape[2], 4:4 + OC] = False
        assert (oparent[mask] == 99).all()
    # eltwise
    a = parent[:, 0:H, 0:W, 0:IC].view(np.int8)
    b = parent[:, 1:1 + H, 2:2 + W, 5:5 + IC]
    pe = orc.ppe(1638, 14, 3, -128, 127)
    for out_f16 in (False, True):
        dense = orc.nce_eltwise(np.ascontiguousarray(a), np.ascontiguousarray(b), pe, 3, 120, 11000, 9000, 17000, 28, subtract=True,
                                out_signed=True, out_f16=out_f16)
        oparent = np.full((N, H + 1, W + 2, IC + 3), 99, dtype=dense.dtype)
        oview = oparent[:, 1:, 1:1 + W, 2:2 + IC]
        orc.nce_eltwise(a, b, pe, 3, 120, 11000, 9000, 17000, 28, subtract=True, out_signed=True, out_f16=out_f16, out=oview)
        assert np.array_equal(oview, dense)
        mask = np.ones(oparent.shape, bool)
        mask[:, 1:, 1:1 + W, 2:2 + IC] = False
        assert (oparent[mask] == 99).all()


def test_nce_eltwise_against_exact_integers_and_real_arithmetic(orc):
    """The eltwise restatement against Python integers (round half even with fractions) and, loosely,
    against the real-valued sum it approximates; multipliers from the reference's golden case
    (tests/unit/vpux_compiler/utils/quantization_tests.cpp style: scales 0.02 / 0.035 -> 0.05)."""
    from fractions import Fraction
    rng = np.random.default_rng(90)
    a = rng.integers(0, 256, 4000, dtype=np.uint8)
    b = rng.integers(-128, 128, 4000).astype(np.int8)
    s1, s2, so = 0.02, 0.035, 0.05
    m1, sh1, _ = orc.approximate(15, s1)
    m2, sh2, _ = orc.approximate(15, s2)
    mo, sho, _ = orc.approximate(15, 1.0 / so)
    shift_in = max(sh1, sh2)
    m1a, m2a = m1 << (shift_in - sh1), m2 << (shift_in - sh2)
    assert m1a < 65536 and m2a < 65536
    zp_a, zp_b, zp_o = 128, -3, 7
    for subtract in (False, True):
        p = orc.ppe(1, 0, zp_o, 0, 255)
        got = orc.nce_eltwise(a, b, p, zp_a, zp_b, m1a, m2a, mo, sho + shift_in, subtract=subtract)
        sign = -1 if subtract else 1
        want = np.empty_like(got)
        real = np.empty(a.size)
        for i in range(a.size):
            acc = (int(a[i]) - zp_a) * m1a + sign * (int(b[i]) - zp_b) * m2a
            t = Fraction(acc * mo, 1 << (sho + shift_in))
            r = round(t)  # Python rounds halves to even
            want[i] = min(255, max(0, r + zp_o))
            real[i] = ((int(a[i]) - zp_a) * s1 + sign * (int(b[i]) - zp_b) * s2) / so + zp_o
        assert np.array_equal(got, want)
        unsat = (real > 1) & (real < 254)
        assert np.abs(got[unsat].astype(np.float64) - real[unsat]).max() <= 1.0


# ---------------------------------------------------------------------------------- activations

def _activation_fp64(op, x, p0, p1):
    """Independent evaluation in fp64 with numpy / scipy (not a retyping of the oracle's branches where a
    smooth closed form exists)."""
    from scipy import special
    x = x.astype(np.float64)
    with np.errstate(all="ignore"):
        return {
            "relu": lambda: np.maximum(x, 0.0),
            "leaky_relu": lambda: np.where(x < 0, x * np.float64(np.float32(p0)), x),
            "clamp": lambda: np.clip(x, np.float32(p0), np.float32(p1)),
            "negative": lambda: -x,
            "abs": lambda: np.abs(x),
            "hswish": lambda: x * np.clip(x + 3.0, 0.0, 6.0) / 6.0,
            "hsigmoid": lambda: np.clip(x + 3.0, 0.0, 6.0) / 6.0,
            "hardsigmoid": lambda: np.clip(np.float64(np.float32(p0)) * x + np.float64(np.float32(p1)), 0.0, 1.0),
            "sigmoid": lambda: special.expit(x),
            "tanh": lambda: np.tanh(x),
            "exp": lambda: np.exp(x),
            "sqrt": lambda: np.sqrt(x),
            "log": lambda: np.log(x),
            "floor": lambda: np.floor(x),
            "ceil": lambda: np.ceil(x),
            "sign": lambda: np.sign(x),
            "elu": lambda: np.where(x < 0, np.float64(np.float32(p0)) * np.expm1(x), x),
            "selu": lambda: np.float64(np.float32(p1)) * np.where(x > 0, x, np.float64(np.float32(p0)) * np.expm1(x)),
            "swish": lambda: x * special.expit(np.float64(np.float32(p0)) * x),
            "mish": lambda: x * np.tanh(np.logaddexp(0.0, x)),
            "softplus": lambda: np.logaddexp(0.0, x),
            "gelu": lambda: x * special.ndtr(x),
            "erf": lambda: special.erf(x),
        }[op]()


ACT_CASES = [("relu", ()), ("leaky_relu", (0.1,)), ("clamp", (-1.5, 6.0)), ("negative", ()), ("abs", ()), ("hswish", ()),
             ("hsigmoid", ()), ("hardsigmoid", (0.2, 0.5)), ("sigmoid", ()), ("tanh", ()), ("exp", ()), ("sqrt", ()),
             ("log", ()), ("floor", ()), ("ceil", ()), ("sign", ()), ("elu", (1.0,)), ("selu", (1.67326, 1.0507)),
             ("swish", (1.0,)), ("mish", ()), ("softplus", ()), ("gelu", ()), ("erf", ())]
ACT_EXACT = {"relu", "leaky_relu", "clamp", "negative", "abs", "hsigmoid", "hardsigmoid", "floor", "ceil", "sign", "sqrt"}


def f16_ulp_distance(a_bits, b_bits):
    """Distance in representable fp16 values (sign-magnitude folded onto a line)."""
    def line(b):
        b = b.astype(np.int32)
        return np.where(b & 0x8000, -(b & 0x7fff), b & 0x7fff)
    return np.abs(line(a_bits) - line(b_bits))


@pytest.mark.parametrize("op,params", ACT_CASES, ids=[c[0] for c in ACT_CASES])
def test_activation_every_f16_value_against_fp64(orc, op, params):
    h = np.arange(65536, dtype=np.uint16)
    h = h[(h & 0x7fff) <= 0x7c00]  # drop NaNs
    p = tuple(params) + (0.0,) * (2 - len(params))
    got = orc.activation_f16(op, h, *p)
    x = orc.f16_to_f32(h)
    want64 = _activation_fp64(op, x, *p)
    # the fp64 result narrowed fp64 -> fp32 -> fp16 with the float16 class's own rounding (pinned by the
    # float16 tests above), so only the activation arithmetic is under test here
    with np.errstate(all="ignore"):
        want = orc.f32_to_f16(want64.astype(np.float32))
    nan = np.isnan(want64)
    assert np.array_equal(((got & 0x7fff) > 0x7c00), nan)
    ok = ~nan
    d = f16_ulp_distance(got[ok], want[ok])
    # one step where fp32 arithmetic and the fp64 evaluation fall on different sides of a rounding
    # boundary; below 2^-14 the float16 class doubles some magnitudes (float16.cpp:74-107), which turns
    # such a difference into a factor of two there
    tiny = np.abs(want64[ok]) < 2.0 ** -14
    if op in ACT_EXACT:
        assert d.max() == 0, (op, d.max())
    assert d[~tiny].max() <= 1, (op, d[~tiny].max(), h[ok][~tiny][np.argmax(d[~tiny])])


def test_activation_special_values(orc):
    f = lambda v: orc.f32_to_f16(np.asarray(v, dtype=np.float32))
    val = lambda op, v, *p: orc.f16_to_f32(orc.activation_f16(op, f(v), *p))
    assert val("relu", [-1.0, -0.0, 0.0, 2.5]).tolist() == [0.0, 0.0, 0.0, 2.5]
    assert val("clamp", [-9.0, 0.25, 9.0], -1.0, 6.0).tolist() == [-1.0, 0.25, 6.0]
    assert val("leaky_relu", [-2.0, 3.0], 0.25).tolist() == [-0.5, 3.0]
    assert val("hswish", [-3.0, 0.0, 3.0, 6.0]).tolist() == [0.0, 0.0, 3.0, 6.0]
    assert val("hsigmoid", [-3.0, 0.0, 3.0]).tolist() == [0.0, 0.5, 1.0]
    assert val("sigmoid", [0.0]).tolist() == [0.5]
    assert val("exp", [0.0]).tolist() == [1.0]
    assert val("tanh", [0.0]).tolist() == [0.0]
    assert val("sign", [-4.0, 0.0, 7.0]).tolist() == [-1.0, 0.0, 1.0]
    assert val("erf", [0.0]).tolist() == [0.0]
    assert val("softplus", [0.0])[0] == np.float32(np.float16(np.log(2.0)))
    # prelu is the binary form of leaky relu
    a = f([-2.0, 3.0, -8.0])
    b = f([0.25, 0.25, 0.5])
    assert orc.f16_to_f32(orc.eltwise_f16("prelu", a, b)).tolist() == [-0.5, 3.0, -4.0]


# ---------------------------------------------------------------------------------- MVN decomposition, MVN-6

def test_mvn1_decomposition_hand_case_and_chain(orc):
    x = orc.f32_to_f16(np.array([1, 2, 3, 4, 10, 10, 10, 10], np.float32).reshape(1, 2, 2, 2))
    s = orc.mvn1_sum(x, False, True)
    assert s.shape == (1, 1, 2, 2) and s[0, 0].tolist() == [[10.0, 40.0], [30.0, 400.0]]
    assert orc.mvn1_sum(x, True, False)[0, 0].tolist() == [[50.0]]
    mv = orc.mvn1_mean_var(s, (1, 2, 2, 2), False, True, 0.0)
    assert mv[0, 0, 0].tolist() == [2.5, 10.0]
    assert mv[0, 0, 1, 0] == np.float32(1.0 / np.sqrt(1.25)) and np.isinf(mv[0, 0, 1, 1])
    mv = orc.mvn1_mean_var(s, (1, 2, 2, 2), False, True, 1e-2)
    y = orc.f16_to_f32(orc.mvn1_norm(x, mv, False, True))
    assert np.allclose(y[0, 0].ravel(), (np.array([1, 2, 3, 4]) - 2.5) / np.sqrt(1.25 + 1e-2), rtol=1e-3)
    assert np.all(y[0, 1] == 0)
    # pooled channel groups: two channels of one group share the statistics of their union
    mvg = orc.mvn1_mean_var(s, (1, 2, 2, 2), False, True, 0.0, group_c=2)
    assert mvg[0, 0, 0].tolist() == [6.25, 6.25]
    assert np.allclose(mvg[0, 0, 1], 1.0 / np.sqrt(430.0 / 8 - 6.25 ** 2))
    # partial sums split over parts add up
    two = np.concatenate([0.25 * s, 0.75 * s], axis=1)
    assert np.array_equal(orc.mvn1_mean_var(two, (1, 2, 2, 2), False, True, 1e-2), orc.mvn1_mean_var(s, (1, 2, 2, 2), False, True, 1e-2))
    # the three steps reproduce the one-kernel MVN (two-pass, double) on random data
    rng = np.random.default_rng(41)
    xr = orc.f32_to_f16((rng.normal(0, 2, (2, 5, 9, 7)) + rng.normal(0, 3, (1, 5, 1, 1))).astype(np.float32))
    for across in (False, True):
        for nv in (False, True):
            mv = orc.mvn1_mean_var(orc.mvn1_sum(xr, across, nv), xr.shape, across, nv, 1e-9)
            got = orc.f16_to_f32(orc.mvn1_norm(xr, mv, across, nv)).astype(np.float64)
            want = orc.f16_to_f32(orc.mvn_f16(xr, across, nv, 1e-9)).astype(np.float64)
            assert np.all(np.abs(got - want) <= 2e-3 * np.abs(want) + 1e-5), (across, nv)


def test_mvn6_against_mvn1_and_hand_cases(orc):
    rng = np.random.default_rng(42)
    x = orc.f32_to_f16(rng.normal(1, 2, (2, 5, 9, 7)).astype(np.float32))
    for axes, across in (((1, 2, 3), True), ((2, 3), False)):
        got = orc.f16_to_f32(orc.mvn6_f16(x, axes, True, 1e-6, 0)).astype(np.float64)
        want = orc.f16_to_f32(orc.mvn_f16(x, across, True, 1e-6)).astype(np.float64)
        assert np.all(np.abs(got - want) <= 1e-3 * np.abs(want) + 1e-6)
    row = orc.f32_to_f16(np.array([[1, 2, 3, 4]], np.float32))
    inside = orc.f16_to_f32(orc.mvn6_f16(row, (1,), True, 0.75, 0))[0]
    outside = orc.f16_to_f32(orc.mvn6_f16(row, (1,), True, 0.75, 1))[0]
    assert np.allclose(inside, (np.array([1, 2, 3, 4]) - 2.5) / np.sqrt(2.0), rtol=1e-3)          # var 1.25 + 0.75
    assert np.allclose(outside, (np.array([1, 2, 3, 4]) - 2.5) / (np.sqrt(1.25) + 0.75), rtol=1e-3)
    assert orc.f16_to_f32(orc.mvn6_f16(row, (1,), False, 0.75, 0))[0].tolist() == [-1.5, -0.5, 0.5, 1.5]
    sc = orc.f32_to_f16(np.array([[2, 2, 0, -1]], np.float32))
    bi = orc.f32_to_f16(np.array([[1]], np.float32))
    assert orc.f16_to_f32(orc.mvn6_f16(row, (1,), False, 0.0, 0, sc, bi))[0].tolist() == [-2.0, 0.0, 1.0, -0.5]


def test_dynamic_dequantize_matches_static_golden_and_broadcasts(orc):
    q = np.array([[-127, 0, 127]], np.int8)
    y = orc.f16_to_f32(orc.dynamic_dequantize(q, np.array([[2.0 / 254.0]], np.float32)))
    assert y.tolist() == [[-1.0, 0.0, 1.0]]                       # content_tests.cpp:754-788 through the tensor-scale form
    q = np.arange(-6, 6, dtype=np.int8).reshape(3, 4)
    sc = np.array([[0.5], [2.0], [0.25]], np.float32)
    zp = np.array([[1], [0], [-2]], np.int8)
    want = (q.astype(np.float64) - zp) * sc
    assert np.array_equal(orc.f16_to_f32(orc.dynamic_dequantize(q, sc, zp)), want.astype(np.float32))
    assert np.array_equal(orc.dynamic_dequantize(q, sc, zp, to_f16=False), want.astype(np.float32))
    # the same numbers as the static per-axis dequantize when scale and zero point are per row
    stat = orc.dequantize(q, sc.ravel().astype(np.float64), zp.ravel().astype(np.int64), to_f16=True, axis=0)
    assert np.array_equal(orc.dynamic_dequantize(q, sc, zp), stat)


def test_dynamic_quantize_onnx_examples(orc):
    """The three worked examples of the ONNX DynamicQuantizeLinear specification."""
    y, sc, zp = orc.dynamic_quantize(np.array([0, 2, -3, -2.5, 1.34, 0.5], np.float32))
    assert np.isclose(sc, 0.0196078438) and zp == 153 and y.tolist() == [153, 255, 0, 26, 221, 179]
    y, sc, zp = orc.dynamic_quantize(np.array([-1.0, -2.1, -1.3, -2.5, -3.34, -4.0], np.float32))
    assert np.isclose(sc, 0.0156862754) and zp == 255 and y.tolist() == [191, 121, 172, 96, 42, 0]
    y, sc, zp = orc.dynamic_quantize(np.array([1, 2.1, 1.3, 2.5, 3.34, 4.0, 1.5, 2.6, 3.9, 4.0, 3.0, 2.345], np.float32).reshape(3, 4))
    assert np.isclose(sc, 0.0156862754) and zp == 0
    assert y.ravel().tolist() == [64, 134, 83, 159, 213, 255, 96, 166, 249, 255, 191, 149]
    y, sc, zp = orc.dynamic_quantize(np.zeros(5, np.float32))
    assert sc == 1.0 and zp == 0 and not y.any()
    # round trip: dequantized values are within half a step of the input
    rng = np.random.default_rng(71)
    x = rng.normal(0.3, 2, 10000).astype(np.float32)
    y, sc, zp = orc.dynamic_quantize(x)
    back = orc.dynamic_dequantize(y, np.full((1,), sc, np.float32), np.full((1,), zp, np.uint8), to_f16=False)
    assert np.all(np.abs(back - x) <= 0.5 * sc * (1 + 1e-5))



def test_eltwise_min_max_special_values(orc):
    """Minimum / Maximum are IEEE minNum / maxNum with -0 below +0 (written out here case by case, not through the
    C library): a NaN operand yields the other operand, two NaNs a NaN, and equal-comparing zeros keep the sign the
    ordering asks for."""
    nan, pz, nz, inf, ninf, one, mone = 0x7e00, 0x0000, 0x8000, 0x7c00, 0xfc00, 0x3c00, 0xbc00
    a = np.array([nan, one, nan, pz, nz, inf, ninf, one, nz, pz], np.uint16)
    b = np.array([one, nan, nan, nz, pz, one, one, mone, nz, pz], np.uint16)
    mn = orc.eltwise_f16("min", a, b)
    mx = orc.eltwise_f16("max", a, b)
    assert mn[:2].tolist() == [one, one] and mx[:2].tolist() == [one, one]
    assert (mn[2] & 0x7fff) > 0x7c00 and (mx[2] & 0x7fff) > 0x7c00
    assert mn[3:].tolist() == [nz, nz, one, ninf, mone, nz, pz]
    assert mx[3:].tolist() == [pz, pz, inf, one, one, nz, pz]
