"""Parity of the HIP ACT-SHAVE kernels with the CPU oracle, through the C ABI, on a real MI355X.

Bars: convert / eltwise / fake_quantize / quantize / dequantize bit-exact (any NaN matches any NaN
where arithmetic produced it); softmax and MVN within relative 2e-3, or one fp16 subnormal step
(2^-24) in absolute terms for results that small."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

REL_TOL = 2e-3
ABS_FLOOR = 2.0 ** -24


def to_dev(bits_or_arr, dev, f16=False):
    import torch
    a = np.ascontiguousarray(bits_or_arr)
    if f16:
        a = a.view(np.float16)
    return torch.from_numpy(a).to(dev)


def f16_bits(t):
    return t.cpu().numpy().view(np.uint16)


def is_nan16(b):
    return (b & 0x7fff) > 0x7c00


def assert_f16_exact(got, want, what=""):
    nan = is_nan16(want)
    assert np.array_equal(is_nan16(got), nan), what
    bad = np.nonzero((got != want) & ~nan)[0] if got.ndim == 1 else np.argwhere((got != want) & ~nan)
    assert len(bad) == 0, "%s: %d mismatches, first at %s: got 0x%04x want 0x%04x" % (
        what, len(bad), bad[0], got[tuple(np.atleast_1d(bad[0]))], want[tuple(np.atleast_1d(bad[0]))])


def assert_close_f16(got_bits, want_bits, orc, what=""):
    g = orc.f16_to_f32(got_bits).astype(np.float64)
    w = orc.f16_to_f32(want_bits).astype(np.float64)
    nan = np.isnan(w)
    assert np.array_equal(np.isnan(g), nan), what
    err = np.abs(g - w)
    tol = np.maximum(REL_TOL * np.abs(w), ABS_FLOOR)
    bad = np.argwhere((err > tol) & ~nan)
    assert len(bad) == 0, "%s: %d outside tolerance, first %s got %r want %r" % (
        what, len(bad), bad[0], g[tuple(bad[0])], w[tuple(bad[0])])


# ---------------------------------------------------------------------------------- convert

def test_convert_f16_to_f32_every_value(rt, orc, dev):
    import torch
    h = np.arange(65536, dtype=np.uint16)
    x = to_dev(h, dev, f16=True)
    y = torch.empty(65536, dtype=torch.float32, device=dev)
    rt.convert(x, y)
    got = y.cpu().numpy()
    want = orc.f16_to_f32(h)
    nan = np.isnan(want)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
    assert np.all(np.isnan(got[nan]))


def test_convert_f32_to_f16_rounding_cases(rt, orc, dev):
    import torch
    from test_oracle import _interesting_f32
    bits = _interesting_f32(np.random.default_rng(21), n_random=3_000_001)  # odd count: ragged tail
    x = to_dev(bits.view(np.float32), dev)
    y = torch.empty(x.shape, dtype=torch.float16, device=dev)
    rt.convert(x, y)
    got = f16_bits(y)
    want = orc.f32_to_f16(bits.view(np.float32))
    assert np.array_equal(got, want)  # NaN payloads and the reference's subnormal doubling included


def test_convert_strided_view_and_4d(rt, orc, dev):
    import torch
    rng = np.random.default_rng(22)
    x = rng.normal(0, 100, (3, 5, 7, 12)).astype(np.float32)
    xd = to_dev(x, dev)
    y = torch.zeros((3, 5, 7, 12), dtype=torch.float16, device=dev)
    rt.convert(xd[:, :, 1:6, 2:9], y[:, :, 1:6, 2:9])  # sub-views with their own strides
    got = f16_bits(y)
    want = np.zeros_like(got)
    want[:, :, 1:6, 2:9] = orc.f32_to_f16(x[:, :, 1:6, 2:9])
    assert np.array_equal(got, want)
    empty = torch.empty((0, 4), dtype=torch.float32, device=dev)
    rt.convert(empty, torch.empty((0, 4), dtype=torch.float16, device=dev))


# ---------------------------------------------------------------------------------- eltwise

@pytest.mark.parametrize("op", ["add", "sub", "mul", "min", "max", "div"])
def test_eltwise_random_bit_patterns(rt, orc, dev, op):
    import torch
    rng = np.random.default_rng(23)
    n = 1_000_003
    a = rng.integers(0, 65536, n).astype(np.uint16)
    b = rng.integers(0, 65536, n).astype(np.uint16)
    if op in ("min", "max"):
        # every pairing of special values: NaN with a number (the number wins), NaN with NaN, zeros of both signs
        # (-0 is below +0), infinities
        sp = np.array([0x7e00, 0xfe00, 0x7c01, 0x0000, 0x8000, 0x7c00, 0xfc00, 0x3c00, 0xbc00, 0x0001, 0x8001], np.uint16)
        a[:sp.size ** 2] = np.repeat(sp, sp.size)
        b[:sp.size ** 2] = np.tile(sp, sp.size)
    out = torch.empty(n, dtype=torch.float16, device=dev)
    rt.eltwise(op, to_dev(a, dev, True), to_dev(b, dev, True), out)
    got, want = f16_bits(out), orc.eltwise_f16(op, a, b)
    if op in ("min", "max"):
        k = 11 * 11
        one_nan = is_nan16(a[:k]) ^ is_nan16(b[:k])
        other = np.where(is_nan16(a[:k]), b[:k], a[:k])
        assert np.array_equal(got[:k][one_nan], other[one_nan])  # a NaN operand yields the other operand
        assert is_nan16(got[:k][is_nan16(a[:k]) & is_nan16(b[:k])]).all()
        assert got[3 * 11 + 4] == (0x8000 if op == "min" else 0x0000) and got[4 * 11 + 3] == got[3 * 11 + 4]  # (+0, -0)
    assert_f16_exact(got, want, op)


def test_eltwise_add_broadcast_and_strides(rt, orc, dev):
    import torch
    rng = np.random.default_rng(24)
    a = orc.f32_to_f16(rng.normal(0, 1, (2, 6, 5, 8)).astype(np.float32))
    b = orc.f32_to_f16(rng.normal(0, 1, (1, 6, 1, 1)).astype(np.float32))
    out = torch.empty((2, 6, 5, 8), dtype=torch.float16, device=dev)
    rt.eltwise("add", to_dev(a, dev, True), to_dev(b, dev, True), out)
    assert_f16_exact(f16_bits(out), orc.eltwise_f16("add", a, b), "bias broadcast")
    s = orc.f32_to_f16(np.array([[[[0.5]]]], np.float32))
    rt.eltwise("mul", to_dev(a, dev, True), to_dev(s, dev, True), out)
    assert_f16_exact(f16_bits(out), orc.eltwise_f16("mul", a, s), "scalar broadcast")
    big = to_dev(a, dev, True)
    o2 = torch.zeros((2, 6, 5, 8), dtype=torch.float16, device=dev)
    rt.eltwise("add", big[:, 1:4], big[:, 2:5], o2[:, 0:3])
    want = np.zeros_like(a)
    want[:, 0:3] = orc.eltwise_f16("add", np.ascontiguousarray(a[:, 1:4]), np.ascontiguousarray(a[:, 2:5]))
    assert_f16_exact(f16_bits(o2), want, "strided views")
    bad = torch.empty((2, 6, 5, 7), dtype=torch.float16, device=dev)
    with pytest.raises(rt.VpxError) as e:
        rt.eltwise("add", big, bad, out)
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT


@pytest.mark.parametrize("shape_a,shape_b", [((37, 1024), (1, 1024)), ((37, 1024), (37, 1)), ((3, 5, 640), (1, 1, 640)),
                                             ((70001, 512), (1, 512)), ((1, 2048), (1, 2048)), ((9, 4, 520), (9, 1, 520))])
def test_eltwise_broadcast_over_rows(rt, orc, dev, shape_a, shape_b):
    """Operands that merge into rows x one inner run (a value per column, or per row): the kernel whose grid walks
    the rows, also past 65535 of them; then the same through a sub-view and for PReLU and FakeQuantize limits."""
    import torch
    rng = np.random.default_rng(25)
    a = orc.f32_to_f16(rng.normal(0, 2, shape_a).astype(np.float32))
    b = orc.f32_to_f16(rng.uniform(0.1, 2, shape_b).astype(np.float32))
    ad, bd = to_dev(a, dev, True), to_dev(b, dev, True)
    out = torch.empty(shape_a, dtype=torch.float16, device=dev)
    for op in ("add", "div"):
        rt.eltwise(op, ad, bd, out)
        assert_f16_exact(f16_bits(out), orc.eltwise_f16(op, a, b), "%s %s %s" % (op, shape_a, shape_b))
        rt.eltwise(op, bd, ad, out)
        assert_f16_exact(f16_bits(out), orc.eltwise_f16(op, b, a), "%s %s %s" % (op, shape_b, shape_a))
    rt.prelu(ad, bd, out)
    assert_f16_exact(f16_bits(out), orc.eltwise_f16("prelu", a, b), "prelu %s %s" % (shape_a, shape_b))
    if len(shape_a) == 2 and shape_a[0] > 4:
        o2 = torch.zeros(shape_a, dtype=torch.float16, device=dev)
        rt.eltwise("add", ad[2:-1], bd if shape_b[0] == 1 else bd[2:-1], o2[2:-1])
        want = np.zeros_like(a)
        want[2:-1] = orc.eltwise_f16("add", a[2:-1], b if shape_b[0] == 1 else b[2:-1])
        assert_f16_exact(f16_bits(o2), want, "rows sub-view")
    lo = orc.f32_to_f16(-b.view(np.float16).astype(np.float32))
    rt.fake_quantize(ad, to_dev(lo, dev, True), bd, to_dev(lo, dev, True), bd, 256, out)
    assert_f16_exact(f16_bits(out), orc.fake_quantize_f16(a, lo, b, lo, b, 256), "fake_quantize limits %s" % (shape_b,))


def test_eltwise_add_f32(rt, dev):
    import torch
    rng = np.random.default_rng(25)
    a = rng.normal(0, 1, 100001).astype(np.float32)
    b = rng.normal(0, 1, 100001).astype(np.float32)
    out = torch.empty(100001, dtype=torch.float32, device=dev)
    rt.eltwise("add", to_dev(a, dev), to_dev(b, dev), out)
    assert np.array_equal(out.cpu().numpy(), a + b)


# ---------------------------------------------------------------------------------- activations

def _act_cases():
    from test_oracle import ACT_CASES
    return ACT_CASES


@pytest.mark.parametrize("op,params", _act_cases(), ids=[c[0] for c in _act_cases()])
def test_activation_every_f16_value_and_f32(rt, orc, dev, op, params):
    """Piecewise-linear activations bit-exact; the ones built on exp / tanh / log / erf within one fp16
    step (device and host libm differ in the last fp32 bits), outside the range below 2^-14 where the
    float16 class's own rounding can double such a difference."""
    import torch
    from test_oracle import ACT_EXACT, f16_ulp_distance
    h = np.tile(np.arange(65536, dtype=np.uint16), 5)[:300_001]  # ragged tail, every value several times
    x = to_dev(h, dev, True)
    out = torch.empty_like(x)
    rt.activation(op, x, out, *params)
    got, want = f16_bits(out), orc.activation_f16(op, h, *params)
    nan = is_nan16(want)
    if op in ACT_EXACT:
        assert_f16_exact(got, want, op)
    else:
        assert np.array_equal(is_nan16(got), nan), op
        with np.errstate(invalid="ignore"):
            w = np.abs(orc.f16_to_f32(want).astype(np.float64))
        check = ~nan & (w >= 2.0 ** -14)
        d = f16_ulp_distance(got[check], want[check])
        assert d.max() <= 1, (op, d.max(), hex(h[check][np.argmax(d)]))
        tiny = ~nan & ~check
        assert np.all(np.abs(orc.f16_to_f32(got[tiny])) <= 2.0 ** -13), op
    # fp32 tensors
    rng = np.random.default_rng(31)
    xf = np.concatenate([rng.normal(0, 3, 70_001), rng.uniform(-12, 12, 30_000), [0.0, -0.0, 1.0, -1.0]]).astype(np.float32)
    of = torch.empty(xf.shape, dtype=torch.float32, device=dev)
    rt.activation(op, to_dev(xf, dev), of, *params)
    gf, wf = of.cpu().numpy(), orc.activation_f32(op, xf, *params)
    if op in ACT_EXACT:
        ok = ~np.isnan(wf)
        assert np.array_equal(np.isnan(gf), np.isnan(wf)) and np.array_equal(gf[ok].view(np.uint32), wf[ok].view(np.uint32)), op
    else:
        assert np.allclose(gf, wf, rtol=3e-6, atol=3e-7, equal_nan=True), (op, np.nanmax(np.abs(gf - wf)))


def test_activation_4d_views_and_errors(rt, orc, dev):
    import torch
    rng = np.random.default_rng(32)
    a = orc.f32_to_f16(rng.normal(0, 2, (2, 6, 5, 8)).astype(np.float32))
    big = to_dev(a, dev, True)
    out = torch.zeros_like(big)
    rt.activation("leaky_relu", big[:, 1:4], out[:, 2:5], 0.1)
    want = np.zeros_like(a)
    want[:, 2:5] = orc.activation_f16("leaky_relu", np.ascontiguousarray(a[:, 1:4]), 0.1)
    assert_f16_exact(f16_bits(out), want, "strided views")
    nhwc = big.permute(0, 2, 3, 1).contiguous().permute(0, 3, 1, 2)
    o2 = torch.empty_like(nhwc)
    rt.activation("clamp", nhwc, o2, -1.0, 1.0, order="NHWC")
    assert_f16_exact(f16_bits(o2.contiguous()), orc.activation_f16("clamp", a, -1.0, 1.0), "NHWC")
    with pytest.raises(rt.VpxError) as e:
        rt.activation("clamp", big, out, 2.0, 1.0)
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT
    with pytest.raises(rt.VpxError) as e:
        rt.activation("relu", big, torch.empty((2, 6, 5, 8), dtype=torch.float32, device=dev))
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT
    rt.activation("relu", torch.empty((0, 4), dtype=torch.float16, device=dev), torch.empty((0, 4), dtype=torch.float16, device=dev))


def test_prelu_per_channel_slope(rt, orc, dev):
    import torch
    rng = np.random.default_rng(33)
    a = orc.f32_to_f16(rng.normal(0, 2, (3, 16, 9, 24)).astype(np.float32))
    slope = orc.f32_to_f16(rng.uniform(0.01, 0.5, (1, 16, 1, 1)).astype(np.float32))
    out = torch.empty((3, 16, 9, 24), dtype=torch.float16, device=dev)
    rt.prelu(to_dev(a, dev, True), to_dev(slope, dev, True), out)
    assert_f16_exact(f16_bits(out), orc.eltwise_f16("prelu", a, slope), "per-channel slope")
    one = orc.f32_to_f16(np.full((1, 1, 1, 1), 0.25, np.float32))
    rt.prelu(to_dev(a, dev, True), to_dev(one, dev, True), out)
    assert_f16_exact(f16_bits(out), orc.activation_f16("leaky_relu", a, 0.25), "scalar slope equals leaky relu")


# ---------------------------------------------------------------------------------- fake_quantize

def _run_fq(rt, dev, c, order=None):
    import torch
    x = to_dev(c["x"], dev, True)
    out = torch.empty_like(x)
    rt.fake_quantize(x, *[to_dev(c[k], dev, True) for k in ("in_lo", "in_hi", "out_lo", "out_hi")], c["levels"], out,
                     order=order)
    return f16_bits(out)


def test_fake_quantize_config_c1(rt, orc, dev):
    from vpux_plugin_amd import configs
    c = configs.c1_fake_quantize()
    got = _run_fq(rt, dev, c)
    want = orc.fake_quantize_f16(c["x"], c["in_lo"], c["in_hi"], c["out_lo"], c["out_hi"], c["levels"])
    assert_f16_exact(got, want, "C1")
    assert len(np.unique(got)) <= 256


@pytest.mark.parametrize("levels", [2, 16, 255, 256, 65536])
def test_fake_quantize_levels_and_every_input(rt, orc, dev, levels):
    h = np.arange(65536, dtype=np.uint16).reshape(1, 1, 256, 256)
    lim = lambda v: orc.f32_to_f16(np.array([v], np.float32)).reshape(1, 1, 1, 1)
    c = {"x": h, "in_lo": lim(-2.5), "in_hi": lim(3.0), "out_lo": lim(-1.0), "out_hi": lim(7.0), "levels": levels}
    got = _run_fq(rt, dev, c)
    want = orc.fake_quantize_f16(h, c["in_lo"], c["in_hi"], c["out_lo"], c["out_hi"], levels)
    assert_f16_exact(got, want, "levels %d" % levels)


def test_fake_quantize_per_channel_limits(rt, orc, dev):
    rng = np.random.default_rng(26)
    x = orc.f32_to_f16(rng.normal(0, 2, (2, 5, 9, 11)).astype(np.float32))
    lo = orc.f32_to_f16(-rng.uniform(0.5, 3, (1, 5, 1, 1)).astype(np.float32))
    hi = orc.f32_to_f16(rng.uniform(0.5, 3, (1, 5, 1, 1)).astype(np.float32))
    one = orc.f32_to_f16(np.array([[[[1.0]]]], np.float32))
    c = {"x": x, "in_lo": lo, "in_hi": hi, "out_lo": lo, "out_hi": one, "levels": 256}
    got = _run_fq(rt, dev, c)
    assert_f16_exact(got, orc.fake_quantize_f16(x, lo, hi, lo, one, 256), "per-channel")


@pytest.mark.parametrize("shape", [(3, 7, 5, 256), (1000, 8), (2, 31, 264), (1, 1, 9, 64), (70000, 16)])
def test_fake_quantize_limits_per_innermost_channel(rt, orc, dev, shape):
    """Channel-minor activations: one limit per innermost channel, some limits a single value; a lane keeps eight
    channels' constants over a run of rows (row counts that do not fill the last run, channel runs shorter than a
    workgroup, results below 2^-15 for the narrowing's slow path)."""
    rng = np.random.default_rng(27)
    ch = shape[-1]
    lshape = (1,) * (len(shape) - 1) + (ch,)
    x = orc.f32_to_f16(rng.normal(0, 2, shape).astype(np.float32))
    lo = orc.f32_to_f16(-rng.uniform(0.5, 3, lshape).astype(np.float32))
    hi = orc.f32_to_f16(rng.uniform(0.5, 3, lshape).astype(np.float32))
    one = orc.f32_to_f16(np.full((1,) * len(shape), 1.0, np.float32))
    tiny_lo = orc.f32_to_f16(rng.uniform(-3e-5, 0, lshape).astype(np.float32))
    tiny_hi = orc.f32_to_f16(rng.uniform(1e-5, 6e-5, lshape).astype(np.float32))
    for levels, ol, oh in ((256, lo, hi), (16, lo, one), (255, tiny_lo, tiny_hi)):
        c = {"x": x, "in_lo": lo, "in_hi": hi, "out_lo": ol, "out_hi": oh, "levels": levels}
        got = _run_fq(rt, dev, c)
        assert_f16_exact(got, orc.fake_quantize_f16(x, lo, hi, ol, oh, levels), "%s levels %d" % (shape, levels))


def test_fake_quantize_rejects_bad_arguments(rt, dev):
    import torch
    x = torch.zeros((1, 2, 3, 4), dtype=torch.float32, device=dev)
    l = torch.zeros((1, 1, 1, 1), dtype=torch.float16, device=dev)
    with pytest.raises(rt.VpxError) as e:
        rt.fake_quantize(x, l, l, l, l, 256, torch.empty_like(x))
    assert e.value.code == rt.ERROR_UNSUPPORTED_FEATURE and "FP16" in e.value.text
    xh = x.half()
    with pytest.raises(rt.VpxError) as e:
        rt.fake_quantize(xh, l, l, l, l, 1, torch.empty_like(xh))
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT


# ---------------------------------------------------------------------------------- quantize / dequantize

@pytest.mark.parametrize("signed,scale,zp", [(False, 0.02, 128), (True, 0.05, 0), (True, 0.003, -21), (False, 1 / 255, 3),
                                             (True, 0.5, 3), (False, 0.25, 100)])
def test_quantize_dequantize(rt, orc, dev, signed, scale, zp):
    import torch
    rng = np.random.default_rng(27)
    # multiples of 1/8: with the power-of-two scales every other one is an exact tie between two levels
    x = orc.f32_to_f16(np.concatenate([rng.normal(0, 3, 200001), np.arange(-70, 70, 0.125), [0.0, -0.0, 1e-4, 65504, -65504, np.inf, -np.inf]])
                       .astype(np.float32))
    qdt = torch.int8 if signed else torch.uint8
    q = torch.empty(x.shape, dtype=qdt, device=dev)
    rt.quantize(to_dev(x, dev, True), q, scale, zp)
    # the kernel receives the scale as shipped in the blob: rounded to the float type of the input
    shipped = float(orc.f16_to_f32(orc.f32_to_f16(np.array([scale], np.float32)))[0])
    want = orc.quantize(x, shipped, zp, signed)
    assert np.array_equal(q.cpu().numpy(), want)
    allq = np.arange(-128, 128, dtype=np.int8) if signed else np.arange(0, 256, dtype=np.uint8)
    qq = np.tile(allq, 1001)[:256003]
    y = torch.empty(qq.shape, dtype=torch.float16, device=dev)
    rt.dequantize(to_dev(qq, dev), y, scale, zp)
    assert_f16_exact(f16_bits(y), orc.dequantize(qq, shipped, zp), "dequantize f16")
    y32 = torch.empty(qq.shape, dtype=torch.float32, device=dev)
    rt.dequantize(to_dev(qq, dev), y32, scale, zp)
    f32scale = float(np.float32(scale))
    assert np.array_equal(y32.cpu().numpy(), orc.dequantize(qq, f32scale, zp, to_f16=False))
    x32 = rng.normal(0, 3, 50001).astype(np.float32)
    q32 = torch.empty(x32.shape, dtype=qdt, device=dev)
    rt.quantize(to_dev(x32, dev), q32, scale, zp)
    assert np.array_equal(q32.cpu().numpy(), orc.quantize(x32, f32scale, zp, signed))


@pytest.mark.parametrize("shape,axis,order", [((2, 6, 5, 7), 1, "NCHW"), ((3, 300, 4, 4), 1, "NCHW"), ((2, 5, 7, 6), 3, "NHWC"),
                                              ((8, 8, 3, 3), 1, "NCHW"), ((16, 64), 1, None), ((700, 3), 0, None),
                                              # one vector per lane: channels shared by a vector, or consecutive channels
                                              ((4, 24, 8, 16), 1, "NCHW"), ((33, 7, 128), 0, None), ((50, 72), 1, None),
                                              ((2, 9, 11, 40), 3, "NHWC"), ((300, 1024), 0, None),
                                              # innermost axis, eight channels per lane: runs shorter and longer than a workgroup
                                              ((1000, 8), 1, None), ((4099, 264), 1, None), ((37, 2056), 1, None)])
def test_quantize_dequantize_per_axis(rt, orc, dev, shape, axis, order):
    """One scale / zero point per slice of `axis`.  The blob does not name the axis: it is the dimension
    whose size equals the parameter count, and the channel dimension when several have it ((8, 8, 3, 3))."""
    import torch
    rng = np.random.default_rng(28 + len(shape) + axis)
    n = shape[axis]
    scales = rng.uniform(0.004, 0.08, n)
    zps = rng.integers(-20, 21, n)
    shipped = orc.f16_to_f32(orc.f32_to_f16(scales.astype(np.float32))).astype(np.float64)
    x = orc.f32_to_f16(rng.normal(0, 3, shape).astype(np.float32))
    q = torch.empty(shape, dtype=torch.int8, device=dev)
    rt.quantize(to_dev(x, dev, True), q, scales, zps, order=order)
    want = orc.quantize(x, shipped, zps, True, axis=axis)
    assert np.array_equal(q.cpu().numpy(), want)
    y = torch.empty(shape, dtype=torch.float16, device=dev)
    rt.dequantize(q, y, scales, zps, order=order)
    assert_f16_exact(f16_bits(y).reshape(-1), orc.dequantize(want, shipped, zps, axis=axis).reshape(-1), "per-axis dequantize")
    y32 = torch.empty(shape, dtype=torch.float32, device=dev)
    rt.dequantize(q, y32, scales, zps, order=order)
    f32scales = scales.astype(np.float32).astype(np.float64)
    assert np.array_equal(y32.cpu().numpy(), orc.dequantize(want, f32scales, zps, to_f16=False, axis=axis))
    # same call again (the parameter table is already on the device), then other parameters of the same count
    rt.quantize(to_dev(x, dev, True), q, scales, zps, order=order)
    assert np.array_equal(q.cpu().numpy(), want)
    scales2 = scales[::-1].copy()
    shipped2 = orc.f16_to_f32(orc.f32_to_f16(scales2.astype(np.float32))).astype(np.float64)
    rt.quantize(to_dev(x, dev, True), q, scales2, zps, order=order)
    assert np.array_equal(q.cpu().numpy(), orc.quantize(x, shipped2, zps, True, axis=axis))
    x32 = rng.normal(0, 3, shape).astype(np.float32)
    q32 = torch.empty(shape, dtype=torch.uint8, device=dev)
    rt.quantize(to_dev(x32, dev), q32, scales, zps + 100, order=order)
    assert np.array_equal(q32.cpu().numpy(), orc.quantize(x32, f32scales, zps + 100, False, axis=axis))


def test_quantize_per_axis_ambiguous_axis_is_refused(rt, dev):
    import torch
    x = torch.zeros((4, 2, 4), dtype=torch.float16, device=dev)  # two dimensions of size 4, neither is the channel
    with pytest.raises(rt.VpxError) as e:
        rt.quantize(x, torch.empty((4, 2, 4), dtype=torch.int8, device=dev), [0.1] * 4, [0] * 4)
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT
    with pytest.raises(rt.VpxError):
        rt.quantize(x, torch.empty((4, 2, 4), dtype=torch.int8, device=dev), [0.1] * 3, [0] * 3)  # no dimension of size 3


# ---------------------------------------------------------------------------------- dynamic_quantize

@pytest.mark.parametrize("shape", [(6,), (3, 4), (1000, 1003), (4096, 1024), (2, 3, 5, 7), (1, 1), (0, 4)])
def test_dynamic_quantize(rt, orc, dev, shape):
    import torch
    rng = np.random.default_rng(64)
    for lo, hi in ((-3.0, 5.0), (1.0, 4.0), (-9.0, -2.0), (0.0, 0.0)):
        x = rng.uniform(lo, hi, shape).astype(np.float32)
        if x.size > 10:
            x.flat[3] = np.nan  # takes no part in the range, quantizes to 0
        out = torch.full(shape, 99, dtype=torch.uint8, device=dev)
        scale = torch.zeros(1, dtype=torch.float32, device=dev)
        zp = torch.zeros(1, dtype=torch.uint8, device=dev)
        rt.dynamic_quantize(to_dev(x, dev), out, scale, zp)
        wy, wsc, wzp = orc.dynamic_quantize(x)
        assert scale.item() == wsc and zp.item() == wzp, (shape, lo, hi, scale.item(), wsc, zp.item(), wzp)
        assert np.array_equal(out.cpu().numpy(), wy), (shape, lo, hi)


# ---------------------------------------------------------------------------------- dynamic_dequantize

DYN_DQ_CASES = [
    # q shape, q dtype, scale shape, scale dtype, zp shape / dtype, out dtype
    # the operand shapes of the reference's lit test (bufferize_sw_ops_to_VPUIP_sw_kernel.mlir:906-929), int8 for its int4
    ((16, 7, 3, 51), np.int8, (16, 1, 3, 1), np.float16, ((16, 7, 1, 51), np.int8), np.float16),
    ((512, 1024), np.int8, (512, 1), np.float16, None, np.float16),                       # per-row scale, vector path
    ((512, 1024), np.int8, (512, 1), np.float16, ((512, 1), np.int8), np.float16),
    ((64, 8, 128), np.int8, (64, 8, 1), np.float16, ((64, 8, 1), np.int8), np.float16),   # group-wise weights
    ((33, 1000), np.uint8, (1, 1000), np.float32, ((1, 1000), np.uint8), np.float16),     # per-column: one value per lane
    ((7, 5, 3), np.int8, (1, 1, 1), np.float16, None, np.float32),
    ((128, 256), np.uint8, (128, 1), np.float32, ((1, 1), np.uint8), np.float32),
]


@pytest.mark.parametrize("case", DYN_DQ_CASES, ids=[str(c[0]) + c[1].__name__ for c in DYN_DQ_CASES])
def test_dynamic_dequantize(rt, orc, dev, case):
    import torch
    shape, qdt, sc_shape, sc_dt, zp_spec, out_dt = case
    rng = np.random.default_rng(61)
    info = np.iinfo(qdt)
    q = rng.integers(info.min, info.max + 1, shape).astype(qdt)
    sc32 = rng.uniform(1e-3, 0.1, sc_shape).astype(np.float32)
    sc32.flat[0] = 2.0 ** -22  # results below 2^-15 take the float16 class's own rounding
    sc = sc32.astype(sc_dt)
    zp = None if zp_spec is None else rng.integers(np.iinfo(zp_spec[1]).min // 2, np.iinfo(zp_spec[1]).max // 2 + 1, zp_spec[0]).astype(zp_spec[1])
    out = torch.empty(shape, dtype=getattr(torch, out_dt.__name__), device=dev)
    rt.dynamic_dequantize(to_dev(q, dev), to_dev(sc, dev), out, None if zp is None else to_dev(zp, dev))
    sc_arg = sc.view(np.uint16) if sc_dt is np.float16 else sc
    if out_dt is np.float16:
        assert_f16_exact(f16_bits(out), orc.dynamic_dequantize(q, sc_arg, zp), str(shape))
    else:
        assert np.array_equal(out.cpu().numpy(), orc.dynamic_dequantize(q, sc_arg, zp, to_f16=False))


def test_dynamic_dequantize_views_and_errors(rt, orc, dev):
    import torch
    rng = np.random.default_rng(62)
    q = rng.integers(-128, 128, (16, 64, 256)).astype(np.int8)
    sc = rng.uniform(1e-3, 0.1, (16, 64, 1)).astype(np.float16)
    qd, sd = to_dev(q, dev), to_dev(sc, dev)
    out = torch.zeros((16, 64, 256), dtype=torch.float16, device=dev)
    rt.dynamic_dequantize(qd[:, 8:24, 64:192], sd[:, 8:24], out[:, 4:20, 128:256])
    want = np.zeros((16, 64, 256), np.uint16)
    want[:, 4:20, 128:256] = orc.dynamic_dequantize(q[:, 8:24, 64:192], sc[:, 8:24].view(np.uint16))
    assert_f16_exact(f16_bits(out), want, "sub-views")
    with pytest.raises(rt.VpxError) as e:
        rt.dynamic_dequantize(qd, to_dev(np.ones((16, 3, 1), np.float16), dev), out)
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT
    with pytest.raises(rt.VpxError) as e:
        rt.dynamic_dequantize(qd.to(torch.int32), sd, out)
    assert e.value.code == rt.ERROR_UNSUPPORTED_FEATURE


# ---------------------------------------------------------------------------------- MVN decomposition

def _mvn_input(orc, rng, shape):
    x = rng.uniform(-8, 8, shape) + rng.normal(0, 2, (1, shape[1], 1, 1))
    return orc.f32_to_f16(x.astype(np.float32))


def _to_layout(a, layout):
    """logical NCHW numpy array -> array in the layout's memory order"""
    return a if layout == "NCHW" else np.ascontiguousarray(a.transpose(0, 2, 3, 1))


@pytest.mark.parametrize("layout", ["NCHW", "NHWC"])
@pytest.mark.parametrize("across", [False, True])
@pytest.mark.parametrize("shape,parts", [((2, 5, 9, 7), 1), ((1, 64, 56, 56), 1), ((3, 40, 33, 31), 3), ((1, 16, 128, 96), 2)])
def test_mvn1_sum(rt, orc, dev, layout, across, shape, parts):
    import torch
    rng = np.random.default_rng(51)
    x = _mvn_input(orc, rng, shape)
    xm = to_dev(_to_layout(x, layout), dev, True)
    for nv in (True, False):
        out_c, out_w = (1 if across else shape[1]), (2 if nv else 1)
        out = torch.full((shape[0], parts, out_w, out_c), float("nan"), dtype=torch.float32, device=dev)
        rt.mvn1_sum(xm, out, across, nv, order=layout)
        got = out.cpu().numpy().astype(np.float64)
        want = orc.mvn1_sum(x, across, nv).astype(np.float64)
        assert not np.isnan(got).any()
        # fp32 accumulation in a fixed tree against double: relative to the sum of magnitudes
        xf = np.abs(orc.f16_to_f32(x).astype(np.float64))
        axes = (1, 2, 3) if across else (2, 3)
        scale = np.stack([xf.sum(axis=axes).reshape(shape[0], -1)] + ([(xf * xf).sum(axis=axes).reshape(shape[0], -1)] if nv else []), axis=1)
        assert np.all(np.abs(got.sum(axis=1) - want[:, 0]) <= 2e-6 * scale), (layout, across, nv)


@pytest.mark.parametrize("out_dtype", ["float32", "float16"])
def test_mvn1_mean_var(rt, orc, dev, out_dtype):
    import torch
    rng = np.random.default_rng(52)
    tdt = getattr(torch, out_dtype)
    ndt = getattr(np, out_dtype)
    for (N, Cc, H, W), across, parts, group_c in (((2, 12, 9, 7), False, 1, 1), ((2, 12, 9, 7), True, 4, 1),
                                                   ((3, 12, 5, 5), False, 2, 4), ((1, 300, 8, 8), False, 3, 1)):
        x = rng.normal(0.5, 2, (N, Cc, H, W))
        c_in = 1 if across else Cc
        axes = (1, 2, 3) if across else (2, 3)
        total = np.stack([x.sum(axis=axes).reshape(N, c_in), (x * x).sum(axis=axes).reshape(N, c_in)], axis=1)  # [N, 2, Cin]
        w = rng.dirichlet(np.ones(parts), size=(N, 2, c_in)).transpose(0, 3, 1, 2)  # split every sum into parts
        sums = (total[:, None] * w).astype(np.float32)
        for nv in (True, False):
            out = torch.empty((N, 1, 2 if nv else 1, c_in if across else Cc), dtype=tdt, device=dev)
            rt.mvn1_mean_var(to_dev(sums[:, :, :2 if nv else 1].copy(), dev), out, (N, Cc, H, W), across, nv, 1e-6, group_c)
            got = out.cpu().numpy().astype(np.float64)
            want = orc.mvn1_mean_var(sums[:, :, :2 if nv else 1], (N, Cc, H, W), across, nv, 1e-6, group_c, ndt).astype(np.float64)
            tol = 2e-6 if out_dtype == "float32" else 1e-3
            assert np.all(np.abs(got - want) <= tol * np.abs(want) + 1e-7), (across, nv, group_c)


@pytest.mark.parametrize("layout", ["NCHW", "NHWC"])
@pytest.mark.parametrize("across", [False, True])
@pytest.mark.parametrize("stat_dtype", ["float32", "float16"])
def test_mvn1_norm_exact(rt, orc, dev, layout, across, stat_dtype):
    import torch
    rng = np.random.default_rng(53)
    for shape in ((2, 5, 9, 7), (2, 24, 16, 40), (1, 3, 64, 100)):
        x = _mvn_input(orc, rng, shape)
        xm = to_dev(_to_layout(x, layout), dev, True)
        for nv in (True, False):
            c = 1 if across else shape[1]
            mv = np.stack([rng.normal(0, 2, (shape[0], c))] + ([rng.uniform(0.1, 3, (shape[0], c))] if nv else []), axis=1)[:, None]
            mv = mv.astype(getattr(np, stat_dtype))
            out = torch.empty_like(xm)
            rt.mvn1_norm(xm, to_dev(mv, dev), out, across, nv, order=layout)
            want = _to_layout(orc.mvn1_norm(x, mv, across, nv), layout)
            assert_f16_exact(f16_bits(out), want, "%s %s %s" % (layout, across, nv))


@pytest.mark.parametrize("layout", ["NCHW", "NHWC"])
@pytest.mark.parametrize("across", [False, True])
def test_mvn1_three_steps_match_the_single_kernel(rt, orc, dev, layout, across):
    import torch
    rng = np.random.default_rng(54)
    shape = (2, 32, 48, 40)
    x = _mvn_input(orc, rng, shape)
    xm = to_dev(_to_layout(x, layout), dev, True)
    c = 1 if across else shape[1]
    sums = torch.empty((shape[0], 2, 2, c), dtype=torch.float32, device=dev)
    mv = torch.empty((shape[0], 1, 2, c), dtype=torch.float32, device=dev)
    out = torch.empty_like(xm)
    rt.mvn1_sum(xm, sums, across, True, order=layout)
    rt.mvn1_mean_var(sums, mv, shape, across, True, 1e-9)
    rt.mvn1_norm(xm, mv, out, across, True, order=layout)
    want = _to_layout(orc.mvn_f16(x, across, True, 1e-9), layout)
    # values next to zero carry the absolute error of the fp32 mean (x - mean cancels): absolute floor
    _assert_mvn6_close(f16_bits(out), want, orc, "three steps vs oracle mvn")
    single = torch.empty_like(xm)
    rt.mvn(xm, single, across, True, 1e-9, order=layout)
    _assert_mvn6_close(f16_bits(out), f16_bits(single), orc, "three steps vs mvn1 kernel")


def test_mvn1_decomposition_errors(rt, dev):
    import torch
    x = torch.zeros((2, 4, 8, 8), dtype=torch.float16, device=dev)
    with pytest.raises(rt.VpxError) as e:
        rt.mvn1_sum(x, torch.empty((2, 1, 2, 3), dtype=torch.float32, device=dev), False, True)
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT
    with pytest.raises(rt.VpxError) as e:
        rt.mvn1_sum(x, torch.empty((2, 1, 2, 4), dtype=torch.float16, device=dev), False, True)
    assert e.value.code == rt.ERROR_UNSUPPORTED_FEATURE
    with pytest.raises(rt.VpxError) as e:
        rt.mvn1_mean_var(torch.zeros((2, 1, 2, 4), dtype=torch.float32, device=dev),
                         torch.empty((2, 1, 2, 4), dtype=torch.float32, device=dev), (2, 4, 8, 8), False, True, 1e-6, group_c=3)
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT
    with pytest.raises(rt.VpxError) as e:
        rt.mvn1_norm(x, torch.zeros((2, 1, 2, 1), dtype=torch.float32, device=dev), torch.empty_like(x), False, True)
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT


# ---------------------------------------------------------------------------------- MVN-6

def _assert_mvn6_close(got_bits, want_bits, orc, what):
    g = orc.f16_to_f32(got_bits).astype(np.float64)
    w = orc.f16_to_f32(want_bits).astype(np.float64)
    bad = np.argwhere(~(np.abs(g - w) <= REL_TOL * np.abs(w) + 2e-5))
    assert len(bad) == 0, "%s: %d outside tolerance, first %s got %r want %r" % (what, len(bad), bad[0], g[tuple(bad[0])], w[tuple(bad[0])])


MVN6_CASES = [
    # shape, axes, scale shape, bias shape
    ((8, 128, 768), (2,), (1, 1, 768), (1, 1, 768)),      # LayerNorm, one wavefront per row
    # LayerNorm over many rows: a team walks 2 or 4 rows with scale / bias in registers; the last workgroup is ragged
    ((70001, 256), (1,), (1, 256), (1, 256)),
    ((131075, 64), (1,), (1, 64), None),
    ((33, 1001, 512), (2,), None, (1, 1, 512)),
    ((65539, 768), (1,), (1, 768), (1, 768)),
    ((32771, 768), (1,), (1, 768), (1, 768)),
    ((3, 11000, 1024), (2,), (1, 1, 1024), (1, 1, 1024)),
    ((40000, 256), (1,), (40000, 256), (1, 256)),         # a scale of full shape is read per row
    # one wavefront per row of up to 3072 values, 3 ... 6 words per lane
    ((301, 1280), (1,), (1, 1280), (1, 1280)),
    ((3, 35, 1536), (2,), (1, 1, 1536), None),
    ((99, 2560), (1,), None, (1, 2560)),
    ((77, 3072), (1,), (1, 3072), (1, 3072)),
    ((45, 1032), (1,), None, None),
    ((21, 5120), (1,), (1, 5120), (1, 5120)),
    ((9, 10240), (1,), None, (1, 10240)),
    ((7, 13824), (1,), (1, 13824), None),
    ((4, 77, 512), (-1,), None, None),
    ((4, 16, 2048), (2,), (1, 1, 2048), None),            # one workgroup per row
    ((2, 8, 8192), (2,), None, (1, 1, 8192)),
    ((2, 6, 4096), (2,), (1, 6, 1), (2, 6, 4096)),        # scale constant along the row, bias of full shape
    ((3, 5, 16, 24), (2, 3), (1, 1, 16, 24), (1, 5, 1, 1)),  # two innermost axes
    ((5, 7, 30), (2,), (1, 1, 30), (1, 1, 30)),           # row not a multiple of 8: generic
    ((4, 6, 10), (1,), (1, 6, 1), None),                  # middle axis: generic
    ((3, 64, 200), (1,), (1, 64, 1), (1, 1, 200)),        # innermost dimension kept: lanes along it
    ((2, 5, 6, 70), (1, 2), (1, 5, 6, 1), None),
    ((2, 3, 4, 5), (1, 3), (1, 3, 1, 5), (1, 1, 1, 5)),   # split axes
    ((3, 2, 11008), (2,), (1, 1, 11008), None),           # rows of up to 16384 stay in the registers of a workgroup
    ((5, 16384), (1,), None, (1, 16384)),
    ((3, 12296), (1,), None, None),
    ((130, 20000), (1,), None, None),                     # many longer rows: a row in LDS, one pass over memory
    ((2, 20000), (1,), None, None),                       # few longer rows: chunked like mvn1 ...
    ((3, 2, 150, 200), (2, 3), None, None),
    ((2, 20001), (1,), None, (1, 20001)),                 # ... or one workgroup per row when there is a bias
    ((6, 1, 64), (1, 2), None, None),                     # unit dimension among the axes
    ((1000, 8), (1,), None, None),                        # packed power-of-two rows: len / 8 lanes per row
    ((77, 5, 32), (2,), None, None),
    ((130, 64), (1,), None, None),
    ((9, 128), (1,), None, None),
    ((33, 16, 16), (1, 2), None, None),
    ((300, 50), (1,), None, None),                        # many short rows, not a multiple of 8: runs of rows per workgroup
    ((64, 3, 7, 7), (2, 3), None, None),
    ((70, 1001), (-1,), None, None),
]


@pytest.mark.parametrize("shape,axes,sc_shape,bi_shape", MVN6_CASES, ids=[str(c[0]) + str(c[1]) for c in MVN6_CASES])
def test_mvn6(rt, orc, dev, shape, axes, sc_shape, bi_shape):
    import torch
    rng = np.random.default_rng(55)
    x = orc.f32_to_f16(rng.normal(0.5, 2, shape).astype(np.float32))
    sc = orc.f32_to_f16(rng.uniform(0.5, 2, sc_shape).astype(np.float32)) if sc_shape else None
    bi = orc.f32_to_f16(rng.normal(0, 1, bi_shape).astype(np.float32)) if bi_shape else None
    xd = to_dev(x, dev, True)
    for nv, eps, mode in ((True, 1e-5, 0), (True, 1e-2, 1), (False, 0.0, 0)):
        out = torch.empty_like(xd)
        rt.mvn6(xd, out, axes, nv, eps, mode, scale=None if sc is None else to_dev(sc, dev, True),
                bias=None if bi is None else to_dev(bi, dev, True))
        _assert_mvn6_close(f16_bits(out), orc.mvn6_f16(x, axes, nv, eps, mode, sc, bi), orc, "%s nv=%s mode=%d" % (shape, nv, mode))


def test_mvn6_strided_rows_and_errors(rt, orc, dev):
    import torch
    rng = np.random.default_rng(56)
    x = orc.f32_to_f16(rng.normal(0, 2, (4, 10, 256)).astype(np.float32))
    xd = to_dev(x, dev, True)
    out = torch.zeros_like(xd)
    rt.mvn6(xd[:, 2:7], out[:, 3:8], (2,), True, 1e-5, 0)  # rows keep their alignment, outer strides differ
    want = np.zeros_like(x)
    want[:, 3:8] = orc.mvn6_f16(np.ascontiguousarray(x[:, 2:7]), (2,), True, 1e-5, 0)
    _assert_mvn6_close(f16_bits(out), want, orc, "row views")
    out.zero_()
    rt.mvn6(xd[:, :, 3:131], out[:, :, 5:133], (2,), True, 1e-5, 0)  # misaligned rows: generic kernel
    want = np.zeros_like(x)
    want[:, :, 5:133] = orc.mvn6_f16(np.ascontiguousarray(x[:, :, 3:131]), (2,), True, 1e-5, 0)
    _assert_mvn6_close(f16_bits(out), want, orc, "misaligned views")
    with pytest.raises(rt.VpxError) as e:
        rt.mvn6(xd, out, (2, 2), True, 1e-5, 0)
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT
    with pytest.raises(rt.VpxError) as e:
        rt.mvn6(xd, out, (2,), True, 1e-5, 0, scale=torch.ones((1, 1, 7), dtype=torch.float16, device=dev))
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT
    with pytest.raises(rt.VpxError) as e:
        rt.mvn6(xd, out, (2,), True, 1e-5, 2)
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT


# ---------------------------------------------------------------------------------- softmax

def _softmax(rt, dev, x_bits, axis, pad=0, packed=True, f32=False):
    import torch
    x = to_dev(x_bits, dev, not f32)
    out = torch.empty_like(x)
    rt.softmax(x, out, axis, pad, packed=packed)
    return out


@pytest.mark.parametrize("shape,axis", [((64, 512), 1), ((3, 5, 1024), 2), ((7, 2048), 1), ((5, 4096), 1), ((33, 40), 1),
                                        ((9, 1000), 1), ((4, 8200), 1), ((2, 3, 4, 4), 3), ((6, 32, 4, 4), 1),
                                        ((5, 17, 300), 1), ((17, 64), 0), ((2, 3, 50, 7), 2),
                                        # rows that are not 16-byte aligned, long rows (one workgroup per row), and beyond
                                        ((65, 500), 1), ((7, 511), 1), ((130, 197), 1), ((300, 192), 1), ((77, 160), 1), ((130, 248), 1), ((3, 1023), 1), ((9, 4099), 1),
                                        ((3, 32768), 1), ((5, 20000), 1), ((6, 8191), 1), ((2, 33000), 1), ((2, 40001), 1),
                                        ((20000, 8), 1), ((17000, 509), 1),
                                        # many short rows: runs of rows through LDS (any length), a ragged last run
                                        ((70, 32), 1), ((3001, 64), 1), ((129, 128), 1), ((2, 50, 197), 2), ((100, 37), 1),
                                        ((77, 3, 5), 2), ((333, 383), 1), ((64, 24), 1), ((50, 16), 1), ((3, 7, 128), 2), ((77, 256), 1),
                                        # rows past the registers of a workgroup: one 1024-lane workgroup per row, two passes
                                        ((3, 40000), 1), ((2, 131072), 1), ((2, 33333), 1),
                                        # 64 or more aligned rows of up to 76 800 values: the row in LDS, one pass over memory
                                        ((70, 50264), 1), ((64, 76800), 1), ((66, 33000), 1),
                                        # outer axis with contiguous inner dimensions: every slab shape (steps x columns x waves)
                                        ((3, 12, 64), 1), ((2, 50, 8, 24), 1), ((2, 200, 520), 1), ((3, 21, 36), 1),
                                        ((2, 100, 4, 5), 1), ((1, 400, 132), 1), ((2, 40, 6), 1), ((1, 200, 30), 1),
                                        ((1, 1000, 66), 1), ((1, 1024, 2, 64), 1), ((1, 1100, 64), 1), ((2, 2, 512, 512), 2),
                                        # outer axis past the slabs: wavefronts along the axis, lanes along the columns
                                        ((4, 2048, 128), 1), ((2, 1500, 70), 1), ((3, 1200, 5, 13), 1), ((2, 4000, 520), 1),
                                        ((5000, 64), 0), ((1, 1030, 1024), 1),
                                        # steps either side of 2048, 63 and 200 columns
                                        ((2, 2047, 64), 1), ((1, 1025, 200), 1), ((2, 2049, 64), 1), ((1, 2048, 1, 63), 1)])
def test_softmax_shapes_and_axes(rt, orc, dev, shape, axis):
    rng = np.random.default_rng(hash((shape, axis)) % 2 ** 32)
    x = rng.normal(0, 3, shape).astype(np.float32)
    x[rng.random(shape) < 0.05] = -60000.0
    xb = orc.f32_to_f16(x)
    want = orc.softmax_f16(xb, axis)
    for packed in (True, False):
        got = f16_bits(_softmax(rt, dev, xb, axis, packed=packed))
        assert_close_f16(got, want, orc, "softmax %s axis %d packed=%s" % (shape, axis, packed))
        assert np.all(got[xb == 0xfb53] == 0)  # masked logits give exact zeros


def test_softmax_padding_fp32_and_subviews(rt, orc, dev):
    import torch
    rng = np.random.default_rng(31)
    x = rng.normal(0, 2, (6, 1000)).astype(np.float32)
    xb = orc.f32_to_f16(x)
    got = f16_bits(_softmax(rt, dev, xb, 1, pad=3))
    assert_close_f16(got, orc.softmax_f16(xb, 1, pad=3), orc, "padSize 3")
    assert np.all(got[:, -3:] == 0)
    got = f16_bits(_softmax(rt, dev, orc.f32_to_f16(x[:, :512]), 1, pad=8))
    assert_close_f16(got, orc.softmax_f16(orc.f32_to_f16(x[:, :512]), 1, pad=8), orc, "padSize 8, wave path")
    y32 = _softmax(rt, dev, x, 1, f32=True).cpu().numpy()
    np.testing.assert_allclose(y32, orc.softmax_f32(x, 1), rtol=REL_TOL, atol=1e-30)
    # long rows: fp32, and fp16 with a padded tail
    xl = rng.normal(0, 2, (3, 9000)).astype(np.float32)
    np.testing.assert_allclose(_softmax(rt, dev, xl, 1, f32=True).cpu().numpy(), orc.softmax_f32(xl, 1), rtol=REL_TOL, atol=1e-30)
    np.testing.assert_allclose(_softmax(rt, dev, xl[:, :8999], 1, f32=True).cpu().numpy(), orc.softmax_f32(xl[:, :8999], 1), rtol=REL_TOL, atol=1e-30)
    xo = rng.normal(0, 2, (3, 70, 200)).astype(np.float32)   # fp32 over an outer axis, with and without a padded tail
    np.testing.assert_allclose(_softmax(rt, dev, xo, 1, f32=True).cpu().numpy(), orc.softmax_f32(xo, 1), rtol=REL_TOL, atol=1e-30)
    np.testing.assert_allclose(_softmax(rt, dev, xo, 1, pad=6, f32=True).cpu().numpy(), orc.softmax_f32(xo, 1, pad=6), rtol=REL_TOL, atol=1e-30)
    xob = orc.f32_to_f16(rng.normal(0, 2, (2, 1300, 96)).astype(np.float32))
    got = f16_bits(_softmax(rt, dev, xob, 1, pad=4))
    assert_close_f16(got, orc.softmax_f16(xob, 1, pad=4), orc, "outer axis, padSize 4")
    assert np.all(got[:, -4:, :] == 0)
    xlb = orc.f32_to_f16(rng.normal(0, 2, (2, 50000)).astype(np.float32))
    got = f16_bits(_softmax(rt, dev, xlb, 1, pad=5))
    assert_close_f16(got, orc.softmax_f16(xlb, 1, pad=5), orc, "long rows, padSize 5")
    assert np.all(got[:, -5:] == 0)
    # rows taken from a wider buffer: strides differ from the compact ones
    wide = to_dev(orc.f32_to_f16(rng.normal(0, 2, (8, 4, 768)).astype(np.float32)), dev, True)
    out = torch.zeros_like(wide)
    rt.softmax(wide[:, 1:3, 128:640], out[:, 1:3, 128:640], 2)
    src = f16_bits(wide)[:, 1:3, 128:640]
    assert_close_f16(f16_bits(out)[:, 1:3, 128:640], orc.softmax_f16(np.ascontiguousarray(src), 2), orc, "sub-view")
    assert torch.count_nonzero(out[:, 0]) == 0 and torch.count_nonzero(out[:, :, :128]) == 0


def test_softmax_config_c2_full_size_properties(rt, orc, dev):
    import torch
    from vpux_plugin_amd import configs
    c = configs.c2_softmax()
    x = to_dev(c["x"], dev, True)
    out = torch.empty_like(x)
    rt.softmax(x, out, c["axis"])
    torch.cuda.synchronize()
    sums = out.float().sum(dim=-1)
    assert float((sums - 1).abs().max()) < 4e-3         # every row is a distribution
    assert bool((out[x == -60000.0] == 0).all())        # masked entries vanish
    assert bool((out >= 0).all())
    # argmax is preserved and the whole tensor matches the oracle (threaded: well under a second of CPU)
    assert bool((out.argmax(dim=-1) == x.argmax(dim=-1)).float().mean() > 0.999)
    assert_close_f16(f16_bits(out), orc.softmax_f16(c["x"], c["axis"]), orc, "C2 whole tensor")


@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("bound,live,axis,pad,compact", [
    ((4, 100, 64), (3, 77, 50), 2, 0, False), ((4, 100, 64), (3, 77, 50), 1, 0, False), ((4, 100, 64), (3, 77, 50), 0, 0, False),
    ((4, 100, 64), (3, 77, 50), 2, 0, True), ((4, 100, 64), (3, 77, 50), 1, 5, True), ((2, 3, 40, 33), (2, 3, 40, 33), 3, 0, False),
    ((2, 3, 40, 33), (1, 2, 17, 9), 2, 0, True), ((8, 700), (5, 513), 1, 13, False), ((600,), (257,), 0, 0, False)])
def test_softmax_bounded_dynamic_shape(rt, orc, dev, dtype, bound, live, axis, pad, compact):
    """SoftmaxModeDynamic: the kernel takes the shape from the memrefs' dims and strides in device memory.  The live tensor
    equals the oracle's softmax of the same values; every element outside it keeps the guard value.  (Parity with the
    SHAVE kernel itself is unpinned: its source is not public.)"""
    import torch
    rng = np.random.default_rng(hash((bound, live, axis)) % 2 ** 32)
    xf = rng.normal(0, 3, bound).astype(np.float32)
    live_sl = tuple(slice(0, n) for n in live)
    if dtype == "f16":
        xb = orc.f32_to_f16(xf)
        x = to_dev(xb, dev, True)
        out = torch.full(bound, 7.0, dtype=torch.float16, device=dev)
    else:
        x = torch.from_numpy(xf).to(dev)
        out = torch.full(bound, 7.0, dtype=torch.float32, device=dev)
    if compact:  # the live tensor lies compactly at the start of both buffers
        n_live = int(np.prod(live))
        src = (xb if dtype == "f16" else xf)[live_sl].reshape(-1).copy()
        flat = x.view(-1)
        flat[:n_live] = to_dev(src, dev, True) if dtype == "f16" else torch.from_numpy(src).to(dev)
    keep = rt.softmax_dynamic(x, out, live, axis, pad, compact=compact)
    torch.cuda.synchronize()
    del keep
    valid = live[axis] - pad
    src_live = (xb if dtype == "f16" else xf)[live_sl]
    cut = tuple(slice(0, valid) if d == axis else slice(None) for d in range(len(live)))
    if dtype == "f16":
        want = np.zeros(live, dtype=np.uint16)
        want[cut] = orc.softmax_f16(np.ascontiguousarray(src_live[cut]), axis)
        got_all = f16_bits(out)
        guard = np.uint16(0x4700)
    else:
        want = np.zeros(live, dtype=np.float32)
        want[cut] = orc.softmax_f32(np.ascontiguousarray(src_live[cut]), axis)
        got_all = out.cpu().numpy()
        guard = np.float32(7.0)
    if compact:
        n_live = int(np.prod(live))
        got = got_all.reshape(-1)[:n_live].reshape(live)
        assert np.all(got_all.reshape(-1)[n_live:] == guard)
    else:
        got = got_all[live_sl]
        mask = np.ones(bound, dtype=bool)
        mask[live_sl] = False
        assert np.all(got_all[mask] == guard)
    if dtype == "f16":
        assert_close_f16(got, want, orc, "dynamic softmax %s of %s axis %d" % (live, bound, axis))
    else:
        assert np.allclose(got, want, rtol=2e-3, atol=1e-7)


def test_softmax_dynamic_shape_larger_than_its_bound_is_cut(rt, orc, dev):
    """Live dims beyond the bound (a producer's mistake) never make the kernel leave the buffers: each is cut to its bound."""
    import torch
    rng = np.random.default_rng(77)
    xb = orc.f32_to_f16(rng.normal(0, 3, (3, 40, 24)).astype(np.float32))
    x = to_dev(xb, dev, True)
    pad_before = torch.full((4096,), 5.0, dtype=torch.float16, device=dev)
    out = torch.full((3, 40, 24), 7.0, dtype=torch.float16, device=dev)
    pad_after = torch.full((4096,), 5.0, dtype=torch.float16, device=dev)
    keep = rt.softmax_dynamic(x, out, (5, 41, 99), 2)
    torch.cuda.synchronize()
    del keep
    assert_close_f16(f16_bits(out), orc.softmax_f16(xb, 2), orc, "dynamic softmax cut to its bound")
    assert bool((pad_before == 5.0).all()) and bool((pad_after == 5.0).all())


def test_softmax_rejects_bad_arguments(rt, dev):
    import torch
    x = torch.zeros((4, 8), dtype=torch.float16, device=dev)
    with pytest.raises(rt.VpxError) as e:
        rt.softmax(x, torch.empty((4, 9), dtype=torch.float16, device=dev), 1)
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT
    with pytest.raises(rt.VpxError) as e:
        rt.softmax(x, torch.empty_like(x), 1, pad_size=8, packed=False)
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT
    # dynamic-shape parameters with static memrefs, and a dynamic memref on a kernel that takes none
    ops = [rt.Operand(x), rt.Operand(torch.empty_like(x))]
    dyn_words = np.asarray([0, 0 | (2 << 32)], dtype=np.uint64).tobytes()
    with pytest.raises(rt.VpxError) as e:
        rt.sw_kernel_launch("softmax", rt.create_kernel_params(ops[:1], ops[1:], dyn_words), ops)
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT
    dyn = [rt.Operand(x, None, dynamic=True), rt.Operand(torch.empty_like(x), None, dynamic=True)]
    for o in dyn:
        o.live_dims = torch.tensor([8, 4], dtype=torch.int32, device=dev)
        o.live_strides = torch.tensor([16, 128], dtype=torch.int64, device=dev)
    with pytest.raises(rt.VpxError) as e:
        rt.sw_kernel_launch("convert", rt.create_kernel_params(dyn[:1], dyn[1:]), dyn)
    assert e.value.code == rt.ERROR_UNSUPPORTED_FEATURE
    with pytest.raises(rt.VpxError) as e:  # static form of the parameters with dynamic memrefs
        rt.sw_kernel_launch("softmax", rt.create_kernel_params(dyn[:1], dyn[1:], np.asarray([0, 0], dtype=np.int64).tobytes()), dyn)
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT


# ---------------------------------------------------------------------------------- MVN

def _mvn(rt, dev, xb, across, nv, eps, order="NCHW"):
    import torch
    x = to_dev(xb, dev, True)
    out = torch.empty_like(x)
    rt.mvn(x, out, across, nv, eps, order=order)
    return f16_bits(out)


@pytest.mark.parametrize("shape", [(2, 3, 8, 8), (1, 16, 64, 64), (3, 7, 5, 9), (2, 64, 33, 31), (1, 2, 1, 4097),
                                   (1, 600, 64, 64),
                                   # many short groups: runs of whole groups per workgroup, odd lengths, a ragged last run
                                   (4, 64, 7, 7), (3, 50, 14, 14), (2, 333, 1, 5), (1, 70, 31, 33), (67, 1, 1, 1), (5, 13, 1, 1024),
                                   (3, 40, 8, 8), (2, 9, 16, 16), (5, 7, 4, 4), (1, 3, 2, 4),   # planes of 8 ... 256 values
                                   # many groups of a few thousand to 76 800 values: the whole group in LDS, one pass over memory
                                   (2, 70, 112, 112), (1, 130, 80, 96), (1, 128, 200, 384), (1, 128, 4104, 1)])
@pytest.mark.parametrize("across", [True, False])
@pytest.mark.parametrize("nv", [True, False])
def test_mvn_nchw(rt, orc, dev, shape, across, nv):
    rng = np.random.default_rng(hash(shape) % 2 ** 32)
    x = (rng.uniform(-8, 8, shape) + rng.normal(0, 2, (1, shape[1], 1, 1))).astype(np.float32)
    xb = orc.f32_to_f16(x)
    got = _mvn(rt, dev, xb, across, nv, 1e-9)
    assert_close_f16_mvn(got, orc.mvn_f16(xb, across, nv, 1e-9), orc, "mvn %s across=%s nv=%s" % (shape, across, nv))


def assert_close_f16_mvn(got_bits, want_bits, orc, what):
    # Normalised values near zero are differences of nearly equal numbers: compare them on the scale
    # of the normalised data (unit variance) as well as relatively.
    g = orc.f16_to_f32(got_bits).astype(np.float64)
    w = orc.f16_to_f32(want_bits).astype(np.float64)
    err = np.abs(g - w)
    scale = max(1.0, float(np.max(np.abs(w))))
    tol = np.maximum(REL_TOL * np.abs(w), REL_TOL * 1e-1 * scale)
    bad = np.argwhere(err > tol)
    assert len(bad) == 0, "%s: %d outside tolerance, first %s got %r want %r" % (
        what, len(bad), bad[0], g[tuple(bad[0])], w[tuple(bad[0])])


@pytest.mark.parametrize("C", [70, 64, 264, 8, 2048])   # multiples of eight take the eight-channels-per-lane sums
@pytest.mark.parametrize("across", [True, False])
def test_mvn_nhwc(rt, orc, dev, across, C):
    rng = np.random.default_rng(41)
    x = (rng.uniform(-8, 8, (2, 9, 7, C)) + rng.normal(0, 2, (1, 1, 1, C))).astype(np.float32)  # N,H,W,C in memory
    xb = orc.f32_to_f16(x)
    got = _mvn(rt, dev, xb, across, True, 1e-9, order="NHWC")
    assert_close_f16_mvn(got, orc.mvn_f16(xb, across, True, 1e-9, layout="NHWC"), orc, "mvn NHWC across=%s" % across)


def test_mvn_config_c3_full_size(rt, orc, dev):
    from vpux_plugin_amd import configs
    c = configs.c3_mvn()
    got = _mvn(rt, dev, c["x"], True, True, c["eps"])
    want = orc.mvn_f16(c["x"], True, True, c["eps"])
    assert_close_f16_mvn(got, want, orc, "C3")
    g = orc.f16_to_f32(got).astype(np.float64).reshape(4, -1)
    assert np.max(np.abs(g.mean(axis=1))) < 1e-3 and np.max(np.abs(g.var(axis=1) - 1)) < 2e-3
    # deterministic: a second run gives the same bits
    assert np.array_equal(got, _mvn(rt, dev, c["x"], True, True, c["eps"]))


@pytest.mark.parametrize("shape", [(4, 64, 64, 64), (1, 3, 72, 200), (3, 5, 40, 104), (7, 2, 64, 40), (2, 33, 97, 8), (1, 128, 128, 128)])
def test_mvn_one_launch_kernel_and_its_fallback(rt, orc, dev, shape):
    """Long groups in one launch (workgroups of a group meet at the group's counter): against the oracle, bit for bit
    against the same kernel when no workgroup waits for the others (each recomputes its group's moments, as a
    workgroup does whose wait runs out), repeated launches (the counters are left at zero), and within tolerance
    against the two-launch kernels."""
    import torch
    rng = np.random.default_rng(sum(shape))
    x = (rng.uniform(-8, 8, shape) + rng.normal(0, 2, (1, shape[1], 1, 1))).astype(np.float32)
    xb = orc.f32_to_f16(x)
    want = orc.mvn_f16(xb, True, True, 1e-9)
    runs = [_mvn(rt, dev, xb, True, True, 1e-9) for _ in range(3)]
    assert_close_f16_mvn(runs[0], want, orc, "one launch %s" % (shape,))
    assert np.array_equal(runs[0], runs[1]) and np.array_equal(runs[0], runs[2])
    rt.set_tuning("VPX_MVN_FUSED", "nowait")
    try:
        alone = _mvn(rt, dev, xb, True, True, 1e-9)
        rt.set_tuning("VPX_MVN_FUSED", None)
        after = _mvn(rt, dev, xb, True, True, 1e-9)  # the counters were left clean by the launch that did not wait
        rt.set_tuning("VPX_MVN_FUSED", "off")
        two = _mvn(rt, dev, xb, True, True, 1e-9)
    finally:
        rt.set_tuning("VPX_MVN_FUSED", None)
    assert np.array_equal(alone, runs[0]) and np.array_equal(after, runs[0])
    assert_close_f16_mvn(two, want, orc, "two launches %s" % (shape,))


def test_mvn_one_launch_kernel_beside_a_launch_that_holds_compute_units(rt, orc, dev):
    """Configuration 3's MVN on one stream while another stream runs a long launch on all but 32 compute units: only
    some of the MVN kernel's workgroups are resident at a time, those wait for records that cannot arrive, their
    bounded wait runs out and they compute their group's moments themselves.  Every kernel exits, and the result is
    the bits of the undisturbed run."""
    import time
    import torch
    from vpux_plugin_amd import configs
    c = configs.c3_mvn()
    x = to_dev(c["x"], dev, True)
    alone, beside = torch.empty_like(x), torch.empty_like(x)
    rt.mvn(x, alone, True, True, c["eps"])
    torch.cuda.synchronize()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    src = torch.zeros((65536,), device=dev, dtype=torch.int8)
    sink = torch.empty((cus * 8192,), device=dev, dtype=torch.uint8)
    a, b = torch.cuda.Stream(), torch.cuda.Stream()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    f0, f1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    rt.set_tuning("VPX_CALIB_BLOCKS", str(max(1, cus - 32)))
    try:
        with torch.cuda.stream(b):
            rt.calib_mfma_i8(src, sink, 200)  # (first launch of the kernel: not under the clock)
        torch.cuda.synchronize()
        with torch.cuda.stream(b):
            f0.record()
            rt.calib_mfma_i8(src, sink, 20000)  # about 9 ms
            f1.record()
        time.sleep(0.002)  # the long launch is running
        with torch.cuda.stream(a):
            e0.record()
            rt.mvn(x, beside, True, True, c["eps"])
            e1.record()
        torch.cuda.synchronize()
    finally:
        rt.set_tuning("VPX_CALIB_BLOCKS", None)
    assert torch.equal(alone, beside)
    long_ms, mvn_ms = f0.elapsed_time(f1), e0.elapsed_time(e1)
    print("MVN beside a %.1f ms launch on %d of %d compute units: %.3f ms" % (long_ms, cus - 32, cus, mvn_ms))
    assert long_ms > 4.0    # the long launch did overlap the MVN
    assert mvn_ms < 50.0    # the waits are bounded


@pytest.mark.parametrize("shape", [(4, 64, 64, 64), (3, 5, 40, 104), (2, 3, 8, 8), (2, 70, 112, 112)])
@pytest.mark.parametrize("fused", [None, "nowait"])
def test_mvn_in_place(rt, orc, dev, shape, fused):
    """Output tensor = input tensor.  Long groups then leave the one-launch kernel alone (a workgroup that recomputes
    its group's moments would read slices other workgroups have already normalised): same bits as out of place."""
    import torch
    rng = np.random.default_rng(sum(shape) + 5)
    xb = orc.f32_to_f16((rng.uniform(-8, 8, shape) + rng.normal(0, 2, (1, shape[1], 1, 1))).astype(np.float32))
    rt.set_tuning("VPX_MVN_FUSED", "off")
    try:
        apart = _mvn(rt, dev, xb, True, True, 1e-9)
        rt.set_tuning("VPX_MVN_FUSED", fused)
        x = to_dev(xb, dev, True)
        rt.mvn(x, x, True, True, 1e-9)
        torch.cuda.synchronize()
    finally:
        rt.set_tuning("VPX_MVN_FUSED", None)
    assert np.array_equal(f16_bits(x), apart)
    assert_close_f16_mvn(apart, orc.mvn_f16(xb, True, True, 1e-9), orc, "in place %s" % (shape,))


def test_mvn_rejects_partial_overlap(rt, dev):
    import torch
    buf = torch.zeros((2 * 4 * 64 * 64 + 64,), dtype=torch.float16, device=dev)
    x = buf[:2 * 4 * 64 * 64].view(2, 4, 64, 64)
    y = buf[64:].view(2, 4, 64, 64)
    with pytest.raises(rt.VpxError) as e:
        rt.mvn(x, y, True, True, 1e-9)
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT


def test_mvn_large_offset_and_constant(rt, orc, dev):
    rng = np.random.default_rng(42)
    x = (1000.0 + rng.normal(0, 1, (2, 4, 64, 64))).astype(np.float32)  # mean >> spread
    xb = orc.f32_to_f16(x)
    assert_close_f16_mvn(_mvn(rt, dev, xb, True, True, 1e-9), orc.mvn_f16(xb, True, True, 1e-9), orc, "offset 1000")
    const = orc.f32_to_f16(np.full((1, 3, 16, 16), 3.5, np.float32))
    assert np.all(_mvn(rt, dev, const, True, True, 1e-9) == 0)


def test_mvn_rejects_bad_arguments(rt, dev):
    import torch
    x = torch.zeros((2, 3, 4), dtype=torch.float16, device=dev)
    with pytest.raises(rt.VpxError) as e:
        rt.mvn(x, torch.empty_like(x), True, True, 1e-9, order="CHW")
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT
    x4 = torch.zeros((2, 3, 4, 5), dtype=torch.float32, device=dev)
    with pytest.raises(rt.VpxError) as e:
        rt.mvn(x4, torch.empty_like(x4), True, True, 1e-9)
    assert e.value.code == rt.ERROR_UNSUPPORTED_FEATURE


# ---------------------------------------------------------------------------------- seeded random shapes

def _random_shape(rng, nd, sizes, budget):
    shape = []
    for _ in range(nd):
        m = max(1, min(int(rng.choice(sizes)), budget))
        shape.append(m)
        budget //= m
    return tuple(shape)


@pytest.mark.parametrize("seed", [7, 8])
def test_random_shapes_softmax(rt, orc, dev, seed):
    rng = np.random.default_rng(seed)
    for i in range(40):
        nd = int(rng.integers(1, 5))
        shape = _random_shape(rng, nd, [1, 2, 3, 5, 8, 17, 64, 100, 257, 512, 1000, 4097], 300000)
        axis = int(rng.integers(0, nd))
        pad = int(rng.integers(0, min(4, shape[axis])))
        print("seed %d case %d: shape %s axis %d pad %d" % (seed, i, shape, axis, pad), flush=True)
        xb = orc.f32_to_f16(rng.normal(0, 3, shape).astype(np.float32))
        want = orc.softmax_f16(xb, axis, pad=pad)
        for packed in (True, False):
            got = f16_bits(_softmax(rt, dev, xb, axis, pad=pad, packed=packed))
            assert_close_f16(got.reshape(want.shape), want, orc, "softmax %s axis %d pad %d" % (shape, axis, pad))


@pytest.mark.parametrize("seed", [7, 8])
def test_random_shapes_eltwise_broadcast(rt, orc, dev, seed):
    import torch
    rng = np.random.default_rng(seed)
    for i in range(40):
        nd = int(rng.integers(1, 5))
        shape = _random_shape(rng, nd, [1, 2, 3, 7, 8, 16, 24, 56, 64, 100, 256], 400000)
        bshape = tuple(s if rng.random() < 0.5 else 1 for s in shape)
        ashape = shape if rng.random() < 0.7 else tuple(s if rng.random() < 0.5 else 1 for s in shape)
        oshape = tuple(max(a, b) for a, b in zip(ashape, bshape))
        op = str(rng.choice(["add", "sub", "mul", "prelu"]))
        print("seed %d case %d: %s %s %s" % (seed, i, op, ashape, bshape), flush=True)
        a = orc.f32_to_f16(rng.normal(0, 2, ashape).astype(np.float32))
        b = orc.f32_to_f16(rng.normal(0, 2, bshape).astype(np.float32))
        out = torch.empty(oshape, dtype=torch.float16, device=dev)
        if op == "prelu":
            rt.prelu(to_dev(a, dev, True), to_dev(b, dev, True), out)
        else:
            rt.eltwise(op, to_dev(a, dev, True), to_dev(b, dev, True), out)
        assert_f16_exact(f16_bits(out), orc.eltwise_f16(op, a, b), "%s %s %s" % (op, ashape, bshape))


@pytest.mark.parametrize("seed", [7, 8])
def test_random_shapes_mvn6(rt, orc, dev, seed):
    import torch
    rng = np.random.default_rng(seed)
    for i in range(25):
        nd = int(rng.integers(2, 5))
        shape = tuple(int(rng.choice([1, 2, 3, 8, 16, 40, 64, 128])) for _ in range(nd))
        axes = tuple(sorted(rng.choice(nd, size=int(rng.integers(1, nd + 1)), replace=False).tolist()))
        sc_shape = tuple(s if rng.random() < 0.5 else 1 for s in shape) if rng.random() < 0.6 else None
        bi_shape = tuple(s if rng.random() < 0.5 else 1 for s in shape) if rng.random() < 0.6 else None
        mode = int(rng.integers(0, 2))
        print("seed %d case %d: %s axes %s scale %s bias %s mode %d" % (seed, i, shape, axes, sc_shape, bi_shape, mode), flush=True)
        x = orc.f32_to_f16(rng.normal(0.5, 2, shape).astype(np.float32))
        sc = orc.f32_to_f16(rng.uniform(0.5, 2, sc_shape).astype(np.float32)) if sc_shape else None
        bi = orc.f32_to_f16(rng.normal(0, 1, bi_shape).astype(np.float32)) if bi_shape else None
        out = torch.empty(shape, dtype=torch.float16, device=dev)
        rt.mvn6(to_dev(x, dev, True), out, axes, True, 1e-3, mode, scale=None if sc is None else to_dev(sc, dev, True),
                bias=None if bi is None else to_dev(bi, dev, True))
        g = orc.f16_to_f32(f16_bits(out)).astype(np.float64)
        w = orc.f16_to_f32(orc.mvn6_f16(x, axes, True, 1e-3, mode, sc, bi)).astype(np.float64)
        # rows of a few elements have statistics of a few values: absolute floor for results next to zero
        assert np.all(np.abs(g - w) <= REL_TOL * np.abs(w) + 2e-4), (shape, axes, float(np.abs(g - w).max()))


@pytest.mark.parametrize("seed", [41, 42])
def test_random_shapes_quantization_family(rt, orc, dev, seed):
    """Per-axis quantize / dequantize on random ranks and axes, dynamic_dequantize with random broadcast patterns."""
    import torch
    rng = np.random.default_rng(seed)
    sizes = [1, 2, 3, 4, 7, 8, 16, 24, 40, 64, 100, 128]
    for i in range(30):
        nd = int(rng.integers(1, 5))
        shape = tuple(int(rng.choice(sizes)) for _ in range(nd))
        cands = [a for a in range(nd) if shape[a] > 1 and shape.count(shape[a]) == 1]
        if not cands:
            continue
        axis = int(rng.choice(cands))
        n = shape[axis]
        print("seed %d per-axis case %d: %s axis %d" % (seed, i, shape, axis), flush=True)
        scales, zps = rng.uniform(0.004, 0.08, n), rng.integers(-20, 21, n)
        shipped = orc.f16_to_f32(orc.f32_to_f16(scales.astype(np.float32))).astype(np.float64)
        x = orc.f32_to_f16(rng.normal(0, 3, shape).astype(np.float32))
        q = torch.empty(shape, dtype=torch.int8, device=dev)
        rt.quantize(to_dev(x, dev, True), q, scales, zps)
        want = orc.quantize(x, shipped, zps, True, axis=axis)
        assert np.array_equal(q.cpu().numpy(), want), (shape, axis)
        y = torch.empty(shape, dtype=torch.float16, device=dev)
        rt.dequantize(q, y, scales, zps)
        assert_f16_exact(f16_bits(y).reshape(-1), orc.dequantize(want, shipped, zps, axis=axis).reshape(-1), "%s axis %d" % (shape, axis))
    for i in range(30):
        nd = int(rng.integers(1, 4))
        shape = tuple(int(rng.choice(sizes)) for _ in range(nd))
        sshape = tuple(s if rng.random() < 0.5 else 1 for s in shape)
        zshape = tuple(s if rng.random() < 0.5 else 1 for s in shape) if rng.random() < 0.6 else None
        print("seed %d dynamic_dequantize case %d: %s scale %s zp %s" % (seed, i, shape, sshape, zshape), flush=True)
        q = rng.integers(-128, 128, shape).astype(np.int8)
        sc = rng.uniform(1e-3, 0.1, sshape).astype(np.float16)
        zp = None if zshape is None else rng.integers(-10, 11, zshape).astype(np.int8)
        out = torch.empty(shape, dtype=torch.float16, device=dev)
        rt.dynamic_dequantize(to_dev(q, dev), to_dev(sc, dev), out, None if zp is None else to_dev(zp, dev))
        assert_f16_exact(f16_bits(out), orc.dynamic_dequantize(q, sc.view(np.uint16), zp), "%s %s %s" % (shape, sshape, zshape))


@pytest.mark.parametrize("seed", [41, 42])
def test_random_shapes_mvn1_and_fake_quantize(rt, orc, dev, seed):
    """mvn1 and its three-step form on random 4-D shapes in both layouts; FakeQuantize with per-tensor / per-channel limits."""
    import torch
    rng = np.random.default_rng(seed)
    for i in range(30):
        N, Cc, H, W = int(rng.integers(1, 4)), int(rng.choice([1, 3, 8, 16, 64, 100])), int(rng.integers(1, 40)), int(rng.integers(1, 40))
        layout, across, nv = str(rng.choice(["NCHW", "NHWC"])), bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        print("seed %d mvn case %d: %s %s across=%s nv=%s" % (seed, i, (N, Cc, H, W), layout, across, nv), flush=True)
        x = orc.f32_to_f16((rng.uniform(-4, 4, (N, Cc, H, W)) + rng.normal(0, 2, (1, Cc, 1, 1))).astype(np.float32))
        xm = _to_layout(x, layout)
        xd = to_dev(xm, dev, True)
        out = torch.empty_like(xd)
        rt.mvn(xd, out, across, nv, 1e-4, order=layout)
        w = orc.f16_to_f32(orc.mvn_f16(xm, across, nv, 1e-4, layout=layout)).astype(np.float64)
        g = orc.f16_to_f32(f16_bits(out)).astype(np.float64)
        # groups of a handful of elements: the tolerance is relative to the normalised scale (1), not to each value
        assert np.all(np.abs(g - w) <= REL_TOL * np.abs(w) + 2e-3), float(np.abs(g - w).max())
        c = 1 if across else Cc
        sums = torch.empty((N, 1, 2 if nv else 1, c), dtype=torch.float32, device=dev)
        mv = torch.empty((N, 1, 2 if nv else 1, c), dtype=torch.float32, device=dev)
        o2 = torch.empty_like(xd)
        rt.mvn1_sum(xd, sums, across, nv, order=layout)
        rt.mvn1_mean_var(sums, mv, (N, Cc, H, W), across, nv, 1e-4)
        rt.mvn1_norm(xd, mv, o2, across, nv, order=layout)
        g2 = orc.f16_to_f32(f16_bits(o2)).astype(np.float64)
        assert np.all(np.abs(g2 - w) <= REL_TOL * np.abs(w) + 2e-3), float(np.abs(g2 - w).max())
    for i in range(20):
        N, Cc, H, W = int(rng.integers(1, 3)), int(rng.choice([1, 3, 8, 16, 64])), int(rng.integers(1, 30)), int(rng.integers(1, 30))
        per_ch, levels = bool(rng.integers(0, 2)), int(rng.choice([2, 16, 255, 256]))
        print("seed %d fake_quantize case %d: %s per_channel=%s levels=%d" % (seed, i, (N, Cc, H, W), per_ch, levels), flush=True)
        lshape = (1, Cc, 1, 1) if per_ch else (1, 1, 1, 1)
        lo, hi = -rng.uniform(0.5, 4, lshape), rng.uniform(0.5, 4, lshape)
        c = {"x": orc.f32_to_f16(rng.normal(0, 2, (N, Cc, H, W)).astype(np.float32)), "levels": levels,
             "in_lo": orc.f32_to_f16(lo.astype(np.float32)), "in_hi": orc.f32_to_f16(hi.astype(np.float32)),
             "out_lo": orc.f32_to_f16(lo.astype(np.float32)), "out_hi": orc.f32_to_f16(hi.astype(np.float32))}
        assert_f16_exact(_run_fq(rt, dev, c), orc.fake_quantize_f16(c["x"], c["in_lo"], c["in_hi"], c["out_lo"], c["out_hi"], levels),
                         "%s per_channel=%s levels=%d" % ((N, Cc, H, W), per_ch, levels))



# ---------------------------------------------------------------------------------- operator -> kernel info -> blob -> launch

def test_operator_attributes_to_launch(rt, orc, dev):
    """The compile-side chain end to end: vpx_get_kernel_info names the entry and serialises the operator's attributes
    (logical axes mapped through the tensor's order), vpx_create_kernel_params builds the blob, the kernel runs it."""
    import torch
    rng = np.random.default_rng(91)
    a = orc.f32_to_f16(rng.normal(0, 2, (2, 5, 7, 16)).astype(np.float32))   # memory order N, H, W, C
    x = to_dev(a, dev, True)

    def run(op, ins, out, order, **attrs):
        ops = [rt.Operand(t, order) for t in ins] + [rt.Operand(out, order)]
        entry, attr_bytes = rt.get_kernel_info(op, ops[0], **attrs)
        rt.sw_kernel_launch(entry, rt.create_kernel_params(ops[:-1], ops[-1:], attr_bytes), ops)
        return f16_bits(out)

    # SoftMax over the logical channel axis of an NHWC tensor: the innermost memory dimension
    got = run("SoftMax", [x], torch.empty_like(x), "NHWC", axis_ind=1)
    assert_close_f16(got, orc.softmax_f16(a, 3), orc, "softmax over C, NHWC")
    # over logical W: memory dimension 2
    got = run("SoftMax", [x], torch.empty_like(x), "NHWC", axis_ind=3)
    assert_close_f16(got, orc.softmax_f16(a, 2), orc, "softmax over W, NHWC")
    # MVN6 over logical H and W (memory dimensions 1 and 2), eps outside the root
    got = run("MVN6", [x], torch.empty_like(x), "NHWC", axes=[2, 3], normalize_variance=1, eps_mode=1, eps=1e-5)
    _assert_mvn6_close(got, orc.mvn6_f16(a, [1, 2], True, 1e-5, 1), orc, "mvn6 over H, W, NHWC")
    # MVN-1 per channel on NCHW, and an activation with two attributes
    b = orc.f32_to_f16(rng.normal(0, 2, (2, 6, 9, 8)).astype(np.float32))
    y = to_dev(b, dev, True)
    got = run("MVN", [y], torch.empty_like(y), "NCHW", across_channels=0, normalize_variance=1, eps=1e-9)
    assert_close_f16(got, orc.mvn_f16(b, False, True, 1e-9), orc, "mvn1")
    got = run("Clamp", [y], torch.empty_like(y), "NCHW", param0=-1.5, param1=0.75)
    assert_f16_exact(got, orc.activation_f16("clamp", b, -1.5, 0.75), "clamp")
    q = torch.empty(y.shape, dtype=torch.uint8, device=dev)
    ops = [rt.Operand(y), rt.Operand(q)]
    entry, attr_bytes = rt.get_kernel_info("Quantize", ops[0], scales=[0.05], zero_points=[128])
    rt.sw_kernel_launch(entry, rt.create_kernel_params(ops[:1], ops[1:], attr_bytes), ops)
    shipped = float(orc.f16_to_f32(orc.f32_to_f16(np.array([0.05], np.float32)))[0])
    assert np.array_equal(q.cpu().numpy(), orc.quantize(b, shipped, 128, False))
