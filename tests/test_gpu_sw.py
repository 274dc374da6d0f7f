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
    if op in ("min", "max"):  # NaN handling of fmin/fmax differs between libm and the GPU; keep NaNs out
        a[is_nan16(a)] = 0x3c00
        b[is_nan16(b)] = 0xbc00
    out = torch.empty(n, dtype=torch.float16, device=dev)
    rt.eltwise(op, to_dev(a, dev, True), to_dev(b, dev, True), out)
    got, want = f16_bits(out), orc.eltwise_f16(op, a, b)
    if op in ("min", "max"):  # +0 / -0 order is unspecified for fmin/fmax
        zero = ((got | want) & 0x7fff) == 0
        got, want = got.copy(), want.copy()
        got[zero] = 0
        want[zero] = 0
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


def test_eltwise_add_f32(rt, dev):
    import torch
    rng = np.random.default_rng(25)
    a = rng.normal(0, 1, 100001).astype(np.float32)
    b = rng.normal(0, 1, 100001).astype(np.float32)
    out = torch.empty(100001, dtype=torch.float32, device=dev)
    rt.eltwise("add", to_dev(a, dev), to_dev(b, dev), out)
    assert np.array_equal(out.cpu().numpy(), a + b)


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

@pytest.mark.parametrize("signed,scale,zp", [(False, 0.02, 128), (True, 0.05, 0), (True, 0.003, -21), (False, 1 / 255, 3)])
def test_quantize_dequantize(rt, orc, dev, signed, scale, zp):
    import torch
    rng = np.random.default_rng(27)
    x = orc.f32_to_f16(np.concatenate([rng.normal(0, 3, 200001), [0.0, -0.0, 1e-4, 65504, -65504, np.inf, -np.inf]])
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
                                              ((8, 8, 3, 3), 1, "NCHW"), ((16, 64), 1, None), ((700, 3), 0, None)])
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


def test_quantize_per_axis_ambiguous_axis_is_refused(rt, dev):
    import torch
    x = torch.zeros((4, 2, 4), dtype=torch.float16, device=dev)  # two dimensions of size 4, neither is the channel
    with pytest.raises(rt.VpxError) as e:
        rt.quantize(x, torch.empty((4, 2, 4), dtype=torch.int8, device=dev), [0.1] * 4, [0] * 4)
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT
    with pytest.raises(rt.VpxError):
        rt.quantize(x, torch.empty((4, 2, 4), dtype=torch.int8, device=dev), [0.1] * 3, [0] * 3)  # no dimension of size 3


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
                                        ((65, 500), 1), ((7, 511), 1), ((130, 197), 1), ((3, 1023), 1), ((9, 4099), 1),
                                        ((3, 32768), 1), ((5, 20000), 1), ((6, 8191), 1), ((2, 33000), 1), ((2, 40001), 1),
                                        ((20000, 8), 1), ((17000, 509), 1),
                                        # outer axis with contiguous inner dimensions: every slab shape (steps x columns x waves)
                                        ((3, 12, 64), 1), ((2, 50, 8, 24), 1), ((2, 200, 520), 1), ((3, 21, 36), 1),
                                        ((2, 100, 4, 5), 1), ((1, 400, 132), 1), ((2, 40, 6), 1), ((1, 200, 30), 1),
                                        ((1, 1000, 66), 1), ((1, 1024, 2, 64), 1), ((1, 1100, 64), 1), ((2, 2, 512, 512), 2)])
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
    # argmax is preserved and a sample of rows matches the oracle
    assert bool((out.argmax(dim=-1) == x.argmax(dim=-1)).float().mean() > 0.999)
    rows = np.random.default_rng(32).integers(0, 8 * 16 * 512, 2048)
    xs = c["x"].reshape(-1, 512)[rows]
    got = f16_bits(out).reshape(-1, 512)[rows]
    assert_close_f16(got, orc.softmax_f16(xs, 1), orc, "C2 sampled rows")


def test_softmax_rejects_bad_arguments(rt, dev):
    import torch
    x = torch.zeros((4, 8), dtype=torch.float16, device=dev)
    with pytest.raises(rt.VpxError) as e:
        rt.softmax(x, torch.empty((4, 9), dtype=torch.float16, device=dev), 1)
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT
    with pytest.raises(rt.VpxError) as e:
        rt.softmax(x, torch.empty_like(x), 1, pad_size=8, packed=False)
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT


# ---------------------------------------------------------------------------------- MVN

def _mvn(rt, dev, xb, across, nv, eps, order="NCHW"):
    import torch
    x = to_dev(xb, dev, True)
    out = torch.empty_like(x)
    rt.mvn(x, out, across, nv, eps, order=order)
    return f16_bits(out)


@pytest.mark.parametrize("shape", [(2, 3, 8, 8), (1, 16, 64, 64), (3, 7, 5, 9), (2, 64, 33, 31), (1, 2, 1, 4097),
                                   (1, 600, 64, 64)])
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


@pytest.mark.parametrize("across", [True, False])
def test_mvn_nhwc(rt, orc, dev, across):
    rng = np.random.default_rng(41)
    x = (rng.uniform(-8, 8, (2, 9, 7, 70)) + rng.normal(0, 2, (1, 1, 1, 70))).astype(np.float32)  # N,H,W,C in memory
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
