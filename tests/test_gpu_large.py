"""Tensors of more than 2^31 elements (the largest an NPU address window of 4 GiB can hold is of this order):
element offsets no longer fit 32 bits.  Each kernel runs once on the whole tensor and once on three
leading-dimension parts of it, whose offsets are small; the two results must be the same bytes.  The rows at
the far end, past the 2^31st element, are also checked against the CPU oracle.  About 13 GiB of device memory."""
import numpy as np
import pytest

from test_gpu_sw import assert_close_f16, assert_f16_exact, f16_bits

pytestmark = pytest.mark.gpu

R, C = 524291, 4099          # 2 149 068 809 elements, rows not a multiple of the vector width
TAIL = 5                     # rows compared with the oracle


@pytest.fixture(scope="module")
def x(dev):
    import torch
    g = torch.Generator(device=dev)
    g.manual_seed(5)
    t = torch.empty((R, C), dtype=torch.float16, device=dev)
    t.normal_(0, 2, generator=g)
    yield t
    del t
    torch.cuda.empty_cache()


def _parts(n, k=3):
    cuts = [0] + [n * i // k + (i * 7) % 5 for i in range(1, k)] + [n]
    return list(zip(cuts[:-1], cuts[1:]))


def _bytes(t):
    import torch
    return t.view({1: torch.uint8, 2: torch.int16, 4: torch.int32}[t.element_size()])


def _whole_and_parts(run, shape, dtype, dev, n0, exact=True):
    """run(out, lo, hi) launches the kernel on [lo, hi) of the leading dimension.  Returns the whole-tensor result.
    exact=False: the parts, which start at other alignments, may take a kernel with other arithmetic -- the two
    results then agree to the tolerance of the operation instead of bit for bit."""
    import torch
    whole = torch.zeros(shape, dtype=dtype, device=dev)
    run(whole, 0, n0)
    parts = torch.zeros(shape, dtype=dtype, device=dev)
    for lo, hi in _parts(n0):
        run(parts, lo, hi)
    torch.cuda.synchronize()
    if exact:
        same = torch.equal(_bytes(whole), _bytes(parts))
    else:
        same = True
        step = 1 << 22                               # compared in pieces: no second full-size fp32 copy
        wf, pf = whole.view(-1), parts.view(-1)
        for lo in range(0, wf.numel(), step * 64):
            a, b = wf[lo:lo + step * 64].float(), pf[lo:lo + step * 64].float()
            same = same and bool(torch.allclose(a, b, rtol=2e-3, atol=2.0 ** -24))
    del parts
    assert same
    return whole


def test_large_convert(rt, orc, dev, x):
    import torch
    out = _whole_and_parts(lambda o, lo, hi: rt.convert(x[lo:hi], o[lo:hi]), (R, C), torch.float32, dev, R)
    assert np.array_equal(out[-TAIL:].cpu().numpy(), orc.f16_to_f32(f16_bits(x[-TAIL:])))


def test_large_eltwise_add(rt, orc, dev, x):
    import torch
    y = torch.roll(x[:4096], 1, 0).repeat(R // 4096 + 1, 1)[:R].contiguous()
    out = _whole_and_parts(lambda o, lo, hi: rt.eltwise("add", x[lo:hi], y[lo:hi], o[lo:hi]), (R, C), torch.float16, dev, R)
    assert_f16_exact(f16_bits(out[-TAIL:]), orc.eltwise_f16("add", f16_bits(x[-TAIL:]), f16_bits(y[-TAIL:])), "add")


def test_large_quantize_dequantize(rt, orc, dev, x):
    import torch
    scale = float(orc.f16_to_f32(orc.f32_to_f16(np.array([0.05], np.float32)))[0])
    q = _whole_and_parts(lambda o, lo, hi: rt.quantize(x[lo:hi], o[lo:hi], 0.05, 128), (R, C), torch.uint8, dev, R)
    assert np.array_equal(q[-TAIL:].cpu().numpy(), orc.quantize(f16_bits(x[-TAIL:]), scale, 128, False))
    out = _whole_and_parts(lambda o, lo, hi: rt.dequantize(q[lo:hi], o[lo:hi], 0.05, 128), (R, C), torch.float16, dev, R)
    assert_f16_exact(f16_bits(out[-TAIL:]), orc.dequantize(q[-TAIL:].cpu().numpy(), scale, 128), "dequantize")


def test_large_fake_quantize_and_activation(rt, orc, dev, x):
    import torch
    lim = [torch.tensor([[v]], dtype=torch.float16, device=dev) for v in (-4.0, 4.0, -4.0, 4.0)]
    out = _whole_and_parts(lambda o, lo, hi: rt.fake_quantize(x[lo:hi], *lim, 256, o[lo:hi]), (R, C), torch.float16, dev, R)
    lim_bits = [f16_bits(t).reshape(-1) for t in lim]
    assert_f16_exact(f16_bits(out[-TAIL:]), orc.fake_quantize_f16(f16_bits(x[-TAIL:]), *lim_bits, 256), "fake_quantize")
    del out
    out = _whole_and_parts(lambda o, lo, hi: rt.activation("hswish", x[lo:hi], o[lo:hi]), (R, C), torch.float16, dev, R)
    assert_close_f16(f16_bits(out[-TAIL:]), orc.activation_f16("hswish", f16_bits(x[-TAIL:])), orc, "hswish")


def test_large_softmax(rt, orc, dev, x):
    import torch
    out = _whole_and_parts(lambda o, lo, hi: rt.softmax(x[lo:hi], o[lo:hi], -1), (R, C), torch.float16, dev, R)
    assert_close_f16(f16_bits(out[-TAIL:]), orc.softmax_f16(f16_bits(x[-TAIL:]), 1), orc, "rows of 4099")
    del out
    rows = 4194309
    x2 = x.view(-1)[: rows * 512].view(rows, 512)
    out = _whole_and_parts(lambda o, lo, hi: rt.softmax(x2[lo:hi], o[lo:hi], -1), (rows, 512), torch.float16, dev, rows)
    assert_close_f16(f16_bits(out[-TAIL:]), orc.softmax_f16(f16_bits(x2[-TAIL:]), 1), orc, "rows of 512")
    del out
    rows = 58082940                                  # short odd rows: runs of rows through LDS
    x4 = x.view(-1)[: rows * 37].view(rows, 37)
    out = _whole_and_parts(lambda o, lo, hi: rt.softmax(x4[lo:hi], o[lo:hi], -1), (rows, 37), torch.float16, dev, rows, exact=False)
    assert_close_f16(f16_bits(out[-TAIL:]), orc.softmax_f16(f16_bits(x4[-TAIL:]), 1), orc, "rows of 37")
    del out
    x3 = x.view(-1)[: 1025 * 64 * 32760].view(1025, 64, 32760)
    out = _whole_and_parts(lambda o, lo, hi: rt.softmax(x3[lo:hi], o[lo:hi], 1), tuple(x3.shape), torch.float16, dev, 1025)
    assert_close_f16(f16_bits(out[-1:, :, -64:]), orc.softmax_f16(np.ascontiguousarray(f16_bits(x3[-1:, :, -64:])), 1), orc,
                     "middle axis")


def test_large_mvn(rt, orc, dev, x):
    import torch
    out = _whole_and_parts(lambda o, lo, hi: rt.mvn6(x[lo:hi], o[lo:hi], [-1], True, 1e-5), (R, C), torch.float16, dev, R)
    want = orc.mvn6_f16(f16_bits(x[-TAIL:]), [1], True, 1e-5, 0)
    assert_close_f16(f16_bits(out[-TAIL:]), want, orc, "mvn6 rows")
    del out
    # per channel: 139 700 groups of 124 x 124
    x2 = x.view(-1)[: 2 * 69850 * 124 * 124].view(2, 69850, 124, 124)
    out = _whole_and_parts(lambda o, lo, hi: rt.mvn(x2[lo:hi], o[lo:hi], False, True, 1e-9), tuple(x2.shape), torch.float16, dev, 2)
    want = orc.mvn_f16(f16_bits(x2[-1:, -3:]), False, True, 1e-9)
    assert_close_f16(f16_bits(out[-1:, -3:]), want, orc, "mvn1 per channel")
    del out
    # per channel, 7 x 7 planes: 43 858 547 short groups
    x4 = x.view(-1)[: 43858547 * 49].view(1, 43858547, 7, 7)
    out = torch.zeros_like(x4)
    rt.mvn(x4, out, False, True, 1e-9)
    want = orc.mvn_f16(f16_bits(x4[:, -4:]), False, True, 1e-9)
    assert_close_f16(f16_bits(out[:, -4:]), want, orc, "mvn1 short groups, far end")
    want = orc.mvn_f16(f16_bits(x4[:, :4]), False, True, 1e-9)
    assert_close_f16(f16_bits(out[:, :4]), want, orc, "mvn1 short groups, near end")
    del out
    # across channels: three groups of 7.2e8 elements, more chunks than one workgroup merges
    x3 = x.view(-1)[: 3 * 26215 * 27307].view(3, 1, 26215, 27307)
    out = _whole_and_parts(lambda o, lo, hi: rt.mvn(x3[lo:hi], o[lo:hi], True, True, 1e-9), tuple(x3.shape), torch.float16, dev, 3)
    last = out[2].view(-1)
    mean = float(last[::7].double().mean())          # every 7th value: 1e8 samples of a unit-variance result
    var = float(last[::7].double().var())
    assert abs(mean) < 1e-3 and abs(var - 1.0) < 2e-3, (mean, var)
    ref = x3[2].view(-1)[-4096:].double()
    stats = x3[2].view(-1).double()
    mu, sd = stats.mean(), stats.var(unbiased=False).sqrt()
    del stats
    assert torch.allclose(last[-4096:].double(), (ref - mu) / sd, rtol=2e-3, atol=2e-3)


def test_large_nce_eltwise_and_matmul(rt, orc, dev):
    import torch
    g = torch.Generator(device=dev)
    g.manual_seed(6)
    H, Cq = 524291, 4096
    a = torch.empty((1, H, 1, Cq), dtype=torch.int8, device=dev)
    b = torch.empty((1, H, 1, Cq), dtype=torch.int8, device=dev)
    a.random_(-128, 128, generator=g)
    b.random_(-128, 128, generator=g)
    in1_mult, in2_mult, out_mult, out_shift = rt.eltwise_quantization_approximation(0.05, 0.04, 0.07, 0)
    ppe = rt.PpeInt(rt.PPE_NOOP, -128, 127, 1, 0, out_mult, out_shift, in1_mult, in2_mult)
    out = _whole_and_parts(lambda o, lo, hi: rt.nce_eltwise(a[:, lo:hi], b[:, lo:hi], o[:, lo:hi], ppe, 3, -5, 7),
                           (1, H, 1, Cq), torch.int8, dev, H)
    want = orc.nce_eltwise(a[:, -TAIL:].cpu().numpy(), b[:, -TAIL:].cpu().numpy(), orc.ppe(1, 0, 7, -128, 127), 3, -5, in1_mult,
                           in2_mult, out_mult, out_shift, out_signed=True)
    assert np.array_equal(out[:, -TAIL:].cpu().numpy(), want)
    del a, b, out
    torch.cuda.empty_cache()

    # [1 048 640 x 64] x [64 x 2112]: 2.2e9 outputs
    M, K, N = 1048640, 64, 2112
    A = torch.empty((M, K), dtype=torch.int8, device=dev)
    B = torch.empty((N, K), dtype=torch.int8, device=dev)
    A.random_(-128, 128, generator=g)
    B.random_(-127, 128, generator=g)
    rng = np.random.default_rng(7)
    wt = rt.make_weights_table(rng.integers(2 ** 14, 2 ** 15, N), rng.integers(18, 24, N), rng.integers(-2 ** 15, 2 ** 15, N).astype(np.int32), K)
    wtd = torch.from_numpy(wt).to(dev)
    p = rt.PpeInt(rt.PPE_LPRELU, -128, 127, 1638, 14)
    want = orc.nce_matmul(A[-64:].cpu().numpy(), B.cpu().numpy(), wt, orc.ppe(1638, 14, 0, -128, 127), zp_a=3)
    # so many rows of a short K take the weights-in-registers kernel by themselves; the tile kernel when that is switched off
    for knob, kernel in ((None, "nce_gemm_regb"), ("off", "nce_gemm_mfma")):
        rt.set_tuning("VPX_GEMM_REGB", knob)
        try:
            out = _whole_and_parts(lambda o, lo, hi: rt.nce_matmul(A[lo:hi], B, wtd, o[lo:hi], p, zp_a=3), (M, N), torch.int8, dev, M)
        finally:
            rt.set_tuning("VPX_GEMM_REGB", None)
        assert rt.nce_last_kernel() == kernel
        assert np.array_equal(out[-64:].cpu().numpy(), want)
        del out
        torch.cuda.empty_cache()
