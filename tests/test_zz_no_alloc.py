"""The allocation-free launch entry point (vpx_sw_kernel_launch_noalloc) against vpx_sw_kernel_launch.

Kernels that need scratch memory take it from a fixed device array instead of a hipMalloc'd block; results must be
the same bits.  Each case runs twice in a row, the second time on a smaller input (the array keeps the first call's
contents).  Collected last: a failure here must not hide the other GPU tests.
"""
import numpy as np
import pytest

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rt():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from vpux_plugin_amd import runtime
    runtime.lib()
    return runtime


def _mvn_pair(rt, shape, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = (torch.rand(shape, device="cuda", generator=g) * 16 - 8).half()
    want, got = torch.empty_like(x), torch.full_like(x, float("nan"))
    rt.mvn(x, want, True, True, 1e-9)
    rt.mvn(x, got, True, True, 1e-9, noalloc=True)
    torch.cuda.synchronize()
    return want, got


def test_mvn1_noalloc_matches_twice(rt):
    # groups of 524288 and then 16384 values: 128 and 4 chunks per group, moments pass through the scratch array
    for shape, seed in (((3, 128, 64, 64), 1), ((2, 16, 32, 32), 2)):
        want, got = _mvn_pair(rt, shape, seed)
        assert torch.equal(want.view(torch.int16), got.view(torch.int16)), shape


def test_dynamic_quantize_noalloc_matches_twice(rt):
    for n, seed in ((1 << 22, 3), (70001, 4)):
        g = torch.Generator(device="cuda").manual_seed(seed)
        x = torch.randn((n,), device="cuda", generator=g) * 3
        outs = []
        for noalloc in (False, True):
            q = torch.zeros((n,), dtype=torch.uint8, device="cuda")
            sc = torch.zeros((1,), dtype=torch.float32, device="cuda")
            zp = torch.zeros((1,), dtype=torch.uint8, device="cuda")
            rt.dynamic_quantize(x, q, sc, zp, noalloc=noalloc)
            torch.cuda.synchronize()
            outs.append((q, sc, zp))
        for a, b in zip(*outs):
            assert torch.equal(a, b), n


def test_per_axis_quantize_noalloc_matches_twice(rt):
    # a parameter set the table cache has not seen: the table is built in the scratch array
    for (rows, ch), seed in (((512, 1000), 5), ((64, 24), 6)):
        rng = np.random.default_rng(seed)
        scales = rng.uniform(0.01, 0.2, ch)
        zps = rng.integers(100, 156, ch)
        g = torch.Generator(device="cuda").manual_seed(seed)
        x = torch.randn((rows, ch), device="cuda", generator=g).half()
        want = torch.empty((rows, ch), dtype=torch.uint8, device="cuda")
        got = torch.zeros_like(want)
        rt.quantize(x, got, scales, zps, noalloc=True)
        rt.quantize(x, want, scales, zps)
        torch.cuda.synchronize()
        assert torch.equal(want, got), (rows, ch)


def test_noalloc_rejects_oversized_scratch(rt):
    # 1.6e9 values in one group are 390 625 chunks of 12-byte moments: more than the 4 MiB array; nothing is launched
    x = torch.empty((1, 1, 40000, 40000), dtype=torch.float16, device="cuda")
    with pytest.raises(rt.VpxError) as e:
        rt.mvn(x, x, True, True, 1e-9, noalloc=True)
    assert e.value.code == rt.ERROR_OUT_OF_MEMORY
    assert "allocation-free" in e.value.text
    torch.cuda.synchronize()
