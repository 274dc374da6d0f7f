"""Bit-exact parity of the NCE task (int8 convolution / matmul + integer PPE) with the CPU oracle,
through the C ABI, on a real MI355X."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def dev_t(a, dev):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def run_task(rt, orc, dev, inp, w, mults, shifts, bias, ppe_kw, zp_in=0, zp_w=0, zp_out=0, strides=(1, 1),
             pads=(0, 0, 0, 0), out_signed=False, mode=None, force=None, rows=None, out_f16=False, out_offset=None):
    """pads = (left, right, top, bottom).  Returns (gpu_out, oracle_out, kernel_name).  With out_offset the output tensor
    starts that many elements into a larger allocation, whose elements either side of it must come back untouched."""
    import torch
    OC, KY, KX, IC = w.shape
    wt = rt.make_weights_table(mults, shifts, bias, KY * KX * IC)
    assert np.array_equal(wt, orc.make_weights_table(mults, shifts, bias, KY * KX * IC))
    mode = mode if mode is not None else rt.PPE_NOOP
    p = rt.PpeInt(mode, ppe_kw["clamp_low"], ppe_kw["clamp_high"], ppe_kw.get("lrelu_mult", 1), ppe_kw.get("lrelu_shift", 0))
    pm, ps = {rt.PPE_NOOP: (1, 0), rt.PPE_LRELU: (0, 0), rt.PPE_LRELUX: (0, 0),
              rt.PPE_LPRELU: (p.lrelu_mult, p.lrelu_shift)}[mode]
    op = orc.ppe(pm, ps, zp_out, p.clamp_low, p.clamp_high)
    N, H, W, _ = inp.shape
    OH = (H + pads[2] + pads[3] - KY) // strides[0] + 1
    OW = (W + pads[0] + pads[1] - KX) // strides[1] + 1
    odt = torch.float16 if out_f16 else (torch.int8 if out_signed else torch.uint8)
    if out_offset is None:
        out = torch.full((N, OH, OW, OC), 77, dtype=odt, device=dev)
    else:
        whole = torch.full((out_offset + N * OH * OW * OC + 64,), 77, dtype=odt, device=dev)
        out = whole[out_offset:out_offset + N * OH * OW * OC].view(N, OH, OW, OC)
    if force in ("regw", "tile", "stream"):  # the LDS-patch kernels only, starting the choice at this one
        rt.set_tuning("VPX_CONV_KERNEL", force)
        rt.set_tuning("VPX_NCE_KERNEL", "conv")
    elif force:
        rt.set_tuning("VPX_NCE_KERNEL", force)
    try:
        rt.nce_task(dev_t(inp, dev), dev_t(w, dev), dev_t(wt, dev), out, p, zp_in=zp_in, zp_w=zp_w, zp_out=zp_out,
                    strides=strides, pads=pads)
        torch.cuda.synchronize()
    finally:
        rt.set_tuning("VPX_NCE_KERNEL", None)
        rt.set_tuning("VPX_CONV_KERNEL", None)
    want = orc.nce_conv(inp, w, wt, op, zp_in=zp_in, zp_w=zp_w, strides=strides,
                        pads=(pads[2], pads[0], pads[3], pads[1]), out_signed=out_signed, rows=rows, out_f16=out_f16)
    got = out.cpu().numpy()
    if out_offset is not None:
        assert bool((whole[:out_offset] == 77).all()) and bool((whole[out_offset + out.numel():] == 77).all()), "wrote outside the output"
    return (got.view(np.uint16) if out_f16 else got), want, rt.nce_last_kernel()


def rand_case(rng, N, H, W, IC, OC, KY, KX, in_u8=True, w_u8=False, shift_lo=12, shift_hi=20):
    inp = rng.integers(0, 256, (N, H, W, IC), dtype=np.uint8) if in_u8 else rng.integers(-128, 128, (N, H, W, IC)).astype(np.int8)
    w = rng.integers(0, 256, (OC, KY, KX, IC), dtype=np.uint8) if w_u8 else rng.integers(-127, 128, (OC, KY, KX, IC)).astype(np.int8)
    mults = rng.integers(2 ** 14, 2 ** 15, OC)
    shifts = rng.integers(shift_lo, shift_hi, OC)
    bias = rng.integers(-2 ** 15, 2 ** 15, OC).astype(np.int32)
    return inp, w, mults, shifts, bias


def patch_kernel(g):
    """The LDS-patch kernel a layer of 64 or 128 input channels takes when asked for the weights-in-registers kernel:
    that one serves 3x3 taps of 64 channels (by itself the dispatcher picks it from about 50 000 output positions on)."""
    return "nce_conv_regw" if (g["IC"], g["KY"], g["KX"]) == (64, 3, 3) else "nce_conv_tile"


# kernels the dispatcher picks only when asked to (or, the first, from a size on): the knob that asks
FORCE_FOR = {"nce_conv_regw": "regw", "nce_conv_mfma16": "gather", "nce_conv_mfma": "gather"}

U8 = {"clamp_low": 0, "clamp_high": 255}
I8 = {"clamp_low": -128, "clamp_high": 127}


@pytest.mark.parametrize("force", [None, "regw", "stream", "gather", "naive"])
@pytest.mark.parametrize("geom", [
    dict(N=2, H=9, W=11, IC=64, OC=64, KY=3, KX=3, strides=(1, 1), pads=(1, 1, 1, 1)),
    dict(N=1, H=14, W=14, IC=32, OC=48, KY=3, KX=3, strides=(2, 2), pads=(0, 1, 0, 1)),
    dict(N=3, H=8, W=5, IC=64, OC=70, KY=1, KX=3, strides=(1, 1), pads=(1, 0, 0, 0)),
    dict(N=1, H=20, W=20, IC=64, OC=32, KY=5, KX=5, strides=(1, 2), pads=(2, 2, 2, 2)),
    dict(N=2, H=30, W=40, IC=128, OC=96, KY=3, KX=3, strides=(1, 1), pads=(1, 1, 1, 1)),
    dict(N=1, H=33, W=70, IC=64, OC=16, KY=3, KX=2, strides=(2, 1), pads=(0, 1, 2, 0)),
    # K too large for the weights of 64 channels to sit in LDS at once: staged a slice at a time
    dict(N=1, H=9, W=9, IC=256, OC=96, KY=3, KX=3, strides=(1, 1), pads=(1, 1, 1, 1)),
    dict(N=1, H=8, W=8, IC=1536, OC=32, KY=1, KX=1, strides=(2, 2), pads=(0, 0, 0, 0)),
    # channel counts that are a multiple of 16 only (stem layers): two taps can share an MFMA step, odd tap counts
    dict(N=2, H=30, W=30, IC=16, OC=64, KY=7, KX=7, strides=(2, 2), pads=(3, 3, 3, 3)),
    dict(N=1, H=10, W=12, IC=48, OC=40, KY=3, KX=3, strides=(1, 1), pads=(1, 1, 1, 1)),
])
def test_conv_paths(rt, orc, dev, geom, force):
    g = dict(geom)
    strides, pads = g.pop("strides"), g.pop("pads")
    tile = g["IC"] in (64, 128)
    lds = g["IC"] % 64 == 0
    gather = "nce_conv_mfma" if g["IC"] % 32 == 0 else "nce_conv_mfma16"
    # (channel counts that are a multiple of 16 but not of 64: the row-patch kernel wherever an LDS kernel may run)
    other = gather if g["IC"] % 64 == 0 else "nce_conv_rows16"
    # (a 1x1 layer without padding is a matmul, with or without a stride, unless its few channels suit the 64-wide tiles better)
    M = g["N"] * ((g["H"] - 1) // strides[0] + 1) * ((g["W"] - 1) // strides[1] + 1)
    matmul = (g["KY"], g["KX"]) == (1, 1) and pads == (0, 0, 0, 0) and g["IC"] % 64 == 0 and (g["OC"] > 64 or (g["OC"] > 48 and g["IC"] >= 192) or M < 1024)
    expect = {None: "nce_gemm_mfma" if matmul else ("nce_conv_tile" if tile else ("nce_conv_stream" if lds else other)),
              "regw": patch_kernel(g) if tile else ("nce_conv_stream" if lds else other),
              "stream": "nce_conv_stream" if lds else other,
              "gather": gather, "naive": "nce_conv_naive"}[force]
    rng = np.random.default_rng(50 + g["H"])
    for in_u8, zp_in, out_signed in ((True, 128, False), (True, 7, True), (False, -5, False), (False, 0, True)):
        inp, w, mults, shifts, bias = rand_case(rng, in_u8=in_u8, **g)
        got, want, name = run_task(rt, orc, dev, inp, w, mults, shifts, bias, I8 if out_signed else U8, zp_in=zp_in,
                                   strides=strides, pads=pads, out_signed=out_signed, force=force)
        assert name == expect
        assert np.array_equal(got, want), "%s zp_in=%d: %d mismatches" % (name, zp_in, int((got != want).sum()))


@pytest.mark.parametrize("geom", [
    dict(N=2, H=17, W=13, IC=128, OC=200, strides=(2, 2)),
    dict(N=3, H=9, W=30, IC=64, OC=70, strides=(1, 2)),
    dict(N=1, H=41, W=7, IC=320, OC=513, strides=(3, 1)),
    dict(N=2, H=56, W=56, IC=256, OC=512, strides=(2, 2)),
])
def test_strided_1x1_layers_take_the_matmul_kernel(rt, orc, dev, geom):
    """A 1x1 convolution with a stride (the shortcut branches of a ResNet) is a matmul over rows picked from the input."""
    g = dict(geom)
    strides = g.pop("strides")
    rng = np.random.default_rng(77 + g["H"])
    for in_u8, zp_in, zp_w, out_signed in ((True, 128, 0, False), (True, 9, 0, True), (False, -5, 0, False), (True, 128, 31, False)):
        inp, w, mults, shifts, bias = rand_case(rng, in_u8=in_u8, KY=1, KX=1, **g)
        kw = dict(I8 if out_signed else U8, lrelu_mult=1638, lrelu_shift=14)
        got, want, name = run_task(rt, orc, dev, inp, w, mults, shifts, bias, kw, zp_in=zp_in, zp_w=zp_w, zp_out=4, strides=strides,
                                   out_signed=out_signed, mode=rt.PPE_LPRELU)
        assert name == "nce_gemm_mfma"
        assert np.array_equal(got, want), "zp_in=%d zp_w=%d: %d mismatches" % (zp_in, zp_w, int((got != want).sum()))


@pytest.mark.parametrize("rows", [1, 2, 3, 5])
@pytest.mark.parametrize("force,kernel", [("regw", "nce_conv_regw"), (None, "nce_conv_tile"), ("stream", "nce_conv_stream")])
def test_conv_patch_tile_heights(rt, orc, dev, rows, force, kernel):
    """The LDS-patch kernels with the tile height forced: tiles that end past the last output row, one-row tiles."""
    rng = np.random.default_rng(55 + rows)
    inp, w, mults, shifts, bias = rand_case(rng, 2, 13, 24, 64, 80, 3, 3)
    rt.set_tuning("VPX_CONV_ROWS", rows)
    try:
        got, want, name = run_task(rt, orc, dev, inp, w, mults, shifts, bias, U8, zp_in=121, zp_out=3,
                                   strides=(1, 1), pads=(1, 1, 1, 1), force=force)
    finally:
        rt.set_tuning("VPX_CONV_ROWS", None)
    assert name == kernel
    assert np.array_equal(got, want), "%d mismatches" % int((got != want).sum())


@pytest.mark.parametrize("ksplit", ["on", "off"])
@pytest.mark.parametrize("geom", [
    # 7 x 7 planes, slices of eight K steps: eight waves, eight shares of K
    dict(N=3, H=7, W=7, IC=512, OC=128, KY=3, KX=3, strides=(1, 1), pads=(1, 1, 1, 1)),
    dict(N=2, H=14, W=14, IC=256, OC=96, KY=3, KX=3, strides=(2, 2), pads=(1, 1, 1, 1)),
    # slices of four K steps: four waves, a quarter each
    dict(N=2, H=8, W=6, IC=128, OC=64, KY=3, KX=3, strides=(1, 1), pads=(1, 1, 1, 1)),
    dict(N=1, H=5, W=9, IC=384, OC=200, KY=2, KX=3, strides=(1, 1), pads=(1, 0, 0, 1)),
    # up to 128 positions a tile: two groups of four waves
    dict(N=2, H=14, W=14, IC=256, OC=64, KY=3, KX=3, strides=(1, 1), pads=(1, 1, 1, 1)),
    dict(N=1, H=9, W=11, IC=768, OC=70, KY=1, KX=1, strides=(1, 1), pads=(1, 1, 0, 0)),
])
def test_streamed_weights_k_split(rt, orc, dev, geom, ksplit):
    """Small planes in the streamed-weights kernel: the waves of a group split the K steps of every weight slice over a
    64 x 64 tile and add their partial sums in LDS (the default), against the same kernel with one 32 x 32 tile per wave."""
    g = dict(geom)
    strides, pads = g.pop("strides"), g.pop("pads")
    rng = np.random.default_rng(90 + g["H"] + g["IC"])
    rt.set_tuning("VPX_STREAM_KSPLIT", None if ksplit == "on" else "off")
    try:
        for in_u8, zp_in, zp_w, w_u8, out_signed, mode, zp_out in ((True, 128, 0, False, False, rt.PPE_LRELU, 0), (True, 9, 131, True, True, rt.PPE_LPRELU, 3),
                                                                   (False, -5, 0, False, False, rt.PPE_NOOP, 4), (False, 0, -7, False, True, rt.PPE_LPRELU, -2)):
            inp, w, mults, shifts, bias = rand_case(rng, in_u8=in_u8, w_u8=w_u8, **g)
            K = w[0].size
            bias = (bias - np.int64(round(K * (inp.mean() - zp_in) * (w.mean() - zp_w)))).astype(np.int32)
            kw = dict(I8 if out_signed else U8, lrelu_mult=1638, lrelu_shift=14)
            got, want, name = run_task(rt, orc, dev, inp, w, mults, shifts, bias, kw, zp_in=zp_in, zp_w=zp_w, zp_out=zp_out, strides=strides,
                                       pads=pads, out_signed=out_signed, mode=mode, force="stream")
            assert name == "nce_conv_stream"
            assert np.array_equal(got, want), "zp_in=%d zp_w=%d: %d mismatches" % (zp_in, zp_w, int((got != want).sum()))
    finally:
        rt.set_tuning("VPX_STREAM_KSPLIT", None)


def test_naive_path_covers_odd_shapes_and_weight_zero_points(rt, orc, dev):
    rng = np.random.default_rng(60)
    inp, w, mults, shifts, bias = rand_case(rng, 2, 6, 7, 5, 9, 3, 2, in_u8=True, w_u8=True)
    got, want, name = run_task(rt, orc, dev, inp, w, mults, shifts, bias, U8, zp_in=100, zp_w=120, zp_out=10,
                               strides=(1, 1), pads=(1, 0, 1, 0))
    assert name == "nce_conv_naive" and np.array_equal(got, want)


@pytest.mark.parametrize("geom,kernel", [
    (dict(N=2, H=9, W=11, IC=64, OC=64, KY=3, KX=3, strides=(1, 1), pads=(1, 1, 1, 1)), "nce_conv_regw"),
    (dict(N=2, H=9, W=11, IC=64, OC=64, KY=3, KX=3, strides=(1, 1), pads=(1, 1, 1, 1)), "nce_conv_tile"),
    (dict(N=1, H=9, W=9, IC=256, OC=96, KY=3, KX=3, strides=(1, 1), pads=(1, 1, 1, 1)), "nce_conv_stream"),
    (dict(N=1, H=14, W=14, IC=32, OC=48, KY=3, KX=3, strides=(2, 2), pads=(0, 1, 0, 1)), "nce_conv_mfma"),
    (dict(N=1, H=14, W=14, IC=32, OC=48, KY=3, KX=3, strides=(2, 2), pads=(0, 1, 0, 1)), "nce_conv_rows16"),
    (dict(N=1, H=12, W=12, IC=16, OC=32, KY=3, KX=3, strides=(1, 1), pads=(1, 1, 1, 1)), "nce_conv_rows16"),
    (dict(N=1, H=12, W=12, IC=16, OC=32, KY=3, KX=3, strides=(1, 1), pads=(1, 1, 1, 1)), "nce_conv_mfma16"),
    (dict(N=1, H=300, W=1, IC=128, OC=520, KY=1, KX=1, strides=(1, 1), pads=(0, 0, 0, 0)), "nce_gemm_mfma"),
])
def test_unsigned_weights_around_128_take_the_mfma_kernels(rt, orc, dev, geom, kernel):
    """u8 weights with zero point 128 are signed weights in unsigned storage: re-biased copy, same kernels."""
    rng = np.random.default_rng(63)
    g = dict(geom)
    strides, pads = g.pop("strides"), g.pop("pads")
    for in_u8, zp_in in ((True, 128), (True, 7), (False, -5)):
        inp, w, mults, shifts, bias = rand_case(rng, in_u8=in_u8, w_u8=True, **g)
        got, want, name = run_task(rt, orc, dev, inp, w, mults, shifts, bias, U8, zp_in=zp_in, zp_w=128, zp_out=3,
                                   strides=strides, pads=pads, force=FORCE_FOR.get(kernel))
        assert name == kernel
        assert np.array_equal(got, want), "%s zp_in=%d: %d mismatches" % (kernel, zp_in, int((got != want).sum()))


WEIGHT_ZP_GEOMS = [
    (dict(N=2, H=9, W=11, IC=64, OC=64, KY=3, KX=3, strides=(1, 1), pads=(1, 1, 1, 1)), "nce_conv_regw"),
    (dict(N=2, H=9, W=11, IC=64, OC=64, KY=3, KX=3, strides=(1, 1), pads=(1, 1, 1, 1)), "nce_conv_tile"),
    (dict(N=2, H=15, W=10, IC=128, OC=40, KY=3, KX=3, strides=(1, 1), pads=(1, 0, 0, 1)), "nce_conv_tile"),
    (dict(N=1, H=9, W=9, IC=256, OC=96, KY=3, KX=3, strides=(1, 1), pads=(1, 1, 1, 1)), "nce_conv_stream"),
    (dict(N=2, H=17, W=13, IC=64, OC=64, KY=3, KX=3, strides=(2, 2), pads=(1, 1, 1, 1)), "nce_conv_regw"),
    (dict(N=2, H=17, W=13, IC=64, OC=64, KY=3, KX=3, strides=(2, 2), pads=(1, 1, 1, 1)), "nce_conv_tile"),
    (dict(N=2, H=12, W=13, IC=64, OC=64, KY=3, KX=2, strides=(2, 1), pads=(1, 1, 1, 1)), "nce_conv_tile"),
    (dict(N=1, H=14, W=14, IC=32, OC=48, KY=3, KX=3, strides=(2, 2), pads=(0, 1, 0, 1)), "nce_conv_mfma"),
    (dict(N=1, H=14, W=14, IC=32, OC=48, KY=3, KX=3, strides=(2, 2), pads=(0, 1, 0, 1)), "nce_conv_rows16"),
    (dict(N=1, H=12, W=12, IC=16, OC=32, KY=3, KX=3, strides=(1, 1), pads=(1, 1, 1, 1)), "nce_conv_rows16"),
    (dict(N=1, H=12, W=12, IC=16, OC=32, KY=3, KX=3, strides=(1, 1), pads=(1, 1, 1, 1)), "nce_conv_mfma16"),
    (dict(N=3, H=40, W=10, IC=64, OC=64, KY=1, KX=1, strides=(1, 1), pads=(0, 0, 0, 0)), "nce_conv_tile"),
    (dict(N=1, H=300, W=1, IC=128, OC=520, KY=1, KX=1, strides=(1, 1), pads=(0, 0, 0, 0)), "nce_gemm_mfma"),
    (dict(N=1, H=777, W=1, IC=1024, OC=300, KY=1, KX=1, strides=(1, 1), pads=(0, 0, 0, 0)), "nce_gemm_mfma"),
    (dict(N=1, H=515, W=1, IC=4160, OC=260, KY=1, KX=1, strides=(1, 1), pads=(0, 0, 0, 0)), "nce_gemm_mfma"),
]


@pytest.mark.parametrize("geom,kernel", WEIGHT_ZP_GEOMS, ids=["%s-%dx%d-ic%d" % (k, g["KY"], g["KX"], g["IC"]) for g, k in WEIGHT_ZP_GEOMS])
def test_weight_zero_points_take_the_mfma_kernels(rt, orc, dev, geom, kernel):
    """Asymmetric weights (mpe_wtbias): the part of the zero point that the signed re-biased copy does not absorb
    enters as one term per output position -- the sum of (activation - zero point) under its window."""
    rng = np.random.default_rng(64)
    g = dict(geom)
    strides, pads = g.pop("strides"), g.pop("pads")
    for in_u8, w_u8, zp_in, zp_w, signed_out in ((True, True, 128, 127, False), (True, True, 3, 255, True), (False, True, -7, 0, False),
                                                 (True, False, 200, -9, True), (False, False, 11, 127, False), (True, True, 128, 77, False)):
        inp, w, mults, shifts, bias = rand_case(rng, in_u8=in_u8, w_u8=w_u8, **g)
        # both zero points shift the accumulators by a large common value: the bias takes it out again and the
        # shifts follow what is left, so that the outputs use the whole range and both PReLU branches
        K = w[0].size
        centre = K * (inp.mean() - zp_in) * (w.mean() - zp_w)
        spread = 3 * np.sqrt(K) * (inp.std() + abs(inp.mean() - zp_in)) * (w.std() + abs(w.mean() - zp_w)) / 2
        bias = (bias - np.int64(round(centre))).astype(np.int32)
        shifts = rng.integers(0, 3, len(shifts)) + max(1, int(np.ceil(np.log2(spread * 2 ** 15 / 128))))
        kw = dict(I8 if signed_out else U8, lrelu_mult=1638, lrelu_shift=14)
        got, want, name = run_task(rt, orc, dev, inp, w, mults, shifts, bias, kw, zp_in=zp_in, zp_w=zp_w, zp_out=-3 if signed_out else 9,
                                   strides=strides, pads=pads, out_signed=signed_out, mode=rt.PPE_LPRELU,
                                   force=FORCE_FOR.get(kernel))
        assert name == kernel
        assert np.array_equal(got, want), "%s zp_in=%d zp_w=%d: %d mismatches" % (kernel, zp_in, zp_w, int((got != want).sum()))
        assert len(np.unique(got)) > 20  # the outputs are spread, not saturated


@pytest.mark.parametrize("geom,kernel", [
    (dict(N=2, H=9, W=11, IC=64, OC=64, KY=3, KX=3, strides=(1, 1), pads=(1, 1, 1, 1)), "nce_conv_regw"),
    (dict(N=2, H=9, W=11, IC=64, OC=64, KY=3, KX=3, strides=(1, 1), pads=(1, 1, 1, 1)), "nce_conv_tile"),
    (dict(N=1, H=9, W=9, IC=256, OC=96, KY=3, KX=3, strides=(1, 1), pads=(1, 1, 1, 1)), "nce_conv_stream"),
    (dict(N=1, H=14, W=14, IC=32, OC=48, KY=3, KX=3, strides=(2, 2), pads=(0, 1, 0, 1)), "nce_conv_mfma"),
    (dict(N=1, H=14, W=14, IC=32, OC=48, KY=3, KX=3, strides=(2, 2), pads=(0, 1, 0, 1)), "nce_conv_rows16"),
    (dict(N=1, H=300, W=1, IC=128, OC=520, KY=1, KX=1, strides=(1, 1), pads=(0, 0, 0, 0)), "nce_gemm_mfma"),
    (dict(N=1, H=700, W=1, IC=512, OC=300, KY=1, KX=1, strides=(1, 1), pads=(0, 0, 0, 0)), "nce_gemm_mfma"),
])
@pytest.mark.parametrize("mode", ["NOOP", "LPRELU", "LRELU"])
def test_negative_multipliers(rt, orc, dev, geom, kernel, mode):
    """Channels whose multiplier is negative (a negative weight scale): the scaled value changes sign, and with it the
    branch of the PReLU stage a given accumulator takes."""
    rng = np.random.default_rng(66)
    g = dict(geom)
    strides, pads = g.pop("strides"), g.pop("pads")
    inp, w, mults, shifts, bias = rand_case(rng, in_u8=True, **g)
    mults = np.where(rng.random(mults.shape) < 0.5, -mults, mults)
    kw = dict(I8, lrelu_mult=1638, lrelu_shift=14)
    got, want, name = run_task(rt, orc, dev, inp, w, mults, shifts, bias, kw, zp_in=120, zp_out=-3, strides=strides, pads=pads,
                               out_signed=True, mode=getattr(rt, "PPE_" + mode), force=FORCE_FOR.get(kernel))
    assert name == kernel
    assert np.array_equal(got, want), "%s %s: %d mismatches" % (kernel, mode, int((got != want).sum()))


@pytest.mark.parametrize("seed,weight_zp", [(1234, False), (99, False), (7, True), (8, True)])
def test_conv_random_geometries(rt, orc, dev, seed, weight_zp):
    """Thirty seeded draws of shape, kernel, stride, padding, types, zero points and PPE mode, whichever kernel they select;
    the last two seeds also draw the weight storage type and a weight zero point."""
    rng = np.random.default_rng(seed)
    for i in range(30):
        IC = int(rng.choice([16, 32, 48, 64, 64, 96, 128, 128, 192, 256, 320, 512]))
        OC = int(rng.integers(1, 200))
        KY, KX = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        SY, SX = int(rng.integers(1, 3)), int(rng.integers(1, 3))
        pl, pr, pt, pb = [int(v) for v in rng.integers(0, 3, 4)]
        pl, pr, pt, pb = min(pl, KX - 1), min(pr, KX - 1), min(pt, KY - 1), min(pb, KY - 1)
        H, W, N = int(rng.integers(KY, 40)), int(rng.integers(KX, 70)), int(rng.integers(1, 4))
        in_u8, out_signed = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        zp_in = int(rng.integers(0, 256)) if in_u8 else int(rng.integers(-128, 128))
        mode = [rt.PPE_NOOP, rt.PPE_LPRELU, rt.PPE_LRELU][int(rng.integers(0, 3))]
        kw = dict(I8 if out_signed else U8, lrelu_mult=int(rng.integers(0, 2048)), lrelu_shift=int(rng.integers(0, 20)))
        what = "seed %d case %d: N=%d H=%d W=%d IC=%d OC=%d K=%dx%d S=%dx%d pads=%s in_u8=%s out_signed=%s zp_in=%d mode=%d" % (
            seed, i, N, H, W, IC, OC, KY, KX, SY, SX, (pl, pr, pt, pb), in_u8, out_signed, zp_in, mode)
        print(what, flush=True)
        w_u8, zp_w = False, 0
        if weight_zp:
            w_u8 = bool(rng.integers(0, 2))
            zp_w = int(rng.integers(0, 256)) if w_u8 else int(rng.integers(-128, 128))
            what += " w_u8=%s zp_w=%d" % (w_u8, zp_w)
        inp, w, mults, shifts, bias = rand_case(rng, N, H, W, IC, OC, KY, KX, in_u8=in_u8, w_u8=w_u8, shift_lo=14, shift_hi=26)
        if weight_zp:  # take the common offset of the accumulators out again, so that the outputs are not saturated
            bias = (bias - np.int64(round(KY * KX * IC * (inp.mean() - zp_in) * (w.mean() - zp_w)))).astype(np.int32)
        got, want, name = run_task(rt, orc, dev, inp, w, mults, shifts, bias, kw, zp_in=zp_in, zp_w=zp_w, zp_out=int(rng.integers(-5, 6)),
                                   strides=(SY, SX), pads=(pl, pr, pt, pb), out_signed=out_signed, mode=mode)
        # (16-channel granularity is served up to K = 1008, the weights of 64 channels in 64 KiB of LDS)
        assert name != "nce_conv_naive" or (IC % 32 != 0 and KY * KX * IC > 1008), what
        assert np.array_equal(got, want), "%s (%s): %d mismatches" % (what, name, int((got != want).sum()))


@pytest.mark.parametrize("seed", [3, 4, 5])
def test_weights_in_registers_conv_random_geometries(rt, orc, dev, seed):
    """The 3x3 x 64-channel kernel that keeps the weights in registers, asked for whatever the layer's size: seeded draws
    of batch, size, stride, padding, channel count (tails of the 64- and 16-channel blocks), tile height, storage types,
    zero points (weights too: the per-position term) and PPE settings on both sides of the short requantisation's
    conditions (slope above 1, odd output zero point, scales above 1/2)."""
    rng = np.random.default_rng(seed)
    for i in range(24):
        OC = int(rng.choice([1, 15, 16, 40, 64, 64, 72, 100, 128, 130]))
        SY, SX = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        pl, pr, pt, pb = [int(v) for v in rng.integers(0, 3, 4)]
        H, W, N = int(rng.integers(3, 45)), int(rng.integers(3, 75)), int(rng.integers(1, 4))
        in_u8, out_signed = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        zp_in = int(rng.integers(0, 256)) if in_u8 else int(rng.integers(-128, 128))
        mode = [rt.PPE_NOOP, rt.PPE_LPRELU, rt.PPE_LRELU][int(rng.integers(0, 3))]
        # slopes: 0, inside (0, 1), exactly 1, above 1 (the multiplier field is unsigned)
        lm, ls = [(0, 0), (1638, 14), (int(rng.integers(1, 2048)), 11), (4, 2), (5, 1), (2047, 3)][int(rng.integers(0, 6))]
        kw = dict(I8 if out_signed else U8, lrelu_mult=lm, lrelu_shift=ls)
        shift_lo, shift_hi = [(14, 26), (10, 16)][int(rng.integers(0, 2))]  # the second range holds scales above 1/2
        w_u8, zp_w = False, 0
        if rng.integers(0, 3) == 0:
            w_u8 = bool(rng.integers(0, 2))
            zp_w = int(rng.integers(0, 256)) if w_u8 else int(rng.integers(-128, 128))
        rows = int(rng.integers(0, 6))  # 0: the dispatcher's choice
        what = "seed %d case %d: N=%d H=%d W=%d OC=%d S=%dx%d pads=%s in_u8=%s out_signed=%s zp_in=%d mode=%d slope=%d/2^%d shifts=%d..%d w_u8=%s zp_w=%d rows=%d" % (
            seed, i, N, H, W, OC, SY, SX, (pl, pr, pt, pb), in_u8, out_signed, zp_in, mode, lm, ls, shift_lo, shift_hi, w_u8, zp_w, rows)
        print(what, flush=True)
        inp, w, mults, shifts, bias = rand_case(rng, N, H, W, 64, OC, 3, 3, in_u8=in_u8, w_u8=w_u8, shift_lo=shift_lo, shift_hi=shift_hi)
        if rng.integers(0, 2):
            mults = np.where(rng.random(mults.shape) < 0.5, -mults, mults)
        bias = (bias - np.int64(round(576 * (inp.mean() - zp_in) * (w.mean() - zp_w)))).astype(np.int32)
        if rows:
            rt.set_tuning("VPX_CONV_ROWS", rows)
        try:
            got, want, name = run_task(rt, orc, dev, inp, w, mults, shifts, bias, kw, zp_in=zp_in, zp_w=zp_w, zp_out=int(rng.integers(-5, 6)),
                                       strides=(SY, SX), pads=(pl, pr, pt, pb), out_signed=out_signed, mode=mode, force="regw")
        finally:
            rt.set_tuning("VPX_CONV_ROWS", None)
        # (weights whose zero point a signed copy cannot absorb with M % 4 != 0 positions, and the like, may take other kernels)
        if zp_w == 0:
            assert name == "nce_conv_regw", what
        assert np.array_equal(got, want), "%s (%s): %d mismatches" % (what, name, int((got != want).sum()))


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_row_patch_conv_random_geometries(rt, orc, dev, seed):
    """The stem-layer kernel (channel counts that are a multiple of 16 but not of 64; input rows resident in LDS, K walked kernel row
    in its natural order, two 16-byte chunks a step): seeded draws of channel count (one, three, five and seven chunks a
    pixel), kernel size up to 7x7 (steps that straddle two kernel rows, odd chunk counts), stride, padding, output channels (tails of the 64- and
    16-channel blocks), tile height and width, storage types, zero points (weights too) and PPE settings on both sides of the
    short requantisation's conditions."""
    rng = np.random.default_rng(seed)
    for i in range(24):
        IC = int(rng.choice([16, 16, 16, 48, 80, 112, 32, 96, 160]))
        OC = int(rng.choice([1, 15, 16, 32, 40, 64, 64, 72, 100, 128, 130, 250, 256]))  # (120 .. 128 of 128, 240 .. 256: blocks of 128 channels where K is short)
        KY, KX = int(rng.integers(1, 8)), int(rng.integers(1, 8))
        SY, SX = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        pl, pr, pt, pb = [int(v) for v in rng.integers(0, 4, 4)]
        pl, pr, pt, pb = min(pl, KX - 1), min(pr, KX - 1), min(pt, KY - 1), min(pb, KY - 1)
        H, W, N = int(rng.integers(KY, 45)), int(rng.integers(KX, 75)), int(rng.integers(1, 4))
        in_u8, out_signed = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        zp_in = int(rng.integers(0, 256)) if in_u8 else int(rng.integers(-128, 128))
        mode = [rt.PPE_NOOP, rt.PPE_LPRELU, rt.PPE_LRELU][int(rng.integers(0, 3))]
        lm, ls = [(0, 0), (1638, 14), (int(rng.integers(1, 2048)), 11), (4, 2), (5, 1), (2047, 3)][int(rng.integers(0, 6))]
        kw = dict(I8 if out_signed else U8, lrelu_mult=lm, lrelu_shift=ls)
        shift_lo, shift_hi = [(14, 26), (10, 16)][int(rng.integers(0, 2))]  # the second range holds scales above 1/2
        w_u8, zp_w = False, 0
        if rng.integers(0, 3) == 0:
            w_u8 = bool(rng.integers(0, 2))
            zp_w = int(rng.integers(0, 256)) if w_u8 else int(rng.integers(-128, 128))
        rows = int(rng.integers(0, 6))  # 0: the dispatcher's choice
        cols = int(rng.choice([0, 0, 7, 20, 33]))  # output columns per tile; 0: the dispatcher's choice (the whole width where it fits)
        what = "seed %d case %d: N=%d H=%d W=%d IC=%d OC=%d K=%dx%d S=%dx%d pads=%s in_u8=%s out_signed=%s zp_in=%d mode=%d slope=%d/2^%d shifts=%d..%d w_u8=%s zp_w=%d rows=%d cols=%d" % (
            seed, i, N, H, W, IC, OC, KY, KX, SY, SX, (pl, pr, pt, pb), in_u8, out_signed, zp_in, mode, lm, ls, shift_lo, shift_hi, w_u8, zp_w, rows, cols)
        print(what, flush=True)
        inp, w, mults, shifts, bias = rand_case(rng, N, H, W, IC, OC, KY, KX, in_u8=in_u8, w_u8=w_u8, shift_lo=shift_lo, shift_hi=shift_hi)
        if rng.integers(0, 2):
            mults = np.where(rng.random(mults.shape) < 0.5, -mults, mults)
        bias = (bias - np.int64(round(KY * KX * IC * (inp.mean() - zp_in) * (w.mean() - zp_w)))).astype(np.int32)
        if rows:
            rt.set_tuning("VPX_CONV_ROWS", rows)
        if cols:
            rt.set_tuning("VPX_CONV_COLS", cols)
        try:
            got, want, name = run_task(rt, orc, dev, inp, w, mults, shifts, bias, kw, zp_in=zp_in, zp_w=zp_w, zp_out=int(rng.integers(-5, 6)),
                                       strides=(SY, SX), pads=(pl, pr, pt, pb), out_signed=out_signed, mode=mode)
        finally:
            rt.set_tuning("VPX_CONV_ROWS", None)
            rt.set_tuning("VPX_CONV_COLS", None)
        # (the kernel wants the weights of 64 channels and the input rows under one output row in LDS together; layers
        # beyond that take the gather or the plain kernel)
        OW = (W + pl + pr - KX) // SX + 1
        steps, m = (KY * KX * IC // 16 + 1) // 2, SX * IC // 16
        row = -(-(((OW - 1) * SX + KX) * IC // 16) // m) * m * 16
        wide = OC > 64 and 128 * (steps * 32 + 16) <= 40 * 1024 and (-(-OC // 128) * 128 - OC) * 8 <= OC
        bn = 32 if OC <= 32 else (128 if wide else 64)  # channels per workgroup
        lds = bn * (steps * 32 + 16) + bn * 32 + 2 * bn * 4 + 16 + (2 * steps + 3) // 4 * 16 + KY * row
        # (multiples of 32 have a gather kernel for any K: they take this one while the weights leave most of LDS to the rows)
        if lds <= 160 * 1024 - 512 and (IC % 32 != 0 or bn * (steps * 32 + 16) <= 100 * 1024):
            assert name == "nce_conv_rows16", what
        assert np.array_equal(got, want), "%s (%s): %d mismatches" % (what, name, int((got != want).sum()))


def test_row_patch_conv_stem_layer(rt, orc, dev):
    """A ResNet stem at a size the oracle still finishes quickly ([2,224,224,16] -> 64, 7x7, stride 2, padding 3): full-width
    rows of 229 pixels in LDS, tiles of several output rows, workgroups that take more than one tile."""
    rng = np.random.default_rng(21)
    inp, w, mults, shifts, bias = rand_case(rng, 2, 224, 224, 16, 64, 7, 7, shift_lo=16, shift_hi=20)
    kw = dict(U8, lrelu_mult=0, lrelu_shift=0)
    for rows in (0, 1, 3):
        if rows:
            rt.set_tuning("VPX_CONV_ROWS", rows)
        try:
            got, want, name = run_task(rt, orc, dev, inp, w, mults, shifts, bias, kw, zp_in=128, zp_out=0, strides=(2, 2),
                                       pads=(3, 3, 3, 3), mode=rt.PPE_LRELU)
        finally:
            rt.set_tuning("VPX_CONV_ROWS", None)
        assert name == "nce_conv_rows16"
        assert np.array_equal(got, want), "rows=%d: %d mismatches" % (rows, int((got != want).sum()))


def test_row_patch_conv_wide_image(rt, orc, dev):
    """A 7x7 stride-2 stem on a 1280-pixel-wide image: the rows under one output row do not fit LDS beside the weights, so
    the kernel walks column tiles (ragged last tile, halo columns on both sides of every tile)."""
    rng = np.random.default_rng(23)
    inp, w, mults, shifts, bias = rand_case(rng, 1, 40, 1280, 16, 64, 7, 7, shift_lo=16, shift_hi=20)
    kw = dict(U8, lrelu_mult=1638, lrelu_shift=14)
    got, want, name = run_task(rt, orc, dev, inp, w, mults, shifts, bias, kw, zp_in=117, zp_out=5, strides=(2, 2), pads=(3, 2, 3, 3),
                               mode=rt.PPE_LPRELU)
    assert name == "nce_conv_rows16"
    assert np.array_equal(got, want), "%d mismatches" % int((got != want).sum())


@pytest.fixture(params=[("8", "256", None), ("8", "256", "on"), ("4", "256", None), ("4", "128", None)], ids=["8w256", "8w256pp", "4w256", "4w128"])
def gemm_waves(request, rt):
    """The shapes of the matmul kernel: 256 x 256 tiles with two waves per SIMD (128 x 64 each; "pp": the two taking turns
    at the MFMAs, where K is a multiple of 256) or one (128 x 128), and 128 x 128 tiles (four waves of 64 x 64), which
    small problems select by themselves."""
    rt.set_tuning("VPX_GEMM_WAVES", request.param[0])
    rt.set_tuning("VPX_GEMM_TILE", request.param[1])
    rt.set_tuning("VPX_GEMM_PINGPONG", request.param[2])
    yield request.param
    rt.set_tuning("VPX_GEMM_WAVES", None)
    rt.set_tuning("VPX_GEMM_TILE", None)
    rt.set_tuning("VPX_GEMM_PINGPONG", None)


@pytest.mark.parametrize("M,K,N", [(256, 64, 256), (300, 128, 520), (1, 64, 1), (513, 256, 77), (1024, 512, 768), (700, 1024, 300)])
def test_matmul_gemm_path(rt, orc, dev, gemm_waves, M, K, N):
    rng = np.random.default_rng(70 + M)
    for in_u8, zp in ((False, 3), (True, 128), (False, 0), (True, 11)):
        a = rng.integers(0, 256, (M, K), dtype=np.uint8) if in_u8 else rng.integers(-128, 128, (M, K)).astype(np.int8)
        b = rng.integers(-127, 128, (N, K)).astype(np.int8)
        mults = rng.integers(2 ** 14, 2 ** 15, N)
        shifts = rng.integers(18, 24, N)
        bias = rng.integers(-2 ** 15, 2 ** 15, N).astype(np.int32)
        kw = dict(I8, lrelu_mult=1638, lrelu_shift=14)
        got, want, name = run_task(rt, orc, dev, a.reshape(1, M, 1, K), b.reshape(N, 1, 1, K), mults, shifts, bias, kw,
                                   zp_in=zp, out_signed=True, mode=rt.PPE_LPRELU)
        assert name == "nce_gemm_mfma"
        assert np.array_equal(got, want), "M=%d K=%d N=%d zp=%d: %d mismatches" % (M, K, N, zp, int((got != want).sum()))


@pytest.fixture(params=["on", "wide"])
def regb_on(rt, request):
    """The weights-in-registers matmul, which by itself serves a short K from some tens of thousands of rows on; "wide":
    with as many channel blocks per wave as it takes from some hundreds of thousands of rows on."""
    rt.set_tuning("VPX_GEMM_REGB", request.param)
    yield request.param
    rt.set_tuning("VPX_GEMM_REGB", None)


@pytest.mark.parametrize("M,K,N", [(4096, 64, 256), (1000, 64, 64), (517, 128, 208), (33, 256, 80), (1, 64, 16), (2050, 256, 528),
                                   (16, 128, 64), (700, 64, 192), (900, 64, 512), (333, 64, 128), (650, 128, 512), (300, 64, 384)])
def test_matmul_weights_in_registers(rt, orc, dev, regb_on, M, K, N):
    """Every PPE form (short with and without a slope, the general integer one through clipping scales, an odd zero
    point and a slope above one), both input types, row and channel counts that end inside a block."""
    rng = np.random.default_rng(170 + M + N)
    cases = [
        (False, 3, dict(I8, lrelu_mult=1638, lrelu_shift=14), rt.PPE_LPRELU, True, 0, (18, 24)),
        (True, 128, dict(U8), rt.PPE_NOOP, False, 0, (16, 22)),
        (True, 11, dict(U8, lrelu_mult=3, lrelu_shift=1), rt.PPE_LPRELU, False, 4, (16, 22)),   # slope 1.5: general
        (False, 0, dict(I8), rt.PPE_LRELU, True, 7, (16, 22)),                                  # odd zero point: general
        (True, 128, dict(clamp_low=10, clamp_high=200), rt.PPE_NOOP, False, 0, (8, 13)),        # scales above 1/2: clipping
    ]
    for in_u8, zp, kw, mode, out_signed, zp_out, (slo, shi) in cases:
        a = rng.integers(0, 256, (M, K), dtype=np.uint8) if in_u8 else rng.integers(-128, 128, (M, K)).astype(np.int8)
        b = rng.integers(-127, 128, (N, K)).astype(np.int8)
        mults = rng.integers(2 ** 14, 2 ** 15, N)
        shifts = rng.integers(slo, shi, N)
        bias = rng.integers(-2 ** 15, 2 ** 15, N).astype(np.int32)
        got, want, name = run_task(rt, orc, dev, a.reshape(1, M, 1, K), b.reshape(N, 1, 1, K), mults, shifts, bias, kw,
                                   zp_in=zp, zp_out=zp_out, out_signed=out_signed, mode=mode)
        assert name == "nce_gemm_regb"
        assert np.array_equal(got, want), "M=%d K=%d N=%d zp=%d mode=%s: %d mismatches" % (M, K, N, zp, mode, int((got != want).sum()))


@pytest.mark.parametrize("M,K,N,w_u8,zp_w", [(900, 64, 256, True, 128), (530, 128, 144, True, 117), (300, 256, 64, False, -5)])
def test_matmul_weights_in_registers_weight_zero_points(rt, orc, dev, regb_on, M, K, N, w_u8, zp_w):
    rng = np.random.default_rng(180 + M)
    a = rng.integers(0, 256, (M, K), dtype=np.uint8)
    b = rng.integers(0, 256, (N, K), dtype=np.uint8) if w_u8 else rng.integers(-127, 128, (N, K)).astype(np.int8)
    mults = rng.integers(2 ** 14, 2 ** 15, N)
    shifts = rng.integers(18, 24, N)
    bias = rng.integers(-2 ** 15, 2 ** 15, N).astype(np.int32)
    got, want, name = run_task(rt, orc, dev, a.reshape(1, M, 1, K), b.reshape(N, 1, 1, K), mults, shifts, bias, dict(U8),
                               zp_in=121, zp_w=zp_w, out_offset=48)
    assert name == "nce_gemm_regb"
    assert np.array_equal(got, want), "%d mismatches" % int((got != want).sum())


def test_matmul_weights_in_registers_leaves_ragged_rows_to_the_tile_kernel(rt, orc, dev, regb_on):
    """Channel counts that are not a multiple of 16 (rows of the result that do not end on a 16-byte piece) and a K it
    does not serve."""
    rng = np.random.default_rng(185)
    for M, K, N in ((300, 64, 77), (300, 192, 128)):
        a = rng.integers(-128, 128, (M, K)).astype(np.int8)
        b = rng.integers(-127, 128, (N, K)).astype(np.int8)
        got, want, name = run_task(rt, orc, dev, a.reshape(1, M, 1, K), b.reshape(N, 1, 1, K), rng.integers(2 ** 14, 2 ** 15, N),
                                   rng.integers(18, 24, N), rng.integers(-2 ** 15, 2 ** 15, N).astype(np.int32), dict(I8), out_signed=True)
        assert name == "nce_gemm_mfma"
        assert np.array_equal(got, want)


@pytest.mark.parametrize("IC,OC", [(64, 256), (64, 48), (128, 64), (256, 64)])
def test_1x1_layer_takes_the_weights_in_registers_matmul_by_itself(rt, orc, dev, IC, OC):
    """[8,112,112,IC] -> OC, 1x1: 100 352 rows of a short K, also where the channels are fewer than a matmul tile is wide."""
    rng = np.random.default_rng(190 + OC)
    inp, w, mults, shifts, bias = rand_case(rng, 8, 112, 112, IC, OC, 1, 1, shift_lo=18, shift_hi=22)
    got, want, name = run_task(rt, orc, dev, inp, w, mults, shifts, bias, dict(U8), zp_in=128)
    assert name == "nce_gemm_regb"
    assert np.array_equal(got, want), "%d mismatches" % int((got != want).sum())


@pytest.mark.parametrize("M,K,N", [(300, 128, 520), (513, 256, 77)])
def test_matmul_gemm_path_f16_output(rt, orc, dev, gemm_waves, M, K, N):
    """The wave-count knob does not reach the fp16-output matmul, which exists with eight waves per large tile only."""
    rng = np.random.default_rng(71 + M)
    for in_u8, zp in ((False, 3), (True, 128)):
        a = rng.integers(0, 256, (M, K), dtype=np.uint8) if in_u8 else rng.integers(-128, 128, (M, K)).astype(np.int8)
        b = rng.integers(-127, 128, (N, K)).astype(np.int8)
        mults = rng.integers(2 ** 14, 2 ** 15, N)
        shifts = rng.integers(18, 24, N)
        bias = rng.integers(-2 ** 15, 2 ** 15, N).astype(np.int32)
        kw = dict(F16_NONE, lrelu_mult=1638, lrelu_shift=14)
        got, want, name = run_task(rt, orc, dev, a.reshape(1, M, 1, K), b.reshape(N, 1, 1, K), mults, shifts, bias, kw,
                                   zp_in=zp, mode=rt.PPE_LPRELU, out_f16=True)
        assert name == "nce_gemm_mfma"
        assert np.array_equal(got, want), "M=%d K=%d N=%d zp=%d: %d mismatches" % (M, K, N, zp, int((got != want).sum()))


@pytest.mark.parametrize("mode", ["NOOP", "LRELU", "LRELUX", "LPRELU"])
def test_ppe_modes_and_rounding_edges(rt, orc, dev, mode):
    """Accumulators chosen to land on ties, on both signs, with shifts from 0 to 40 and output zero points."""
    rng = np.random.default_rng(80)
    M, K, N = 256, 64, 256
    a = rng.integers(-4, 5, (M, K)).astype(np.int8)
    b = rng.integers(-4, 5, (N, K)).astype(np.int8)
    mults = np.where(np.arange(N) % 3 == 0, 1 << 14, rng.integers(2 ** 14, 2 ** 15, N))
    shifts = np.arange(N) % 41
    bias = rng.integers(-64, 64, N).astype(np.int32)
    md = getattr(rt, "PPE_" + mode)
    kw = dict(clamp_low=-100, clamp_high=90, lrelu_mult=1638 if mode == "LPRELU" else 1, lrelu_shift=14 if mode == "LPRELU" else 0)
    got, want, _ = run_task(rt, orc, dev, a.reshape(1, M, 1, K), b.reshape(N, 1, 1, K), mults, shifts, bias, kw, zp_in=1,
                            zp_out=-7, out_signed=True, mode=md)
    assert np.array_equal(got, want)
    assert got.min() >= -100 and got.max() <= 90


@pytest.mark.parametrize("G,M,K,N,in_u8,zp_a,w_u8,zp_b,out_f16,kernel", [
    (3, 300, 128, 520, False, 3, False, 0, False, "nce_gemm_mfma"),    # one launch, column sums of all groups in one pass
    (5, 64, 64, 48, True, 121, False, 0, False, "nce_gemm_mfma"),      # 128 x 128 tiles, short K
    (2, 256, 192, 320, True, 7, True, 131, False, "nce_gemm_mfma"),    # weight zero point: per-position term, M % 4 == 0
    (2, 130, 128, 96, False, -2, False, 0, True, "nce_gemm_mfma"),     # fp16 output
    (3, 33, 128, 80, True, 9, True, 120, False, "nce_gemm_mfma"),      # weight zero point with M % 4 != 0: group after group
    (2, 40, 48, 72, False, 1, False, 0, False, "nce_conv_rows16"),     # K not a multiple of 64: group after group
])
def test_grouped_matmul_one_task(rt, orc, dev, G, M, K, N, in_u8, zp_a, w_u8, zp_b, out_f16, kernel):
    """VPU.NCE.MatMul with G groups ([G,1,K,M,1] x [G,N,K,1,1], weight table [G,N,1,1,4]) as one task: bit-exact against
    G separate runs of the oracle."""
    import torch
    rng = np.random.default_rng(400 + G * M)
    a = rng.integers(0, 256, (G, M, K), dtype=np.uint8) if in_u8 else rng.integers(-128, 128, (G, M, K)).astype(np.int8)
    b = rng.integers(0, 256, (G, N, K), dtype=np.uint8) if w_u8 else rng.integers(-127, 128, (G, N, K)).astype(np.int8)
    wt = np.stack([rt.make_weights_table(rng.integers(2 ** 14, 2 ** 15, N), rng.integers(16, 22, N),
                                         rng.integers(-2 ** 15, 2 ** 15, N).astype(np.int32), K) for _ in range(G)])
    if out_f16:
        ppe, op = rt.PpeInt(rt.PPE_LPRELU, -(2 ** 31), 2 ** 31 - 1, 1638, 14), orc.ppe(1638, 14, 0, -(2 ** 31), 2 ** 31 - 1)
    else:
        ppe, op = rt.PpeInt(rt.PPE_LPRELU, -128, 127, 1638, 14), orc.ppe(1638, 14, 5, -128, 127)
    out = torch.full((G, M, N), 77, dtype=torch.float16 if out_f16 else torch.int8, device=dev)
    rt.nce_matmul(dev_t(a, dev), dev_t(b, dev), dev_t(wt, dev), out, ppe, zp_a=zp_a, zp_b=zp_b, zp_out=0 if out_f16 else 5)
    torch.cuda.synchronize()
    assert rt.nce_last_kernel() == kernel
    got = out.cpu().numpy()
    for g in range(G):
        want = orc.nce_matmul(a[g], b[g], wt[g], op, zp_a=zp_a, zp_b=zp_b, out_f16=out_f16)
        gg = got[g].view(np.uint16) if out_f16 else got[g]
        assert np.array_equal(gg, want), "group %d: %d mismatches" % (g, int((gg != want).sum()))


F16_NONE = {"clamp_low": -(2 ** 31), "clamp_high": 2 ** 31 - 1}


@pytest.mark.parametrize("mode", ["NOOP", "LPRELU", "LRELU", "LRELUX"])
@pytest.mark.parametrize("geom,kernel,force", [
    (dict(N=1, H=700, W=1, IC=128, OC=520, KY=1, KX=1), "nce_gemm_mfma", "tile256"),     # 256 x 256 tiles, ragged edges
    (dict(N=1, H=130, W=1, IC=64, OC=200, KY=1, KX=1), "nce_gemm_mfma", None),           # 128 x 128 tiles
    (dict(N=1, H=300, W=1, IC=128, OC=77, KY=1, KX=1), "nce_gemm_mfma", None),           # rows of an odd length: no 16-byte stores
    (dict(N=1, H=333, W=1, IC=192, OC=301, KY=1, KX=1), "nce_gemm_mfma", "tile256"),     # the same with both halves of a 256-row tile ragged
    (dict(N=2, H=9, W=11, IC=64, OC=70, KY=3, KX=3), "nce_conv_tile", None),             # convolution: input patch in LDS, 128-byte staging rows
    (dict(N=2, H=9, W=11, IC=64, OC=70, KY=3, KX=3), "nce_conv_mfma", "gather"),         # the gather kernel
    (dict(N=2, H=13, W=10, IC=128, OC=136, KY=3, KX=3), "nce_conv_tile", None),
    (dict(N=1, H=9, W=9, IC=256, OC=96, KY=3, KX=3), "nce_conv_stream", None),           # streamed weights, K split over two groups of waves
    (dict(N=3, H=7, W=7, IC=512, OC=72, KY=3, KX=3), "nce_conv_stream", None),           # ... over eight waves
    (dict(N=2, H=30, W=33, IC=192, OC=40, KY=3, KX=3), "nce_conv_stream", None),         # ... one tile per wave
    (dict(N=1, H=10, W=12, IC=48, OC=40, KY=3, KX=3), "nce_conv_rows16", None),          # input rows in LDS, two 16-byte stores per position and lane
    (dict(N=2, H=31, W=40, IC=16, OC=72, KY=3, KX=3), "nce_conv_rows16", None),
    (dict(N=1, H=10, W=12, IC=48, OC=40, KY=3, KX=3), "nce_conv_mfma16", "gather"),
    (dict(N=2, H=6, W=7, IC=5, OC=9, KY=3, KX=2), "nce_conv_naive", None),
    (dict(N=1, H=40, W=1, IC=64, OC=96, KY=1, KX=1), "nce_conv_naive", "naive"),
])
def test_f16_output_s1715_path(rt, orc, dev, geom, kernel, force, mode):
    """fp16 output of an integer convolution / matmul ("INT32 s17.15 fixed-point convert to FP16"): bit-exact against the
    oracle on every kernel that serves it.  Parity unpinned against silicon, like the integer PPE."""
    rng = np.random.default_rng(300 + geom["H"])
    conv = geom["KY"] > 1
    pads, strides = ((1, 1, 1, 1) if conv else (0, 0, 0, 0)), (1, 1)
    md = getattr(rt, "PPE_" + mode)
    for in_u8, zp_in, zp_w, shift_lo, shift_hi in ((True, 128, 0, 14, 24), (False, -4, 0, 8, 30), (True, 9, 3, 16, 22)):
        if zp_w and geom["IC"] % 16:
            zp_w = 0
        inp, w, mults, shifts, bias = rand_case(rng, in_u8=in_u8, shift_lo=shift_lo, shift_hi=shift_hi, **geom)
        kw = dict(F16_NONE, lrelu_mult=1638, lrelu_shift=14)
        if mode == "LRELUX":
            kw["clamp_high"] = orc.pack_clamp_f16(0.0, 6.0)
        if force == "tile256":
            rt.set_tuning("VPX_GEMM_TILE", 256)
        try:
            got, want, name = run_task(rt, orc, dev, inp, w, mults, shifts, bias, kw, zp_in=zp_in, zp_w=zp_w, strides=strides,
                                       pads=pads, mode=md, force=None if force == "tile256" else force, out_f16=True)
        finally:
            rt.set_tuning("VPX_GEMM_TILE", None)
        assert name == kernel
        assert np.array_equal(got, want), "%s %s zp_in=%d: %d mismatches" % (name, mode, zp_in, int((got != want).sum()))
        vals = got.view(np.float16).astype(np.float32)
        if mode in ("LRELU", "LRELUX"):
            assert vals.min() >= 0.0
        if mode == "LRELUX":
            assert vals.max() <= 6.0 and (vals == 6.0).any()


@pytest.mark.parametrize("seed", [41, 42])
def test_f16_output_conv_random_geometries(rt, orc, dev, seed):
    """fp16 outputs of convolutions whichever kernel the layer selects (tile and streamed-weights kernels stage 128 bytes
    a position, the gather kernels store from registers): seeded draws of shape, kernel, stride, padding, channel counts
    (odd ones: no 16-byte stores), zero points, PPE mode and fp16 clamp."""
    rng = np.random.default_rng(seed)
    for i in range(24):
        IC = int(rng.choice([16, 32, 64, 64, 128, 128, 192, 256, 512]))
        OC = int(rng.choice([8, 24, 63, 64, 72, 100, 128, 130]))
        KY, KX = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        SY, SX = int(rng.integers(1, 3)), int(rng.integers(1, 3))
        pl, pr, pt, pb = [int(v) for v in rng.integers(0, 2, 4)]
        pl, pr, pt, pb = min(pl, KX - 1), min(pr, KX - 1), min(pt, KY - 1), min(pb, KY - 1)
        H, W, N = int(rng.integers(KY, 30)), int(rng.integers(KX, 40)), int(rng.integers(1, 4))
        in_u8 = bool(rng.integers(0, 2))
        zp_in = int(rng.integers(0, 256)) if in_u8 else int(rng.integers(-128, 128))
        w_u8, zp_w = False, 0
        if rng.integers(0, 3) == 0:
            w_u8 = bool(rng.integers(0, 2))
            zp_w = int(rng.integers(0, 256)) if w_u8 else int(rng.integers(-128, 128))
        mode = ["NOOP", "LPRELU", "LRELU", "LRELUX"][int(rng.integers(0, 4))]
        kw = dict(F16_NONE, lrelu_mult=int(rng.integers(0, 2048)), lrelu_shift=int(rng.integers(8, 16)))
        if mode == "LRELUX":
            kw["clamp_high"] = orc.pack_clamp_f16(0.0, 6.0)
        what = "seed %d case %d: N=%d H=%d W=%d IC=%d OC=%d K=%dx%d S=%dx%d pads=%s in_u8=%s zp_in=%d w_u8=%s zp_w=%d mode=%s" % (
            seed, i, N, H, W, IC, OC, KY, KX, SY, SX, (pl, pr, pt, pb), in_u8, zp_in, w_u8, zp_w, mode)
        print(what, flush=True)
        inp, w, mults, shifts, bias = rand_case(rng, N, H, W, IC, OC, KY, KX, in_u8=in_u8, w_u8=w_u8, shift_lo=10, shift_hi=26)
        if rng.integers(0, 2):
            mults = np.where(rng.random(mults.shape) < 0.5, -mults, mults)
        bias = (bias - np.int64(round(KY * KX * IC * (inp.mean() - zp_in) * (w.mean() - zp_w)))).astype(np.int32)
        got, want, name = run_task(rt, orc, dev, inp, w, mults, shifts, bias, kw, zp_in=zp_in, zp_w=zp_w, strides=(SY, SX),
                                   pads=(pl, pr, pt, pb), mode=getattr(rt, "PPE_" + mode), out_f16=True)
        assert np.array_equal(got, want), "%s (%s): %d mismatches" % (what, name, int((got != want).sum()))


@pytest.mark.parametrize("out_f16", [False, True])
@pytest.mark.parametrize("geom,kernel,force", [
    (dict(N=2, H=20, W=24, IC=64, KY=1, KX=1), "nce_gemm_mfma", None),
    (dict(N=2, H=20, W=24, IC=64, KY=3, KX=3), "nce_conv_regw", "regw"),
    (dict(N=2, H=20, W=24, IC=128, KY=3, KX=3), "nce_conv_tile", None),
    (dict(N=3, H=7, W=7, IC=256, KY=3, KX=3), "nce_conv_stream", None),       # the K steps split over the waves
    (dict(N=1, H=30, W=33, IC=192, KY=3, KX=3), "nce_conv_stream", None),     # one tile per wave
    (dict(N=2, H=20, W=24, IC=48, KY=1, KX=1), "nce_conv_rows16", None),
    (dict(N=2, H=20, W=24, IC=16, KY=3, KX=3), "nce_conv_rows16", None),
    (dict(N=1, H=12, W=10, IC=64, KY=3, KX=3), "nce_conv_mfma", "gather"),
    (dict(N=1, H=12, W=10, IC=48, KY=3, KX=3), "nce_conv_mfma16", "gather"),
])
def test_output_rows_that_are_not_whole_16_byte_pieces(rt, orc, dev, geom, kernel, force, out_f16):
    """Channel counts whose output rows are a multiple of 8, 4, 2 or 1 bytes only, in tensors that start 0, 8, 4 or an odd
    number of bytes past an aligned address: the kernels store such rows in the largest pieces row length and base allow,
    and the elements either side of the tensor stay as they were."""
    rng = np.random.default_rng(640 + geom["IC"] + geom["KY"])
    pads = (1, 1, 1, 1) if geom["KY"] > 1 else (0, 0, 0, 0)
    for OC, offset in ((72, 0), (72, 8), (72, 4), (100, 0), (100, 4), (120, 16), (200, 8), (36, 0), (70, 2), (37, 1), (72, 3), (88, 0)):
        if out_f16:
            offset = (offset + 1) // 2 if offset % 2 == 0 else offset  # elements of two bytes: 0, 8, 4, 2 bytes and odd element counts
        inp, w, mults, shifts, bias = rand_case(rng, OC=OC, shift_lo=14, shift_hi=22, **geom)
        kw = dict(F16_NONE if out_f16 else U8, lrelu_mult=1638, lrelu_shift=14)
        got, want, name = run_task(rt, orc, dev, inp, w, mults, shifts, bias, kw, zp_in=128, zp_out=0 if out_f16 else 3, pads=pads,
                                   mode=rt.PPE_LPRELU, force=force, out_f16=out_f16, out_offset=offset)
        assert name == ("nce_conv_tile" if out_f16 and kernel == "nce_conv_regw" else kernel)  # (no fp16 output from that one)
        assert np.array_equal(got, want), "%s OC=%d offset=%d: %d mismatches" % (name, OC, offset, int((got != want).sum()))


def test_f16_output_scale_is_weight_scale_times_input_scale(rt, orc, dev):
    """With the weight table built for a float output (no output scale) the result is the real-valued convolution:
    sum (q_in - zp) * s_in * q_w * s_w, within the 15-bit multiplier's and fp16's precision."""
    import torch
    rng = np.random.default_rng(311)
    M, K, N = 64, 128, 192
    a = rng.integers(0, 256, (M, K), dtype=np.uint8)
    b = rng.integers(-127, 128, (N, K)).astype(np.int8)
    s_in, zp = 0.02, 128
    s_w = np.exp(rng.uniform(np.log(1e-3), np.log(2e-2), N))
    wt = rt.get_weights_table(s_in, 1.0, s_w, None, N, weights_ptr_step=K)
    out = torch.empty((M, N), dtype=torch.float16, device=dev)
    rt.nce_matmul(dev_t(a, dev), dev_t(b, dev), dev_t(wt, dev), out, rt.retrieve_ppe_int(rt.POSTOP_NONE, None), zp_a=zp)
    torch.cuda.synchronize()
    real = ((a.astype(np.float64) - zp) * s_in) @ (b.astype(np.float64) * s_w[:, None]).T
    got = out.cpu().numpy().astype(np.float64)
    assert np.all(np.abs(got - real) <= np.abs(real) * (2.0 ** -10 + 2.0 ** -13) + 2.0 ** -14)
    want = orc.nce_matmul(a, b, wt, orc.ppe(1, 0, 0, -(2 ** 31), 2 ** 31 - 1), zp_a=zp, out_f16=True)
    assert np.array_equal(out.cpu().numpy().view(np.uint16), want)


def test_conv_config_c4_full_size(rt, orc, dev):
    from vpux_plugin_amd import configs
    c = configs.c4_conv()
    got, want, name = run_task(rt, orc, dev, c["input"], c["weights"], c["mult"], c["shift"], c["bias"],
                               {"clamp_low": c["clamp"][0], "clamp_high": c["clamp"][1]}, zp_in=c["zp_in"],
                               strides=c["strides"], pads=c["pads"])
    assert name == "nce_conv_regw"
    assert np.array_equal(got, want), "%d mismatches" % int((got != want).sum())
    assert 0 < (got == 0).mean() < 0.9  # the ReLU clamp is active and the output is not saturated flat


def test_matmul_config_c5_full_size_and_chain(rt, orc, dev):
    """Full [4096x4096]x[4096x11008]: the MFMA result is compared bit for bit with the CPU oracle over the whole
    tensor (run here, all host threads), with the committed checksums of the oracle's result
    (tests/golden/c5_matmul_checksum.json, written by tests/golden/make_c5_checksum.py) and with the naive device
    path; then Dequantize and the fp16 Add, likewise over the whole tensors."""
    import hashlib
    import json
    import torch
    from vpux_plugin_amd import configs
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "golden", "c5_matmul_checksum.json")) as f:
        gold = json.load(f)
    sha = lambda arr: hashlib.sha256(np.ascontiguousarray(arr).tobytes()).hexdigest()
    c = configs.c5_matmul()
    M, K = c["a"].shape
    N = c["b_nk"].shape[0]
    wt = rt.make_weights_table(c["mult"], c["shift"], c["bias"], K)
    p = rt.PpeInt(rt.PPE_LPRELU, c["clamp"][0], c["clamp"][1], c["lrelu_mult"], c["lrelu_shift"])
    a, b, wtd = dev_t(c["a"], dev), dev_t(c["b_nk"], dev), dev_t(wt, dev)
    out = torch.empty((M, N), dtype=torch.int8, device=dev)
    rt.nce_matmul(a, b, wtd, out, p, zp_a=c["zp_a"], zp_out=c["zp_out"])
    assert rt.nce_last_kernel() == "nce_gemm_mfma"
    out2 = torch.empty_like(out)
    rt.set_tuning("VPX_NCE_KERNEL", "naive")
    try:
        rt.nce_matmul(a, b, wtd, out2, p, zp_a=c["zp_a"], zp_out=c["zp_out"])
        assert rt.nce_last_kernel() == "nce_conv_naive"
    finally:
        rt.set_tuning("VPX_NCE_KERNEL", None)
    torch.cuda.synchronize()
    assert bool((out == out2).all())
    got = out.cpu().numpy()
    # committed checksums of the oracle's full result: the bytes, and row / column sums that localise a difference
    g = gold["matmul_i8"]
    assert int(got.astype(np.int64).sum()) == g["sum"]
    assert sha(got.astype(np.int64).sum(axis=1)) == g["row_sums_sha256"]
    assert sha(got.astype(np.int64).sum(axis=0)) == g["col_sums_sha256"]
    assert sha(got) == g["sha256"]
    # the oracle itself, whole tensor
    op = orc.ppe(c["lrelu_mult"], c["lrelu_shift"], c["zp_out"], *c["clamp"])
    want = orc.nce_matmul(c["a"], c["b_nk"], wt, op, zp_a=c["zp_a"])
    assert np.array_equal(got, want), "%d mismatches" % int((got != want).sum())
    hist = np.bincount(got.astype(np.int64).ravel() + 128, minlength=256)
    assert hist[0] / got.size < 0.05 and hist[255] / got.size < 0.05 and (hist > 0).sum() > 100  # spans i8
    # C5 chain: Dequantize to fp16, then fp16 Add of the residual
    deq = torch.empty((M, N), dtype=torch.float16, device=dev)
    rt.dequantize(out, deq, c["deq_scale"], c["deq_zp"])
    res = dev_t(c["residual"].view(np.float16), dev)
    y = torch.empty_like(deq)
    rt.eltwise("add", deq, res, y)
    torch.cuda.synchronize()
    shipped = float(orc.f16_to_f32(orc.f32_to_f16(np.array([c["deq_scale"]], np.float32)))[0])
    deq_bits = deq.cpu().numpy().view(np.uint16)
    assert np.array_equal(deq_bits, orc.dequantize(got, shipped, c["deq_zp"]))
    assert sha(deq_bits) == gold["dequantize_f16_bits"]["sha256"]
    y_bits = y.cpu().numpy().view(np.uint16)
    assert np.array_equal(y_bits, orc.eltwise_f16("add", deq_bits, c["residual"]))
    assert sha(y_bits) == gold["add_f16_bits"]["sha256"]


@pytest.mark.parametrize("subtract", [False, True])
@pytest.mark.parametrize("mode", ["NOOP", "LPRELU"])
def test_nce_eltwise(rt, orc, dev, subtract, mode):
    """Quantized residual add / subtract: every combination of operand signedness, odd and even output
    zero points, partial clamp windows, ragged sizes and an unaligned view."""
    import torch
    rng = np.random.default_rng(95)
    in1_mult, in2_mult, out_mult, out_shift = rt.eltwise_quantization_approximation(0.02, 0.035, 0.05, 1 if subtract else 0)
    md = getattr(rt, "PPE_" + mode)
    pm, ps = (1638, 14) if mode == "LPRELU" else (1, 0)
    for a_signed, b_signed, out_signed, zp1, zp2, zpo, clamp, shape in (
            (False, True, False, 128, -3, 7, (0, 255), (2, 9, 11, 64)),
            (True, True, True, 0, 5, 0, (-128, 127), (1, 7, 5, 33)),
            (True, False, True, -7, 100, -20, (-100, 90), (3, 4, 4, 16)),
            (False, False, False, 3, 250, 128, (128, 255), (1, 1, 1, 5))):
        a = rng.integers(-128, 128, shape).astype(np.int8) if a_signed else rng.integers(0, 256, shape, dtype=np.uint8)
        b = rng.integers(-128, 128, shape).astype(np.int8) if b_signed else rng.integers(0, 256, shape, dtype=np.uint8)
        ppe = rt.PpeInt(md, clamp[0], clamp[1], pm, ps, out_mult, out_shift, in1_mult, in2_mult)
        out = torch.full(shape, 99, dtype=torch.int8 if out_signed else torch.uint8, device=dev)
        rt.nce_eltwise(dev_t(a, dev), dev_t(b, dev), out, ppe, zp1, zp2, zpo, subtract=subtract)
        torch.cuda.synchronize()
        assert rt.nce_last_kernel() == "nce_eltwise_kernel"
        want = orc.nce_eltwise(a, b, orc.ppe(pm if mode == "LPRELU" else 1, ps, zpo, clamp[0], clamp[1]), zp1, zp2, in1_mult,
                               in2_mult, out_mult, out_shift, subtract=subtract, out_signed=out_signed)
        got = out.cpu().numpy()
        assert np.array_equal(got, want), "%s: %d mismatches" % (shape, int((got != want).sum()))
        # a negative output multiplier (negative output scale) flips which sums take the PReLU branch
        ppe = rt.PpeInt(md, clamp[0], clamp[1], pm, ps, -out_mult, out_shift, in1_mult, in2_mult)
        rt.nce_eltwise(dev_t(a, dev), dev_t(b, dev), out, ppe, zp1, zp2, zpo, subtract=subtract)
        want = orc.nce_eltwise(a, b, orc.ppe(pm if mode == "LPRELU" else 1, ps, zpo, clamp[0], clamp[1]), zp1, zp2, in1_mult,
                               in2_mult, -out_mult, out_shift, subtract=subtract, out_signed=out_signed)
        got = out.cpu().numpy()
        assert np.array_equal(got, want), "%s, negative multiplier: %d mismatches" % (shape, int((got != want).sum()))


@pytest.mark.parametrize("subtract", [False, True])
@pytest.mark.parametrize("mode", ["NOOP", "LPRELU", "LRELU", "LRELUX"])
def test_nce_eltwise_f16_output(rt, orc, dev, subtract, mode):
    """The quantized add / subtract with an fp16 output (the sum through the s17.15 fixed-point PPE, no output zero point):
    operand signedness, ragged sizes, an unaligned view, both signs of the output multiplier, an fp16 clamp."""
    import torch
    rng = np.random.default_rng(96)
    in1_mult, in2_mult, out_mult, out_shift = rt.eltwise_quantization_approximation(0.02, 0.035, 0.05, 1 if subtract else 0)
    md = getattr(rt, "PPE_" + mode)
    hi = orc.pack_clamp_f16(0.0, 6.0) if mode == "LRELUX" else 2 ** 31 - 1
    for a_signed, b_signed, zp1, zp2, shape, mult in ((False, True, 128, -3, (2, 9, 11, 64), out_mult), (True, True, 0, 5, (1, 7, 5, 33), -out_mult),
                                                      (True, False, -7, 100, (3, 4, 4, 16), out_mult), (False, False, 3, 250, (1, 1, 1, 5), out_mult)):
        a = rng.integers(-128, 128, shape).astype(np.int8) if a_signed else rng.integers(0, 256, shape, dtype=np.uint8)
        b = rng.integers(-128, 128, shape).astype(np.int8) if b_signed else rng.integers(0, 256, shape, dtype=np.uint8)
        ppe = rt.PpeInt(md, -(2 ** 31), hi, 1638, 14, mult, out_shift, in1_mult, in2_mult)
        out = torch.full(shape, 99, dtype=torch.float16, device=dev)
        rt.nce_eltwise(dev_t(a, dev), dev_t(b, dev), out, ppe, zp1, zp2, 0, subtract=subtract)
        torch.cuda.synchronize()
        assert rt.nce_last_kernel() == "nce_eltwise_kernel"
        pm, ps = {"NOOP": (1, 0), "LPRELU": (1638, 14), "LRELU": (0, 0), "LRELUX": (0, 0)}[mode]
        op = orc.ppe(pm, ps, 0, -(2 ** 31), hi)
        want = orc.nce_eltwise(a, b, op, zp1, zp2, in1_mult, in2_mult, mult, out_shift, subtract=subtract, out_f16=True)
        got = out.cpu().numpy().view(np.uint16)
        assert np.array_equal(got, want), "%s: %d mismatches" % (shape, int((got != want).sum()))
        vals = got.view(np.float16).astype(np.float32)
        if mode in ("LRELU", "LRELUX"):
            assert vals.min() >= 0.0
        if mode == "LRELUX":
            assert vals.max() <= 6.0
    # an unaligned view: one value per lane
    base = torch.zeros(1 + 2 * 5 * 3 * 16, dtype=torch.float16, device=dev)
    view = base[1:].view(2, 5, 3, 16)
    a = rng.integers(0, 256, (2, 5, 3, 16), dtype=np.uint8)
    b = rng.integers(0, 256, (2, 5, 3, 16), dtype=np.uint8)
    ppe = rt.PpeInt(md, -(2 ** 31), hi, 1638, 14, out_mult, out_shift, in1_mult, in2_mult)
    rt.nce_eltwise(dev_t(a, dev), dev_t(b, dev), view, ppe, 120, 131, 0, subtract=subtract)
    torch.cuda.synchronize()
    pm, ps = {"NOOP": (1, 0), "LPRELU": (1638, 14), "LRELU": (0, 0), "LRELUX": (0, 0)}[mode]
    want = orc.nce_eltwise(a, b, orc.ppe(pm, ps, 0, -(2 ** 31), hi), 120, 131, in1_mult, in2_mult, out_mult, out_shift, subtract=subtract,
                           out_f16=True)
    assert np.array_equal(view.cpu().numpy().view(np.uint16), want)
    assert float(base[0]) == 0.0


def test_nce_eltwise_full_size_residual(rt, orc, dev):
    """[4096, 11008] i8 + i8 -> i8, the quantized form of the C5 residual add, whole tensor against the oracle."""
    import torch
    rng = np.random.default_rng(96)
    shape = (1, 4096, 1, 11008)
    a = rng.integers(-128, 128, shape).astype(np.int8)
    b = rng.integers(-128, 128, shape).astype(np.int8)
    in1_mult, in2_mult, out_mult, out_shift = rt.eltwise_quantization_approximation(0.05, 0.04, 0.07, 0)
    ppe = rt.PpeInt(rt.PPE_NOOP, -128, 127, 1, 0, out_mult, out_shift, in1_mult, in2_mult)
    out = torch.empty(shape, dtype=torch.int8, device=dev)
    rt.nce_eltwise(dev_t(a, dev), dev_t(b, dev), out, ppe, 3, -2, 0)
    torch.cuda.synchronize()
    want = orc.nce_eltwise(a, b, orc.ppe(1, 0, 0, -128, 127), 3, -2, in1_mult, in2_mult, out_mult, out_shift, out_signed=True)
    got = out.cpu().numpy()
    assert np.array_equal(got, want), "%d mismatches" % int((got != want).sum())
    assert 0.001 < (np.abs(got.astype(np.int32)) == 127).mean() + (got == -128).mean() < 0.5


def test_nce_rejects_bad_descriptors(rt, dev):
    import torch
    inp = torch.zeros((1, 4, 4, 16), dtype=torch.uint8, device=dev)
    w = torch.zeros((8, 3, 3, 16), dtype=torch.int8, device=dev)
    wt = torch.zeros((8, 4), dtype=torch.int32, device=dev)
    out = torch.zeros((1, 2, 2, 8), dtype=torch.uint8, device=dev)
    ok = rt.PpeInt(rt.PPE_NOOP, 0, 255, 1, 0)
    with pytest.raises(rt.VpxError) as e:
        rt.nce_task(inp, w, wt, out, rt.PpeInt(rt.PPE_NOOP, 10, 5, 1, 0))
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT and "clamp" in e.value.text
    with pytest.raises(rt.VpxError) as e:
        rt.nce_task(inp, w, wt, out, rt.PpeInt(5, 0, 255, 1, 0))  # ADD is not an integer-pipeline activation mode
    assert e.value.code == rt.ERROR_UNSUPPORTED_FEATURE
    with pytest.raises(rt.VpxError) as e:
        rt.nce_task(inp, w, wt, out, rt.PpeInt(rt.PPE_LPRELU, 0, 255, 4096, 3))
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT
    with pytest.raises(rt.VpxError) as e:
        rt.nce_task(inp.float(), w, wt, out, ok)
    with pytest.raises(rt.VpxError) as e:  # a float output has no zero point
        rt.nce_task(inp, w, wt, out.half(), ok, zp_out=3)
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT and "zero point" in e.value.text
    big_k = torch.zeros((8, 7, 7, 16), dtype=torch.int8, device=dev)
    with pytest.raises(rt.VpxError) as e:
        rt.nce_task(inp, big_k, wt, out, ok)
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT and "fit" in e.value.text


def test_c_abi_host_example(rt):
    """The C++ host example drives softmax, an NCE matmul + PPE and dequantize through the C ABI alone
    (its own process, the system HIP runtime, no Python in the loop) and checks them against host arithmetic."""
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(rt.__file__)), "examples", "c_abi_host")
    assert os.path.exists(exe), "build the library first (vpux_plugin_amd/build.py)"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "OK" in r.stdout and "0 mismatches" in r.stdout


def test_chain_replayed_from_a_hip_graph(rt, orc, dev):
    """MatMul + PPE -> Dequantize -> fp16 Add (with a non-zero activation zero point, so the zero-point
    term is in play) captured once into a HIP graph and replayed several
    times with eager launches and synchronisations in between: every replay must reproduce the eager result."""
    import torch
    rng = np.random.default_rng(97)
    M, K, N = 512, 256, 384
    a = dev_t(rng.integers(-128, 128, (M, K)).astype(np.int8), dev)
    b = dev_t(rng.integers(-127, 128, (N, K)).astype(np.int8), dev)
    wt = dev_t(rt.make_weights_table(rng.integers(2 ** 14, 2 ** 15, N), rng.integers(20, 23, N),
                                     rng.integers(-500, 500, N).astype(np.int32), K), dev)
    res = torch.randn((M, N), device=dev).half()
    ppe = rt.PpeInt(rt.PPE_LPRELU, -128, 127, 1638, 14)

    def chain(q, deq, y):
        rt.nce_matmul(a, b, wt, q, ppe, zp_a=3)
        rt.dequantize(q, deq, 0.05, 0)
        rt.eltwise("add", deq, res, y)

    def buffers():
        return (torch.zeros((M, N), dtype=torch.int8, device=dev), torch.zeros((M, N), dtype=torch.float16, device=dev),
                torch.zeros((M, N), dtype=torch.float16, device=dev))

    eager = buffers()
    chain(*eager)
    torch.cuda.synchronize()
    captured = buffers()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        chain(*captured)  # first use of this stream sizes the library's workspace: not allowed while capturing
        stream.synchronize()
        for t in captured:
            t.zero_()
        with torch.cuda.graph(graph, stream=stream):
            chain(*captured)
    torch.cuda.synchronize()
    for replay in range(4):
        for t in captured:
            t.fill_(7)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want, what in zip(captured, eager, ("matmul", "dequantize", "add")):
            assert torch.equal(got, want), "replay %d: %s differs from the eager result" % (replay, what)
        scratch = buffers()
        chain(*scratch)  # eager work between replays, on the default stream
        torch.cuda.synchronize()
        assert torch.equal(scratch[2], eager[2])


def test_workspace_reserve_release_and_cold_capture(rt, orc, dev):
    """A launch that needs scratch memory on a capturing stream the library has not seen is refused (it would have to
    call hipMalloc inside the capture); after vpx_workspace_reserve the same capture goes through and replays to the
    eager result; vpx_workspace_release frees the block and the next launch allocates afresh."""
    import torch
    rng = np.random.default_rng(98)
    x = torch.from_numpy(rng.normal(0, 2, (2, 64, 64, 64)).astype(np.float16)).to(dev)  # 64 chunks per group: chunk moments in scratch
    eager = torch.empty_like(x)
    rt.mvn(x, eager, True, True, 1e-9)
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    y = torch.zeros_like(x)
    graph = torch.cuda.CUDAGraph()
    refused = []
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            try:
                rt.mvn(x, y, True, True, 1e-9)
            except rt.VpxError as err:
                refused.append(err)
            y.fill_(1)  # the capture itself stays valid and is ended normally
    assert len(refused) == 1 and refused[0].code == rt.ERROR_UNSUPPORTED_FEATURE and "vpx_workspace_reserve" in refused[0].text
    del graph
    torch.cuda.synchronize()
    rt.workspace_reserve(1 << 16, stream=stream)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            rt.mvn(x, y, True, True, 1e-9)
    for _ in range(3):
        y.fill_(3)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y.view(torch.int16), eager.view(torch.int16))
    del graph
    rt.workspace_release(stream=stream)
    rt.workspace_release(stream=stream)  # nothing left: still succeeds
    with torch.cuda.stream(stream):
        y.fill_(5)
        rt.mvn(x, y, True, True, 1e-9)  # allocates a fresh block
        # per-axis quantize tables are cached per stream and released with it
        q = torch.empty((64, 24), dtype=torch.uint8, device=dev)
        h = torch.from_numpy(rng.normal(0, 1, (64, 24)).astype(np.float16)).to(dev)
        sc, zp = rng.uniform(0.01, 0.1, 24), rng.integers(100, 150, 24)
        rt.quantize(h, q, sc, zp)
        q2 = torch.empty_like(q)
        rt.quantize(h, q2, sc, zp)  # cache hit
    stream.synchronize()
    assert torch.equal(y.view(torch.int16), eager.view(torch.int16)) and torch.equal(q, q2)
    rt.workspace_release(stream=stream)
    with torch.cuda.stream(stream):
        q3 = torch.empty_like(q)
        rt.quantize(h, q3, sc, zp)  # table rebuilt after the release
    stream.synchronize()
    assert torch.equal(q, q3)
    rt.workspace_release(stream=stream)


def test_two_host_threads_on_their_own_streams(rt, orc, dev):
    """The launch functions keep no shared state but a per-(device, stream) workspace: two host threads, each on its own
    stream, run the matmul, MVN (chunk moments in the workspace or the sync area) and softmax
    many times over different data; every result must equal the one computed alone."""
    import threading
    import torch

    def make(seed):
        rng = np.random.default_rng(seed)
        M, K, N = 384, 256, 320
        d = {
            "a": dev_t(rng.integers(-128, 128, (M, K)).astype(np.int8), dev),
            "b": dev_t(rng.integers(-127, 128, (N, K)).astype(np.int8), dev),
            "wt": dev_t(rt.make_weights_table(rng.integers(2 ** 14, 2 ** 15, N), rng.integers(20, 23, N),
                                              rng.integers(-500, 500, N).astype(np.int32), K), dev),
            "x": torch.from_numpy(rng.normal(0, 2, (2, 8, 64, 64)).astype(np.float16)).to(dev),
            "s": torch.from_numpy(rng.normal(0, 3, (512, 512)).astype(np.float16)).to(dev),
            "zp": int(seed % 5) + 1,
        }
        return d

    ppe = rt.PpeInt(rt.PPE_LPRELU, -128, 127, 1638, 14)

    def run(d, stream):
        q = torch.empty((384, 320), dtype=torch.int8, device=dev)
        y = torch.empty_like(d["x"])
        p = torch.empty_like(d["s"])
        rt.nce_matmul(d["a"], d["b"], d["wt"], q, ppe, zp_a=d["zp"], stream=stream)
        rt.mvn(d["x"], y, True, True, 1e-6, stream=stream)
        rt.softmax(d["s"], p, 1, stream=stream)
        return q, y, p

    data = [make(11), make(12)]
    alone = []
    for d in data:
        out = run(d, torch.cuda.current_stream())
        torch.cuda.synchronize()
        alone.append([t.clone() for t in out])
    errors = []

    def worker(i):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for it in range(40):
                    out = run(data[i], stream)
                    stream.synchronize()
                    for got, want, what in zip(out, alone[i], ("matmul", "mvn", "softmax")):
                        if not torch.equal(got, want):
                            errors.append("thread %d iteration %d: %s differs" % (i, it, what))
                            return
        except Exception as e:  # surfaced by the assertion below
            errors.append("thread %d: %r" % (i, e))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors



def test_mfma_calibration_loop(rt, dev):
    """The register-only MFMA loop the bench calibrates the int8 roofline with: its operation count is what it says
    (the accumulators hold exactly `iters` times the products of the fragments it loaded)."""
    import torch
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    rng = np.random.default_rng(11)
    src = rng.integers(-128, 128, 65536, dtype=np.int8)
    sink = torch.zeros((cus, 8, 64, 4), dtype=torch.int32, device=dev)
    iters = 37
    ops = rt.calib_mfma_i8(dev_t(src, dev), sink, iters, False)
    torch.cuda.synchronize()
    assert ops == iters * 16 * 2 * 32 * 32 * 32 * 8 * cus
    got = sink.cpu().numpy().astype(np.int64)
    assert np.array_equal(got[0], got[-1])          # every compute unit ran the same loop
    s = src.astype(np.int64)
    m = np.arange(32)
    for wave in range(8):
        def colsum(base):
            # sum over the 32 rows of a fragment, per lane half c and byte t
            off = base + (wave & 3) * 2048 + m[:, None, None] * 64 + ((np.arange(2)[None, :, None] ^ ((m[:, None, None] >> 2) & 3)) << 4) \
                + np.arange(16)[None, None, :]
            return s[off].sum(axis=0)
        want = 0
        for h in range(2):
            sa = sum(colsum(i * 8192 + h * 32) for i in range(4))
            sb = sum(colsum(32768 + j * 8192 + h * 32) for j in range(2))
            want += int((sa * sb).sum())
        want *= iters
        assert (int(got[0, wave].sum()) - want) % (1 << 32) == 0, wave
    # with the fragment reads: zeros stay zeros, and a launch is deterministic
    z = torch.zeros(65536, dtype=torch.int8, device=dev)
    rt.calib_mfma_i8(z, sink, 5, True)
    torch.cuda.synchronize()
    assert int(sink.abs().max()) == 0
    a = torch.empty_like(sink)
    rt.calib_mfma_i8(dev_t(src, dev), sink, 9, True)
    rt.calib_mfma_i8(dev_t(src, dev), a, 9, True)
    torch.cuda.synchronize()
    assert torch.equal(a, sink) and int(sink.abs().max()) > 0
    with pytest.raises(RuntimeError):
        rt.calib_mfma_i8(dev_t(src, dev), sink, 0, False)
