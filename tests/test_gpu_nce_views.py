"""NCE tasks whose input and output are views of larger tensors (a channel slice, a window in H or W): the operand
strides of the task, bit-exact against the CPU oracle on every device kernel, with the parent tensors' elements
outside the view checked untouched.  The NPU reads a task's input out of its parent tensor and writes its output
through the buffer's strides (runtime_dpu_parser_imports.cpp.inc:850-852, 1031-1090)."""
import zlib

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GUARD = 77


def seed(*parts):
    return zlib.crc32(repr(parts).encode())


def dev_t(a, dev):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


# how the task's tensor sits in its parent: (rows before, rows after, columns before, columns after, channels before, channels after)
VIEWS = {
    "dense": (0, 0, 0, 0, 0, 0),
    "chan16": (0, 0, 0, 0, 16, 32),     # a channel slice at a 16-byte boundary (Concat elided)
    "chan_odd": (0, 0, 0, 0, 5, 6),     # the same at an odd channel: no 16-byte access lines up
    "rows": (2, 1, 0, 0, 0, 0),         # a band of rows of a taller tensor (a layer tiled over H)
    "window": (1, 2, 3, 1, 0, 0),       # a window in H and W
    "window_chan": (1, 1, 2, 3, 16, 16),
}


def make_view(rng, shape, kind, dtype, fill=None):
    """(parent array, view of the task's shape inside it)."""
    N, H, W, Cn = shape
    t, b, l, r, c0, c1 = VIEWS[kind]
    pshape = (N, H + t + b, W + l + r, Cn + c0 + c1)
    if fill is not None:
        parent = np.full(pshape, fill, dtype=dtype)
    elif dtype == np.uint8:
        parent = rng.integers(0, 256, pshape, dtype=np.uint8)
    else:
        parent = rng.integers(-128, 128, pshape).astype(np.int8)
    return parent, parent[:, t:t + H, l:l + W, c0:c0 + Cn]


def torch_view(tp, shape, kind):
    N, H, W, Cn = shape
    t, b, l, r, c0, c1 = VIEWS[kind]
    return tp[:, t:t + H, l:l + W, c0:c0 + Cn]


def run_views(rt, orc, dev, rng, g, in_kind, out_kind, in_u8=True, out_signed=False, out_f16=False, zp_in=None, zp_w=0,
              force=None, mode="LPRELU", tuning=()):
    import torch
    N, H, W, IC, OC, KY, KX = (g[k] for k in ("N", "H", "W", "IC", "OC", "KY", "KX"))
    strides, pads = g.get("strides", (1, 1)), g.get("pads", (0, 0, 0, 0))
    OH = (H + pads[2] + pads[3] - KY) // strides[0] + 1
    OW = (W + pads[0] + pads[1] - KX) // strides[1] + 1
    if zp_in is None:
        zp_in = 128 if in_u8 else -5
    inp_parent, inp = make_view(rng, (N, H, W, IC), in_kind, np.uint8 if in_u8 else np.int8)
    w = rng.integers(-127, 128, (OC, KY, KX, IC)).astype(np.int8) if zp_w == 0 else rng.integers(0, 256, (OC, KY, KX, IC), dtype=np.uint8)
    mults = rng.integers(2 ** 14, 2 ** 15, OC)
    shifts = rng.integers(14, 22, OC)
    bias = rng.integers(-2 ** 15, 2 ** 15, OC).astype(np.int32)
    wt = rt.make_weights_table(mults, shifts, bias, KY * KX * IC)
    odt = np.uint16 if out_f16 else (np.int8 if out_signed else np.uint8)
    clamp = (-(2 ** 31), 2 ** 31 - 1) if out_f16 else ((-128, 127) if out_signed else (0, 255))
    md = getattr(rt, "PPE_" + mode)
    pm, ps = {"NOOP": (1, 0), "LRELU": (0, 0), "LPRELU": (1638, 14)}[mode]
    p = rt.PpeInt(md, clamp[0], clamp[1], 1638, 14)
    zp_out = 0 if out_f16 else 3
    # the oracle writes its view of a guard-filled parent; the device must produce the same parent
    guard = np.array(GUARD, dtype=np.uint8).astype(odt) if not out_f16 else np.uint16(0x3c00)
    want_parent, want_view = make_view(rng, (N, OH, OW, OC), out_kind, odt, fill=guard)
    orc.nce_conv(inp, w, wt, orc.ppe(pm, ps, zp_out, clamp[0], clamp[1]), zp_in=zp_in, zp_w=zp_w, strides=strides,
                 pads=(pads[2], pads[0], pads[3], pads[1]), out_signed=out_signed, out_f16=out_f16, out=want_view)
    # ... and equals the dense computation on a packed copy of the view
    dense = orc.nce_conv(np.ascontiguousarray(inp), w, wt, orc.ppe(pm, ps, zp_out, clamp[0], clamp[1]), zp_in=zp_in, zp_w=zp_w,
                         strides=strides, pads=(pads[2], pads[0], pads[3], pads[1]), out_signed=out_signed, out_f16=out_f16)
    assert np.array_equal(want_view, dense)

    tin_parent = dev_t(inp_parent, dev)
    tout_parent = torch.from_numpy(np.full(want_parent.shape, guard, dtype=odt).view(np.float16 if out_f16 else odt)).to(dev)
    tin = torch_view(tin_parent, (N, H, W, IC), in_kind)
    tout = torch_view(tout_parent, (N, OH, OW, OC), out_kind)
    knobs = list(tuning)
    if force in ("regw", "tile", "stream"):
        knobs += [("VPX_CONV_KERNEL", force), ("VPX_NCE_KERNEL", "conv")]
    elif force:
        knobs += [("VPX_NCE_KERNEL", force)]
    for k, v in knobs:
        rt.set_tuning(k, v)
    try:
        rt.nce_task(tin, dev_t(w, dev), dev_t(wt, dev), tout, p, zp_in=zp_in, zp_w=zp_w, zp_out=zp_out, strides=strides, pads=pads)
        torch.cuda.synchronize()
    finally:
        for k, _ in knobs:
            rt.set_tuning(k, None)
    got_parent = tout_parent.cpu().numpy()
    if out_f16:
        got_parent = got_parent.view(np.uint16)
    name = rt.nce_last_kernel()
    t, b, l, r, c0, c1 = VIEWS[out_kind]
    got_view = got_parent[:, t:t + OH, l:l + OW, c0:c0 + OC]
    assert np.array_equal(got_view, want_view), "%s in=%s out=%s: %d mismatches inside the view" % (
        name, in_kind, out_kind, int((got_view != want_view).sum()))
    assert np.array_equal(got_parent, want_parent), "%s in=%s out=%s: wrote outside the view" % (name, in_kind, out_kind)
    return name


# one geometry per device kernel, with the knob that sends it there
FAMILIES = {
    "gemm256": (dict(N=2, H=20, W=16, IC=128, OC=300, KY=1, KX=1), None, (("VPX_GEMM_TILE", "256"),), "nce_gemm_mfma"),
    "gemm256w4": (dict(N=1, H=24, W=24, IC=64, OC=260, KY=1, KX=1), None, (("VPX_GEMM_TILE", "256"), ("VPX_GEMM_WAVES", "4")), "nce_gemm_mfma"),
    "gemm128": (dict(N=1, H=13, W=21, IC=320, OC=200, KY=1, KX=1), None, (("VPX_GEMM_TILE", "128"),), "nce_gemm_mfma"),
    "gemm_shortk": (dict(N=3, H=9, W=10, IC=64, OC=130, KY=1, KX=1), None, (("VPX_GEMM_TILE", "128"),), "nce_gemm_mfma"),
    "gemm_stride2": (dict(N=2, H=17, W=13, IC=128, OC=200, KY=1, KX=1, strides=(2, 2)), None, (), "nce_gemm_mfma"),
    "regw": (dict(N=2, H=9, W=11, IC=64, OC=64, KY=3, KX=3, pads=(1, 1, 1, 1)), "regw", (), "nce_conv_regw"),
    "regw_s2": (dict(N=1, H=15, W=14, IC=64, OC=70, KY=3, KX=3, strides=(2, 2), pads=(0, 1, 1, 0)), "regw", (), "nce_conv_regw"),
    "tile": (dict(N=2, H=12, W=10, IC=128, OC=96, KY=3, KX=3, pads=(1, 1, 1, 1)), None, (), "nce_conv_tile"),
    "tile5x5": (dict(N=1, H=20, W=20, IC=64, OC=32, KY=5, KX=5, strides=(1, 2), pads=(2, 2, 2, 2)), None, (), "nce_conv_tile"),
    "stream": (dict(N=1, H=9, W=9, IC=256, OC=96, KY=3, KX=3, pads=(1, 1, 1, 1)), None, (), "nce_conv_stream"),
    "stream_ksplit": (dict(N=2, H=7, W=7, IC=512, OC=128, KY=3, KX=3, pads=(1, 1, 1, 1)), None, (), "nce_conv_stream"),
    "rows16": (dict(N=2, H=30, W=30, IC=16, OC=64, KY=7, KX=7, strides=(2, 2), pads=(3, 3, 3, 3)), None, (), "nce_conv_rows16"),
    "rows16_48": (dict(N=1, H=10, W=12, IC=48, OC=40, KY=3, KX=3, pads=(1, 1, 1, 1)), None, (), "nce_conv_rows16"),
    "rows16_cols": (dict(N=1, H=12, W=200, IC=16, OC=32, KY=3, KX=3, strides=(1, 2), pads=(1, 1, 1, 1)), None, (("VPX_CONV_COLS", "40"),), "nce_conv_rows16"),
    "gather": (dict(N=2, H=9, W=11, IC=96, OC=70, KY=3, KX=3, pads=(1, 1, 1, 1)), "gather", (), "nce_conv_mfma"),
    "gather16": (dict(N=1, H=10, W=12, IC=48, OC=40, KY=3, KX=3, pads=(1, 1, 1, 1)), "gather", (), "nce_conv_mfma16"),
    "naive": (dict(N=2, H=6, W=7, IC=10, OC=9, KY=3, KX=2, pads=(1, 0, 0, 1)), None, (), "nce_conv_naive"),
}

COMBOS = [("chan16", "chan16"), ("window", "chan_odd"), ("window_chan", "window"), ("rows", "window_chan"), ("dense", "rows")]


@pytest.mark.parametrize("in_kind,out_kind", COMBOS)
@pytest.mark.parametrize("family", sorted(FAMILIES))
def test_views_on_every_kernel(rt, orc, dev, family, in_kind, out_kind):
    g, force, tuning, kernel = FAMILIES[family]
    rng = np.random.default_rng(seed(family, in_kind, out_kind))
    for in_u8, out_signed in ((True, False), (False, True)):
        name = run_views(rt, orc, dev, rng, g, in_kind, out_kind, in_u8=in_u8, out_signed=out_signed, force=force, tuning=tuning)
        assert name == kernel


@pytest.mark.parametrize("knob", ["on", "wide"])
@pytest.mark.parametrize("N,in_kind,out_kind,kernel", [
    (2, "chan16", "chan16", "nce_gemm_regb"), (2, "dense", "chan16", "nce_gemm_regb"), (2, "chan16", "dense", "nce_gemm_regb"),
    (1, "rows", "rows", "nce_gemm_regb"),
    # rows that are not a fixed pitch apart, or that do not start on 16 bytes: the tile kernel
    (2, "window", "chan16", "nce_gemm_mfma"), (2, "chan16", "window", "nce_gemm_mfma"), (2, "chan16", "chan_odd", "nce_gemm_mfma")])
def test_views_on_the_weights_in_registers_matmul(rt, orc, dev, knob, N, in_kind, out_kind, kernel):
    """It serves operands whose rows are a fixed pitch apart (channel slices, a band of rows of one image)."""
    rng = np.random.default_rng(seed("regb", knob, N, in_kind, out_kind))
    for IC, OC in ((64, 208), (128, 128), (256, 64)):
        g = dict(N=N, H=20, W=16, IC=IC, OC=OC, KY=1, KX=1)
        for in_u8, out_signed in ((True, False), (False, True)):
            name = run_views(rt, orc, dev, rng, g, in_kind, out_kind, in_u8=in_u8, out_signed=out_signed, tuning=(("VPX_GEMM_REGB", knob),))
            assert name == kernel


@pytest.mark.parametrize("in_kind,out_kind", [("chan16", "chan_odd"), ("window_chan", "window_chan"), ("window", "chan16")])
@pytest.mark.parametrize("family", ["gemm256", "gemm128", "tile", "stream", "rows16", "rows16_48", "gather", "gather16", "naive"])
def test_views_with_an_fp16_output(rt, orc, dev, family, in_kind, out_kind):
    g, force, tuning, kernel = FAMILIES[family]
    rng = np.random.default_rng(seed(family, in_kind, out_kind, 16))
    name = run_views(rt, orc, dev, rng, g, in_kind, out_kind, out_f16=True, force=force, tuning=tuning, mode="LRELU")
    assert name == kernel


@pytest.mark.parametrize("in_kind,out_kind", [("window_chan", "chan16"), ("rows", "window")])
@pytest.mark.parametrize("family", ["gemm256", "gemm_stride2", "regw", "tile", "stream", "rows16_48", "gather"])
def test_views_with_a_weight_zero_point(rt, orc, dev, family, in_kind, out_kind):
    """The term of the weight zero point sums the input pixels under every window: it reads the view too."""
    g, force, tuning, kernel = FAMILIES[family]
    rng = np.random.default_rng(seed(family, in_kind, out_kind, 31))
    name = run_views(rt, orc, dev, rng, g, in_kind, out_kind, zp_in=9, zp_w=131, force=force, tuning=tuning)
    assert name == kernel


@pytest.mark.parametrize("family", ["gemm256", "regw", "rows16"])
def test_an_input_view_off_the_16_byte_grid_takes_the_general_kernel(rt, orc, dev, family):
    g, force, tuning, kernel = FAMILIES[family]
    rng = np.random.default_rng(5)
    assert run_views(rt, orc, dev, rng, g, "chan_odd", "chan16", force=None, tuning=()) == "nce_conv_naive"


def test_matmul_on_a_column_block_of_a_wider_matrix(rt, orc, dev):
    """A [M, K] block of a [M, K + ...] matrix times B into a column block of a wider result: leading dimensions."""
    import torch
    rng = np.random.default_rng(11)
    M, K, N = 300, 128, 520
    big_a = rng.integers(-128, 128, (M, K + 64)).astype(np.int8)
    b = rng.integers(-127, 128, (N, K)).astype(np.int8)
    wt = rt.make_weights_table(rng.integers(2 ** 14, 2 ** 15, N), rng.integers(18, 24, N), rng.integers(-2 ** 15, 2 ** 15, N).astype(np.int32), K)
    big_out = torch.full((M, N + 48), GUARD, dtype=torch.int8, device=dev)
    ta = dev_t(big_a, dev)
    rt.nce_task(ta[:, 32:32 + K].unflatten(0, (1, M)).unsqueeze(2), dev_t(b.reshape(N, 1, 1, K), dev), dev_t(wt, dev),
                big_out[:, 16:16 + N].unflatten(0, (1, M)).unsqueeze(2), rt.PpeInt(rt.PPE_LPRELU, -128, 127, 1638, 14), zp_in=3)
    torch.cuda.synchronize()
    assert rt.nce_last_kernel() == "nce_gemm_mfma"
    want = orc.nce_matmul(np.ascontiguousarray(big_a[:, 32:32 + K]), b, wt, orc.ppe(1638, 14, 0, -128, 127), zp_a=3)
    got = big_out.cpu().numpy()
    assert np.array_equal(got[:, 16:16 + N], want)
    assert (got[:, :16] == GUARD).all() and (got[:, 16 + N:] == GUARD).all()


@pytest.mark.parametrize("out_f16", [False, True])
@pytest.mark.parametrize("kinds", [("chan16", "window", "chan_odd"), ("window_chan", "dense", "chan16"), ("dense", "chan_odd", "window_chan"),
                                   ("rows", "rows", "rows")])
def test_eltwise_on_views(rt, orc, dev, kinds, out_f16):
    import torch
    rng = np.random.default_rng(seed(kinds, out_f16))
    in1_mult, in2_mult, out_mult, out_shift = rt.eltwise_quantization_approximation(0.02, 0.035, 0.05, 0)
    for shape, a_signed, b_signed, out_signed, subtract in (((2, 5, 7, 40), False, True, False, False), ((1, 6, 4, 64), True, False, True, True),
                                                            ((3, 2, 3, 7), True, True, False, False)):
        a_parent, a = make_view(rng, shape, kinds[0], np.int8 if a_signed else np.uint8)
        b_parent, b = make_view(rng, shape, kinds[1], np.int8 if b_signed else np.uint8)
        odt = np.uint16 if out_f16 else (np.int8 if out_signed else np.uint8)
        clamp = (-(2 ** 31), 2 ** 31 - 1) if out_f16 else ((-128, 127) if out_signed else (0, 255))
        zpo = 0 if out_f16 else 5
        guard = np.uint16(0x3c00) if out_f16 else np.array(GUARD, dtype=np.uint8).astype(odt)
        want_parent, want_view = make_view(rng, shape, kinds[2], odt, fill=guard)
        orc.nce_eltwise(a, b, orc.ppe(1638, 14, zpo, clamp[0], clamp[1]), 3, -2 if b_signed else 120, in1_mult, in2_mult, out_mult, out_shift,
                        subtract=subtract, out_signed=out_signed, out_f16=out_f16, out=want_view)
        dense = orc.nce_eltwise(np.ascontiguousarray(a), np.ascontiguousarray(b), orc.ppe(1638, 14, zpo, clamp[0], clamp[1]), 3,
                                -2 if b_signed else 120, in1_mult, in2_mult, out_mult, out_shift, subtract=subtract, out_signed=out_signed,
                                out_f16=out_f16)
        assert np.array_equal(want_view, dense)
        ta, tb = dev_t(a_parent, dev), dev_t(b_parent, dev)
        tout = torch.from_numpy(np.full(want_parent.shape, guard, dtype=odt).view(np.float16 if out_f16 else odt)).to(dev)
        ppe = rt.PpeInt(rt.PPE_LPRELU, clamp[0], clamp[1], 1638, 14, out_mult, out_shift, in1_mult, in2_mult)
        views = [torch_view(t_, shape, k) for t_, k in zip((ta, tb, tout), kinds)]
        rt.nce_eltwise(views[0], views[1], views[2], ppe, 3, -2 if b_signed else 120, zpo, subtract=subtract)
        torch.cuda.synchronize()
        # (a band of rows of a single image is a dense tensor)
        assert rt.nce_last_kernel() == ("nce_eltwise_kernel" if all(v.is_contiguous() for v in views) else "nce_eltwise_views_kernel")
        got = tout.cpu().numpy()
        got = got.view(np.uint16) if out_f16 else got
        assert np.array_equal(got, want_parent), "%s %s: %d mismatches" % (kinds, shape, int((got != want_parent).sum()))


def test_view_descriptors_are_validated(rt, dev):
    import torch
    inp = torch.zeros((1, 8, 8, 64), dtype=torch.uint8, device=dev)
    w = torch.zeros((64, 1, 1, 64), dtype=torch.int8, device=dev)
    wt = torch.zeros((64, 4), dtype=torch.int32, device=dev)
    out = torch.zeros((1, 8, 8, 64), dtype=torch.uint8, device=dev)
    ok = rt.PpeInt(rt.PPE_NOOP, 0, 255, 1, 0)

    def task(in_strides=None, out_strides=None, groups=0):
        import ctypes as C
        t = rt.NceTask()
        t.task_type = 0
        t.groups = groups
        t.input, t.weights, t.weight_table, t.output = inp.data_ptr(), w.data_ptr(), wt.data_ptr(), out.data_ptr()
        t.input_type, t.weights_type, t.output_type = rt.NN_U8, rt.NN_I8, rt.NN_U8
        t.N, t.H, t.W, t.IC, t.OC = 1, 8, 8, 64, 64
        t.kernel_size[0] = t.kernel_size[1] = t.kernel_strides[0] = t.kernel_strides[1] = 1
        t.ppe = ok
        for field, vals in ((t.input_strides, in_strides), (t.output_strides, out_strides)):
            for i, v in enumerate(vals or ()):
                field[i] = v
        return rt.lib().vpx_nce_task(C.byref(t), None)

    assert task() == 0
    assert task(in_strides=(4096, 512, 64, 1), out_strides=(4096, 512, 64, 1)) == 0      # the dense strides, spelled out
    assert task(in_strides=(4096, 512, 64, 2)) == rt.ERROR_INVALID_ARGUMENT               # channels must be contiguous
    assert task(out_strides=(4096, 512, 32, 1)) == rt.ERROR_INVALID_ARGUMENT              # pixels overlap
    assert task(out_strides=(4096, 256, 64, 1)) == rt.ERROR_INVALID_ARGUMENT              # rows overlap
    assert task(in_strides=(4096, 512, -64, 1)) == rt.ERROR_INVALID_ARGUMENT
    assert task(in_strides=(8192, 1024, 128, 1), groups=2) == rt.ERROR_UNSUPPORTED_FEATURE  # a grouped task takes dense operands
    torch.cuda.synchronize()
