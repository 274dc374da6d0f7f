"""Host-side logic of the product library against the reference's golden vectors and the oracle:
parameter packing, scale approximation, weights table, PPE attribute, C-ABI surface.  No GPU and no
compute entry point is called here."""
import ctypes as C
import json
import os
import re
import struct

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
with open(os.path.join(HERE, "golden", "reference_goldens.json")) as f:
    GOLD = json.load(f)


def test_library_exports_every_declared_symbol(rt):
    L = rt.lib()
    declared = set()
    for header in ("vpx_runtime.h", "vpx_compiler_utils.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        declared |= set(re.findall(r"VPX_API[^;(]*?\b(vpx_\w+)\s*\(", text))
    assert declared, "no declarations found"
    assert declared == set(rt.EXPORTS)
    for name in sorted(declared):
        assert getattr(L, name) is not None, name
    assert L.vpx_get_version() == 1
    names = [L.vpx_sw_kernel_name(i).decode() for i in range(L.vpx_sw_kernel_count())]
    for must in ("softmax", "mvn1", "fake_quantize", "quantize", "dequantize", "convert", "eltwise_add", "mvn1_sum", "mvn1_mean_var",
                 "mvn1_norm", "mvn6", "dynamic_quantize", "dynamic_dequantize", "prelu_fp16", "leaky_relu_fp16", "activation_relu",
                 "activation_clamp"):
        assert must in names and L.vpx_sw_kernel_supported(must.encode()) == 1
    # every entry the Python binding can name exists in the library
    for entry, _ in rt.ACTIVATIONS.values():
        assert entry in names, entry
    assert len(names) == len(set(names))
    assert L.vpx_sw_kernel_supported(b"no_such_kernel") == 0
    assert L.vpx_sw_kernel_name(10 ** 6) is None


def test_memref_struct_is_36_bytes_packed():
    # sw_params::MemRefData, common_types.h:85-101
    text = open(os.path.join(ROOT, "include", "vpx_sw_params.h")).read()
    assert "#pragma pack(push, 1)" in text
    from vpux_plugin_amd import runtime as rt
    dims = (C.c_int32 * 1)(4)
    strides = (C.c_int64 * 1)(16)
    d = rt.TensorDesc(1, dims, strides, rt.NN_FP16, 0x1, rt.LOC_DDR)
    ins = (rt.TensorDesc * 1)(d)
    size = C.c_size_t(0)
    rt.check(rt.lib().vpx_create_kernel_params(ins, 1, ins, 1, None, 0, None, C.byref(size)))
    assert size.value == 2 * 36 + 2 * (4 + 8)


def test_error_codes_without_gpu(rt):
    L = rt.lib()
    assert L.vpx_sw_kernel_launch(None, None, 0, None, 0, None) == rt.ERROR_INVALID_NULL_HANDLE
    assert b"null" in L.vpx_get_last_error()
    blob = b"\0" * 72
    addrs = (rt.MemRefAddr * 2)()
    assert L.vpx_sw_kernel_launch(b"bogus_kernel", blob, len(blob), addrs, 2, None) == rt.ERROR_UNSUPPORTED_FEATURE
    assert b"bogus_kernel" in L.vpx_get_last_error()
    # wrong operand count, short blob, zero-rank memref: all rejected before anything touches the device
    assert L.vpx_sw_kernel_launch(b"convert", blob, len(blob), addrs, 3, None) == rt.ERROR_INVALID_ARGUMENT
    assert L.vpx_sw_kernel_launch(b"convert", blob, 10, addrs, 2, None) == rt.ERROR_INVALID_ARGUMENT
    assert L.vpx_sw_kernel_launch(b"convert", blob, len(blob), addrs, 2, None) == rt.ERROR_INVALID_ARGUMENT
    # kernels with optional operands find the end of their memref list by a marker word
    assert L.vpx_sw_kernel_launch(b"mvn6", blob, len(blob), addrs, 2, None) == rt.ERROR_INVALID_ARGUMENT
    assert b"marker" in L.vpx_get_last_error()
    assert L.vpx_sw_kernel_launch(b"dynamic_dequantize", blob, len(blob), addrs, 2, None) == rt.ERROR_INVALID_ARGUMENT
    marked = b"\0" * 36 + struct.pack("<q", 2 ** 63 - 1) + b"\0" * 28  # one memref, then the delimiter: too few operands
    assert L.vpx_sw_kernel_launch(b"dynamic_dequantize", marked, len(marked), addrs, 1, None) == rt.ERROR_INVALID_ARGUMENT
    # activation attributes must be present
    short = b"\0" * 72
    assert L.vpx_sw_kernel_launch(b"activation_clamp", short, len(short), addrs, 2, None) == rt.ERROR_INVALID_ARGUMENT
    assert L.vpx_nce_task(None, None) == rt.ERROR_INVALID_NULL_HANDLE
    t = rt.NceTask()
    assert L.vpx_nce_task(C.byref(t), None) == rt.ERROR_INVALID_NULL_HANDLE  # null buffers
    t.task_type = 1  # DWCONV
    assert L.vpx_nce_task(C.byref(t), None) == rt.ERROR_UNSUPPORTED_FEATURE
    t.task_type = 4  # ELTWISE: implemented, so the null buffers are what is refused
    assert L.vpx_nce_task(C.byref(t), None) == rt.ERROR_INVALID_NULL_HANDLE


def test_half_conversion_matches_oracle(rt, orc):
    L = rt.lib()
    rng = np.random.default_rng(11)
    bits = np.concatenate([rng.integers(0, 1 << 32, 200000, dtype=np.uint64).astype(np.uint32),
                           (np.arange(90, 150, dtype=np.uint32)[:, None] << 23 |
                            np.array([0, 1, 0xfff, 0x1000, 0x1001, 0x7ff000, 0x7fffff, 0x7fe000, 0x3000],
                                     dtype=np.uint32)[None, :]).ravel()])
    x = bits.view(np.float32)
    want = orc.f32_to_f16(x)
    got = np.array([L.vpx_float_to_half_bits(C.c_float(float(v))) if not np.isnan(v) else 0 for v in x[:20000]],
                   dtype=np.uint16)
    ok = ~np.isnan(x[:20000])
    assert np.array_equal(got[ok], want[:20000][ok])
    tail = x[200000:]
    got_t = np.array([L.vpx_float_to_half_bits(C.c_float(float(v))) for v in tail], dtype=np.uint16)
    assert np.array_equal(got_t, want[200000:])
    for h in (0, 1, 0x3ff, 0x400, 0x3c00, 0x7bff, 0x7c00, 0x8001, 0xfbff):
        assert L.vpx_half_bits_to_float(h) == orc.f16_to_f32(np.array([h], np.uint16))[0]


def test_approximate_goldens_and_oracle(rt, orc):
    for c in GOLD["approximate"]["cases"]:
        assert rt.approximate(c["bits"], c["target"]) == (c["mult"], c["shift"], 0), c
    rng = np.random.default_rng(12)
    for t in np.exp(rng.uniform(np.log(1e-9), np.log(1000.0), 500)):
        for bits in (11, 15):
            assert rt.approximate(bits, float(t)) == orc.approximate(bits, float(t))
    # exponent above the bit width needs a post shift, which the reference refuses
    with pytest.raises(rt.VpxError) as e:
        rt.approximate(15, 2.0 ** 20)
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT and "post-shift" in e.value.text


def test_eltwise_approximation_goldens(rt):
    for c in GOLD["eltwise_approximation"]["cases"]:
        got = rt.eltwise_quantization_approximation(c["in1"], c["in2"], c["out"])
        assert got == (c["in1_mult"], c["in2_mult"], c["out_mult"], c["out_shift"]), c
    with pytest.raises(rt.VpxError):
        rt.eltwise_quantization_approximation(0.01, -0.01, 0.05)  # one negative scale on ADD


def test_weights_table(rt, orc):
    for c in GOLD["weights_table_layout"]["ptr_step_cases"]:
        t = rt.get_weights_table(0.5, 0.25, [0.125], None, c["OC"], weights_ptr_step=c["step"])
        if "expected_ptrs" in c:
            assert t[:, 0].tolist() == c["expected_ptrs"]
        else:
            assert [t[0, 0], t[1, 0], t[-2, 0], t[-1, 0]] == c["expected_first_last"]
        assert np.all(t[:, 1] == 0xFFFFFF) and np.all(t[:, 3] == 0)
    # per-channel scales: word 2 = mult << 16 | shift << 8 of approximate(w_scale * in_scale / out_scale),
    # word 3 = round(bias / (in_scale * w_scale))
    rng = np.random.default_rng(13)
    OC = 37
    ws = np.exp(rng.uniform(np.log(1e-4), np.log(0.1), OC))
    bias = rng.normal(0, 3, OC)
    in_s, out_s = 0.02, 0.05
    t = rt.get_weights_table(in_s, out_s, ws, bias, OC, weights_ptr_step=576)
    for oc in range(OC):
        m, s, _ = orc.approximate(15, ws[oc] * in_s / out_s)
        assert t[oc, 2] == orc.wt_pack_scale(s, m)
        assert t[oc, 3] == int(np.round(bias[oc] / (in_s * ws[oc])))
        assert t[oc, 0] == oc * 576
    with pytest.raises(rt.VpxError):
        rt.get_weights_table(in_s, out_s, ws, bias, OC, weights_ptr_step=24)  # not 16-byte aligned
    with pytest.raises(rt.VpxError):
        rt.get_weights_table(in_s, out_s, ws[:5], bias, OC)
    assert np.array_equal(rt.make_weights_table([20000, 30000], [20, 24], [5, -7], 64),
                          orc.make_weights_table([20000, 30000], [20, 24], [5, -7], 64))


def test_ppe_int_attr_goldens(rt):
    g = GOLD["ppe_int_attr"]
    u8 = g["u8_type"]
    u8t = (u8["scale"], u8["zero_point"], u8["storage_min"], u8["storage_max"])
    modes = {"NOOP": rt.PPE_NOOP, "LRELU": rt.PPE_LRELU, "LRELUX": rt.PPE_LRELUX, "LPRELU": rt.PPE_LPRELU}
    ops = {"NONE": rt.POSTOP_NONE, "RELU": rt.POSTOP_RELU, "CLAMP": rt.POSTOP_CLAMP, "LEAKY_RELU": rt.POSTOP_LEAKY_RELU}
    for c in g["cases"]:
        p = rt.retrieve_ppe_int(ops[c["post_op"]], u8t if c["out"] == "u8" else None, c.get("param0", 0.0),
                                c.get("param1", 0.0))
        if "clamp_high_unpacked_f16" in c:
            # two fp16 bit patterns in one word, low bound in the upper half (the reference's test unpacks it the same way)
            halves = np.array([(p.clamp_high >> 16) & 0xffff, p.clamp_high & 0xffff], dtype=np.uint16).view(np.float16)
            assert [float(v) for v in halves] == c["clamp_high_unpacked_f16"], c
            c = dict(c, clamp_high=p.clamp_high)
        assert (p.mode, p.clamp_low, p.clamp_high, p.lrelu_mult, p.lrelu_shift) == \
               (modes[c["mode"]], c["clamp_low"], c["clamp_high"], c["lrelu_mult"], c["lrelu_shift"]), c
    # ReLU on a float output selects LRELU; slope 0 LeakyReLU has multiplier 0; clamp [0, 6] on u8 zp 0 is LRELUX
    assert rt.retrieve_ppe_int(rt.POSTOP_RELU, None).mode == rt.PPE_LRELU
    assert rt.retrieve_ppe_int(rt.POSTOP_LEAKY_RELU, u8t, 0.0).lrelu_mult == 0
    p = rt.retrieve_ppe_int(rt.POSTOP_CLAMP, (0.05, 0, 0, 255), 0.0, 6.0)
    assert (p.mode, p.clamp_low, p.clamp_high) == (rt.PPE_LRELUX, 0, 120)


def test_softmax_packed_params_golden(rt):
    g = GOLD["softmax_packed_params"]
    shape = g["shape_nchw"]
    dims = list(reversed(shape))
    strides = [1]
    for d in dims[:-1]:
        strides.append(strides[-1] * d)
    axis, pad = g["attrs_before"]
    words = rt.generate_softmax_attr(dims, strides, strides, axis, pad)
    assert [int(w) for w in words] == g["expected_words"]
    # the BASELINE softmax shape [8,16,512,512], last axis: inner mode, rows fused to 65536 x 512
    dims = [512, 512, 16, 8]
    strides = [1, 512, 512 * 512, 512 * 512 * 16]
    w = [int(v) for v in rt.generate_softmax_attr(dims, strides, strides, 0, 0)]
    assert w[0] == 0 and w[1] == (3 << 32 | 1)
    assert [(v & 0xffffffff) for v in w[2::2]] == [512, 65536, 1]
    assert [(v & 0xffffffff) for v in w[3::2]] == [1, 512, 33554432]
    # innermost axis of 2 or 4 contiguous elements selects the hard-coded inner mode
    w = [int(v) for v in rt.generate_softmax_attr([4, 10, 3], [1, 4, 40], [1, 4, 40], 0, 0)]
    assert w[1] & 0xffffffff == 2
    # a strided innermost axis is presented as an outer axis over a unit inner dimension
    w = [int(v) for v in rt.generate_softmax_attr([8, 5], [2, 16], [2, 16], 0, 0)]
    assert (w[0] & 0xffffffff, w[1] & 0xffffffff) == (1, 3) and w[2] & 0xffffffff == 1


def test_softmax_packed_params_describe_the_same_rows(rt):
    """Whatever the packing drops or fuses, walking the packed levels must visit exactly the (input offset, output offset)
    pairs of the original tensor, and the packed axis must group them into the original softmax rows."""
    import itertools
    rng = np.random.default_rng(77)
    for case in range(300):
        rank = int(rng.integers(1, 6))
        dims = [int(rng.choice([1, 1, 2, 3, 4, 5])) for _ in range(rank)]
        axis = int(rng.integers(0, rank))

        def strides_for(gap_prob):
            st, run = [], int(rng.choice([1, 1, 1, 2, 3]))
            for d in dims:
                st.append(run)
                run *= d
                if rng.random() < gap_prob:
                    run *= int(rng.integers(2, 4))
            return st
        si, so = strides_for(0.3), strides_for(0.3 if case % 2 else 0.0)
        pad = 0
        w = [int(v) for v in rt.generate_softmax_attr(dims, si, so, axis, pad)]
        p_axis, p_pad = w[0] & 0xffffffff, w[0] >> 32
        mode, nd = w[1] & 0xffffffff, w[1] >> 32
        assert nd >= 3 and len(w) == 2 + 2 * nd and p_pad == pad
        pd = [v & 0xffffffff for v in w[2::2]]
        assert pd == [v >> 32 for v in w[2::2]]
        psi, pso = [v & 0xffffffff for v in w[3::2]], [v >> 32 for v in w[3::2]]

        def rows(dd, a, s_in, s_out):
            out = set()
            others = [range(n) if k != a else [0] for k, n in enumerate(dd)]
            for idx in itertools.product(*others):
                base_i = sum(i * s for i, s in zip(idx, s_in))
                base_o = sum(i * s for i, s in zip(idx, s_out))
                out.add(tuple((base_i + k * s_in[a], base_o + k * s_out[a]) for k in range(dd[a])))
            return out
        assert rows(dims, axis, si, so) == rows(pd, p_axis, psi, pso), (dims, si, so, axis, w)
        # variant selection: outer axis -> 3; inner axis -> 1, or 2 for packed rows of 2 or 4 values
        if p_axis != 0:
            assert mode == 3
        else:
            assert psi[0] == 1 and pso[0] == 1
            tiny = pd[0] in (2, 4) and psi[1] == pd[0] and psi[2] == pso[2]
            assert mode == (2 if tiny else 1)
        # nothing left to fuse: above the axis no two real levels are gapless in both operands (unit levels are padding)
        for k in range(p_axis + 1, nd - 1):
            if pd[k + 1] != 1:
                assert not (psi[k + 1] == psi[k] * pd[k] and pso[k + 1] == pso[k] * pd[k]), (dims, si, so, axis, w)


def test_eltwise_approximation_properties(rt):
    """The four integers must reproduce in_scale / out_scale for both inputs, fit their registers, and give both inputs
    the same shift (that is what lets the datapath add before the output multiplier)."""
    rng = np.random.default_rng(78)
    for _ in range(400):
        s1, s2, so = (float(np.exp(rng.uniform(np.log(2e-3), np.log(0.5)))) for _ in range(3))
        try:
            m1, m2, mo, sh = rt.eltwise_quantization_approximation(s1, s2, so)
        except rt.VpxError:
            continue
        assert 0 <= m1 <= 65535 and 0 <= m2 <= 65535 and 0 < mo <= 32767 and 0 <= sh <= 63
        for m, sc in ((m1, s1), (m2, s2)):
            got = m * mo / 2.0 ** sh
            # the smaller input's factor may have been shifted down: its relative error is bounded by one unit of that factor
            assert abs(got - sc / so) <= (sc / so) * (2.0 ** -13 + 1.0 / max(m, 1)), (s1, s2, so, m1, m2, mo, sh)
    # both scales negative: an add folds the sign into the output multiplier
    m1, m2, mo, sh = rt.eltwise_quantization_approximation(-0.02, -0.03, 0.05)
    p1, p2, po, ps = rt.eltwise_quantization_approximation(0.02, 0.03, 0.05)
    # (a negative scale's multiplier is floored away from zero, so its magnitude may be one more)
    assert 0 <= m1 - p1 <= 1 and 0 <= m2 - p2 <= 1 and (mo, sh) == (-po, ps)
    # a multiply (type 2) folds a single negative sign
    m1, m2, mo, sh = rt.eltwise_quantization_approximation(-0.02, 0.03, 0.05, 2)
    assert 0 <= m1 - p1 <= 1 and m2 == p2 and (mo, sh) == (-po, ps)
    # scales too far apart for either alignment are refused
    with pytest.raises(rt.VpxError):
        rt.eltwise_quantization_approximation(1e-12, 1e-12, 1e8)


def test_softmax_first_form_axis_convention():
    g = GOLD["softmax_first_form"]
    nd = len(g["shape_nchw"])
    # computeReverseMemDim (sw_kernel.cpp:29-40): nDims - 1 - memory position of the logical axis
    assert nd - 1 - g["axisInd"] == g["expected_attrs"][0] and g["padSize"] == g["expected_attrs"][1]


def test_quant_params_packing(rt, orc):
    # fp16 packing: four values per word, zero points shipped as floats too (sw_kernel.cpp:97-163)
    w = rt.get_quant_params_attr([0.5, 0.25, 2.0, 1.0, 0.125], [1, 2, 3, 4, 128], rt.NN_FP16)
    assert int(w[0]) == 5 and len(w) == 1 + 2 + 2
    h = lambda v: int(orc.f32_to_f16(np.array([v], np.float32))[0])
    assert int(w[1]) == h(0.5) | h(0.25) << 16 | h(2.0) << 32 | h(1.0) << 48
    assert int(w[2]) == h(0.125)
    assert int(w[3]) == h(1) | h(2) << 16 | h(3) << 32 | h(4) << 48
    assert int(w[4]) == h(128)
    w = rt.get_quant_params_attr([0.1], [-21], rt.NN_FP32)
    f = lambda v: struct.unpack("<I", struct.pack("<f", v))[0]
    assert [int(v) for v in w] == [1, f(0.1), f(-21.0)]


def test_kernel_params_blob_layout(rt):
    # MemRefData[in..., out...] | attrs | in dims | in strides | out dims | out strides
    def desc(dims, dtype, order, elem_bits):
        d = (C.c_int32 * len(dims))(*dims)
        st, acc = [], elem_bits
        for v in dims:
            st.append(acc)
            acc *= v
        s = (C.c_int64 * len(dims))(*st)
        return rt.TensorDesc(len(dims), d, s, dtype, order, rt.LOC_DDR), d, s

    a, *_k1 = desc([56, 56, 64, 1], rt.NN_FP16, 0x4321, 16)
    lim, *_k2 = desc([1, 1, 1, 1], rt.NN_FP16, 0x4321, 16)
    ins = (rt.TensorDesc * 5)(a, lim, lim, lim, lim)
    outs = (rt.TensorDesc * 1)(a)
    attrs = struct.pack("<q", 256)
    size = C.c_size_t(0)
    rt.check(rt.lib().vpx_create_kernel_params(ins, 5, outs, 1, attrs, len(attrs), None, C.byref(size)))
    assert size.value == 6 * 36 + 8 + 6 * 4 * (4 + 8)
    buf = C.create_string_buffer(size.value)
    rt.check(rt.lib().vpx_create_kernel_params(ins, 5, outs, 1, attrs, len(attrs), buf, C.byref(size)))
    raw = buf.raw
    data_addr, is_static, nd, dims_addr, strides_addr, dtype, order, loc = struct.unpack_from("<IIIIIIQI", raw, 0)
    assert (data_addr, is_static, nd, dims_addr, strides_addr, dtype, order, loc) == (0, 1, 4, 0, 0, 2, 0x4321, 1)
    assert struct.unpack_from("<q", raw, 6 * 36)[0] == 256
    tail = 6 * 36 + 8
    assert struct.unpack_from("<4i", raw, tail) == (56, 56, 64, 1)                    # first input dims
    assert struct.unpack_from("<4q", raw, tail + 5 * 16) == (16, 16 * 56, 16 * 56 * 56, 16 * 56 * 56 * 64)
    assert struct.unpack_from("<4i", raw, tail + 5 * 16 + 5 * 32) == (56, 56, 64, 1)  # output dims
    # a buffer that is too small is refused and the needed size reported
    small = C.create_string_buffer(8)
    sz = C.c_size_t(8)
    assert rt.lib().vpx_create_kernel_params(ins, 5, outs, 1, attrs, len(attrs), small, C.byref(sz)) == \
        rt.ERROR_INVALID_ARGUMENT
    assert sz.value == size.value


def test_dynamic_dequantize_blob_matches_the_lit_golden(rt):
    """bufferize_sw_ops_to_VPUIP_sw_kernel.mlir:906-929: operands (input, scale, zero point, output), attrs = [INT64_MAX]."""
    def desc(dims, dtype, elem_bits):
        d = (C.c_int32 * len(dims))(*dims)
        st, acc = [], elem_bits
        for v in dims:
            st.append(acc)
            acc *= v
        s = (C.c_int64 * len(dims))(*st)
        return rt.TensorDesc(len(dims), d, s, dtype, 0x4321, rt.LOC_DDR), d, s

    q, *_k1 = desc([51, 3, 7, 16], rt.NN_I8, 8)
    sc, *_k2 = desc([1, 3, 1, 16], rt.NN_FP16, 16)
    zp, *_k3 = desc([51, 1, 7, 16], rt.NN_I8, 8)
    out, *_k4 = desc([51, 3, 7, 16], rt.NN_FP16, 16)
    ins = (rt.TensorDesc * 3)(q, sc, zp)
    outs = (rt.TensorDesc * 1)(out)
    attrs = struct.pack("<q", 9223372036854775807)
    size = C.c_size_t(0)
    rt.check(rt.lib().vpx_create_kernel_params(ins, 3, outs, 1, attrs, len(attrs), None, C.byref(size)))
    buf = C.create_string_buffer(size.value)
    rt.check(rt.lib().vpx_create_kernel_params(ins, 3, outs, 1, attrs, len(attrs), buf, C.byref(size)))
    # the delimiter is the first word after the four MemRefData records: that is how the kernel counts its operands
    assert struct.unpack_from("<q", buf.raw, 4 * 36)[0] == 2 ** 63 - 1
    for i in range(4):
        assert struct.unpack_from("<q", buf.raw, i * 36)[0] != 2 ** 63 - 1



def test_get_kernel_info_against_lit_goldens_and_the_operator_wrappers(rt):
    """Operator attributes -> entry name + attribute bytes, as SwKernelOp::getKernelInfo derives them."""
    import torch
    i64 = lambda *v: struct.pack("<%dq" % len(v), *v)
    f32 = lambda v: struct.pack("<f", v)
    x = torch.empty((1, 1, 1, 1000), dtype=torch.float16)
    # bufferize_sw_ops_to_VPUIP_sw_kernel.mlir:203-211 (axisInd = 3, padSize = 3 -> [0, 3]) and :225-242 (-> [0, 0])
    assert rt.get_kernel_info("SoftMax", x, axis_ind=3, pad_size=3) == ("softmax", i64(0, 3))
    assert rt.get_kernel_info("SoftMax", x, axis_ind=3) == ("softmax", i64(0, 0))
    assert rt.get_kernel_info("SoftMax", x.float(), axis_ind=-1)[0] == "softmaxFp32"
    # the axis is a logical one: channels of an NHWC tensor are the innermost memory dimension
    nhwc = rt.Operand(torch.empty((2, 5, 7, 16), dtype=torch.float16), "NHWC")
    assert rt.get_kernel_info("SoftMax", nhwc, axis_ind=1)[1] == i64(0, 0)
    assert rt.get_kernel_info("SoftMax", nhwc, axis_ind=3)[1] == i64(1, 0)
    assert rt.get_kernel_info("SoftMax", nhwc, axis_ind=0)[1] == i64(3, 0)
    # dialect/VPUIP/ops/sw_kernel.mlir:42 (attrs = [false, true, 6.0892105102539063E-4]); a true i1 is -1
    assert rt.get_kernel_info("MVN", across_channels=0, normalize_variance=1, eps=6.0892105102539063E-4) == (
        "mvn1", i64(0, -1) + f32(6.0892105102539063E-4))
    # tile_act_shave_kernel_task.mlir:240 (MVN1Sum, attrs = [true, true])
    assert rt.get_kernel_info("MVN1Sum", across_channels=1, normalize_variance=1) == ("mvn1_sum", i64(-1, -1))
    assert rt.get_kernel_info("MVN1Normalize", across_channels=0, normalize_variance=1) == ("mvn1_norm", i64(0, -1))
    assert rt.get_kernel_info("MVN1MeanVar", orig_shape=[1, 32, 21846, 1], across_channels=1, normalize_variance=1, group_c=1,
                              eps=1e-9) == ("mvn1_mean_var", i64(1, 32, 21846, 1, -1, -1, 1) + f32(1e-9))
    # MVN6: marker, operand mask, then the axes as innermost-first memory positions
    entry, attrs = rt.get_kernel_info("MVN6", nhwc, axes=[2, 3], normalize_variance=1, eps_mode=1, eps=1e-5, has_scale=1)
    assert entry == "mvn6" and attrs == i64(-2 ** 63, 1 | 2 | 8, -1, 1) + f32(1e-5) + i64(2, 2, 1)
    # bufferize_sw_ops_to_VPUIP_sw_kernel.mlir:906-929
    assert rt.get_kernel_info("DynamicDequantize") == ("dynamic_dequantize", i64(2 ** 63 - 1))
    assert rt.get_kernel_info("FakeQuantize", levels=256) == ("fake_quantize", i64(256))
    entry, attrs = rt.get_kernel_info("Quantize", x, scales=[0.5, 0.25, 2.0], zero_points=[1, 2, 3])
    assert entry == "quantize" and attrs == rt.get_quant_params_attr([0.5, 0.25, 2.0], [1, 2, 3], rt.NN_FP16).tobytes()
    assert rt.get_kernel_info("Dequantize", x.float(), scales=[0.5], zero_points=[7])[1] == rt.get_quant_params_attr(
        [0.5], [7], rt.NN_FP32).tobytes()
    assert rt.get_kernel_info("LeakyRelu", param0=0.1) == ("leaky_relu_fp16", f32(0.1))
    assert rt.get_kernel_info("Clamp", param0=-1.5, param1=6.0) == ("activation_clamp", f32(-1.5) + f32(6.0))
    # every entry the builder names is one the library launches, with the number of float attributes its wrapper sends
    ops = {"Convert": "convert", "Add": "eltwise_add", "Subtract": "eltwise_sub", "Multiply": "eltwise_mul", "Divide": "eltwise_div",
           "Minimum": "eltwise_min", "Maximum": "eltwise_max", "PRelu": "prelu_fp16", "DynamicQuantize": "dynamic_quantize",
           "ReLU": "relu", "LeakyRelu": "leaky_relu", "Clamp": "clamp", "Negative": "negative", "Abs": "abs", "HSwish": "hswish",
           "HSigmoid": "hsigmoid", "HardSigmoid": "hardsigmoid", "Sigmoid": "sigmoid", "Tanh": "tanh", "Exp": "exp",
           "Sqrt": "sqrt", "Log": "log", "Floor": "floor", "Ceiling": "ceil", "Sign": "sign", "Elu": "elu", "Selu": "selu",
           "Swish": "swish", "Mish": "mish", "SoftPlus": "softplus", "Gelu": "gelu", "Erf": "erf"}
    for op, short in ops.items():
        entry, attrs = rt.get_kernel_info(op, param0=0.5, param1=2.0)
        assert rt.lib().vpx_sw_kernel_supported(entry.encode()) == 1, op
        if short in rt.ACTIVATIONS:
            assert (entry, len(attrs)) == (rt.ACTIVATIONS[short][0], 4 * rt.ACTIVATIONS[short][1]), op
        else:
            assert entry == short and attrs == b"", op
    with pytest.raises(rt.VpxError) as e:
        rt.get_kernel_info("TopK")
    assert e.value.code == rt.ERROR_UNSUPPORTED_FEATURE
    with pytest.raises(rt.VpxError) as e:
        rt.get_kernel_info("SoftMax", x, axis_ind=4)
    assert e.value.code == rt.ERROR_INVALID_ARGUMENT
