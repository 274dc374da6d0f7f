"""ctypes view of the CPU oracle (oracle/vpx_oracle.c) -- TEST INFRASTRUCTURE ONLY.

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import
this package.  The product package never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libvpx_oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libref_float16.so")


def build(force=False):
    """Compile the oracle (and oracle/_ref when the reference checkout is present)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-B", "-C", _HERE, "all"])


class _PPE(C.Structure):
    _fields_ = [("prelu_mult", C.c_int32), ("prelu_shift", C.c_int32), ("zp_out", C.c_int32),
                ("clamp_low", C.c_int32), ("clamp_high", C.c_int32)]


class _Conv(C.Structure):
    _fields_ = [(n, C.c_int64) for n in ("N", "H", "W", "IC", "OC", "KY", "KX", "stride_y", "stride_x", "pad_top",
                                          "pad_left", "pad_bottom", "pad_right")] + \
               [(n, C.c_int32) for n in ("in_signed", "w_signed", "out_signed", "zp_in", "zp_w")] + [("ppe", _PPE)] + \
               [("in_strides", C.c_int64 * 3), ("out_strides", C.c_int64 * 3)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        L.orc_f32_to_f16.restype = C.c_uint16
        L.orc_f32_to_f16.argtypes = [C.c_float]
        L.orc_f16_to_f32.restype = C.c_float
        L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_fake_quantize.restype = C.c_float
        L.orc_fake_quantize.argtypes = [C.c_float] * 6
        L.orc_dequantize_value.restype = C.c_float
        L.orc_dequantize_value.argtypes = [C.c_int64, C.c_double, C.c_int64]
        L.orc_quantize_value.restype = C.c_int64
        L.orc_quantize_value.argtypes = [C.c_double, C.c_double, C.c_int64, C.c_int64, C.c_int64]
        L.orc_approximate.restype = C.c_int
        L.orc_approximate.argtypes = [C.c_int, C.c_double] + [C.POINTER(C.c_int64)] * 3
        L.orc_wt_pack_scale.restype = C.c_int32
        L.orc_wt_pack_scale.argtypes = [C.c_uint8, C.c_int16]
        L.orc_ppe_requant.restype = C.c_int32
        L.orc_ppe_requant.argtypes = [C.c_int32] * 4 + [C.POINTER(_PPE)]
        L.orc_num_threads.restype = C.c_int
        _lib = L
    return _lib


def ref_lib():
    """The reference's own float16.cpp compiled in place (None when it was not built)."""
    if not os.path.exists(_REF_PATH):
        return None
    L = C.CDLL(_REF_PATH)
    L.ref_f32_to_f16.restype = C.c_uint16
    L.ref_f32_to_f16.argtypes = [C.c_float]
    L.ref_f16_to_f32.restype = C.c_float
    L.ref_f16_to_f32.argtypes = [C.c_uint16]
    L.ref_f16_add.restype = C.c_uint16
    L.ref_f16_add.argtypes = [C.c_uint16, C.c_uint16]
    return L


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _i64(seq):
    return (C.c_int64 * len(seq))(*[int(v) for v in seq])


def set_num_threads(n):
    lib().orc_set_num_threads(C.c_int(n))


def num_threads():
    return lib().orc_num_threads()


# ---- fp16 ----------------------------------------------------------------------------------

def f32_to_f16(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().orc_convert_f32_to_f16(_p(x), _p(out), C.c_size_t(x.size))
    return out


def f16_to_f32(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, dtype=np.float32)
    lib().orc_convert_f16_to_f32(_p(h), _p(out), C.c_size_t(h.size))
    return out


# ---- elementwise -----------------------------------------------------------------------------

def fake_quantize_f16(x, in_lo, in_hi, out_lo, out_hi, levels):
    """x and limits are uint16 (fp16 bit patterns) arrays of equal rank; limits broadcast NUMPY style."""
    x = np.ascontiguousarray(x, dtype=np.uint16)
    lims = [np.ascontiguousarray(l, dtype=np.uint16) for l in (in_lo, in_hi, out_lo, out_hi)]
    rank = x.ndim
    lims = [l.reshape((1,) * (rank - l.ndim) + l.shape) for l in lims]
    y = np.empty_like(x)
    ptrs = (C.c_void_p * 4)(*[l.ctypes.data for l in lims])
    lim_dims = _i64([d for l in lims for d in l.shape])
    lib().orc_fake_quantize_f16(_p(x), _p(y), C.c_int(rank), _i64(x.shape), ptrs, lim_dims, C.c_int64(levels))
    return y


def _axis_view(shape, axis):
    if axis is None:
        return 1, 1, int(np.prod(shape, dtype=np.int64))
    outer = int(np.prod(shape[:axis], dtype=np.int64))
    inner = int(np.prod(shape[axis + 1:], dtype=np.int64))
    return outer, int(shape[axis]), inner


def quantize(x, scales, zps, signed, qmin=None, qmax=None, axis=None):
    """x: uint16 (fp16 bits) or float32 array -> int8/uint8 (createQuantizeFn semantics)."""
    scales = np.atleast_1d(np.asarray(scales, dtype=np.float64))
    zps = np.atleast_1d(np.asarray(zps, dtype=np.int64))
    if qmin is None:
        qmin = -128 if signed else 0
    if qmax is None:
        qmax = 127 if signed else 255
    outer, ax, inner = _axis_view(x.shape, axis)
    assert ax == scales.size == zps.size
    q = np.empty(x.shape, dtype=np.int8 if signed else np.uint8)
    if x.dtype == np.uint16:
        fn = lib().orc_quantize_f16
    else:
        x = np.ascontiguousarray(x, dtype=np.float32)
        fn = lib().orc_quantize_f32
    x = np.ascontiguousarray(x)
    fn(_p(x), _p(q), C.c_int(int(signed)), C.c_int64(outer), C.c_int64(ax), C.c_int64(inner), _p(scales), _p(zps),
       C.c_int64(qmin), C.c_int64(qmax))
    return q


def dequantize(q, scales, zps, to_f16=True, axis=None):
    scales = np.atleast_1d(np.asarray(scales, dtype=np.float64))
    zps = np.atleast_1d(np.asarray(zps, dtype=np.int64))
    q = np.ascontiguousarray(q)
    signed = q.dtype == np.int8
    outer, ax, inner = _axis_view(q.shape, axis)
    assert ax == scales.size == zps.size
    if to_f16:
        y = np.empty(q.shape, dtype=np.uint16)
        lib().orc_dequantize_f16(_p(q), C.c_int(int(signed)), _p(y), C.c_int64(outer), C.c_int64(ax), C.c_int64(inner),
                                 _p(scales), _p(zps))
    else:
        y = np.empty(q.shape, dtype=np.float32)
        lib().orc_dequantize_f32(_p(q), C.c_int(int(signed)), _p(y), C.c_int64(outer), C.c_int64(ax), C.c_int64(inner),
                                 _p(scales), _p(zps))
    return y


ELT_OPS = {"add": 0, "sub": 1, "mul": 2, "min": 3, "max": 4, "div": 5, "prelu": 6}

ACT_OPS = {name: i for i, name in enumerate(
    ["relu", "leaky_relu", "clamp", "negative", "abs", "hswish", "hsigmoid", "hardsigmoid", "sigmoid", "tanh", "exp",
     "sqrt", "log", "floor", "ceil", "sign", "elu", "selu", "swish", "mish", "softplus", "gelu", "erf"])}


def activation_f16(op, x, p0=0.0, p1=0.0):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    y = np.empty_like(x)
    lib().orc_activation_f16(C.c_int(ACT_OPS[op]), C.c_float(p0), C.c_float(p1), _p(x), _p(y), C.c_int64(x.size))
    return y


def activation_f32(op, x, p0=0.0, p1=0.0):
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty_like(x)
    lib().orc_activation_f32(C.c_int(ACT_OPS[op]), C.c_float(p0), C.c_float(p1), _p(x), _p(y), C.c_int64(x.size))
    return y


def eltwise_f16(op, a, b):
    a = np.ascontiguousarray(a, dtype=np.uint16)
    b = np.ascontiguousarray(b, dtype=np.uint16)
    rank = max(a.ndim, b.ndim)
    a = a.reshape((1,) * (rank - a.ndim) + a.shape)
    b = b.reshape((1,) * (rank - b.ndim) + b.shape)
    shape = tuple(max(x, y) for x, y in zip(a.shape, b.shape))
    y = np.empty(shape, dtype=np.uint16)
    lib().orc_eltwise_f16(C.c_int(ELT_OPS[op]), _p(a), _p(b), _p(y), C.c_int(rank), _i64(shape), _i64(a.shape),
                          _i64(b.shape))
    return y


# ---- reductions --------------------------------------------------------------------------------

def softmax_f16(x, axis, pad=0):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    outer, ax, inner = _axis_view(x.shape, axis % x.ndim)
    y = np.empty_like(x)
    lib().orc_softmax_f16(_p(x), _p(y), C.c_int64(outer), C.c_int64(ax), C.c_int64(inner), C.c_int64(pad))
    return y


def softmax_f32(x, axis, pad=0):
    x = np.ascontiguousarray(x, dtype=np.float32)
    outer, ax, inner = _axis_view(x.shape, axis % x.ndim)
    y = np.empty_like(x)
    lib().orc_softmax_f32(_p(x), _p(y), C.c_int64(outer), C.c_int64(ax), C.c_int64(inner), C.c_int64(pad))
    return y


def mvn_f16(x, across_channels, normalize_variance, eps, layout="NCHW"):
    """x: uint16 array, 4-D in memory order given by layout ("NCHW" or "NHWC")."""
    x = np.ascontiguousarray(x, dtype=np.uint16)
    y = np.empty_like(x)
    if layout == "NCHW":
        N, Cc, H, W = x.shape
        sn, sc, ss = Cc * H * W, H * W, 1
    elif layout == "NHWC":
        N, H, W, Cc = x.shape
        sn, sc, ss = H * W * Cc, 1, Cc
    else:
        raise ValueError(layout)
    lib().orc_mvn_f16(_p(x), _p(y), C.c_int64(N), C.c_int64(Cc), C.c_int64(H * W), C.c_int64(sn), C.c_int64(sc),
                      C.c_int64(ss), C.c_int(int(across_channels)), C.c_int(int(normalize_variance)), C.c_float(eps))
    return y


def dynamic_quantize(x):
    """VPU.DynamicQuantize (ops.td:6646-6660) with the arithmetic of ONNX DynamicQuantizeLinear, in float32: the range
    [min(0, min x), max(0, max x)] maps onto 0..255; returns (uint8 values, float32 scale, uint8 zero point).
    "parity unpinned": the reference holds the signature only; pinned by the ONNX specification's examples."""
    x = np.asarray(x, dtype=np.float32)
    with np.errstate(all="ignore"):
        lo = np.float32(min(0.0, np.nanmin(x, initial=0.0)))
        hi = np.float32(max(0.0, np.nanmax(x, initial=0.0)))
        scale = np.float32(1.0) if hi == lo else np.float32((hi - lo) / np.float32(255.0))
        zp = np.uint8(np.rint(np.clip(np.float32(0.0) - lo / scale, 0.0, 255.0)))
        v = np.rint(x / scale) + np.float32(zp)
        y = np.where(np.isnan(v), 0.0, np.clip(v, 0.0, 255.0)).astype(np.uint8)
    return y, scale, zp


def dynamic_dequantize(q, scale, zero_point=None, to_f16=True):
    """VPU.DynamicDequantize (ops.td:7780-7819): (q - zp) * scale with NUMPY-broadcast scale / zero-point tensors, in
    fp32, then the float16 class's rounding for fp16 output.  scale: float32 array or uint16 fp16 bits.
    "parity unpinned" against the SHAVE kernel; pinned by the static dequantize golden (content_tests.cpp:754-788)."""
    q = np.asarray(q)
    sc = f16_to_f32(scale) if np.asarray(scale).dtype == np.uint16 else np.asarray(scale, dtype=np.float32)
    z = np.zeros((1,) * q.ndim, np.int32) if zero_point is None else np.asarray(zero_point).astype(np.int32)
    r = ((q.astype(np.int32) - z).astype(np.float32) * sc).astype(np.float32)
    return f32_to_f16(r) if to_f16 else r


# The three-step decomposition of MVN-1 (decompose_mvn.cpp:82-129; ops.td:3659-3845), in numpy.  Tensors are
# logical [N,C,H,W] arrays; statistics tensors are in their memory order [N, parts, 2 or 1, C or 1].
# "parity unpinned" like mvn_f16: the reference holds no vectors for these kernels.  Pinned by the tests through
# hand-computed cases and through mvn1_norm(mvn1_mean_var(mvn1_sum(x))) == mvn_f16(x).

def mvn1_sum(x_bits, across_channels, normalize_variance):
    """{sum, sum of squares} per group, accumulated in double and rounded to float32; one part."""
    x = f16_to_f32(np.asarray(x_bits, dtype=np.uint16)).astype(np.float64)
    axes = (1, 2, 3) if across_channels else (2, 3)
    terms = [x.sum(axis=axes)] + ([(x * x).sum(axis=axes)] if normalize_variance else [])
    out = np.stack([t.reshape(x.shape[0], -1) for t in terms], axis=1)  # [N, W, C]
    return out[:, None].astype(np.float32)


def mvn1_mean_var(sums, orig_shape, across_channels, normalize_variance, eps, group_c=1, out_dtype=np.float32):
    """sums: float32 [N, parts, 2 or 1, C or 1] -> {mean, 1/sqrt(var + eps)} [N, 1, 2 or 1, C or 1]; channels are
    pooled in consecutive groups of group_c (the op's internal reshape)."""
    s = np.asarray(sums, dtype=np.float32).astype(np.float64).sum(axis=1)  # [N, W, Cin]
    N, Cc, H, W = orig_shape
    if across_channels:
        pooled = s.sum(axis=2, keepdims=True)
        count = float(Cc * H * W)
    else:
        g = s.reshape(s.shape[0], s.shape[1], Cc // group_c, group_c).sum(axis=3, keepdims=True)
        pooled = np.broadcast_to(g, g.shape[:3] + (group_c,)).reshape(s.shape[0], s.shape[1], Cc)
        count = float(group_c * H * W)
    mean = pooled[:, 0] / count
    rows = [mean]
    if normalize_variance:
        var = np.maximum(pooled[:, 1] / count - mean * mean, 0.0)
        with np.errstate(divide="ignore"):
            rows.append(1.0 / np.sqrt(var + np.float64(np.float32(eps))))
    out = np.stack(rows, axis=1)[:, None].astype(np.float32)
    return out.astype(out_dtype)


def mvn1_norm(x_bits, mean_var, across_channels, normalize_variance):
    """(x - mean) * inv in float32, rounded to fp16 (IEEE); mean_var [N, 1, 2 or 1, C or 1] of fp16 or fp32."""
    x = f16_to_f32(np.asarray(x_bits, dtype=np.uint16))
    mv = np.asarray(mean_var).astype(np.float32)
    mean = mv[:, 0, 0, :, None, None]
    inv = mv[:, 0, 1, :, None, None] if normalize_variance else np.float32(1.0)
    with np.errstate(all="ignore"):
        return ((x - mean) * inv).astype(np.float32).astype(np.float16).view(np.uint16)


def mvn6_f16(x_bits, axes, normalize_variance, eps, eps_mode, scale_bits=None, bias_bits=None):
    """OpenVINO MVN-6 over `axes` of an array indexed in memory order: y = (x - mean) / sqrt(var + eps) (eps_mode 0,
    INSIDE_SQRT) or (x - mean) / (sqrt(var) + eps) (1, OUTSIDE_SQRT), then the fused y * scale + bias with NUMPY
    broadcast (fuse_mvn6_scale_bias.cpp); double statistics, one rounding to fp16 (IEEE)."""
    x = f16_to_f32(np.asarray(x_bits, dtype=np.uint16)).astype(np.float64)
    axes = tuple(int(a) % x.ndim for a in axes)
    mean = x.mean(axis=axes, keepdims=True)
    y = x - mean
    if normalize_variance:
        var = (y * y).mean(axis=axes, keepdims=True)
        e = np.float64(np.float32(eps))
        y = y / (np.sqrt(var + e) if eps_mode == 0 else np.sqrt(var) + e)
    if scale_bits is not None:
        y = y * f16_to_f32(np.asarray(scale_bits, dtype=np.uint16)).astype(np.float64)
    if bias_bits is not None:
        y = y + f16_to_f32(np.asarray(bias_bits, dtype=np.uint16)).astype(np.float64)
    with np.errstate(all="ignore"):
        return y.astype(np.float32).astype(np.float16).view(np.uint16)


# ---- integer path --------------------------------------------------------------------------------

def approximate(bits, target):
    m, s, p = C.c_int64(), C.c_int64(), C.c_int64()
    rc = lib().orc_approximate(C.c_int(bits), C.c_double(target), C.byref(m), C.byref(s), C.byref(p))
    if rc != 0:
        raise OverflowError(target)
    return m.value, s.value, p.value


def wt_pack_scale(shift, mult):
    return lib().orc_wt_pack_scale(C.c_uint8(shift), C.c_int16(mult))


def make_weights_table(mults, shifts, biases, weight_step):
    """[OC,4] int32 table as NCESparsity::getWeightsTable lays it out (nce_sparsity.cpp:195-231)."""
    oc = len(mults)
    wt = np.zeros((oc, 4), dtype=np.int32)
    wt[:, 0] = np.arange(oc, dtype=np.int64) * weight_step
    wt[:, 1] = 0xFFFFFF
    wt[:, 2] = [wt_pack_scale(int(s), int(m)) for m, s in zip(mults, shifts)]
    wt[:, 3] = biases
    return wt


def ppe(prelu_mult=1, prelu_shift=0, zp_out=0, clamp_low=-(2 ** 31), clamp_high=2 ** 31 - 1):
    return _PPE(prelu_mult, prelu_shift, zp_out, clamp_low, clamp_high)


def ppe_requant(acc, bias, mult, shift, p):
    return lib().orc_ppe_requant(C.c_int32(acc), C.c_int32(bias), C.c_int32(mult), C.c_int32(shift), C.byref(p))


def ppe_requant_f16(acc, bias, mult, shift, p):
    """fp16 bit pattern of the s17.15 fixed-point output path."""
    fn = lib().orc_ppe_requant_f16
    fn.restype = C.c_uint16
    return fn(C.c_int32(acc), C.c_int32(bias), C.c_int32(mult), C.c_int32(shift), C.byref(p))


def pack_clamp_f16(lo, hi):
    """Two fp16 bounds in one int32 as the compiler packs them for a float output: 0xllllhhhh built by adding the
    sign-extended 16-bit patterns (ppe_utils.hpp:57-73)."""
    lo_b, hi_b = (int(np.array([v], dtype=np.float32).astype(np.float16).view(np.int16)[0]) for v in (lo, hi))
    v = ((lo_b << 16) + hi_b) & 0xffffffff
    return v - (1 << 32) if v & 0x80000000 else v


def _nhw_strides(x):
    """N, H, W strides in elements of a 4-D array whose channels are contiguous (a view of a larger tensor)."""
    assert x.ndim == 4 and (x.shape[3] == 1 or x.strides[3] == x.itemsize)
    return tuple(int(v) // x.itemsize for v in x.strides[:3])


def nce_conv(inp, w, wt, p, zp_in=0, zp_w=0, strides=(1, 1), pads=(0, 0, 0, 0), out_signed=False, rows=None,
             want_acc=False, out_f16=False, out=None):
    """inp NHWC int8/uint8, w [OC,KY,KX,IC] int8/uint8, wt [OC,4] int32; pads = (top,left,bottom,right).

    rows=(row0,nrows) computes only those flattened output rows (the rest of the result is zero).
    inp may be a view of a larger array (channels contiguous): it is read in place through its strides.  `out`, when
    given, is the array to write, likewise a view if wanted; elements of its parent outside the view are not touched."""
    w = np.ascontiguousarray(w)
    wt = np.ascontiguousarray(wt, dtype=np.int32)
    N, H, W, IC = inp.shape
    OC, KY, KX, IC2 = w.shape
    assert IC == IC2
    d = _Conv(N, H, W, IC, OC, KY, KX, strides[0], strides[1], pads[0], pads[1], pads[2], pads[3],
              int(inp.dtype == np.int8), int(w.dtype == np.int8), 2 if out_f16 else int(out_signed), zp_in, zp_w, p)
    OH = (H + pads[0] + pads[2] - KY) // strides[0] + 1
    OW = (W + pads[1] + pads[3] - KX) // strides[1] + 1
    odt = np.uint16 if out_f16 else (np.int8 if out_signed else np.uint8)
    if not inp.flags.c_contiguous:
        for i, v in enumerate(_nhw_strides(inp)):
            d.in_strides[i] = v
    if out is None:
        out = np.zeros((N, OH, OW, OC), dtype=odt)
    else:
        assert out.shape == (N, OH, OW, OC) and out.dtype == odt
        if not out.flags.c_contiguous:
            for i, v in enumerate(_nhw_strides(out)):
                d.out_strides[i] = v
    acc = np.zeros((N, OH, OW, OC), dtype=np.int32) if want_acc else None
    row0, nrows = rows if rows is not None else (0, N * OH * OW)
    lib().orc_nce_conv_rows(C.byref(d), _p(inp), _p(w), _p(wt), _p(out), _p(acc) if want_acc else None,
                            C.c_int64(row0), C.c_int64(nrows))
    return (out, acc) if want_acc else out


def nce_eltwise(a, b, p, zp_a, zp_b, mult_a, mult_b, out_mult, out_shift, subtract=False, out_signed=False, out_f16=False,
                out=None):
    """Quantized add / subtract of two 8-bit tensors of the same shape (the NCE ELTWISE task); out_f16: fp16 bit patterns."""
    assert a.shape == b.shape
    if out is not None or not (a.flags.c_contiguous and b.flags.c_contiguous):
        # views of larger arrays (channels contiguous), read and written in place
        odt = np.uint16 if out_f16 else (np.int8 if out_signed else np.uint8)
        if out is None:
            out = np.zeros(a.shape, dtype=odt)
        assert out.shape == a.shape and out.dtype == odt and a.ndim == 4
        lib().orc_nce_eltwise_views(_p(a), C.c_int(int(a.dtype == np.int8)), _p(b), C.c_int(int(b.dtype == np.int8)), _p(out),
                                    C.c_int(2 if out_f16 else int(out_signed)), _i64(a.shape), _i64(_nhw_strides(a)),
                                    _i64(_nhw_strides(b)), _i64(_nhw_strides(out)), C.c_int32(zp_a), C.c_int32(zp_b),
                                    C.c_int32(mult_a), C.c_int32(mult_b), C.c_int(int(subtract)), C.c_int32(out_mult),
                                    C.c_int32(out_shift), C.byref(p))
        return out
    if out_f16:
        out = np.zeros(a.shape, dtype=np.uint16)
        lib().orc_nce_eltwise_f16(_p(a), C.c_int(int(a.dtype == np.int8)), _p(b), C.c_int(int(b.dtype == np.int8)), _p(out),
                                  C.c_int64(a.size), C.c_int32(zp_a), C.c_int32(zp_b), C.c_int32(mult_a), C.c_int32(mult_b),
                                  C.c_int(int(subtract)), C.c_int32(out_mult), C.c_int32(out_shift), C.byref(p))
        return out
    out = np.zeros(a.shape, dtype=np.int8 if out_signed else np.uint8)
    lib().orc_nce_eltwise(_p(a), C.c_int(int(a.dtype == np.int8)), _p(b), C.c_int(int(b.dtype == np.int8)), _p(out),
                          C.c_int(int(out_signed)), C.c_int64(a.size), C.c_int32(zp_a), C.c_int32(zp_b),
                          C.c_int32(mult_a), C.c_int32(mult_b), C.c_int(int(subtract)), C.c_int32(out_mult),
                          C.c_int32(out_shift), C.byref(p))
    return out


def nce_matmul(a, b_nk, wt, p, zp_a=0, zp_b=0, out_signed=True, rows=None, want_acc=False, out_f16=False):
    """A [M,K] x B stored [N,K] -> [M,N]: the 1x1-convolution form NCE.MatMul lowers to (ops.td:228-357)."""
    M, K = a.shape
    Nn, K2 = b_nk.shape
    assert K == K2
    r = nce_conv(a.reshape(1, M, 1, K), b_nk.reshape(Nn, 1, 1, K), wt, p, zp_in=zp_a, zp_w=zp_b,
                 out_signed=out_signed, rows=rows, want_acc=want_acc, out_f16=out_f16)
    if want_acc:
        return r[0].reshape(M, Nn), r[1].reshape(M, Nn)
    return r.reshape(M, Nn)
