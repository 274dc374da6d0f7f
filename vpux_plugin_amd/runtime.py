"""ctypes binding of libvpx_amd.so and thin operator wrappers over torch device tensors.

torch is used for device memory and streams only; every computation goes through the C ABI
declared in include/vpx_runtime.h.  There is no fallback: a missing library raises at import of
this module's `lib()`.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libvpx_amd.so")

# sw_params::DataType codes (include/vpx_sw_params.h)
NN_FP32, NN_FP16, NN_U8, NN_I32, NN_I8 = 1, 2, 7, 9, 11
ORDER = {"NCHW": 0x4321, "NHWC": 0x2431, "NCWH": 0x3421, "NWHC": 0x2341, "CHW": 0x321, "HWC": 0x132, "NC": 0x21, "C": 0x1}
LOC_DDR = 1

SUCCESS = 0
ERROR_OUT_OF_MEMORY = 0x70000002
ERROR_UNSUPPORTED_FEATURE = 0x78000003
ERROR_INVALID_ARGUMENT = 0x78000004
ERROR_INVALID_NULL_HANDLE = 0x78000005
ERROR_UNKNOWN = 0x7FFFFFFE

PPE_NOOP, PPE_LRELU, PPE_LRELUX, PPE_LPRELU = 3, 13, 14, 15
POSTOP_NONE, POSTOP_RELU, POSTOP_CLAMP, POSTOP_LEAKY_RELU = 0, 1, 2, 3


class VpxError(RuntimeError):
    def __init__(self, code, text):
        super().__init__("vpx error 0x%x: %s" % (code & 0xFFFFFFFF, text))
        self.code = code
        self.text = text


class MemRefAddr(C.Structure):
    _fields_ = [("data", C.c_void_p), ("dims", C.POINTER(C.c_int32)), ("strides", C.POINTER(C.c_int64))]


class TensorDesc(C.Structure):
    _fields_ = [("num_dims", C.c_uint32), ("dims", C.POINTER(C.c_int32)), ("strides", C.POINTER(C.c_int64)),
                ("data_type", C.c_uint32), ("dims_order", C.c_uint64), ("location", C.c_uint32), ("dynamic_shape", C.c_uint32)]


class PpeInt(C.Structure):
    _fields_ = [("mode", C.c_int32), ("clamp_low", C.c_int32), ("clamp_high", C.c_int32), ("lrelu_mult", C.c_int32),
                ("lrelu_shift", C.c_int32), ("quant_mult", C.c_int32), ("quant_shift", C.c_int32),
                ("in1_quant_mult", C.c_int32), ("in2_quant_mult", C.c_int32)]


class OpAttrs(C.Structure):
    """vpx_op_attrs_t: the operator attributes vpx_get_kernel_info reads."""
    _fields_ = [("axis_ind", C.c_int64), ("pad_size", C.c_int64), ("across_channels", C.c_int32),
                ("normalize_variance", C.c_int32), ("eps", C.c_float), ("eps_mode", C.c_int32),
                ("axes", C.POINTER(C.c_int64)), ("num_axes", C.c_uint32), ("has_scale", C.c_int32), ("has_bias", C.c_int32),
                ("orig_shape", C.POINTER(C.c_int64)), ("group_c", C.c_int64), ("levels", C.c_int64),
                ("scales", C.POINTER(C.c_double)), ("zero_points", C.POINTER(C.c_int64)), ("num_quant_params", C.c_uint32),
                ("param0", C.c_float), ("param1", C.c_float)]


class QuantType(C.Structure):
    _fields_ = [("is_quantized", C.c_int32), ("scale", C.c_double), ("zero_point", C.c_int64),
                ("storage_min", C.c_int64), ("storage_max", C.c_int64)]


class NceTask(C.Structure):
    _fields_ = [("task_type", C.c_int32), ("input", C.c_void_p), ("weights", C.c_void_p), ("weight_table", C.c_void_p),
                ("output", C.c_void_p), ("input_type", C.c_int32), ("weights_type", C.c_int32),
                ("output_type", C.c_int32), ("N", C.c_int64), ("H", C.c_int64), ("W", C.c_int64), ("IC", C.c_int64),
                ("OC", C.c_int64), ("kernel_size", C.c_int32 * 2), ("kernel_strides", C.c_int32 * 2),
                ("kernel_padding", C.c_int32 * 4), ("zp_in", C.c_int32), ("zp_w", C.c_int32), ("zp_out", C.c_int32),
                ("ppe", PpeInt), ("eltwise_type", C.c_int32), ("groups", C.c_int32),
                ("input_strides", C.c_int64 * 4), ("weights_strides", C.c_int64 * 4), ("output_strides", C.c_int64 * 4)]


NCE_CONV, NCE_ELTWISE = 0, 4
ELTWISE_ADD, ELTWISE_SUBTRACT = 0, 1


# every symbol include/vpx_runtime.h and include/vpx_compiler_utils.h declare
EXPORTS = ["vpx_get_last_error", "vpx_get_version", "vpx_sw_kernel_launch", "vpx_sw_kernel_launch_noalloc", "vpx_sw_kernel_supported",
           "vpx_sw_kernel_count", "vpx_sw_kernel_name", "vpx_nce_task", "vpx_nce_last_kernel", "vpx_set_tuning", "vpx_workspace_reserve", "vpx_workspace_release", "vpx_calib_mfma_i8", "vpx_calib_coissue", "vpx_approximate",
           "vpx_eltwise_quantization_approximation", "vpx_wt_get_scale", "vpx_wt_get_bias", "vpx_get_weights_table",
           "vpx_retrieve_ppe_int", "vpx_generate_softmax_attr", "vpx_get_quant_params_attr", "vpx_create_kernel_params", "vpx_get_kernel_info",
           "vpx_float_to_half_bits", "vpx_half_bits_to_float"]

_lib = None


def _load_hip_runtime():
    """libvpx_amd.so leaves the HIP runtime symbols undefined so that it binds to whichever single
    runtime the process holds.  Under Python that is the copy bundled with torch (a second,
    system-wide copy in the same process does not see the GPU); without torch, the ROCm install."""
    candidates = []
    try:
        import torch
        candidates.append(os.path.join(os.path.dirname(torch.__file__), "lib", "libamdhip64.so"))
    except ImportError:
        pass
    candidates += [os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "lib", "libamdhip64.so")]
    for path in candidates:
        if os.path.exists(path):
            return C.CDLL(path, mode=C.RTLD_GLOBAL)
    raise RuntimeError("no libamdhip64.so found (looked in %s)" % ", ".join(candidates))


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is missing: build it with `python -m vpux_plugin_amd.build` "
                               "(there is no CPU fallback)" % LIB_PATH)
        _load_hip_runtime()
        L = C.CDLL(LIB_PATH)
        L.vpx_get_last_error.restype = C.c_char_p
        L.vpx_get_version.restype = C.c_uint32
        L.vpx_sw_kernel_name.restype = C.c_char_p
        L.vpx_sw_kernel_name.argtypes = [C.c_uint32]
        L.vpx_sw_kernel_count.restype = C.c_uint32
        L.vpx_sw_kernel_supported.argtypes = [C.c_char_p]
        L.vpx_nce_last_kernel.restype = C.c_char_p
        L.vpx_sw_kernel_launch.argtypes = [C.c_char_p, C.c_void_p, C.c_size_t, C.POINTER(MemRefAddr), C.c_uint32,
                                           C.c_void_p]
        L.vpx_sw_kernel_launch_noalloc.argtypes = L.vpx_sw_kernel_launch.argtypes
        L.vpx_nce_task.argtypes = [C.POINTER(NceTask), C.c_void_p]
        L.vpx_set_tuning.argtypes = [C.c_char_p, C.c_char_p]
        L.vpx_workspace_reserve.argtypes = [C.c_void_p, C.c_size_t]
        L.vpx_workspace_release.argtypes = [C.c_void_p]
        L.vpx_calib_mfma_i8.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.POINTER(C.c_int64), C.c_void_p]
        L.vpx_approximate.argtypes = [C.c_int, C.c_double] + [C.POINTER(C.c_int64)] * 3
        L.vpx_eltwise_quantization_approximation.argtypes = [C.c_double] * 3 + [C.c_int] + [C.POINTER(C.c_int64)] * 4
        L.vpx_wt_get_scale.restype = C.c_int32
        L.vpx_wt_get_scale.argtypes = [C.c_uint8, C.c_int16]
        L.vpx_wt_get_bias.argtypes = [C.c_double, C.POINTER(C.c_int32)]
        L.vpx_get_weights_table.argtypes = [C.c_double, C.c_double, C.c_void_p, C.c_size_t, C.c_void_p, C.c_int64,
                                            C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_void_p]
        L.vpx_retrieve_ppe_int.argtypes = [C.c_int, C.c_double, C.c_double, C.POINTER(QuantType), C.POINTER(PpeInt)]
        L.vpx_generate_softmax_attr.argtypes = [C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64,
                                                C.c_void_p, C.POINTER(C.c_uint32)]
        L.vpx_get_quant_params_attr.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_void_p,
                                                C.POINTER(C.c_uint32)]
        L.vpx_create_kernel_params.argtypes = [C.POINTER(TensorDesc), C.c_uint32, C.POINTER(TensorDesc), C.c_uint32,
                                               C.c_void_p, C.c_size_t, C.c_void_p, C.POINTER(C.c_size_t)]
        L.vpx_get_kernel_info.argtypes = [C.c_char_p, C.POINTER(OpAttrs), C.POINTER(TensorDesc), C.c_char_p, C.c_size_t,
                                          C.c_void_p, C.POINTER(C.c_size_t)]
        L.vpx_float_to_half_bits.restype = C.c_uint16
        L.vpx_float_to_half_bits.argtypes = [C.c_float]
        L.vpx_half_bits_to_float.restype = C.c_float
        L.vpx_half_bits_to_float.argtypes = [C.c_uint16]
        _lib = L
    return _lib


def check(rc):
    if rc != SUCCESS:
        raise VpxError(rc, lib().vpx_get_last_error().decode())


# ---- host-side helpers (compile-time arithmetic) ---------------------------------------------------

def approximate(bits, target):
    m, s, p = C.c_int64(), C.c_int64(), C.c_int64()
    check(lib().vpx_approximate(bits, target, C.byref(m), C.byref(s), C.byref(p)))
    return m.value, s.value, p.value


def eltwise_quantization_approximation(in1, in2, out, eltwise_type=0):
    v = [C.c_int64() for _ in range(4)]
    check(lib().vpx_eltwise_quantization_approximation(in1, in2, out, eltwise_type, *[C.byref(x) for x in v]))
    return tuple(x.value for x in v)


def get_weights_table(in_scale, out_scale, weight_scales, bias, OC, weights_ptr=0, weights_ptr_step=16,
                      sparsity_ptr=0xFFFFFF, sparsity_ptr_step=0):
    ws = np.ascontiguousarray(np.atleast_1d(weight_scales), dtype=np.float64)
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float64)
    table = np.zeros((OC, 4), dtype=np.int32)
    check(lib().vpx_get_weights_table(in_scale, out_scale, ws.ctypes.data, ws.size, None if b is None else b.ctypes.data,
                                      OC, weights_ptr, weights_ptr_step, sparsity_ptr, sparsity_ptr_step,
                                      table.ctypes.data))
    return table


def make_weights_table(mults, shifts, biases, weights_ptr_step=16):
    """[OC,4] int32 table from explicit per-channel multiplier / shift / int32 bias."""
    oc = len(mults)
    t = np.zeros((oc, 4), dtype=np.int32)
    t[:, 0] = (np.arange(oc, dtype=np.int64) * weights_ptr_step).astype(np.int32)
    t[:, 1] = 0xFFFFFF
    t[:, 2] = [lib().vpx_wt_get_scale(int(s), int(m)) for m, s in zip(mults, shifts)]
    t[:, 3] = biases
    return t


def retrieve_ppe_int(post_op, out_type=None, param0=0.0, param1=0.0):
    """out_type: None (float output) or (scale, zero_point, storage_min, storage_max)."""
    q = QuantType(0, 1.0, 0, 0, 0) if out_type is None else QuantType(1, *out_type)
    p = PpeInt()
    check(lib().vpx_retrieve_ppe_int(post_op, param0, param1, C.byref(q), C.byref(p)))
    return p


def generate_softmax_attr(dims, in_strides, out_strides, axis, pad_size=0):
    """dims/strides innermost first (strides in elements); returns the packed uint64 words."""
    d = np.ascontiguousarray(dims, dtype=np.int64)
    si = np.ascontiguousarray(in_strides, dtype=np.int64)
    so = np.ascontiguousarray(out_strides, dtype=np.int64)
    words = np.zeros(2 + 2 * 16, dtype=np.uint64)
    n = C.c_uint32()
    check(lib().vpx_generate_softmax_attr(d.size, d.ctypes.data, si.ctypes.data, so.ctypes.data, axis, pad_size,
                                          words.ctypes.data, C.byref(n)))
    return words[:n.value].copy()


def get_quant_params_attr(scales, zero_points, float_type):
    s = np.ascontiguousarray(np.atleast_1d(scales), dtype=np.float64)
    z = np.ascontiguousarray(np.atleast_1d(zero_points), dtype=np.int64)
    words = np.zeros(1 + 2 * ((s.size + 1) // 2) + 2, dtype=np.uint64)
    n = C.c_uint32()
    check(lib().vpx_get_quant_params_attr(s.ctypes.data, z.ctypes.data, s.size, float_type, words.ctypes.data,
                                          C.byref(n)))
    return words[:n.value].copy()


def get_kernel_info(op, operand=None, axes=None, orig_shape=None, scales=None, zero_points=None, **fields):
    """(entry name, attribute bytes) of a VPU operator, as SwKernelOp::getKernelInfo derives them.  `operand` is the
    Operand (or torch tensor) whose order and element type the derivation reads; list-valued attributes are keywords."""
    a = OpAttrs()
    keep = []
    for k, v in fields.items():
        setattr(a, k, v)
    if axes is not None:
        arr = (C.c_int64 * len(axes))(*axes)
        keep.append(arr)
        a.axes, a.num_axes = arr, len(axes)
    if orig_shape is not None:
        arr = (C.c_int64 * 4)(*orig_shape)
        keep.append(arr)
        a.orig_shape = arr
    if scales is not None:
        sc, zp = (C.c_double * len(scales))(*scales), (C.c_int64 * len(scales))(*zero_points)
        keep += [sc, zp]
        a.scales, a.zero_points, a.num_quant_params = sc, zp, len(scales)
    desc = None
    if operand is not None:
        operand = operand if isinstance(operand, Operand) else Operand(operand)
        desc = C.byref(operand.desc)
    entry = C.create_string_buffer(64)
    size = C.c_size_t(0)
    check(lib().vpx_get_kernel_info(op.encode(), C.byref(a), desc, entry, len(entry), None, C.byref(size)))
    buf = C.create_string_buffer(max(size.value, 1))
    check(lib().vpx_get_kernel_info(op.encode(), C.byref(a), desc, entry, len(entry), buf, C.byref(size)))
    return entry.value.decode(), buf.raw[:size.value]


def half_bits(v):
    return lib().vpx_float_to_half_bits(C.c_float(v))


def half_to_float(bits):
    return lib().vpx_half_bits_to_float(C.c_uint16(bits))


# ---- kernel parameter blobs ------------------------------------------------------------------------

def _torch_dtype_code(t):
    import torch
    return {torch.float16: NN_FP16, torch.float32: NN_FP32, torch.uint8: NN_U8, torch.int8: NN_I8,
            torch.int32: NN_I32}[t.dtype]


class Operand:
    """A device tensor seen as a memref: `t` is indexed in MEMORY order (outermost first); its torch
    strides may describe a sub-view.  `order` is the NDOrder code / name of the logical layout."""

    def __init__(self, t, order=None, dynamic=False):
        self.t = t
        nd = t.dim()
        if order is None:
            order = {4: "NCHW", 3: "CHW", 2: "NC", 1: "C"}.get(nd, None)
            order = ORDER[order] if order else int("".join("%x" % (nd - i) for i in range(nd)), 16)
        elif isinstance(order, str):
            order = ORDER[order]
        self.order = order
        bits = t.element_size() * 8
        self.dims = (C.c_int32 * nd)(*[int(s) for s in reversed(t.shape)])
        self.strides = (C.c_int64 * nd)(*[int(s) * bits for s in reversed(t.stride())])
        self.desc = TensorDesc(nd, self.dims, self.strides, _torch_dtype_code(t), order, LOC_DDR, 1 if dynamic else 0)
        self.live_dims = self.live_strides = None  # dynamic shapes: device tensors (int32 dims, int64 strides in bits)


def create_kernel_params(inputs, outputs, attrs=b""):
    ins = (TensorDesc * len(inputs))(*[o.desc for o in inputs])
    outs = (TensorDesc * len(outputs))(*[o.desc for o in outputs])
    size = C.c_size_t(0)
    check(lib().vpx_create_kernel_params(ins, len(inputs), outs, len(outputs), attrs, len(attrs), None, C.byref(size)))
    buf = C.create_string_buffer(size.value)
    check(lib().vpx_create_kernel_params(ins, len(inputs), outs, len(outputs), attrs, len(attrs), buf, C.byref(size)))
    return buf.raw[:size.value]


def _stream_handle(stream):
    import torch
    if stream is None:
        stream = torch.cuda.current_stream()
    return C.c_void_p(stream.cuda_stream)


NOALLOC_SCRATCH_BYTES = 4 << 20  # VPX_NOALLOC_SCRATCH_BYTES


def sw_kernel_launch(entry, blob, operands, stream=None, side_dims=False, noalloc=False):
    """Launch `entry` with the serialized blob; operands supply the device addresses.  With
    side_dims=True dims/strides travel in the address table instead of the blob tail; with noalloc=True
    the call goes through vpx_sw_kernel_launch_noalloc (fixed scratch array, no device allocation)."""
    addrs = (MemRefAddr * len(operands))()
    for i, o in enumerate(operands):
        addrs[i].data = o.t.data_ptr()
        if o.live_dims is not None:
            addrs[i].dims = C.cast(C.c_void_p(o.live_dims.data_ptr()), C.POINTER(C.c_int32))
            addrs[i].strides = C.cast(C.c_void_p(o.live_strides.data_ptr()), C.POINTER(C.c_int64))
        elif side_dims:
            addrs[i].dims = C.cast(o.dims, C.POINTER(C.c_int32))
            addrs[i].strides = C.cast(o.strides, C.POINTER(C.c_int64))
    fn = lib().vpx_sw_kernel_launch_noalloc if noalloc else lib().vpx_sw_kernel_launch
    check(fn(entry.encode(), blob, len(blob), addrs, len(operands), _stream_handle(stream)))


def _i64(*vals):
    return np.asarray(vals, dtype=np.int64).tobytes()


# ---- operator wrappers (VPU op -> kernel entry + attributes, as SwKernelOp::getKernelInfo does) -------

def convert(x, out, order=None, stream=None):
    ops = [Operand(x, order), Operand(out, order)]
    sw_kernel_launch("convert", create_kernel_params(ops[:1], ops[1:]), ops, stream)
    return out


def eltwise(kind, a, b, out, order=None, stream=None):
    ops = [Operand(a, order), Operand(b, order), Operand(out, order)]
    sw_kernel_launch("eltwise_" + kind, create_kernel_params(ops[:2], ops[2:]), ops, stream)
    return out


# kernel entry and number of float attributes of each unary activation (sw_kernel.cpp getKernelInfo)
ACTIVATIONS = {
    "relu": ("activation_relu", 0), "leaky_relu": ("leaky_relu_fp16", 1), "clamp": ("activation_clamp", 2),
    "negative": ("activation_negative", 0), "abs": ("activation_abs", 0), "hswish": ("activation_hswish", 0),
    "hsigmoid": ("activation_hsigmoid", 0), "hardsigmoid": ("activation_hardsigmoid", 2),
    "sigmoid": ("activation_sigmoid", 0), "tanh": ("activation_tanh", 0), "exp": ("activation_exp", 0),
    "sqrt": ("activation_sqrt", 0), "log": ("activation_log", 0), "floor": ("activation_floor", 0),
    "ceil": ("activation_ceil", 0), "sign": ("activation_sign", 0), "elu": ("activation_elu", 1),
    "selu": ("activation_selu", 2), "swish": ("activation_swish", 1), "mish": ("activation_mish", 0),
    "softplus": ("activation_softplus", 0), "gelu": ("activation_gelu", 0), "erf": ("activation_erf", 0),
}


def activation(kind, x, out, *params, order=None, stream=None):
    entry, n_attrs = ACTIVATIONS[kind]
    if len(params) != n_attrs:
        raise ValueError(f"{kind} takes {n_attrs} attributes, got {len(params)}")
    ops = [Operand(x, order), Operand(out, order)]
    attrs = np.asarray(params, dtype=np.float32).tobytes()
    sw_kernel_launch(entry, create_kernel_params(ops[:1], ops[1:], attrs), ops, stream)
    return out


def prelu(x, slope, out, order=None, stream=None):
    ops = [Operand(x, order), Operand(slope, order), Operand(out, order)]
    sw_kernel_launch("prelu_fp16", create_kernel_params(ops[:2], ops[2:]), ops, stream)
    return out


def fake_quantize(x, in_lo, in_hi, out_lo, out_hi, levels, out, order=None, stream=None):
    ops = [Operand(t, order) for t in (x, in_lo, in_hi, out_lo, out_hi, out)]
    sw_kernel_launch("fake_quantize", create_kernel_params(ops[:5], ops[5:], _i64(levels)), ops, stream)
    return out


def quantize(x, out, scale, zero_point, order=None, stream=None, noalloc=False):
    ops = [Operand(x, order), Operand(out, order)]
    attrs = get_quant_params_attr(scale, zero_point, _torch_dtype_code(x)).tobytes()
    sw_kernel_launch("quantize", create_kernel_params(ops[:1], ops[1:], attrs), ops, stream, noalloc=noalloc)
    return out


def dequantize(q, out, scale, zero_point, order=None, stream=None):
    ops = [Operand(q, order), Operand(out, order)]
    attrs = get_quant_params_attr(scale, zero_point, _torch_dtype_code(out)).tobytes()
    sw_kernel_launch("dequantize", create_kernel_params(ops[:1], ops[1:], attrs), ops, stream)
    return out


def mvn(x, out, across_channels, normalize_variance, eps, order="NCHW", stream=None, noalloc=False):
    ops = [Operand(x, order), Operand(out, order)]
    # a true boolean attribute serialises as int64 -1 (sign-extended i1)
    attrs = _i64(-1 if across_channels else 0, -1 if normalize_variance else 0) + np.float32(eps).tobytes()
    sw_kernel_launch("mvn1", create_kernel_params(ops[:1], ops[1:], attrs), ops, stream, noalloc=noalloc)
    return out


def _bool_attr(v):
    return -1 if v else 0


def mvn1_sum(x, out, across_channels, normalize_variance, order="NCHW", stream=None):
    """out: float32 statistics tensor in memory order [N, parts, 2 or 1, C or 1] (the NHWC storage of the
    op's logical [N, C or 1, parts, 2 or 1] result)."""
    ops = [Operand(x, order), Operand(out, "NHWC")]
    attrs = _i64(_bool_attr(across_channels), _bool_attr(normalize_variance))
    sw_kernel_launch("mvn1_sum", create_kernel_params(ops[:1], ops[1:], attrs), ops, stream)
    return out


def mvn1_mean_var(sums, out, orig_shape, across_channels, normalize_variance, eps, group_c=1, stream=None):
    ops = [Operand(sums, "NHWC"), Operand(out, "NHWC")]
    attrs = _i64(*orig_shape, _bool_attr(across_channels), _bool_attr(normalize_variance), group_c) + np.float32(eps).tobytes()
    sw_kernel_launch("mvn1_mean_var", create_kernel_params(ops[:1], ops[1:], attrs), ops, stream)
    return out


def mvn1_norm(x, mean_var, out, across_channels, normalize_variance, order="NCHW", stream=None):
    ops = [Operand(x, order), Operand(mean_var, "NHWC"), Operand(out, order)]
    attrs = _i64(_bool_attr(across_channels), _bool_attr(normalize_variance))
    sw_kernel_launch("mvn1_norm", create_kernel_params(ops[:2], ops[2:], attrs), ops, stream)
    return out


def dynamic_quantize(x, out, scale, zero_point, order=None, stream=None, noalloc=False):
    """x: float32; out: uint8 of x's shape; scale: float32[1]; zero_point: uint8[1] (all written by the kernel)."""
    ops = [Operand(x, order), Operand(out, order), Operand(scale), Operand(zero_point)]
    sw_kernel_launch("dynamic_quantize", create_kernel_params(ops[:1], ops[1:]), ops, stream, noalloc=noalloc)
    return out, scale, zero_point


def dynamic_dequantize(q, scale, out, zero_point=None, order=None, stream=None):
    """scale (fp16 / fp32) and the optional zero point (int8 / uint8) are tensors of q's rank that broadcast onto it."""
    ins = [Operand(q, order), Operand(scale, order)] + ([Operand(zero_point, order)] if zero_point is not None else [])
    ops = ins + [Operand(out, order)]
    sw_kernel_launch("dynamic_dequantize", create_kernel_params(ins, ops[-1:], _i64(2 ** 63 - 1)), ops, stream)
    return out


def mvn6(x, out, axes, normalize_variance, eps, eps_mode=0, scale=None, bias=None, order=None, stream=None):
    """axes index x in memory order (outermost first), like torch dims; eps_mode 0 = inside the square root,
    1 = outside.  scale / bias: optional tensors of x's rank, broadcast NUMPY-style."""
    nd = x.dim()
    ins = [Operand(x, order)] + [Operand(t, order) for t in (scale, bias) if t is not None]
    ops = ins + [Operand(out, order)]
    mask = 1 | (2 if scale is not None else 0) | (4 if bias is not None else 0) | 8
    mem_axes = [nd - 1 - (a % nd) for a in axes]
    attrs = (_i64(-(2 ** 63), mask, _bool_attr(normalize_variance), eps_mode) + np.float32(eps).tobytes() +
             _i64(len(mem_axes), *mem_axes))
    sw_kernel_launch("mvn6", create_kernel_params(ins, ops[-1:], attrs), ops, stream)
    return out


def softmax(x, out, axis, pad_size=0, order=None, packed=True, stream=None):
    """axis indexes x in memory order (outermost first), like a torch dim."""
    nd = x.dim()
    axis = axis % nd
    ops = [Operand(x, order), Operand(out, order)]
    rev_axis = nd - 1 - axis
    if packed:
        bits = x.element_size() * 8
        dims = [int(d) for d in ops[0].dims]
        si = [int(s) // bits for s in ops[0].strides]
        so = [int(s) // bits for s in ops[1].strides]
        attrs = generate_softmax_attr(dims, si, so, rev_axis, pad_size).tobytes()
    else:
        attrs = _i64(rev_axis, pad_size)
    entry = "softmaxFp32" if _torch_dtype_code(x) == NN_FP32 else "softmax"
    sw_kernel_launch(entry, create_kernel_params(ops[:1], ops[1:], attrs), ops, stream)
    return out


def softmax_dynamic(x, out, live_shape, axis, pad_size=0, compact=False, stream=None):
    """Softmax over a tensor whose shape is only bounded at compile time: x / out are the buffers of the bound shape,
    `live_shape` (memory order, like x.shape) the shape at run time.  The live dims and strides are put in device memory
    and the kernel reads them there; compact=True lays the live tensor out compactly at the start of the buffers,
    otherwise it keeps the bound buffer's strides.  Returns the (dims, in strides, out strides) device tensors."""
    import torch
    nd = x.dim()
    axis = axis % nd
    ops = [Operand(x, None, dynamic=True), Operand(out, None, dynamic=True)]
    bits = x.element_size() * 8
    dims = [int(d) for d in reversed(live_shape)]
    held = []
    for o in ops:
        if compact:
            st, acc = [], 1
            for d in dims:
                st.append(acc * bits)
                acc *= d
        else:
            st = [int(v) for v in o.strides]
        o.live_dims = torch.tensor(dims, dtype=torch.int32, device=x.device)
        o.live_strides = torch.tensor(st, dtype=torch.int64, device=x.device)
        held += [o.live_dims, o.live_strides]
    w0 = (nd - 1 - axis) | (int(pad_size) << 32)
    w1 = 0 | (nd << 32)  # SoftmaxModeDynamic = 0
    attrs = np.asarray([w0, w1], dtype=np.uint64).tobytes()
    entry = "softmaxFp32" if _torch_dtype_code(x) == NN_FP32 else "softmax"
    sw_kernel_launch(entry, create_kernel_params(ops[:1], ops[1:], attrs), ops, stream)
    return held


def _view_strides(field, x):
    """N, H, W, C strides (elements) of a 4-D tensor that is a view of a larger one; a contiguous tensor leaves the
    field zeroed, which is the task's dense default."""
    if not x.is_contiguous():
        for i, v in enumerate(x.stride()[-4:]):
            field[i] = v


def nce_task(inp, weights, weight_table, out, ppe, zp_in=0, zp_w=0, zp_out=0, strides=(1, 1),
             pads=(0, 0, 0, 0), stream=None, groups=None):
    """inp NHWC, weights [OC,KY,KX,IC], weight_table [OC,4] int32 (device), out NHWC.
    pads = (left, right, top, bottom).  With groups=G every tensor carries a leading dimension of G
    (dense), and the G tasks go down in one call.  inp and out may be views of larger tensors (a channel slice,
    a window in H or W): their strides go into the task."""
    if groups is not None:
        assert inp.shape[0] == weights.shape[0] == weight_table.shape[0] == out.shape[0] == groups
        assert all(x.is_contiguous() for x in (inp, weights, weight_table, out))
    N, H, W, IC = inp.shape[-4:]
    OC, KY, KX, IC2 = weights.shape[-4:]
    assert IC == IC2
    t = NceTask()
    t.task_type = 0
    t.groups = groups or 0
    t.input, t.weights, t.weight_table, t.output = inp.data_ptr(), weights.data_ptr(), weight_table.data_ptr(), out.data_ptr()
    t.input_type, t.weights_type, t.output_type = (_torch_dtype_code(x) for x in (inp, weights, out))
    t.N, t.H, t.W, t.IC, t.OC = N, H, W, IC, OC
    t.kernel_size[0], t.kernel_size[1] = KY, KX
    t.kernel_strides[0], t.kernel_strides[1] = strides
    for i in range(4):
        t.kernel_padding[i] = pads[i]
    t.zp_in, t.zp_w, t.zp_out = zp_in, zp_w, zp_out
    t.ppe = ppe
    if groups is None:
        assert weights.is_contiguous() and weight_table.is_contiguous()
        _view_strides(t.input_strides, inp)
        _view_strides(t.output_strides, out)
    check(lib().vpx_nce_task(C.byref(t), _stream_handle(stream)))
    return out


def nce_eltwise(in1, in2, out, ppe, zp_in1=0, zp_in2=0, zp_out=0, subtract=False, stream=None):
    """Quantized add / subtract of two NHWC 8-bit tensors of one shape (NCE ELTWISE task); `ppe` carries
    quant_mult / quant_shift / in1_quant_mult / in2_quant_mult."""
    assert in1.shape == in2.shape == out.shape and in1.dim() == 4
    N, H, W, IC = in1.shape
    t = NceTask()
    t.task_type = NCE_ELTWISE
    t.eltwise_type = ELTWISE_SUBTRACT if subtract else ELTWISE_ADD
    t.input, t.weights, t.weight_table, t.output = in1.data_ptr(), in2.data_ptr(), None, out.data_ptr()
    t.input_type, t.weights_type, t.output_type = (_torch_dtype_code(x) for x in (in1, in2, out))
    t.N, t.H, t.W, t.IC, t.OC = N, H, W, IC, IC
    t.kernel_size[0] = t.kernel_size[1] = t.kernel_strides[0] = t.kernel_strides[1] = 1
    t.zp_in, t.zp_w, t.zp_out = zp_in1, zp_in2, zp_out
    t.ppe = ppe
    _view_strides(t.input_strides, in1)
    _view_strides(t.weights_strides, in2)
    _view_strides(t.output_strides, out)
    check(lib().vpx_nce_task(C.byref(t), _stream_handle(stream)))
    return out


def nce_matmul(a, b_nk, weight_table, out, ppe, zp_a=0, zp_b=0, zp_out=0, stream=None):
    """A [M,K] x B stored [N,K] -> out [M,N]: NCE.MatMul as the 1x1 convolution task.  Three-dimensional operands
    (A [G,M,K], B [G,N,K], weight table [G,N,4], out [G,M,N]) are the operator's grouped form, one call."""
    if a.dim() == 3:
        G, M, K = a.shape
        Nn = b_nk.shape[1]
        return nce_task(a.view(G, 1, M, 1, K), b_nk.view(G, Nn, 1, 1, K), weight_table, out.view(G, 1, M, 1, Nn), ppe,
                        zp_in=zp_a, zp_w=zp_b, zp_out=zp_out, stream=stream, groups=G)
    M, K = a.shape
    Nn, _ = b_nk.shape
    return nce_task(a.view(1, M, 1, K), b_nk.view(Nn, 1, 1, K), weight_table, out.view(1, M, 1, Nn), ppe, zp_in=zp_a,
                    zp_w=zp_b, zp_out=zp_out, stream=stream)


def set_tuning(knob, value=None):
    """Override the NCE dispatcher (tests, tuning): knob is a VPX_* name, value a string or None for the default."""
    check(lib().vpx_set_tuning(knob.encode(), None if value is None else str(value).encode()))


def calib_mfma_i8(operands, sink, iters, fragment_reads=False, stream=None):
    """Enqueue the int8 MFMA calibration loop (operands: 64 KiB on the device, sink: 8 KiB per compute unit);
    returns the integer operations the launch performs."""
    ops = C.c_int64(0)
    check(lib().vpx_calib_mfma_i8(operands.data_ptr(), sink.data_ptr(), int(iters), int(bool(fragment_reads)), C.byref(ops),
                                  _stream_handle(stream)))
    return ops.value


COISSUE_KINDS = ["v_fma_f64", "v_fma_f32", "v_add_u32", "v_mul_lo_u32", "v_mad_u64_u32", "v_cvt_f64_i32"]


def calib_coissue(valu_kind, wide_mfma, mode, iters, sink, stream=None):
    """Enqueue the co-issue calibration loop (vpx_calib_coissue; sink: 8 KiB per compute unit on the device)."""
    check(lib().vpx_calib_coissue(int(valu_kind), int(bool(wide_mfma)), int(mode), int(iters), C.c_void_p(sink.data_ptr()),
                                  _stream_handle(stream)))


def workspace_reserve(nbytes, stream=None):
    """Grow the library's scratch block of `stream` on the current device to at least nbytes."""
    check(lib().vpx_workspace_reserve(_stream_handle(stream), nbytes))


def workspace_release(stream=None):
    """Wait for `stream`, then free its scratch block and cached per-axis tables."""
    check(lib().vpx_workspace_release(_stream_handle(stream)))


def nce_last_kernel():
    return lib().vpx_nce_last_kernel().decode()
