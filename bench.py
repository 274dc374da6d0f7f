#!/usr/bin/env python3
"""Benchmark of the vpux hot path on one MI355X.

A step is one pass of the selected configuration's hot path over one batch of synthetic input that
is already resident in HBM.  The headline workload is BASELINE configuration 5's int8 matmul
(A[4096,4096] x B[4096,11008] with the integer PPE), the largest configuration and the one the
metric's first clause (int8 TOP/s) is quoted on; the same run appends `other_configs` with the
remaining BASELINE configurations (C1 FakeQuantize, C2 softmax, C3 MVN, C4 conv, C5 dequantize and
C5 add), each with its own roofline and CPU baseline.

Every configuration is timed over a rotation of separate buffer sets whose total is at least 1 GiB
(four times the 256 MB Infinity Cache), so a step does not find its operands in cache; the same-buffers
figure, a HIP-graph replay and a steady-state figure (200 launches after 50 ms of the same launches) are
reported beside it as named extras.  The JSON line on stdout holds numbers; the descriptions and notes of
the configurations go to stderr.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c5_matmul] [--only] [--no-cpu] [--extra]
"""
import argparse
import ctypes as C
import itertools
import json
import os
import sys
import time

import numpy as np

HBM_PEAK_GBS = 8000.0     # MI355X HBM3E, published
I8_PEAK_TOPS = 5000.0     # MI355X dense int8 MFMA, published

METRIC = "int8 conv/matmul TOPS (% MFMA peak); SW-kernel GB/s (% HBM peak)"

# Bytes moved through L2 per step.  These are NOT measured in this run: they are the rocprofv3 FETCH_SIZE /
# WRITE_SIZE counters of an earlier run of the same workload, scaled by a plain copy of known size
# (profiles/<workload>__*.md hold those runs and their commands); the JSON line labels them as such.
MEASURED_TRAFFIC = {
    "c1_fake_quantize": 888450, "c2_softmax": 134261983, "c3_mvn": 17043564, "c4_conv": 14905457,
    "c5_matmul": 339731998, "c5_dequantize": 135262411, "c5_eltwise_add": 270552950, "c5_nce_eltwise": 135260008,
    "calib_copy": 134217728, "calib_int_mm": 534882288, "x_mvn6_layernorm": 268523883, "x_activation_hswish": 180471319,
    "x_mvn1_three_steps": 25341653, "x_stem_conv": 67131551, "x_small_plane_conv": 20886567, "x_large_conv": 54593192,
    "x_wide_conv": 58724921, "x_pointwise_conv": 36744405, "x_softmax_outer_axis": 402620437, "x_mvn_nhwc_per_channel": 317063410,
}


def _dev(a, f16=False):
    import torch
    a = np.ascontiguousarray(a)
    if f16:
        a = a.view(np.float16)
    return torch.from_numpy(a).cuda()


class Workload:
    """name, description, a zero-argument `step` that enqueues one pass on the current stream,
    algorithmic bytes and ops per step, roofline bound and the CPU-oracle sample runner."""

    def __init__(self, name, desc, step, bytes_per_step, ops_per_step, bound, dtype, kernel, cpu_sample=None,
                 cpu_units=(1, 1, "full tensor")):
        self.name, self.desc, self.step = name, desc, step
        self.bytes, self.ops, self.bound, self.dtype, self.kernel = bytes_per_step, ops_per_step, bound, dtype, kernel
        # cpu_sample(oracle, units) -> (callable, work in bytes or ops); cpu_units = (first sample, whole workload, what a unit is)
        self.cpu_sample, self.cpu_units = cpu_sample, cpu_units


def _prebuilt_sw_launch(rt, entry, blob, operands):
    """Bind everything once so that a step is a single foreign call."""
    import torch
    L = rt.lib()
    addrs = (rt.MemRefAddr * len(operands))()
    for i, o in enumerate(operands):
        addrs[i].data = o.t.data_ptr()
    name = entry.encode()
    n = len(operands)
    size = len(blob)

    def step():
        rc = L.vpx_sw_kernel_launch(name, blob, size, addrs, n, C.c_void_p(torch.cuda.current_stream().cuda_stream))
        if rc:
            rt.check(rc)
    step.keep = (addrs, operands, blob)
    return step


def make_c1(rt):
    import torch
    from vpux_plugin_amd import configs
    c = configs.c1_fake_quantize()
    x = _dev(c["x"], True)
    out = torch.empty_like(x)
    ops = [rt.Operand(t) for t in (x, *[_dev(c[k], True) for k in ("in_lo", "in_hi", "out_lo", "out_hi")], out)]
    blob = rt.create_kernel_params(ops[:5], ops[5:], np.int64(c["levels"]).tobytes())
    n = x.numel()

    def cpu(orc, frac):
        return lambda: orc.fake_quantize_f16(c["x"], c["in_lo"], c["in_hi"], c["out_lo"], c["out_hi"], 256), n * 4
    return Workload("c1_fake_quantize", "FakeQuantize fp16 NCHW [1,64,56,56], per-tensor, 256 levels, +-4",
                    _prebuilt_sw_launch(rt, "fake_quantize", blob, ops), n * 4, 0, "hbm", "f16", "stream_kernel<FqMap>", cpu,
                    (1, 1, "full tensor"))


def make_c2(rt):
    import torch
    from vpux_plugin_amd import configs
    c = configs.c2_softmax()
    x = _dev(c["x"], True)
    out = torch.empty_like(x)
    ops = [rt.Operand(x), rt.Operand(out)]
    dims = [int(d) for d in ops[0].dims]
    st = [int(s) // 16 for s in ops[0].strides]
    attrs = rt.generate_softmax_attr(dims, st, st, 0, 0).tobytes()
    blob = rt.create_kernel_params(ops[:1], ops[1:], attrs)
    n = x.numel()

    def cpu(orc, rows):
        xs = np.ascontiguousarray(c["x"].reshape(-1, 512)[:rows])
        return lambda: orc.softmax_f16(xs, 1), xs.size * 4
    return Workload("c2_softmax", "Softmax fp16 last axis [8,16,512,512], 5% of logits masked to -60000",
                    _prebuilt_sw_launch(rt, "softmax", blob, ops), n * 4, 0, "hbm", "f16", "softmax_rows_f16", cpu,
                    (2048, 65536, "rows"))


def make_c3(rt):
    import torch
    from vpux_plugin_amd import configs
    c = configs.c3_mvn()
    x = _dev(c["x"], True)
    out = torch.empty_like(x)
    ops = [rt.Operand(x, "NCHW"), rt.Operand(out, "NCHW")]
    attrs = np.asarray([-1, -1], dtype=np.int64).tobytes() + np.float32(c["eps"]).tobytes()
    blob = rt.create_kernel_params(ops[:1], ops[1:], attrs)
    n = x.numel()

    def cpu(orc, groups):
        xs = np.ascontiguousarray(c["x"][:groups])
        return lambda: orc.mvn_f16(xs, True, True, c["eps"]), xs.size * 4
    return Workload("c3_mvn", "MVN fp16 across C,H,W [4,256,64,64], eps 1e-9, normalize_variance",
                    _prebuilt_sw_launch(rt, "mvn1", blob, ops), n * 4, 0, "hbm", "f16", "mvn_fused_kernel", cpu,
                    (1, 4, "batch elements"))


def make_softmax_outer(rt):
    """Softmax over an outer axis too long for the register slabs: [32,2048,1024] fp16 over axis 1."""
    import torch
    g = torch.Generator(device="cuda").manual_seed(11)
    x = (torch.randn((32, 2048, 1024), device="cuda", generator=g) * 3).half()
    out = torch.empty_like(x)
    ops = [rt.Operand(x), rt.Operand(out)]
    dims = [int(d) for d in ops[0].dims]
    st = [int(s) // 16 for s in ops[0].strides]
    attrs = rt.generate_softmax_attr(dims, st, st, 1, 0).tobytes()  # axis counted from the innermost dimension
    blob = rt.create_kernel_params(ops[:1], ops[1:], attrs)
    return Workload("x_softmax_outer_axis", "Softmax fp16 [32,2048,1024] over axis 1 (2048 steps, rows of 1024 contiguous)",
                    _prebuilt_sw_launch(rt, "softmax", blob, ops), x.numel() * 4, 0, "hbm", "f16", "softmax_cols")


def make_mvn_nhwc(rt):
    """MVN per channel on a channel-minor tensor: [16,112,112,256] fp16 stored NHWC."""
    import torch
    g = torch.Generator(device="cuda").manual_seed(12)
    x = (torch.rand((16, 112, 112, 256), device="cuda", generator=g) * 16 - 8).half()
    out = torch.empty_like(x)
    ops = [rt.Operand(x, "NHWC"), rt.Operand(out, "NHWC")]  # (operands are indexed in memory order)
    attrs = np.asarray([0, -1], dtype=np.int64).tobytes() + np.float32(1e-9).tobytes()
    blob = rt.create_kernel_params(ops[:1], ops[1:], attrs)
    return Workload("x_mvn_nhwc_per_channel", "MVN fp16 per channel, NHWC storage [16,112,112,256], normalize_variance",
                    _prebuilt_sw_launch(rt, "mvn1", blob, ops), x.numel() * 4, 0, "hbm", "f16", "mvn_nhwc kernels")


def _nce_step(rt, task):
    import torch
    L = rt.lib()

    def step():
        rc = L.vpx_nce_task(C.byref(task), C.c_void_p(torch.cuda.current_stream().cuda_stream))
        if rc:
            rt.check(rc)
    return step


def _nce_task(rt, inp, w, wt, out, ppe, zp_in, zp_out, strides, pads):
    N, H, W, IC = inp.shape
    OC, KY, KX, _ = w.shape
    t = rt.NceTask()
    t.task_type = 0
    t.input, t.weights, t.weight_table, t.output = inp.data_ptr(), w.data_ptr(), wt.data_ptr(), out.data_ptr()
    t.input_type, t.weights_type, t.output_type = (rt._torch_dtype_code(v) for v in (inp, w, out))
    t.N, t.H, t.W, t.IC, t.OC = N, H, W, IC, OC
    t.kernel_size[0], t.kernel_size[1] = KY, KX
    t.kernel_strides[0], t.kernel_strides[1] = strides
    for i in range(4):
        t.kernel_padding[i] = pads[i]
    t.zp_in, t.zp_w, t.zp_out = zp_in, 0, zp_out
    t.ppe = ppe
    return t


def make_c4(rt):
    import torch
    from vpux_plugin_amd import configs
    c = configs.c4_conv()
    inp, w = _dev(c["input"]), _dev(c["weights"])
    wt_h = rt.make_weights_table(c["mult"], c["shift"], c["bias"], 9 * 64)
    wt = _dev(wt_h)
    out = torch.empty((32, 56, 56, 64), dtype=torch.uint8, device="cuda")
    ppe = rt.PpeInt(rt.PPE_NOOP, c["clamp"][0], c["clamp"][1], 1, 0)
    task = _nce_task(rt, inp, w, wt, out, ppe, c["zp_in"], c["zp_out"], c["strides"], c["pads"])
    step = _nce_step(rt, task)
    step.keep = (inp, w, wt, out, task)
    ops = 2 * 32 * 56 * 56 * 64 * 9 * 64
    nbytes = inp.numel() + out.numel() + w.numel() + wt.numel() * 4

    def cpu(orc, rows):
        p = orc.ppe(1, 0, 0, 0, 255)
        return lambda: orc.nce_conv(c["input"], c["weights"], wt_h, p, zp_in=128, pads=(1, 1, 1, 1), rows=(0, rows)), \
            2 * rows * 64 * 9 * 64
    return Workload("c4_conv", "int8 Conv 3x3 s1 p1 NHWC [32,56,56,64] u8 zp128 x [64,3,3,64] i8, PPE ReLU clamp [0,255]",
                    step, nbytes, ops, "mfma", "int8", "nce_conv_regw", cpu, (3136, 100352, "output positions"))


def make_conv64(rt, name, N, H, W):
    """3x3, 64 -> 64 channels, stride 1, padding 1, ReLU: the C4 layer at other sizes (not a BASELINE config)."""
    import torch
    g = torch.Generator(device="cuda").manual_seed(17)
    inp = torch.randint(0, 256, (N, H, W, 64), dtype=torch.uint8, device="cuda", generator=g)
    w = torch.randint(-127, 128, (64, 3, 3, 64), dtype=torch.int8, device="cuda", generator=g)
    rng = np.random.default_rng(17)
    wt = _dev(rt.make_weights_table(rng.integers(2 ** 14, 2 ** 15, 64), rng.integers(20, 25, 64),
                                    rng.integers(-2 ** 15, 2 ** 15, 64).astype(np.int32), 9 * 64))
    out = torch.empty((N, H, W, 64), dtype=torch.uint8, device="cuda")
    ppe = rt.PpeInt(rt.PPE_NOOP, 0, 255, 1, 0)
    task = _nce_task(rt, inp, w, wt, out, ppe, 128, 0, (1, 1), (1, 1, 1, 1))
    step = _nce_step(rt, task)
    step.keep = (inp, w, wt, out, task)
    ops = 2 * N * H * W * 64 * 9 * 64
    return Workload(name, "int8 Conv 3x3 s1 p1 NHWC [%d,%d,%d,64] u8 zp128 x [64,3,3,64] i8, ReLU clamp (not a BASELINE config)" % (N, H, W),
                    step, inp.numel() + out.numel() + w.numel() + wt.numel() * 4, ops, "mfma", "int8", "nce_conv_regw")


def make_pointwise(rt):
    """1x1, 64 -> 256 channels (the expansion layer of a ResNet-50 stage-2 block): bound by its 26 MB of output
    (not a BASELINE config)."""
    import torch
    N, H, W, IC, OC = 32, 56, 56, 64, 256
    g = torch.Generator(device="cuda").manual_seed(19)
    inp = torch.randint(0, 256, (N, H, W, IC), dtype=torch.uint8, device="cuda", generator=g)
    w = torch.randint(-127, 128, (OC, 1, 1, IC), dtype=torch.int8, device="cuda", generator=g)
    rng = np.random.default_rng(19)
    wt = _dev(rt.make_weights_table(rng.integers(2 ** 14, 2 ** 15, OC), rng.integers(18, 23, OC),
                                    rng.integers(-2 ** 15, 2 ** 15, OC).astype(np.int32), IC))
    out = torch.empty((N, H, W, OC), dtype=torch.uint8, device="cuda")
    ppe = rt.PpeInt(rt.PPE_NOOP, 0, 255, 1, 0)
    task = _nce_task(rt, inp, w, wt, out, ppe, 128, 0, (1, 1), (0, 0, 0, 0))
    step = _nce_step(rt, task)
    step.keep = (inp, w, wt, out, task)
    ops = 2 * N * H * W * IC * OC
    return Workload("x_pointwise_conv", "int8 Conv 1x1 NHWC [32,56,56,64] u8 zp128 x [256,1,1,64] i8, ReLU clamp (not a BASELINE config)",
                    step, inp.numel() + out.numel() + w.numel() + wt.numel() * 4, ops, "hbm", "int8", "nce_gemm_regb")


def make_stem(rt):
    """The first layer of a ResNet-50 with the image channels padded to 16: not a BASELINE config."""
    import torch
    N, H, IC, OC, K = 32, 224, 16, 64, 7
    g = torch.Generator(device="cuda").manual_seed(9)
    inp = torch.randint(0, 256, (N, H, H, IC), dtype=torch.uint8, device="cuda", generator=g)
    w = torch.randint(-127, 128, (OC, K, K, IC), dtype=torch.int8, device="cuda", generator=g)
    wt = _dev(rt.make_weights_table(np.full(OC, 20000), np.full(OC, 22), np.zeros(OC, np.int32), K * K * IC))
    out = torch.empty((N, H // 2, H // 2, OC), dtype=torch.uint8, device="cuda")
    ppe = rt.PpeInt(rt.PPE_LRELU, 0, 255, 1, 0)
    task = _nce_task(rt, inp, w, wt, out, ppe, 128, 0, (2, 2), (3, 3, 3, 3))
    step = _nce_step(rt, task)
    step.keep = (inp, w, wt, out, task)
    ops = 2 * N * (H // 2) * (H // 2) * OC * K * K * IC
    return Workload("x_stem_conv", "int8 Conv 7x7 s2 p3 NHWC [32,224,224,16] u8 zp128 x [64,7,7,16] i8, ReLU (not a BASELINE config)",
                    step, inp.numel() + out.numel() + w.numel() + wt.numel() * 4, ops, "mfma", "int8", "nce_conv_rows16")


def make_small_plane_conv(rt):
    """A late ResNet-50 layer, 3x3 over 7x7 planes of 512 channels: not a BASELINE config."""
    import torch
    N, H, IC, OC, K = 32, 7, 512, 512, 3
    g = torch.Generator(device="cuda").manual_seed(10)
    inp = torch.randint(0, 256, (N, H, H, IC), dtype=torch.uint8, device="cuda", generator=g)
    w = torch.randint(-127, 128, (OC, K, K, IC), dtype=torch.int8, device="cuda", generator=g)
    wt = _dev(rt.make_weights_table(np.full(OC, 20000), np.full(OC, 24), np.zeros(OC, np.int32), K * K * IC))
    out = torch.empty((N, H, H, OC), dtype=torch.uint8, device="cuda")
    ppe = rt.PpeInt(rt.PPE_LRELU, 0, 255, 1, 0)
    task = _nce_task(rt, inp, w, wt, out, ppe, 128, 0, (1, 1), (1, 1, 1, 1))
    step = _nce_step(rt, task)
    step.keep = (inp, w, wt, out, task)
    ops = 2 * N * H * H * OC * K * K * IC
    return Workload("x_small_plane_conv", "int8 Conv 3x3 s1 p1 NHWC [32,7,7,512] u8 zp128 x [512,3,3,512] i8, ReLU (not a BASELINE config)",
                    step, inp.numel() + out.numel() + w.numel() + wt.numel() * 4, ops, "mfma", "int8", "nce_conv_stream")


_C5_CACHE = {}


def _c5_quantized(M, N):
    """Stand-in for the matmul's i8 output (uniform codes), generated once on the host."""
    if "q" not in _C5_CACHE:
        _C5_CACHE["q"] = np.random.default_rng(55).integers(-128, 128, (M, N), dtype=np.int8)
    return _C5_CACHE["q"]


def _c5_dequantized(M, N):
    """The dequantized tensor the residual is added to: code * 0.05, exact in fp16 for |code| <= 128 after rounding."""
    if "deq" not in _C5_CACHE:
        _C5_CACHE["deq"] = (_c5_quantized(M, N).astype(np.float32) * np.float32(0.05)).astype(np.float16).view(np.uint16)
    return _C5_CACHE["deq"]


def make_c5(rt, part="matmul"):
    import torch
    from vpux_plugin_amd import configs
    c = configs.c5_matmul()
    M, K = c["a"].shape
    N = c["b_nk"].shape[0]
    if part == "matmul":
        a, b = _dev(c["a"]), _dev(c["b_nk"])
        wt_h = rt.make_weights_table(c["mult"], c["shift"], c["bias"], K)
        wt = _dev(wt_h)
        out = torch.empty((M, N), dtype=torch.int8, device="cuda")
        ppe = rt.PpeInt(rt.PPE_LPRELU, c["clamp"][0], c["clamp"][1], c["lrelu_mult"], c["lrelu_shift"])
        task = _nce_task(rt, a.view(1, M, 1, K), b.view(N, 1, 1, K), wt, out.view(1, M, 1, N), ppe, c["zp_a"],
                         c["zp_out"], (1, 1), (0, 0, 0, 0))
        step = _nce_step(rt, task)
        step.keep = (a, b, wt, out, task)

        def cpu(orc, rows):
            p = orc.ppe(c["lrelu_mult"], c["lrelu_shift"], 0, -128, 127)
            a_s = np.ascontiguousarray(c["a"][:rows])
            return lambda: orc.nce_matmul(a_s, c["b_nk"], wt_h, p, zp_a=c["zp_a"]), 2 * rows * K * N
        return Workload("c5_matmul", "int8 MatMul A[4096,4096] zp3 x B[4096,11008], PPE per-column + LeakyReLU 0.1 -> i8",
                        step, M * K + N * K + M * N + N * 16, 2 * M * K * N, "mfma", "int8", "nce_gemm_mfma", cpu,
                        (8, 4096, "rows of A"))
    q_h = _c5_quantized(M, N)
    q = _dev(q_h)
    if part == "nce_eltwise":
        # the quantized form of the same residual add: i8 + i8 -> i8 on the NCE eltwise path
        res_q = torch.randint(-128, 128, (M, N), dtype=torch.int8, device="cuda")
        out_q = torch.empty_like(q)
        m1, m2, mo, so = rt.eltwise_quantization_approximation(0.05, 0.04, 0.07, 0)
        t = rt.NceTask()
        t.task_type, t.eltwise_type = rt.NCE_ELTWISE, rt.ELTWISE_ADD
        t.input, t.weights, t.weight_table, t.output = q.data_ptr(), res_q.data_ptr(), None, out_q.data_ptr()
        t.input_type = t.weights_type = t.output_type = rt.NN_I8
        t.N, t.H, t.W, t.IC, t.OC = 1, M, 1, N, N
        t.kernel_size[0] = t.kernel_size[1] = t.kernel_strides[0] = t.kernel_strides[1] = 1
        t.zp_in, t.zp_w, t.zp_out = 3, -2, 0
        t.ppe = rt.PpeInt(rt.PPE_NOOP, -128, 127, 1, 0, mo, so, m1, m2)
        step = _nce_step(rt, t)
        step.keep = (q, res_q, out_q, t)
        return Workload("c5_nce_eltwise", "NCE eltwise add i8 + i8 -> i8 [4096,11008] (quantized residual; not a BASELINE config)",
                        step, M * N * 3, 0, "hbm", "int8", "nce_eltwise_kernel")
    deq = torch.empty((M, N), dtype=torch.float16, device="cuda")
    if part == "dequant":
        ops = [rt.Operand(q), rt.Operand(deq)]
        blob = rt.create_kernel_params(ops[:1], ops[1:], rt.get_quant_params_attr(c["deq_scale"], c["deq_zp"], rt.NN_FP16).tobytes())

        def cpu(orc, rows):
            qs = np.ascontiguousarray(q_h[:rows])
            return lambda: orc.dequantize(qs, [c["deq_scale"]], [c["deq_zp"]], to_f16=True), qs.size * 3
        return Workload("c5_dequantize", "Dequantize i8 -> fp16 [4096,11008], per-tensor",
                        _prebuilt_sw_launch(rt, "dequantize", blob, ops), M * N * 3, 0, "hbm", "f16", "stream_kernel<DequantFn>",
                        cpu, (256, 4096, "rows"))
    res = _dev(c["residual"], True)
    y = torch.empty_like(deq)
    deq_h = _c5_dequantized(M, N)
    deq.copy_(_dev(deq_h, True))
    ops = [rt.Operand(deq), rt.Operand(res), rt.Operand(y)]
    blob = rt.create_kernel_params(ops[:2], ops[2:])

    def cpu(orc, rows):
        a_s, b_s = np.ascontiguousarray(deq_h[:rows]), np.ascontiguousarray(c["residual"][:rows])
        return lambda: orc.eltwise_f16("add", a_s, b_s), a_s.size * 6
    return Workload("c5_eltwise_add", "Eltwise Add fp16 [4096,11008] + residual",
                    _prebuilt_sw_launch(rt, "eltwise_add", blob, ops), M * N * 6, 0, "hbm", "f16", "stream_kernel<EltFn add>",
                    cpu, (256, 4096, "rows"))


def make_copy(rt):
    """fp16 -> fp16 `convert` of the softmax tensor: a plain copy of known size, the yardstick the
    FETCH_SIZE / WRITE_SIZE counters of the other kernels are scaled by."""
    import torch
    x = torch.zeros((8, 16, 512, 512), dtype=torch.float16, device="cuda")
    out = torch.empty_like(x)
    ops = [rt.Operand(x), rt.Operand(out)]
    blob = rt.create_kernel_params(ops[:1], ops[1:])
    n = x.numel()
    return Workload("calib_copy", "copy fp16 [8,16,512,512] (counter calibration)",
                    _prebuilt_sw_launch(rt, "convert", blob, ops), n * 4, 0, "hbm", "f16", "stream_kernel<Copy>")


def make_layernorm(rt):
    """mvn6 over the last axis with the fused scale and bias (a LayerNorm): not a BASELINE config."""
    import torch
    rows, width = 16384, 4096
    g = torch.Generator(device="cuda").manual_seed(7)
    x = torch.randn((rows, width), device="cuda", generator=g).half()
    sc = torch.rand((1, width), device="cuda", generator=g).half()
    bi = torch.rand((1, width), device="cuda", generator=g).half()
    out = torch.empty_like(x)
    ops = [rt.Operand(t) for t in (x, sc, bi, out)]
    attrs = (np.asarray([-(2 ** 63), 15, -1, 0], dtype=np.int64).tobytes() + np.float32(1e-5).tobytes() +
             np.asarray([1, 0], dtype=np.int64).tobytes())
    blob = rt.create_kernel_params(ops[:3], ops[3:], attrs)
    return Workload("x_mvn6_layernorm", "MVN-6 fp16 over the last axis [16384,4096] with scale and bias (not a BASELINE config)",
                    _prebuilt_sw_launch(rt, "mvn6", blob, ops), x.numel() * 4 + width * 4, 0, "hbm", "f16", "mvn6_rows_kernel")


def make_activation(rt):
    """hswish on the C5-sized tensor: not a BASELINE config."""
    import torch
    x = torch.randn((4096, 11008), device="cuda", generator=torch.Generator(device="cuda").manual_seed(8)).half()
    out = torch.empty_like(x)
    ops = [rt.Operand(x), rt.Operand(out)]
    blob = rt.create_kernel_params(ops[:1], ops[1:])
    return Workload("x_activation_hswish", "activation_hswish fp16 [4096,11008] (not a BASELINE config)",
                    _prebuilt_sw_launch(rt, "activation_hswish", blob, ops), x.numel() * 4, 0, "hbm", "f16", "stream_kernel<ActFn>")


def make_mvn_steps(rt):
    """The compiler's three-step form of C3: mvn1_sum -> mvn1_mean_var -> mvn1_norm (not a BASELINE config)."""
    import torch
    from vpux_plugin_amd import configs
    c = configs.c3_mvn()
    x = _dev(c["x"], True)
    N, Cc, H, W = x.shape
    out = torch.empty_like(x)
    sums = torch.empty((N, 1, 2, 1), dtype=torch.float32, device="cuda")
    mv = torch.empty((N, 1, 2, 1), dtype=torch.float32, device="cuda")
    flags = np.asarray([-1, -1], dtype=np.int64).tobytes()
    o1 = [rt.Operand(x, "NCHW"), rt.Operand(sums, "NHWC")]
    o2 = [rt.Operand(sums, "NHWC"), rt.Operand(mv, "NHWC")]
    o3 = [rt.Operand(x, "NCHW"), rt.Operand(mv, "NHWC"), rt.Operand(out, "NCHW")]
    a2 = np.asarray([N, Cc, H, W, -1, -1, 1], dtype=np.int64).tobytes() + np.float32(c["eps"]).tobytes()
    steps = [_prebuilt_sw_launch(rt, "mvn1_sum", rt.create_kernel_params(o1[:1], o1[1:], flags), o1),
             _prebuilt_sw_launch(rt, "mvn1_mean_var", rt.create_kernel_params(o2[:1], o2[1:], a2), o2),
             _prebuilt_sw_launch(rt, "mvn1_norm", rt.create_kernel_params(o3[:2], o3[2:], flags), o3)]

    def step():
        for f in steps:
            f()
    step.keep = steps
    return Workload("x_mvn1_three_steps", "mvn1_sum -> mvn1_mean_var -> mvn1_norm fp16 [4,256,64,64] (not a BASELINE config)",
                    step, x.numel() * 4, 0, "hbm", "f16", "mvn_norm_runs_kernel")


def make_int_mm(rt):
    """The vendor library's int8 GEMM (torch._int_mm, hipBLASLt) on the C5 operands, int32 output and no PPE: the yardstick
    for what this part sustains on uniform random int8 data, beside which nce_gemm_mfma is read."""
    import torch
    from vpux_plugin_amd import configs
    c = configs.c5_matmul()
    a, b_nk = _dev(c["a"]), _dev(c["b_nk"])
    M, K = a.shape
    N = b_nk.shape[0]
    b = b_nk.t()
    out = torch.empty((M, N), dtype=torch.int32, device="cuda")

    def step():
        torch._int_mm(a, b, out=out)
    step.keep = (a, b_nk, out)
    return Workload("calib_int_mm", "torch._int_mm (hipBLASLt) i8 [4096,4096] x [4096,11008] -> i32, no PPE (vendor yardstick)",
                    step, 0, 2 * M * K * N, "mfma", "int8", "hipBLASLt")


def make_mfma_loop(rt, operands, fragment_reads):
    """`v_mfma_i32_32x32x32_i8` alone (or with the matmul kernel's LDS fragment reads) on every compute unit: the rate the
    part sustains on these operand bytes before anything comes from global memory."""
    import torch
    if operands == "random":
        g = torch.Generator(device="cuda").manual_seed(5)
        src = torch.randint(-128, 128, (65536,), device="cuda", generator=g, dtype=torch.int8)
    else:
        src = torch.zeros((65536,), device="cuda", dtype=torch.int8)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    sink = torch.empty((cus * 8192,), device="cuda", dtype=torch.uint8)
    iters = 2000
    ops = rt.calib_mfma_i8(src, sink, iters, fragment_reads)
    torch.cuda.synchronize()

    def step():
        rt.calib_mfma_i8(src, sink, iters, fragment_reads)
    step.keep = (src, sink)
    name = "calib_mfma_%s%s" % (operands, "_lds" if fragment_reads else "")
    desc = "loop of v_mfma_i32_32x32x32_i8 on %s int8 operands, two waves per SIMD, %s" % (
        operands, "with the matmul kernel's twelve LDS fragment reads per sixteen MFMAs" if fragment_reads else "registers only")
    return Workload(name, desc, step, 0, ops, "mfma", "int8", "calib_mfma_i8_kernel")


MAKERS = {
    "calib_copy": make_copy,
    "calib_int_mm": make_int_mm,
    "calib_mfma_random": lambda rt: make_mfma_loop(rt, "random", False),
    "calib_mfma_random_lds": lambda rt: make_mfma_loop(rt, "random", True),
    "calib_mfma_zero": lambda rt: make_mfma_loop(rt, "zero", False),
    "calib_mfma_zero_lds": lambda rt: make_mfma_loop(rt, "zero", True),
    "c1_fake_quantize": make_c1,
    "c2_softmax": make_c2,
    "c3_mvn": make_c3,
    "c4_conv": make_c4,
    "c5_matmul": lambda rt: make_c5(rt, "matmul"),
    "c5_dequantize": lambda rt: make_c5(rt, "dequant"),
    "c5_eltwise_add": lambda rt: make_c5(rt, "add"),
    "c5_nce_eltwise": lambda rt: make_c5(rt, "nce_eltwise"),
    "x_mvn6_layernorm": make_layernorm,
    "x_activation_hswish": make_activation,
    "x_mvn1_three_steps": make_mvn_steps,
    "x_softmax_outer_axis": make_softmax_outer,
    "x_mvn_nhwc_per_channel": make_mvn_nhwc,
    "x_stem_conv": make_stem,
    "x_pointwise_conv": make_pointwise,
    "x_large_conv": lambda rt: make_conv64(rt, "x_large_conv", 128, 56, 56),
    "x_wide_conv": lambda rt: make_conv64(rt, "x_wide_conv", 32, 112, 112),
    "x_small_plane_conv": make_small_plane_conv,
}


def time_steps(step, steps, warmup, graph=False):
    """Returns (wall ms per step, device ms per step from events on the launch stream)."""
    import torch
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    if graph:
        g = torch.cuda.CUDAGraph()
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            step()  # first use of a stream may size the library's scratch buffer: not allowed while capturing
        s.synchronize()
        with torch.cuda.stream(s):
            with torch.cuda.graph(g, stream=s):
                for _ in range(steps):
                    step()
        torch.cuda.current_stream().wait_stream(s)
        g.replay()
        torch.cuda.synchronize()
        run = g.replay
    else:
        def run(seq=(step,) * steps):
            for f in seq:
                f()
    # events are recorded on the stream the steps are launched on (the current stream)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    run()
    e1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return (t1 - t0) * 1e3 / steps, e0.elapsed_time(e1) / steps


def steady_state(step, dev_ms, launches=200, lead_ms=50.0):
    """Device ms per step of `launches` steps that follow at least `lead_ms` of the same steps without a pause: what a
    long run settles at, where a short one still sees clocks and caches ramp."""
    import torch
    lead = int(min(200000, max(1, lead_ms / max(dev_ms, 1e-4)))) + 1
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    for _ in range(lead):
        step()
    e0.record()
    for _ in range(launches):
        step()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / launches


def roofline(w, dev_ms):
    traffic = MEASURED_TRAFFIC.get(w.name)
    if w.bound == "hbm":
        achieved = w.bytes / (dev_ms * 1e-3) / 1e9
        return {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                "kernel": w.kernel, "algorithmic_bytes": w.bytes}
    achieved = w.ops / (dev_ms * 1e-3) / 1e12
    return {"bound": "mfma", "achieved": round(achieved, 2), "peak": I8_PEAK_TOPS, "unit": "TOP/s",
            "frac": round(achieved / I8_PEAK_TOPS, 4), "traffic": traffic,
            "kernel": w.kernel, "algorithmic_ops": w.ops}


def value_of(w, ms):
    if w.bound == "hbm":
        return w.bytes / (ms * 1e-3) / 1e9, "GB/s"
    return w.ops / (ms * 1e-3) / 1e12, "TOP/s"


def cpu_baseline(w, budget_s=8.0, one_thread_s=2.5):
    """Times the CPU oracle on a bounded sample of the same workload: all host threads, then one thread."""
    import oracle
    if w.cpu_sample is None:
        return None
    cores = min(oracle.num_threads(), int(os.environ.get("OMP_NUM_THREADS", "1024")))
    units, full, what = w.cpu_units
    fn, work = w.cpu_sample(oracle, units)
    t0 = time.perf_counter()
    fn()
    dt = time.perf_counter() - t0
    # grow the sample towards the time budget (at most the full workload), then repeat it to fill the budget
    scale = int(min(full // units, max(1, budget_s / max(dt, 1e-4))))
    if scale > 1:
        units *= scale
        fn, work = w.cpu_sample(oracle, units)
        t0 = time.perf_counter()
        fn()
        dt = time.perf_counter() - t0
    reps = int(max(1, min(5000, budget_s / max(dt, 1e-5))))
    t0 = time.perf_counter()
    for _ in range(reps):
        fn()
    dt = (time.perf_counter() - t0) / reps
    div = 1e9 if w.bound == "hbm" else 1e12
    unit = "GB/s" if w.bound == "hbm" else "TOP/s"
    val = work / dt / div
    sample = "full tensor" if units == full else "%d of %d %s" % (units, full, what)
    # a sample sized for the one-thread budget
    units1 = max(1, int(units * min(1.0, one_thread_s / max(dt * cores, 1e-6))))
    fn1, work1 = w.cpu_sample(oracle, units1)
    oracle.set_num_threads(1)
    try:
        t0 = time.perf_counter()
        n1 = 0
        while n1 < reps and (n1 == 0 or time.perf_counter() - t0 < one_thread_s):
            fn1()
            n1 += 1
        dt1 = (time.perf_counter() - t0) / n1
    finally:
        oracle.set_num_threads(cores)
    return {"value": round(val, 4), "unit": unit, "cores": cores, "kind": "port",
            "sample": "%s, %d repetition(s), %.3f s per repetition, %.1f s in total" % (sample, reps, dt, reps * dt),
            "value_one_thread": round(work1 / dt1 / div, 4)}


CACHE_BYTES = 256 << 20   # Infinity Cache of the part
ROTATION_BYTES = 4 * CACHE_BYTES  # what the buffer sets of a configuration add up to, at least
MAX_SETS = 2048


def footprint(w):
    """Bytes one buffer set of a workload occupies (what a step touches)."""
    return w.bytes if w.bytes else 1 << 30


def build_sets(name, rt, rotate):
    """The workload plus as many further copies on separate buffers as the rotation asks for: by default enough that
    their total is at least four times the Infinity Cache, so that a set has left the cache when its turn comes again."""
    w = MAKERS[name](rt)
    n = rotate if rotate > 0 else min(MAX_SETS, max(2, -(-ROTATION_BYTES // footprint(w))))
    sets = [w] + [MAKERS[name](rt) for _ in range(n - 1)]
    ring = itertools.cycle([x.step for x in sets])

    def step():
        next(ring)()
    return w, sets, step


def measure(name, rt, steps, warmup, rotate, cpu, extras=True):
    """One configuration: rotated eager timing (the figure of record), then the same-buffers and HIP-graph extras."""
    import torch
    w, sets, step = build_sets(name, rt, rotate)
    wall_ms, dev_ms = time_steps(step, steps, warmup)
    value, unit = value_of(w, wall_ms)
    rec = {"value": round(value, 2), "unit": unit, "dtype": w.dtype, "steps": steps, "warmup": warmup,
           "launch": "eager", "buffer_sets": len(sets), "buffer_bytes_total": len(sets) * footprint(w),
           "ms_per_step": round(wall_ms, 6), "device_ms_per_step": round(dev_ms, 6), "roofline": roofline(w, dev_ms)}
    if extras:
        _, same_ms = time_steps(w.step, steps, min(warmup, 5))
        _, graph_ms = time_steps(step, steps, 2, graph=True)
        steady_ms = steady_state(step, dev_ms)
        rec["extras"] = {"same_buffers_device_ms_per_step": round(same_ms, 6),
                         "same_buffers_frac": roofline(w, same_ms)["frac"],
                         "graph_device_ms_per_step": round(graph_ms, 6),
                         "graph_frac": roofline(w, graph_ms)["frac"],
                         "steady_state_device_ms_per_step": round(steady_ms, 6),
                         "steady_state_frac": roofline(w, steady_ms)["frac"]}
    if cpu:
        rec["cpu_baseline"] = cpu_baseline(w)
    del sets, step
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    return w, rec


# What bounds a configuration besides its roofline, said in the line itself.
NOTES = {
    "c1_fake_quantize": "0.8 MB per launch: launch-bound, not bandwidth-bound. An empty kernel of the same grid takes 2.6 us, the "
                        "kernel 2.5-3 us (graph_device_ms_per_step); the eager figure of record is the host's launch rate over "
                        "418 separate parameter blobs. A single launch of this size cannot reach 0.70 of the HBM peak (that would be 0.14 us).",
    "c3_mvn": "16 MB in one launch of 8.2 us, of which about 2.6 us are the launch floor; 0.70 of the HBM peak would be 3.0 us end to end.",
    "c4_conv": "7.4 GOP: about 1.5 us of MFMA time and 1.5 us of HBM time. Measured by early returns: an empty kernel of this grid "
               "1.6 us, the tile's loads back after 4.0 us, operands staged after 6.1 us, MFMAs + requantisation + stores 3.5 us "
               "(on this part vector-ALU work does not run under MFMAs of the same SIMD, so the PPE's 5.5 instructions per value add to the MFMA time).",
    "c5_matmul": "power-limited: the part runs this kernel at 1.83-1.86 GHz on random int8 operands (2.4 GHz on zeros), where the "
                 "dense int8 peak is 3.9 POP/s; frac is against the 5.0 POP/s of 2.4 GHz. mfma_calibration in this line is what "
                 "a bare loop of the same MFMA sustains on this part: about 0.98 of the peak on zeros, 0.68 on random int8 operands, "
                 "0.62 with this kernel's LDS fragment reads added.",
}

HEADLINE = "c5_matmul"
OTHER_CONFIGS = ["c1_fake_quantize", "c2_softmax", "c3_mvn", "c4_conv", "c5_dequantize", "c5_eltwise_add"]
EXTRA_CONFIGS = ["c5_nce_eltwise", "x_mvn6_layernorm", "x_activation_hswish", "x_mvn1_three_steps", "x_stem_conv", "x_small_plane_conv"]


def coissue_table(rt, iters=20000):
    """vpx_calib_coissue over every vector instruction kind and both MFMA shapes: nanoseconds per round when every wave
    multiplies, when every wave runs the vector instructions, when the two waves of a SIMD do one each, and when every
    wave does both (four vector instructions behind each MFMA).  One JSON line."""
    import torch
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    sink = torch.empty((cus * 8192,), device="cuda", dtype=torch.uint8)
    rows = []
    for wide in (1, 0):
        for kind, name in enumerate(rt.COISSUE_KINDS):
            ns = []
            for mode in range(4):
                rt.calib_coissue(kind, wide, mode, 200, sink)
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                rt.calib_coissue(kind, wide, mode, iters, sink)
                e1.record()
                torch.cuda.synchronize()
                ns.append(round(e0.elapsed_time(e1) * 1e6 / iters, 1))
            rows.append({"mfma": "32x32x32" if wide else "16x16x64", "valu": name, "ns_per_round_all_mfma": ns[0], "ns_per_round_all_valu": ns[1],
                         "ns_per_round_one_wave_each": ns[2], "ns_per_round_both_in_every_wave": ns[3]})
    print(json.dumps({"workload": "calib_coissue", "round": "16 int8 MFMAs per multiplying wave, 64 vector instructions per vector wave, two waves per SIMD",
                      "rows": rows}), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default=HEADLINE, choices=sorted(MAKERS) + ["calib_coissue"])
    ap.add_argument("--only", action="store_true", help="measure the headline workload only (no other_configs)")
    ap.add_argument("--extra", action="store_true", help="also measure the workloads beside the BASELINE configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baselines")
    ap.add_argument("--rotate", type=int, default=0, metavar="N",
                    help="number of separate buffer sets a workload cycles through (default 0: as many as make their "
                         "total reach 4 x the 256 MB Infinity Cache; 1: the same buffers every step)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this path runs on one GPU only (every kernel shards without exchange, so N GPUs would run N independent copies); "
                 "run it with --gpus 1")
    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    from vpux_plugin_amd import runtime as rt
    rt.lib()
    torch.cuda.set_device(0)

    if args.workload == "calib_coissue":
        coissue_table(rt)
        return
    t_start = time.perf_counter()
    w, rec = measure(args.workload, rt, args.steps, args.warmup, args.rotate, cpu=not args.no_cpu)
    texts = {w.name: {"description": w.desc, "note": NOTES.get(w.name)}}
    line = {
        "metric": METRIC, "value": rec["value"], "unit": rec["unit"], "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": rec["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": w.dtype, "data": "synthetic",
        "config": {"workload": w.name, "launch": "eager", "buffer_sets": rec["buffer_sets"],
                   "buffer_bytes_total": rec["buffer_bytes_total"]},
        "device_ms_per_step": rec["device_ms_per_step"],
        "roofline": rec["roofline"],
        "extras": rec.get("extras"),
        "traffic_source": "roofline.traffic: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of an earlier run (profiles/<workload>__*.md), not measured in this run",
    }
    if "cpu_baseline" in rec:
        line["cpu_baseline"] = rec["cpu_baseline"]
    if not args.only:
        others = {}
        names = [n for n in OTHER_CONFIGS + [HEADLINE] + (EXTRA_CONFIGS if args.extra else []) if n != args.workload]
        for name in names:
            steps = min(args.steps, 100) if name == "c5_matmul" else args.steps
            ow, r = measure(name, rt, steps, min(args.warmup, 10), args.rotate, cpu=not args.no_cpu)
            others[name] = r
            texts[name] = {"description": ow.desc, "note": NOTES.get(name)}
            sys.stderr.write("bench.py: %s done at %.0f s\n" % (name, time.perf_counter() - t_start))
            sys.stderr.flush()
        line["other_configs"] = others
        # configuration 5 end to end: the matmul, the dequantize of its result and the residual add, one after the other
        parts = {n: (rec if n == args.workload else others.get(n)) for n in ("c5_matmul", "c5_dequantize", "c5_eltwise_add")}
        if all(parts.values()):
            line["c5_chain"] = {"device_ms": round(sum(p["device_ms_per_step"] for p in parts.values()), 6),
                                "steady_state_device_ms": round(sum(p["extras"]["steady_state_device_ms_per_step"] for p in parts.values()), 6),
                                "parts": list(parts)}
        # what the part sustains today, beside the kernels it bounds: a plain copy for the HBM side (rotated like the
        # configurations), register-only loops of the int8 MFMA for the matrix side
        calib = {}
        hbm = {}
        cw, cr = measure("calib_copy", rt, args.steps, min(args.warmup, 10), args.rotate, cpu=False, extras=False)
        hbm["calib_copy"] = {"device_ms_per_step": cr["device_ms_per_step"], "achieved": cr["roofline"]["achieved"], "unit": "GB/s",
                               "frac_of_peak": cr["roofline"]["frac"], "buffer_sets": cr["buffer_sets"]}
        texts["calib_copy"] = {"description": cw.desc, "note": None}
        for name in ("calib_mfma_zero", "calib_mfma_random", "calib_mfma_random_lds"):
            cw = MAKERS[name](rt)
            _, ms = time_steps(cw.step, 50, 5)
            calib[name] = {"device_ms_per_step": round(ms, 6), "achieved": round(cw.ops / (ms * 1e-3) / 1e12, 1),
                           "unit": "TOP/s", "frac_of_peak": round(cw.ops / (ms * 1e-3) / 1e12 / I8_PEAK_TOPS, 4)}
            texts[name] = {"description": cw.desc, "note": None}
        line["hbm_calibration"] = hbm
        line["mfma_calibration"] = calib
    sys.stderr.write("bench.py: descriptions %s\n" % json.dumps(texts))
    sys.stderr.flush()
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
