/*
 * C ABI of the MI355X execution library for the vpux hot path: ACT-SHAVE software kernels and
 * the NCE/DPU quantized convolution / matmul with the integer PPE.
 *
 * Every entry point takes plain pointers and sizes, is asynchronous on the caller's HIP stream
 * (passed as void*, NULL = default stream), is safe to call from several host threads and owns
 * no caller buffer.  Return values follow the reference's compiler C API
 * (src/vpux_driver_compiler/include/npu_driver_compiler.h:94-103); the text of the last failure
 * on the calling thread is available from vpx_get_last_error (the role of
 * vclLogHandleGetString, npu_driver_compiler.h:287).
 */
#ifndef VPX_RUNTIME_H_
#define VPX_RUNTIME_H_

#include <stddef.h>
#include <stdint.h>

#include "vpx_sw_params.h"

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define VPX_API __attribute__((visibility("default")))
#else
#define VPX_API
#endif

/* SUCCESS, OUT_OF_MEMORY, INVALID_ARGUMENT, INVALID_NULL_HANDLE and UNKNOWN carry the numeric values of the
 * vcl_result_t members of the same name (npu_driver_compiler.h:94-103).  UNSUPPORTED_FEATURE is this library's
 * own (vcl_result_t has no such member; the value is the one Level Zero gives ZE_RESULT_ERROR_UNSUPPORTED_FEATURE,
 * the family vcl_result_t's numbering follows).  VCL_RESULT_ERROR_IO and VCL_RESULT_ERROR_INVALID_IR have no use
 * here (no file or IR handling) and are not mirrored. */
typedef enum vpx_result_t {
    VPX_RESULT_SUCCESS = 0,
    VPX_RESULT_ERROR_OUT_OF_MEMORY = 0x70000002,
    VPX_RESULT_ERROR_UNSUPPORTED_FEATURE = 0x78000003,
    VPX_RESULT_ERROR_INVALID_ARGUMENT = 0x78000004,
    VPX_RESULT_ERROR_INVALID_NULL_HANDLE = 0x78000005,
    VPX_RESULT_ERROR_UNKNOWN = 0x7ffffffe
} vpx_result_t;

/* Text of the last error returned to the calling thread ("" when none). */
VPX_API const char* vpx_get_last_error(void);

/* Library version: major << 16 | minor. */
VPX_API uint32_t vpx_get_version(void);

/* ------------------------------------------------------------------------------------------
 * Boundary A: ACT-SHAVE software kernels.
 *
 * Replaces the firmware call `entry(paramsPtr)` made by the ACT-SHAVE management kernel for a
 * VpuActKernelInvocation (src/vpux_compiler/src/dialect/VPUMI37XX/ops/act_kernel_invo.cpp:21-48).
 * `entry` is the kernel's ELF stem as chosen by SwKernelOp::getKernelInfo
 * (src/vpux_compiler/src/dialect/VPUIP/IR/ops/sw_kernel.cpp); `params` is the byte blob the
 * compiler serialises for that kernel (layout in vpx_sw_params.h) and is read on the host during
 * the call.  addrs[i] carries the 64-bit device address of memref i (inputs first, then outputs),
 * which on the NPU firmware relocation would have patched into MemRefData::dataAddr.  dims and
 * strides may be NULL: they are then read from the tail of the blob, where
 * KernelParamsOp::serialize appends them (VPUMI37XX/ops/kernel_params.cpp:19-73).
 * ------------------------------------------------------------------------------------------ */
typedef struct vpx_memref_addr_t {
    void* data;             /* device memory */
    const int32_t* dims;    /* host memory, innermost first, or NULL */
    const int64_t* strides; /* host memory, bits, innermost first, or NULL */
} vpx_memref_addr_t;
/* A memref whose MemRefData has isStatic = 0 (a bounded dynamic shape; `softmax` / `softmaxFp32` with the
 * [axis, padSize], [SoftmaxModeDynamic, rank] form of their parameters, update_sw_kernel_params.cpp:48-55): the blob's
 * own dims and strides are the bounds, and `dims` / `strides` above must point at DEVICE memory holding the live
 * values -- what MemRefData::dimsAddr / stridesAddr point at on the NPU, written by whatever produced the shape.
 * They are read by the kernel, not during the call; elements outside the live shape are left untouched.  The SHAVE
 * kernel's source is not public: that the live strides are taken as found (compact over the live shape or those of
 * the bound buffer, whichever the producer wrote) is this library's reading. */

VPX_API int vpx_sw_kernel_launch(const char* entry, const void* params, size_t params_size,
                                 const vpx_memref_addr_t* addrs, uint32_t num_addrs, void* stream);

/* The same launch for callers that cannot allocate device memory (code under HIP graph capture on a stream the
 * library has not seen, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference.  Kernels that need scratch memory (mvn1 / mvn6 chunk moments, the MVN-1 decomposition's partial sums,
 * dynamic_quantize's range pass, per-axis quantize / dequantize tables) take it from one fixed array of
 * VPX_NOALLOC_SCRATCH_BYTES in device memory that the library holds on every device it runs on; a launch that
 * would need more returns VPX_RESULT_ERROR_OUT_OF_MEMORY and enqueues nothing (the library keeps a further 128 KiB of
 * counters behind it for kernels whose workgroups meet inside one launch).  The call performs no hipMalloc /
 * hipFree.  All calls on one device share that array and it keeps the previous call's contents: calls through
 * this entry point that may overlap on one device (different streams, or different threads) race; order them on
 * one stream.  Arguments, results and errors are otherwise those of vpx_sw_kernel_launch. */
#define VPX_NOALLOC_SCRATCH_BYTES (4u << 20)
VPX_API int vpx_sw_kernel_launch_noalloc(const char* entry, const void* params, size_t params_size,
                                         const vpx_memref_addr_t* addrs, uint32_t num_addrs, void* stream);

/* Scratch memory of vpx_sw_kernel_launch and vpx_nce_task (no counterpart in the reference, whose kernels get
 * their buffers from the compiler's memory scheduler).  The library keeps one block per (device, stream handle) and
 * grows it with hipMalloc when a launch needs more: mvn1 / mvn6 / mvn1_sum with several chunks per group (12 bytes
 * per 4096 values), dynamic_quantize, per-axis quantize / dequantize tables, and an NCE task with a non-zero
 * activation zero point, unsigned weights or a weight zero point (4 bytes per output channel and per output
 * position, plus a signed copy of unsigned weights).  A launch on a capturing stream that would have to grow the
 * block returns VPX_RESULT_ERROR_UNSUPPORTED_FEATURE instead.
 * vpx_workspace_reserve grows the block of `stream` on the current device to at least `bytes` ahead of time (before
 * a capture, or to keep hipMalloc out of a serving loop).  vpx_workspace_release waits for the stream, then frees
 * its block, the blocks it outgrew and the per-axis tables cached for it; the next launch allocates afresh.
 * Blocks are keyed by the stream HANDLE: release before destroying a stream (a new stream may get the same
 * handle), and do not run one handle's work concurrently from several threads' per-thread streams.  A graph captured
 * on a stream records the addresses of that stream's block, counter area and cached tables: destroy such graphs
 * before releasing the stream's workspace (and replay them on no other stream).  Every block is freed even when one
 * hipFree fails; the first failure is what the call returns. */
VPX_API int vpx_workspace_reserve(void* stream, size_t bytes);
VPX_API int vpx_workspace_release(void* stream);

/* 1 when `entry` names a kernel this library implements, else 0. */
VPX_API int vpx_sw_kernel_supported(const char* entry);

/* Number of implemented entries; name of entry i (NULL when out of range). */
VPX_API uint32_t vpx_sw_kernel_count(void);
VPX_API const char* vpx_sw_kernel_name(uint32_t i);

/* ------------------------------------------------------------------------------------------
 * Boundary B: NCE cluster task (DPU).
 *
 * Replaces one VPUIP.NCEClusterTask of task_type CONV
 * (src/vpux_compiler/tblgen/vpux/compiler/dialect/VPUIP/ops.td:651-750), the form
 * VPU.NCE.Convolution and VPU.NCE.MatMul lower to (tblgen/.../VPU/ops.td:138-357).
 *   input   NHWC  [N][H][W][IC]   u8 or i8
 *   weights OYXI  [OC][KY][KX][IC] u8 or i8, one dense set per output channel
 *   weight_table [OC][4] int32 as built by NCESparsity::getWeightsTable
 *       (src/vpux_compiler/src/dialect/VPU/utils/nce_sparsity.cpp:195-231): word 2 holds
 *       mult << 16 | shift << 8, word 3 the int32 bias
 *       (src/vpux_compiler/src/NPU37XX/dialect/VPU/impl/nce_sparsity_converters.cpp:14-41);
 *       words 0 and 1 (weight / sparsity pointers) are NPU addresses and are ignored
 *   output  NHWC  [N][OH][OW][OC] u8 or i8
 * input and output may be strided views of larger tensors (input_strides / output_strides below).
 * A matmul A[M][K] x B[N][K] -> [M][N] is the task N=1, H=M, W=1, IC=K, OC=N, 1x1 kernel.
 *
 * task_type ELTWISE (the quantized residual add of a network): `weights` is the second input,
 * same shape and layout as `input`, zero point zp_w; OC = IC; weight_table, kernel_* are not used.
 *   acc = (in1 - zp_in) * in1_quant_mult +/- (in2 - zp_w) * in2_quant_mult       (int32)
 *   t = acc * quant_mult, PReLU stage as above, r = round_half_even(t / 2^quant_shift) + zp_out, clamp
 * ("input1 * MULT1 --> + --> * MULT_OUT >> SHIFT_OUT", quantization.cpp:461-462).
 * Arithmetic: acc = sum (in - zp_in) * (w - zp_w) over the taps inside the image (padding adds 0),
 * then the integer PPE in the order the compiler programs it
 * (src/vpux_compiler/src/NPU40XX/dialect/VPUIPDPU/transforms/passes/expand_dpu_config/
 * expand_dpu_config_invariant_ppe.cpp:322-380): t = (acc + bias) * mult; if t < 0 then
 * t *= prelu_mult and shift += prelu_shift; r = round_half_even(t / 2^shift) + zp_out;
 * clamp to [clamp_low, clamp_high]; saturate to the output type.
 *
 * output_type VPX_NN_FP16 (CONV and ELTWISE tasks; "INT32 s17.15 fixed-point convert to FP16",
 * src/vpux_compiler/src/dialect/VPUMI37XX/ops/external/runtime_dpu_parser_imports.cpp.inc:546-574): the same
 * pipeline with the round stage keeping 15 fractional bits, fx = round_half_even(t / 2^(shift - 15)) saturated to
 * 32 bits; the output is fx * 2^-15 narrowed to fp16 with one round-to-nearest-even (infinity from 65520 up).
 * The weight table then holds mult / shift of w_scale * in_scale (no output scale, nce_sparsity.cpp:112-126),
 * zp_out must be 0, clamp_low is not used and clamp_high packs two fp16 bounds as 0xllllhhhh
 * (include/vpux/compiler/dialect/VPU/utils/ppe_utils.hpp:36-87; INT32_MAX = no clamp), as
 * vpx_retrieve_ppe_int produces them for a float output.
 * ------------------------------------------------------------------------------------------ */

/* VPUIP::NCETaskType (tblgen/.../VPUIP/attributes.td:56-70) */
typedef enum vpx_nce_task_type_t { VPX_NCE_CONV = 0, VPX_NCE_ELTWISE = 4 } vpx_nce_task_type_t;

/* VPU::EltwiseType values the ELTWISE task implements (tblgen/.../VPU/attributes.td:237-252) */
typedef enum vpx_eltwise_type_t { VPX_ELTWISE_ADD = 0, VPX_ELTWISE_SUBTRACT = 1 } vpx_eltwise_type_t;

/* VPU::PPEMode values used by the integer pipeline (tblgen/.../VPU/attributes.td:327-369) */
typedef enum vpx_ppe_mode_t {
    VPX_PPE_NOOP = 3,
    VPX_PPE_LRELU = 13,
    VPX_PPE_LRELUX = 14,
    VPX_PPE_LPRELU = 15
} vpx_ppe_mode_t;

/* The PPEIntAttr fields the integer convolution path consumes (attributes.td:399-430). */
typedef struct vpx_ppe_int_t {
    int32_t mode; /* vpx_ppe_mode_t */
    int32_t clamp_low;
    int32_t clamp_high;
    int32_t lrelu_mult;
    int32_t lrelu_shift;
    /* ELTWISE tasks only (a CONV task takes its scale from the weight table and ignores these):
     * the per-tensor output and input multipliers EltwiseQuantizationApproximation produces
     * (src/vpux_compiler/src/utils/quantization.cpp:455-516, ppe_factory.cpp:300-310) */
    int32_t quant_mult;
    int32_t quant_shift;
    int32_t in1_quant_mult;
    int32_t in2_quant_mult;
} vpx_ppe_int_t;

typedef struct vpx_nce_task_t {
    int32_t task_type; /* vpx_nce_task_type_t */
    const void* input;
    const void* weights;
    const int32_t* weight_table;
    void* output;
    int32_t input_type;   /* VPX_NN_U8 or VPX_NN_I8 */
    int32_t weights_type; /* VPX_NN_U8 or VPX_NN_I8 */
    int32_t output_type;  /* VPX_NN_U8, VPX_NN_I8, or VPX_NN_FP16 */
    int64_t N, H, W, IC;  /* input shape */
    int64_t OC;
    int32_t kernel_size[2];    /* KY, KX */
    int32_t kernel_strides[2]; /* SY, SX */
    int32_t kernel_padding[4]; /* left, right, top, bottom (VPU_PaddingAttr order) */
    int32_t zp_in, zp_w, zp_out;
    vpx_ppe_int_t ppe;
    int32_t eltwise_type; /* vpx_eltwise_type_t, ELTWISE tasks only */
    /* VPU.NCE.MatMul's group dimension (tblgen/vpux/compiler/dialect/VPU/ops.td:228-357: input [G,1,K,M,1],
     * weights [G,N,K,1,1], weight table [G,N,1,1,4], all GNHWC in memory): `groups` independent CONV tasks of the
     * shape above whose inputs, weights, weight tables and outputs lie one after the other, densely, behind the four
     * pointers.  0 and 1 both mean a single task.  A matmul the MFMA matmul kernel serves is one launch for all
     * groups (the group on the grid's second dimension). */
    int32_t groups;
    /* Operand strides in ELEMENTS, in the order N, H, W, C: the strides of the operand's memref
     * (src/vpux_compiler/tblgen/vpux/compiler/dialect/VPUIP/ops.td:651-700).  The NPU writes a task's output into the
     * buffer its bit strides describe -- the ODU's te_dim_z is stride_x / stride_z, the channel pitch of the BUFFER, not
     * the task's channel count (src/vpux_compiler/src/dialect/VPUMI37XX/ops/external/runtime_dpu_parser_imports.cpp.inc:
     * 1031-1090) -- and reads its input out of the parent tensor's dimensions (:850-852); that is how the compiler
     * elides Concat (a task writes channels [c0, c0 + OC) of a wider tensor) and tiles a layer over H or W (a task
     * reads a window of a larger tensor).  Here the pointer names the operand's first element and the strides say how
     * far apart its images, rows and pixels lie.  All four zero = dense NHWC (the default: every field an existing
     * caller leaves zeroed).  Otherwise C must be 1 and the others must keep the operand's elements apart, outermost
     * largest (W >= channels, H >= (width - 1) * W + channels, N likewise).  `weights_strides` describes the second
     * input of an ELTWISE task; the weights of a CONV task are always dense.  Strides need groups <= 1.
     * The MFMA kernels read 16 bytes at a time: an input whose base address or strides are not multiples of 16 bytes
     * runs on the general kernel (correct, slow).  Outputs may sit anywhere. */
    int64_t input_strides[4];
    int64_t weights_strides[4];
    int64_t output_strides[4];
} vpx_nce_task_t;

VPX_API int vpx_nce_task(const vpx_nce_task_t* task, void* stream);

/* Testing and tuning hook (no counterpart in the reference): overrides how vpx_nce_task picks its device kernel.
 * `knob` is one of "VPX_NCE_KERNEL" (naive | gather | conv), "VPX_GEMM_TILE" (128 | 256), "VPX_GEMM_WAVES" (4 | 8),
 * "VPX_GEMM_REGB" (on | wide | off: the weights-in-registers matmul for a K of 64, 128 or 256, which by itself serves layers of
 * many rows; wide: with as many channel blocks per wave as it otherwise takes from some hundreds of thousands of rows on),
 * "VPX_GEMM_PINGPONG" (on: the two waves of a SIMD take turns at the MFMAs of the large matmul tile; measured slower, off by default),
 * "VPX_CONV_KERNEL" (regw | tile | stream), "VPX_CONV_ROWS" (n), "VPX_CONV_COLS" (n), "VPX_CONV_WAVES" (4 | 8), "VPX_STREAM_KSPLIT" (off: the streamed-weights
 * convolution kernel gives every wave a 32 x 32 tile also on small planes, instead of splitting K over the waves of a group),
 * "VPX_MVN_FUSED" (off: long MVN groups take
 * the two-launch kernels; nowait: the one-launch kernel's workgroups do not wait for each other and each recomputes its
 * group's statistics, the path taken when they are not all resident), "VPX_CALIB_BLOCKS" (n: workgroups of
 * vpx_calib_mfma_i8, by default one per compute unit); `value` NULL or "" restores the default.
 * Environment variables of the same names give the initial values; they are read once, at the first NCE task or the
 * first call of this function, never during a launch.  Process-wide; results do not depend on any of them. */
VPX_API int vpx_set_tuning(const char* knob, const char* value);

/* Measurement aid (no counterpart in the reference): a loop of `v_mfma_i32_32x32x32_i8` alone on every compute unit,
 * eight waves of 128 x 64 register tiles as in the matmul kernel, sixteen MFMAs per wave and iteration; with
 * `fragment_reads` non-zero each wave also reads the twelve 16-byte LDS fragments those MFMAs consume.  It shows what the
 * part sustains on the given operand bytes before anything comes from global memory (the shader clock depends on the
 * data), which is what the matmul's fraction of the nominal peak has to be read against.
 * `operands`: 64 KiB of device memory, copied to LDS by every workgroup; `sink`: 8 KiB per compute unit of device memory
 * that receives the accumulators; `*ops` (may be NULL) is set to the integer operations the launch performs. */
VPX_API int vpx_calib_mfma_i8(const void* operands, void* sink, int iters, int fragment_reads, int64_t* ops, void* stream);

/* Measurement aid (no counterpart in the reference): whether vector-ALU instructions of one wave run under the MFMAs of
 * the other wave of its SIMD.  One workgroup of eight waves (two per SIMD) per compute unit; a round is sixteen int8 MFMAs
 * (`wide_mfma` non-zero: 32x32x32, else 16x16x64) for a wave that multiplies and sixty-four instructions of `valu_kind`
 * (0 v_fma_f64, 1 v_fma_f32, 2 v_add_u32, 3 v_mul_lo_u32, 4 v_mad_u64_u32, 5 v_cvt_f64_i32) for a wave that does not.
 * `mode` 0: every wave multiplies; 1: every wave runs the vector instructions; 2: waves 0-3 multiply while waves 4-7 run
 * the vector instructions; 3: every wave does both, four vector instructions behind each MFMA.  `sink`: 8 KiB of device
 * memory per compute unit.  The caller times the launch; time / iters is the length of a round. */
VPX_API int vpx_calib_coissue(int valu_kind, int wide_mfma, int mode, int iters, void* sink, void* stream);

/* Name of the device kernel the last successful vpx_nce_task on this thread dispatched to
 * ("" before the first); for tests and profiles. */
VPX_API const char* vpx_nce_last_kernel(void);

#ifdef __cplusplus
}
#endif
#endif
