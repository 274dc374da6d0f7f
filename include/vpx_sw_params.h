/*
 * Byte-level description of the parameter blob an ACT-SHAVE software kernel receives.
 *
 * The layouts here are an ABI shared with the compiler that serialises the blob, so field
 * names, order, widths and enum values are fixed by the reference:
 *   - MemRefData, DataType, NDOrder codes, Location, INT64_MAX memref-list delimiter:
 *       sw_runtime_kernels/kernels/inc/common_types.h:18-151
 *   - blob = MemRefData[inputs..., outputs...] | attributes | input dims | input strides |
 *            output dims | output strides:
 *       src/vpux_compiler/src/dialect/VPUMI37XX/kernel_params_utils.cpp:228-310 and
 *       src/vpux_compiler/src/dialect/VPUMI37XX/ops/kernel_params.cpp:19-73
 *   - attribute encoding (integer/bool -> int64 sign-extended, float -> float32, arrays flattened):
 *       kernel_params_utils.cpp:104-125
 *
 * On the NPU the 32-bit *Addr fields are patched by firmware relocation.  A GPU pointer does not
 * fit, so the launcher takes the addresses in a side table (vpx_memref_addr_t in vpx_runtime.h)
 * and leaves the *Addr fields untouched.
 */
#ifndef VPX_SW_PARAMS_H_
#define VPX_SW_PARAMS_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { VPX_MAX_ND_DIMS = 15, VPX_MAX_KERNEL_INPUTS = 8, VPX_MAX_KERNEL_OUTPUTS = 8 };

/* sw_params::DataType (common_types.h:24-45) */
typedef enum vpx_data_type_t {
    VPX_NN_FP64 = 0,
    VPX_NN_FP32 = 1,
    VPX_NN_FP16 = 2,
    VPX_NN_FP8 = 3,
    VPX_NN_U64 = 4,
    VPX_NN_U32 = 5,
    VPX_NN_U16 = 6,
    VPX_NN_U8 = 7,
    VPX_NN_I64 = 8,
    VPX_NN_I32 = 9,
    VPX_NN_I16 = 10,
    VPX_NN_I8 = 11,
    VPX_NN_I4 = 12,
    VPX_NN_I2 = 13,
    VPX_NN_BIN = 14,
    VPX_NN_BF16 = 15,
    VPX_NN_UNDEFINED = 16,
    VPX_NN_U4 = 17
} vpx_data_type_t;

/* Packed permutation ("inverted code" of the compiler's DimsOrder, src/vpux_compiler/src/core/
 * attributes/dims_order.cpp:391-401): reading hex digits from the least significant one gives the
 * logical dimension (index + 1) stored outermost ... innermost. */
typedef uint64_t vpx_nd_order_t;
#define VPX_ORDER_NCHW 0x4321ull
#define VPX_ORDER_NHWC 0x2431ull
#define VPX_ORDER_NCWH 0x3421ull
#define VPX_ORDER_NWHC 0x2341ull
#define VPX_ORDER_CHW 0x321ull
#define VPX_ORDER_HWC 0x132ull
#define VPX_ORDER_NC 0x21ull
#define VPX_ORDER_C 0x1ull

/* sw_params::Location (common_types.h:75) */
typedef enum vpx_location_t { VPX_LOC_NONE = 0, VPX_LOC_DDR = 1, VPX_LOC_NN_CMX = 2 } vpx_location_t;

#pragma pack(push, 1)
/* sw_params::MemRefData (common_types.h:85-101), 36 bytes */
typedef struct vpx_memref_data_t {
    uint32_t dataAddr;    /* NPU window offset; ignored here, see vpx_memref_addr_t */
    uint32_t isStatic;    /* 1: static shape */
    uint32_t numDims;
    uint32_t dimsAddr;    /* -> int32 dims[numDims], innermost first */
    uint32_t stridesAddr; /* -> int64 strides[numDims] in BITS, innermost first */
    uint32_t dataType;    /* vpx_data_type_t */
    uint64_t dimsOrder;   /* vpx_nd_order_t */
    uint32_t location;    /* vpx_location_t */
} vpx_memref_data_t;
#pragma pack(pop)

/* A memref list of a kernel with optional operands ends with this 64-bit word (common_types.h:141-151). */
#define VPX_MEMREF_LIST_END INT64_MAX

/* Softmax "mode" word written by the compiler's parameter update
 * (src/vpux_compiler/src/dialect/VPUIP/transforms/passes/update_sw_kernel_params.cpp:21-26). */
typedef enum vpx_softmax_mode_t {
    VPX_SOFTMAX_DYNAMIC = 0,
    VPX_SOFTMAX_INNER = 1,
    VPX_SOFTMAX_INNER_HARDCODED = 2,
    VPX_SOFTMAX_OUTER = 3
} vpx_softmax_mode_t;

/*
 * Attribute area per kernel entry (bytes that follow the MemRefData array):
 *
 *   convert        in, out                           | (none)
 *   eltwise_add    in1, in2, out                     | (none)      (also _sub _mul _min _max _div)
 *   fake_quantize  in, inLow, inHigh, outLow, outHigh, out | int64 levels
 *   quantize       in, out                           | int64 n; uint64 scales[ceil(n/P)]; uint64 zeroPoints[ceil(n/P)]
 *   dequantize     in, out                           | same as quantize
 *       scales and zero points are both stored as floating point values of the non-quantized
 *       operand's type, P = 4 (fp16) or 2 (fp32) per 64-bit word, zero padded
 *       (src/vpux_compiler/src/dialect/VPUIP/IR/ops/sw_kernel.cpp:97-163)
 *   mvn1           in, out                           | int64 acrossChannels; int64 normalizeVariance; float eps
 *       a true boolean attribute is the int64 value -1 (sign-extended i1)
 *   softmax        in, out                           | either int64 axis (counted from the innermost memory
 *       dimension), int64 padSize (sw_kernel.cpp:730-745), or the packed form
 *       uint64 w[2 + 2*ndims]: w0 = axis | padSize << 32, w1 = mode | ndims << 32, then per dimension
 *       (innermost first) dim | dim << 32 and inStride | outStride << 32 in elements
 *       (update_sw_kernel_params.cpp:36-147)
 *   mvn1_sum       in, sums                          | int64 acrossChannels; int64 normalizeVariance
 *       sums: f32 [N, C or 1, parts, 2 or 1] in NHWC order = {sum, sum of squares} (sw_kernel.cpp:964-968;
 *       src/vpux_compiler/tblgen/vpux/compiler/dialect/VPU/ops.td:3659-3715)
 *   mvn1_mean_var  sums, meanVar                     | int64 origShape[4]; int64 acrossChannels; int64 normalizeVariance;
 *       int64 groupC; float eps (sw_kernel.cpp:969-981); meanVar: f16/f32 [N, C or 1, 1, 2 or 1] in NHWC order
 *       = {mean, 1/sqrt(var + eps)}
 *   mvn1_norm      in, meanVar, out                  | int64 acrossChannels; int64 normalizeVariance (sw_kernel.cpp:982-986)
 *   mvn6           in, [scale], [bias], out, marker  | the memref list ends at an INT64_MIN word, which opens the
 *       attributes: int64 marker; int64 mask (bit 0 input, 1 scale, 2 bias, 3 output); int64 normalizeVariance;
 *       int64 epsMode (0 inside, 1 outside the square root); float eps; int64 numAxes; int64 memAxes[numAxes]
 *       (axes counted from the innermost memory dimension; sw_kernel.cpp:164-185, 987-1004)
 *   activation_<name>, leaky_relu_fp16  in, out      | the op's float attributes as 32-bit floats, in order:
 *       leaky_relu_fp16 {negative_slope}; activation_clamp {min, max}; activation_hardsigmoid {alpha, beta};
 *       activation_elu {alpha}; activation_selu {alpha, lambda}; activation_swish {beta}; none for relu, negative,
 *       abs, hswish, hsigmoid, sigmoid, tanh, exp, sqrt, log, floor, ceil, sign, mish, softplus, gelu, erf
 *       (sw_kernel.cpp:650-941, 1266-1285, 1689-1845)
 *   dynamic_quantize    in, out, scale, zeroPoint    | (none); f32 in, u8 out, one f32 scale and one u8 zero point, all three
 *       written by the kernel (sw_kernel.cpp:1177-1179; arithmetic of ONNX DynamicQuantizeLinear)
 *   dynamic_dequantize  in, scale, [zeroPoint], out  | int64 INT64_MAX (ends the memref list; sw_kernel.cpp:1180-1183,
 *       sw_runtime_kernels/kernels/inc/common_types.h:141-151); out = (in - zeroPoint) * scale, scale and
 *       zero point broadcast onto the input
 *   prelu_fp16     in, slope, out                    | (none); slope broadcasts NUMPY-style (sw_kernel.cpp:1102-1104)
 */

#ifdef __cplusplus
}
#endif
#endif
