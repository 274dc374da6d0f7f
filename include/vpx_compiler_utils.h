/*
 * Host-side helpers that produce what the execution entry points of vpx_runtime.h consume, with
 * the arithmetic of the reference compiler: scale approximation, weights-table words, the integer
 * PPE attribute of a fused post-op, and the ACT-SHAVE parameter blobs.  They exist so that tests,
 * benchmarks and integrators without the compiler at hand can build byte-identical inputs.
 */
#ifndef VPX_COMPILER_UTILS_H_
#define VPX_COMPILER_UTILS_H_

#include <stddef.h>
#include <stdint.h>

#include "vpx_runtime.h"

#ifdef __cplusplus
extern "C" {
#endif

/* approximate<>(bits, target): mantissa/exponent split of a real scale into mult * 2^-shift
 * (src/vpux_compiler/include/vpux/compiler/utils/quantization.hpp:65-78).  bits = 15 is
 * QuantizationApproximation (src/vpux_compiler/src/utils/quantization.cpp:426-433), bits = 11 is
 * PReLUApproximation (:530-540).  A non-zero post_shift is reported, as the reference throws on it,
 * with VPX_RESULT_ERROR_INVALID_ARGUMENT. */
VPX_API int vpx_approximate(int bits, double target, int64_t* mult, int64_t* shift, int64_t* post_shift);

/* EltwiseQuantizationApproximation (quantization.cpp:455-516): input multipliers aligned to a
 * common shift that is folded into the output shift.  eltwise_type: 0 ADD, 1 SUBTRACT, 2 MULTIPLY. */
VPX_API int vpx_eltwise_quantization_approximation(double in1_scale, double in2_scale, double out_scale,
                                                   int eltwise_type, int64_t* in1_mult, int64_t* in2_mult,
                                                   int64_t* out_mult, int64_t* out_shift);

/* arch37xx::getScale / getBias for quantized input
 * (src/vpux_compiler/src/NPU37XX/dialect/VPU/impl/nce_sparsity_converters.cpp:14-41). */
VPX_API int32_t vpx_wt_get_scale(uint8_t shift, int16_t mult);
VPX_API int vpx_wt_get_bias(double real_val, int32_t* bias);

/* NCESparsity::getWeightsTable for quantized input and output
 * (src/vpux_compiler/src/dialect/VPU/utils/nce_sparsity.cpp:36-136,195-231, getRescaledBias :317-346).
 *   in_scale, out_scale : per-tensor scales; weight_scales[n_weight_scales] (1 or OC entries)
 *   bias : OC real-valued biases or NULL
 *   weights_ptr / weights_ptr_step, sparsity_ptr / sparsity_ptr_step : table words 0 and 1
 *   table : OC * 4 int32 */
VPX_API int vpx_get_weights_table(double in_scale, double out_scale, const double* weight_scales,
                                  size_t n_weight_scales, const double* bias, int64_t OC, int32_t weights_ptr,
                                  int32_t weights_ptr_step, int32_t sparsity_ptr, int32_t sparsity_ptr_step,
                                  int32_t* table);

/* PPE attribute of a convolution / matmul with a fused post-op on a quantized or float output
 * (PpeFactory::retrieveNonEltwisePPEAttribute and its callbacks,
 * src/vpux_compiler/src/NPU37XX/dialect/VPU/impl/ppe_factory.cpp:123-257). */
typedef enum vpx_post_op_t { VPX_POSTOP_NONE = 0, VPX_POSTOP_RELU = 1, VPX_POSTOP_CLAMP = 2, VPX_POSTOP_LEAKY_RELU = 3 } vpx_post_op_t;
typedef struct vpx_quant_type_t {
    int32_t is_quantized; /* 0: float output (clamps stay at the int32 limits) */
    double scale;
    int64_t zero_point;
    int64_t storage_min, storage_max;
} vpx_quant_type_t;
VPX_API int vpx_retrieve_ppe_int(int post_op, double param0, double param1, const vpx_quant_type_t* out_type,
                                 vpx_ppe_int_t* ppe);

/* generateVpuipSoftmaxAttr (src/vpux_compiler/src/dialect/VPUIP/transforms/passes/
 * update_sw_kernel_params.cpp:36-147).  dims (int32), in/out strides (in elements), all innermost
 * first; axis counted from the innermost memory dimension.  words must hold 2 + 2*16 entries;
 * *n_words receives the number written. */
VPX_API int vpx_generate_softmax_attr(uint32_t ndims, const int64_t* dims, const int64_t* in_strides,
                                      const int64_t* out_strides, int64_t axis, int64_t pad_size, uint64_t* words,
                                      uint32_t* n_words);

/* getQuantParamsAttr / packAsFpIntoU64 (src/vpux_compiler/src/dialect/VPUIP/IR/ops/sw_kernel.cpp:97-163):
 * words = [n, packed scales..., packed zero points...], packed as fp16 (float_type VPX_NN_FP16, four
 * per word) or fp32 (two per word).  words must hold 1 + 2*ceil(n/2) entries. */
VPX_API int vpx_get_quant_params_attr(const double* scales, const int64_t* zero_points, uint32_t n,
                                      uint32_t float_type, uint64_t* words, uint32_t* n_words);

/* KernelParamsSerializer::createKernelParams + KernelParamsOp::serialize
 * (src/vpux_compiler/src/dialect/VPUMI37XX/kernel_params_utils.cpp:228-310,
 *  src/vpux_compiler/src/dialect/VPUMI37XX/ops/kernel_params.cpp:19-73):
 * MemRefData per operand (inputs then outputs), attribute bytes, then all input dims, input strides,
 * output dims, output strides.  dims/strides are given innermost first, strides in bits.
 * Returns the blob size through *blob_size; blob may be NULL to query it. */
typedef struct vpx_tensor_desc_t {
    uint32_t num_dims;
    const int32_t* dims;    /* innermost first */
    const int64_t* strides; /* bits, innermost first */
    uint32_t data_type;     /* vpx_data_type_t */
    uint64_t dims_order;    /* vpx_nd_order_t */
    uint32_t location;      /* vpx_location_t */
    uint32_t dynamic_shape; /* non-zero: dims / strides are upper bounds, MemRefData::isStatic is written as 0 and the live
                               values are read from device memory when the kernel runs (softmax only) */
} vpx_tensor_desc_t;
VPX_API int vpx_create_kernel_params(const vpx_tensor_desc_t* inputs, uint32_t n_inputs,
                                     const vpx_tensor_desc_t* outputs, uint32_t n_outputs, const void* attrs,
                                     size_t attrs_size, void* blob, size_t* blob_size);

/* SwKernelOp::getKernelInfo (src/vpux_compiler/src/dialect/VPUIP/IR/ops/sw_kernel.cpp:640-1850) for the operators this
 * library serves: from the name of a VPU operator ("SoftMax", "MVN", "MVN1Sum", "MVN1MeanVar", "MVN1Normalize", "MVN6",
 * "FakeQuantize", "Quantize", "Dequantize", "DynamicQuantize", "DynamicDequantize", "Convert", "Add", "Subtract",
 * "Multiply", "Divide", "Minimum", "Maximum", "PRelu", "ReLU", "LeakyRelu", "Clamp", "Negative", "Abs", "HSwish",
 * "HSigmoid", "HardSigmoid", "Sigmoid", "Tanh", "Exp", "Sqrt", "Log", "Floor", "Ceiling", "Sign", "Elu", "Selu", "Swish",
 * "Mish", "SoftPlus", "Gelu", "Erf") and its attributes to the firmware entry name and the serialised attribute
 * bytes that vpx_create_kernel_params appends to the MemRefData records: int64 per integer or boolean attribute (a
 * true i1 sign-extends to -1), float32 per float attribute, arrays flattened (kernel_params_utils.cpp:104-125).
 * `input` is the first operand: its element type selects softmaxFp32 and the packing of quantization parameters
 * (for Dequantize pass the OUTPUT tensor, whose float type packs them), its order maps logical axes to the
 * innermost-first memory positions the kernels take (computeReverseMemDim, sw_kernel.cpp:29-40).
 * Only the fields the operator reads are looked at.  attr_bytes may be NULL to query *attr_size. */
typedef struct vpx_op_attrs_t {
    int64_t axis_ind;            /* SoftMax: logical axis, negative counts from the end */
    int64_t pad_size;            /* SoftMax: trailing elements of the axis to ignore */
    int32_t across_channels;     /* MVN, MVN1Sum, MVN1MeanVar, MVN1Normalize */
    int32_t normalize_variance;  /* the MVN family and MVN6 */
    float eps;                   /* MVN, MVN1MeanVar, MVN6 */
    int32_t eps_mode;            /* MVN6: 0 inside the square root, 1 outside */
    const int64_t* axes;         /* MVN6: logical axes */
    uint32_t num_axes;
    int32_t has_scale, has_bias; /* MVN6: optional operands present */
    const int64_t* orig_shape;   /* MVN1MeanVar: the four dimensions of the tensor being normalised */
    int64_t group_c;             /* MVN1MeanVar: channels per group after the internal reshape (1 without one) */
    int64_t levels;              /* FakeQuantize */
    const double* scales;        /* Quantize / Dequantize: parameters of the quantized element type */
    const int64_t* zero_points;
    uint32_t num_quant_params;
    float param0, param1;        /* LeakyRelu slope; Clamp min, max; Elu x; Selu alpha, lambda; Swish beta;
                                    HardSigmoid alpha, beta */
} vpx_op_attrs_t;
VPX_API int vpx_get_kernel_info(const char* op, const vpx_op_attrs_t* attrs, const vpx_tensor_desc_t* input, char* entry,
                                size_t entry_capacity, void* attr_bytes, size_t* attr_size);

/* RNE fp32 -> fp16 bit pattern and back, the rule of vpux::type::float16
 * (src/vpux_utils/src/core/type/float16.cpp:30-144). */
VPX_API uint16_t vpx_float_to_half_bits(float v);
VPX_API float vpx_half_bits_to_float(uint16_t bits);

#ifdef __cplusplus
}
#endif
#endif
