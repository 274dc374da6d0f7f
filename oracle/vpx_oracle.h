/*
 * CPU oracle for the vpux hot path -- TEST INFRASTRUCTURE ONLY.
 *
 * This library restates, in plain C, the arithmetic of the reference's hot
 * path (SHAVE software kernels and the NCE/DPU integer pipeline).  It exists
 * to check the HIP kernels and to be timed as the CPU baseline.  Nothing in
 * the product library links, loads or calls it.
 *
 * All reference citations are relative to the reference checkout root.
 *
 * Pinning status (what fixes each function besides its own formula):
 *   orc_f32_to_f16 / orc_f16_to_f32 : reference unit-test bit patterns
 *       (tests/unit/vpux_utils/core/float16_tests.cpp:9-106), the compiled
 *       reference float16.cpp (oracle/_ref), numpy float16.
 *   orc_fake_quantize, orc_quantize_value : reference goldens
 *       (tests/unit/vpux_compiler/dialect/const/content_tests.cpp:2440-2540).
 *   orc_dequantize_value : content_tests.cpp:754-788.
 *   orc_approximate : ppe_factory_tests.cpp goldens and the lit goldens in
 *       tests/lit/NPU/conversion/passes/IE2VPU/convert_IE_to_VPU_NCE_37XX_40XX.mlir.
 *   orc_softmax_f16, orc_mvn_f16 : no reference vectors exist (kernel sources
 *       are absent from the reference); pinned by closed forms and an fp64
 *       brute force.  Numerics are "parity unpinned" against the SHAVE kernels.
 *   orc_ppe_requant : the bit-level rounding of the DPU is silicon; the
 *       formula follows the PPE op emission order and is "parity unpinned"
 *       against hardware.  Integer accumulation itself is exact arithmetic.
 */
#ifndef VPX_ORACLE_H_
#define VPX_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- fp16 (src/vpux_utils/src/core/type/float16.cpp:30-144) ---- */
uint16_t orc_f32_to_f16(float v);      /* bit-exact with the reference class, its subnormal-range deviation included */
uint16_t orc_f32_to_f16_ieee(float v); /* plain IEEE RNE; rounds softmax / MVN results */
float orc_f16_to_f32(uint16_t h);
void orc_convert_f32_to_f16(const float* in, uint16_t* out, size_t n);
void orc_convert_f16_to_f32(const uint16_t* in, float* out, size_t n);

/* ---- FakeQuantize (src/vpux_compiler/src/utils/quantization.cpp:995-1003) ---- */
float orc_fake_quantize(float x, float in_lo, float in_hi, float out_lo, float out_hi, float levels);
/* x, y: compact arrays of `rank` dims (outermost first).  Each limit i in
 * {in_lo,in_hi,out_lo,out_hi} has dims lim_dims[i*rank .. i*rank+rank) that are
 * either 1 or equal to dims[] (NUMPY broadcast). */
void orc_fake_quantize_f16(const uint16_t* x, uint16_t* y, int rank, const int64_t* dims, const uint16_t* const lims[4],
                           const int64_t* lim_dims, int64_t levels);

/* ---- Quantize / Dequantize (const/attributes/quantize.cpp:91-106, quantization.hpp:208-210) ---- */
float orc_dequantize_value(int64_t q, double scale, int64_t zp);
int64_t orc_quantize_value(double x, double scale, int64_t zp, int64_t qmin, int64_t qmax);
/* per-axis form: element idx = (o*axis_size + a)*inner + i uses scales[a], zps[a]; axis_size==1 is per-tensor */
void orc_quantize_f16(const uint16_t* x, void* q, int out_is_signed, int64_t outer, int64_t axis_size, int64_t inner,
                      const double* scales, const int64_t* zps, int64_t qmin, int64_t qmax);
void orc_quantize_f32(const float* x, void* q, int out_is_signed, int64_t outer, int64_t axis_size, int64_t inner,
                      const double* scales, const int64_t* zps, int64_t qmin, int64_t qmax);
void orc_dequantize_f16(const void* q, int in_is_signed, uint16_t* y, int64_t outer, int64_t axis_size, int64_t inner,
                        const double* scales, const int64_t* zps);
void orc_dequantize_f32(const void* q, int in_is_signed, float* y, int64_t outer, int64_t axis_size, int64_t inner,
                        const double* scales, const int64_t* zps);

/* ---- Eltwise fp16 (float16.hpp:123-126: fp32 op then RNE) ---- */
enum { ORC_ELT_ADD = 0, ORC_ELT_SUB = 1, ORC_ELT_MUL = 2, ORC_ELT_MIN = 3, ORC_ELT_MAX = 4, ORC_ELT_DIV = 5,
       ORC_ELT_PRELU = 6 /* a < 0 ? a * b : a */ };

/* Unary activations (OpenVINO operator definitions; p0, p1 = the op's float attributes in the
 * order the compiler serialises them).  "parity unpinned" against the SHAVE kernels, whose sources
 * are not public; pinned by special values and an independent fp64 evaluation in the tests. */
enum {
    ORC_ACT_RELU = 0, ORC_ACT_LEAKY_RELU, ORC_ACT_CLAMP, ORC_ACT_NEGATIVE, ORC_ACT_ABS, ORC_ACT_HSWISH,
    ORC_ACT_HSIGMOID, ORC_ACT_HARDSIGMOID, ORC_ACT_SIGMOID, ORC_ACT_TANH, ORC_ACT_EXP, ORC_ACT_SQRT,
    ORC_ACT_LOG, ORC_ACT_FLOOR, ORC_ACT_CEIL, ORC_ACT_SIGN, ORC_ACT_ELU, ORC_ACT_SELU, ORC_ACT_SWISH,
    ORC_ACT_MISH, ORC_ACT_SOFTPLUS, ORC_ACT_GELU, ORC_ACT_ERF
};
float orc_activation(int op, float x, float p0, float p1);
void orc_activation_f16(int op, float p0, float p1, const uint16_t* x, uint16_t* y, int64_t n);
void orc_activation_f32(int op, float p0, float p1, const float* x, float* y, int64_t n);
/* NUMPY broadcast: a_dims/b_dims entries are 1 or dims[] */
void orc_eltwise_f16(int op, const uint16_t* a, const uint16_t* b, uint16_t* y, int rank, const int64_t* dims,
                     const int64_t* a_dims, const int64_t* b_dims);

/* ---- Softmax (OpenVINO Softmax-8 semantics; VPU.SoftMax ops.td:2638-2676) ----
 * tensor viewed as [outer][axis][inner] compact; the last `pad` entries of the
 * axis are ignored on input and written as 0. */
void orc_softmax_f16(const uint16_t* x, uint16_t* y, int64_t outer, int64_t axis, int64_t inner, int64_t pad);
void orc_softmax_f32(const float* x, float* y, int64_t outer, int64_t axis, int64_t inner, int64_t pad);

/* ---- MVN-1 (VPU.MVN ops.td:3600-3652; eps inside sqrt) ----
 * element (n,c,s) lives at n*stride_n + c*stride_c + s*stride_s. */
void orc_mvn_f16(const uint16_t* x, uint16_t* y, int64_t N, int64_t C, int64_t S, int64_t stride_n, int64_t stride_c,
                 int64_t stride_s, int across_channels, int normalize_variance, float eps);

/* ---- scale approximation (include/vpux/compiler/utils/quantization.hpp:65-78) ---- */
/* returns 0 on success, -1 if the multiplier does not fit int32 */
int orc_approximate(int bits, double target, int64_t* mult, int64_t* shift, int64_t* post_shift);

/* ---- weights table words (NPU37XX/dialect/VPU/impl/nce_sparsity_converters.cpp:14-41) ---- */
int32_t orc_wt_pack_scale(uint8_t shift, int16_t mult);
void orc_wt_unpack_scale(int32_t word, int32_t* mult, int32_t* shift);

/* ---- integer PPE (NPU40XX/.../expand_dpu_config_invariant_ppe.cpp:322-380) ---- */
typedef struct {
    int32_t prelu_mult;  /* NOOP: 1, LRELU/LRELUX: 0, LPRELU: lrelu_mult */
    int32_t prelu_shift; /* NOOP/LRELU/LRELUX: 0, LPRELU: lrelu_shift */
    int32_t zp_out;
    int32_t clamp_low;
    int32_t clamp_high;
} orc_ppe_t;
int32_t orc_ppe_requant(int32_t acc, int32_t bias, int32_t mult, int32_t shift, const orc_ppe_t* ppe);
/* fp16 output (s17.15 fixed point converted to fp16, runtime_dpu_parser_imports.cpp.inc:546-574): returns the bit
 * pattern; zp_out is not used, clamp_low is ignored and clamp_high holds two fp16 bounds as 0xllllhhhh
 * (ppe_utils.hpp:36-87), INT32_MAX meaning none */
uint16_t orc_ppe_requant_f16(int32_t acc, int32_t bias, int32_t mult, int32_t shift, const orc_ppe_t* ppe);

/* ---- NCE convolution / matmul (VPU.NCE.Convolution ops.td:138-226, NCE.MatMul :228-357) ----
 * in  : NHWC [N][H][W][IC] 8-bit (signed flag), zero point zp_in
 * w   : OYXI [OC][KY][KX][IC] 8-bit (signed flag), zero point zp_w
 * wt  : weights table [OC][4] int32 (word 2 = mult/shift, word 3 = bias)
 * out : NHWC [N][OH][OW][OC] 8-bit; returns int32 accumulators too when acc_out != NULL */
typedef struct {
    int64_t N, H, W, IC, OC, KY, KX;
    int64_t stride_y, stride_x, pad_top, pad_left, pad_bottom, pad_right;
    int32_t in_signed, w_signed, out_signed; /* out_signed: 0 = u8, 1 = i8, 2 = fp16 (16-bit output elements) */
    int32_t zp_in, zp_w;
    orc_ppe_t ppe;
    /* Strides of the input and the output in elements, for images, rows and pixels (N, H, W; a pixel's channels are
     * contiguous): the operands of a task may be views of larger tensors, as the NPU's are
     * (VPUMI37XX/ops/external/runtime_dpu_parser_imports.cpp.inc:850-852, 1031-1090).  All three zero = dense NHWC.
     * acc_out stays dense. */
    int64_t in_strides[3];
    int64_t out_strides[3];
} orc_conv_t;
void orc_nce_conv(const orc_conv_t* d, const void* in, const void* w, const int32_t* wt, void* out, int32_t* acc_out);
/* only rows [row0,row0+nrows) of the flattened N*OH*OW output are produced (into out + row0*OC) */
void orc_nce_conv_rows(const orc_conv_t* d, const void* in, const void* w, const int32_t* wt, void* out,
                       int32_t* acc_out, int64_t row0, int64_t nrows);

/* ---- NCE eltwise add / subtract (EltwiseQuantizationApproximation, utils/quantization.cpp:455-516) ----
 * acc = (a - zp_a) * mult_a +/- (b - zp_b) * mult_b, then the integer PPE with bias 0 and the
 * per-tensor out_mult / out_shift.  "parity unpinned" against silicon like orc_ppe_requant. */
void orc_nce_eltwise(const void* a, int a_signed, const void* b, int b_signed, void* out, int out_signed, int64_t n,
                     int32_t zp_a, int32_t zp_b, int32_t mult_a, int32_t mult_b, int subtract, int32_t out_mult,
                     int32_t out_shift, const orc_ppe_t* ppe);

/* The same task with an fp16 output (the PPE of orc_ppe_requant_f16; no output zero point). */
void orc_nce_eltwise_f16(const void* a, int a_signed, const void* b, int b_signed, uint16_t* out, int64_t n, int32_t zp_a,
                         int32_t zp_b, int32_t mult_a, int32_t mult_b, int subtract, int32_t out_mult, int32_t out_shift,
                         const orc_ppe_t* ppe);

/* Both on views of larger tensors: dims = {N, H, W, C}; strides of a, b and out in elements for N, H, W (channels
 * contiguous).  out_kind: 0 = u8, 1 = i8, 2 = fp16 (as orc_conv_t.out_signed). */
void orc_nce_eltwise_views(const void* a, int a_signed, const void* b, int b_signed, void* out, int out_kind,
                           const int64_t dims[4], const int64_t a_strides[3], const int64_t b_strides[3],
                           const int64_t out_strides[3], int32_t zp_a, int32_t zp_b, int32_t mult_a, int32_t mult_b,
                           int subtract, int32_t out_mult, int32_t out_shift, const orc_ppe_t* ppe);

int orc_num_threads(void);
void orc_set_num_threads(int n);

#ifdef __cplusplus
}
#endif
#endif
