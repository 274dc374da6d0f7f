// Host-side mirror of the reference compiler's parameter derivation for the hot path
// (declarations and reference citations in include/vpx_compiler_utils.h).
#include "vpx_compiler_utils.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <string>
#include <vector>

namespace vpx {
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
std::string& last_error();
}  // namespace vpx

namespace vpx {
namespace host {

// ---- fp16 ----------------------------------------------------------------------------------
// Round to nearest even by adding the rounding constant to the bit pattern, then shifting.
// Like vpux::type::float16 (src/vpux_utils/src/core/type/float16.cpp:74-107), a value below 2^-15
// whose mantissa is at least 0x7ff000 is rounded as if it were twice as large: the reference's
// first rounding step bumps the exponent and its subnormal branch then reuses the old mantissa.
uint16_t floatToHalfBits(float v) {
    uint32_t x;
    std::memcpy(&x, &v, 4);
    if ((x & 0x7f800000u) != 0 && (x & 0x7f800000u) <= (111u << 23) && (x & 0x7fffffu) >= 0x7ff000u) x += 1u << 23;
    const uint32_t sign = (x >> 16) & 0x8000u;
    x &= 0x7fffffffu;
    if (x >= 0x7f800000u) {  // Inf / NaN
        if (x == 0x7f800000u) return (uint16_t)(sign | 0x7c00u);
        const uint32_t payload = (x & 0x7fffffu) >> 13;
        return (uint16_t)(sign | 0x7c00u | (payload ? payload : 1u));
    }
    if (x < 0x00800000u) return (uint16_t)sign;  // fp32 zero / subnormal
    if (x >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);  // >= 65520 rounds to infinity
    if (x >= 0x38800000u) {                                   // normal half
        const uint32_t odd = (x >> 13) & 1u;
        x += 0xfffu + odd;
        return (uint16_t)(sign | ((x - 0x38000000u) >> 13));
    }
    if (x < 0x33000000u) return (uint16_t)sign;  // < 2^-25: underflow to zero
    // subnormal half: align the mantissa so that one unit is 2^-24
    const int e = (int)(x >> 23);
    uint32_t m = (x & 0x7fffffu) | 0x800000u;
    const int shift = 126 - e;  // 14 .. 24
    const uint32_t rem_mask = (1u << shift) - 1u, half = 1u << (shift - 1);
    const uint32_t rem = m & rem_mask;
    m >>= shift;
    if (rem > half || (rem == half && (m & 1u))) m++;
    return (uint16_t)(sign | m);
}

float halfBitsToFloat(uint16_t h) {
    const uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
    float mag;
    if (e == 0) mag = std::ldexp((float)m, -24);
    else if (e == 31) {
        uint32_t bits = 0x7f800000u | (m << 13);
        std::memcpy(&mag, &bits, 4);
    } else mag = std::ldexp((float)(m | 0x400u), (int)e - 25);
    return (h & 0x8000u) ? -mag : mag;
}

// ---- scale approximation ---------------------------------------------------------------------
struct Approximation {
    int64_t mult = 0, shift = 0, postShift = 0;
};

Approximation approximate(int bits, double target) {
    int exponent = 0;
    const double mantissa = std::frexp(target, &exponent);
    Approximation a;
    // floor: rounding could give 2^bits, which the multiplier register cannot hold
    a.mult = (int64_t)std::floor(mantissa * std::pow(2.0, bits));
    a.shift = exponent > bits ? 0 : bits - exponent;
    a.postShift = exponent > bits ? bits - exponent : 0;
    return a;
}

// ---- PPE attribute -----------------------------------------------------------------------------
// absolute comparison at float epsilon (src/vpux_utils/include/vpux/utils/core/numeric.hpp:56-58)
bool isFloatEqual(float a, float b) {
    return std::fabs(a - b) <= std::numeric_limits<float>::epsilon();
}

}  // namespace host
}  // namespace vpx

using namespace vpx;
using namespace vpx::host;

extern "C" {

uint16_t vpx_float_to_half_bits(float v) {
    return floatToHalfBits(v);
}
float vpx_half_bits_to_float(uint16_t bits) {
    return halfBitsToFloat(bits);
}

int vpx_approximate(int bits, double target, int64_t* mult, int64_t* shift, int64_t* post_shift) {
    if (!mult || !shift || !post_shift) return fail(VPX_RESULT_ERROR_INVALID_NULL_HANDLE, "approximate: null output");
    if (bits < 1 || bits > 31 || !std::isfinite(target))
        return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT, "approximate: cannot approximate %g with %d bits", target, bits);
    const Approximation a = approximate(bits, target);
    *mult = a.mult;
    *shift = a.shift;
    *post_shift = a.postShift;
    if (a.postShift != 0)
        return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT,
                    "%g approximates to multiplier %lld >> %lld with a further post-shift of %lld; this path has no post-shift stage",
                    target, (long long)a.mult, (long long)a.shift, (long long)a.postShift);
    return VPX_RESULT_SUCCESS;
}

// Two input scales and the inverse output scale as 15-bit multipliers with shifts, brought to the form the eltwise
// datapath has: both inputs multiplied by 16-bit unsigned factors, one shared shift after the output multiplier
// (quantization.cpp:455-516).  The two input shifts are equalised by scaling one factor: up to the larger shift when
// the factor still fits 16 bits and the summed shift fits the 6-bit field, otherwise down to the smaller one.
int vpx_eltwise_quantization_approximation(double in1_scale, double in2_scale, double out_scale, int eltwise_type,
                                           int64_t* in1_mult, int64_t* in2_mult, int64_t* out_mult, int64_t* out_shift) {
    if (!in1_mult || !in2_mult || !out_mult || !out_shift)
        return fail(VPX_RESULT_ERROR_INVALID_NULL_HANDLE, "eltwise approximation: null output");
    constexpr int64_t kShiftFieldMax = (1 << 6) - 1;
    constexpr int64_t kFactorMax = (1 << 16) - 1;
    enum { kAdd = 0, kSubtract = 1, kMultiply = 2 };

    const Approximation src[2] = {approximate(15, in1_scale), approximate(15, in2_scale)};
    const Approximation dst = approximate(15, 1.0 / out_scale);
    if (src[0].postShift || src[1].postShift || dst.postShift)
        return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT, "eltwise approximation: a scale needs a post-shift, which the datapath lacks");

    // signs: the input factors are unsigned, so a negative pair is folded into the output multiplier
    int64_t factor[2] = {src[0].mult, src[1].mult};
    int64_t result_mult = dst.mult;
    const int negatives = (factor[0] < 0) + (factor[1] < 0);
    if (negatives) {
        const bool sum_like = eltwise_type == kAdd || eltwise_type == kSubtract;
        if (sum_like && negatives == 1)
            return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT,
                        "eltwise approximation: input multipliers %lld and %lld differ in sign, which an add / subtract cannot express",
                        (long long)factor[0], (long long)factor[1]);
        if (sum_like || (eltwise_type == kMultiply && negatives == 1)) result_mult = -result_mult;
        for (int64_t& f : factor) f = (int64_t)(uint16_t)(f < 0 ? -f : f);
    }

    const int64_t hi = std::max(src[0].shift, src[1].shift), lo = std::min(src[0].shift, src[1].shift);
    bool up = hi + dst.shift <= kShiftFieldMax;
    for (int k = 0; k < 2 && up; k++) up = factor[k] <= (kFactorMax >> (hi - src[k].shift));
    int64_t common;
    if (up) {
        common = hi;
        for (int k = 0; k < 2; k++) factor[k] = (int64_t)(uint16_t)(factor[k] << (hi - src[k].shift));
    } else if (lo + dst.shift < kShiftFieldMax) {
        common = lo;
        for (int k = 0; k < 2; k++) factor[k] = (int64_t)(uint16_t)(factor[k] >> (src[k].shift - lo));
    } else {
        return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT,
                    "eltwise approximation: shifts %lld / %lld with output shift %lld do not fit the 6-bit shift field",
                    (long long)src[0].shift, (long long)src[1].shift, (long long)dst.shift);
    }
    *in1_mult = factor[0];
    *in2_mult = factor[1];
    *out_mult = result_mult;
    *out_shift = dst.shift + common;
    return VPX_RESULT_SUCCESS;
}

int32_t vpx_wt_get_scale(uint8_t shift, int16_t mult) {
    const int32_t PPE_SHIFT_OFFSET = 8, PPE_MULT_OFFSET = 16;
    return (int32_t)(((uint32_t)shift << PPE_SHIFT_OFFSET) | ((uint32_t)(int32_t)mult << PPE_MULT_OFFSET));
}

int vpx_wt_get_bias(double real_val, int32_t* bias) {
    const double r = std::round(real_val);
    if (!(r > (double)std::numeric_limits<int32_t>::min() && r < (double)std::numeric_limits<int32_t>::max()))
        return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT, "a bias divided by its rescale factor does not fit 32 bits");
    *bias = (int32_t)r;
    return VPX_RESULT_SUCCESS;
}

int vpx_get_weights_table(double in_scale, double out_scale, const double* weight_scales, size_t n_weight_scales,
                          const double* bias, int64_t OC, int32_t weights_ptr, int32_t weights_ptr_step,
                          int32_t sparsity_ptr, int32_t sparsity_ptr_step, int32_t* table) {
    if (!weight_scales || !table) return fail(VPX_RESULT_ERROR_INVALID_NULL_HANDLE, "getWeightsTable: null argument");
    if (n_weight_scales != 1 && (int64_t)n_weight_scales != OC)
        return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT, "getWeightsTable: %zu weight scales cannot broadcast to %lld channels",
                    n_weight_scales, (long long)OC);
    for (int64_t oc = 0; oc < OC; oc++) {
        const int32_t wptr = weights_ptr + (int32_t)oc * weights_ptr_step;
        const int32_t sptr = sparsity_ptr + (int32_t)oc * sparsity_ptr_step;
        if (wptr % 16 != 0) return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT, "weightsPtrs[%lld] must be multiple of 16, got %d", (long long)oc, wptr);
        if (sptr != 0xFFFFFF && sptr % 16 != 0)
            return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT, "sparsityPtrs[%lld] must be aligned to 16, got %d", (long long)oc, sptr);
        const double ws = weight_scales[n_weight_scales == 1 ? 0 : oc];
        const double rescale = (ws * in_scale) / out_scale;
        const Approximation a = approximate(15, rescale);
        if (a.postShift != 0)
            return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT,
                        "%g approximates to multiplier %lld >> %lld with a further post-shift of %lld; this path has no post-shift stage",
                        rescale, (long long)a.mult, (long long)a.shift, (long long)a.postShift);
        if (a.shift > 255 || a.mult > 32767 || a.mult < -32768)
            return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT, "scale %g does not fit the multiplier / shift fields", rescale);
        int32_t b = 0;
        if (bias) {
            const int rc = vpx_wt_get_bias(bias[oc] / (ws * in_scale), &b);
            if (rc) return rc;
        }
        table[oc * 4 + 0] = wptr;
        table[oc * 4 + 1] = sptr;
        table[oc * 4 + 2] = vpx_wt_get_scale((uint8_t)a.shift, (int16_t)a.mult);
        table[oc * 4 + 3] = b;
    }
    return VPX_RESULT_SUCCESS;
}

int vpx_retrieve_ppe_int(int post_op, double param0, double param1, const vpx_quant_type_t* out_type, vpx_ppe_int_t* ppe) {
    if (!out_type || !ppe) return fail(VPX_RESULT_ERROR_INVALID_NULL_HANDLE, "retrievePPEAttribute: null argument");
    // neutral values (VPU_PPEIntAttr description, tblgen/.../VPU/attributes.td:399-414)
    ppe->mode = VPX_PPE_NOOP;
    ppe->clamp_low = std::numeric_limits<int32_t>::min();
    ppe->clamp_high = std::numeric_limits<int32_t>::max();
    ppe->lrelu_mult = 1;
    ppe->lrelu_shift = 0;
    ppe->quant_mult = 1;  // the eltwise-only fields: neutral
    ppe->quant_shift = 0;
    ppe->in1_quant_mult = 1;
    ppe->in2_quant_mult = 1;
    const bool q = out_type->is_quantized != 0;
    switch (post_op) {
    case VPX_POSTOP_NONE:
        if (q) {
            ppe->clamp_low = (int32_t)out_type->storage_min;
            ppe->clamp_high = (int32_t)out_type->storage_max;
        }
        return VPX_RESULT_SUCCESS;
    case VPX_POSTOP_RELU:
        if (q) {
            ppe->clamp_low = (int32_t)out_type->zero_point;
            ppe->clamp_high = (int32_t)out_type->storage_max;
        } else {
            ppe->mode = VPX_PPE_LRELU;
        }
        return VPX_RESULT_SUCCESS;
    case VPX_POSTOP_CLAMP: {
        if (!q) {
            // fp16 output: both bounds as fp16 bit patterns in clamp_high (0xllllhhhh, the sign-extended patterns
            // added, ppe_utils.hpp:57-73), clamp_low stays at its neutral value; a maximum that fp16 cannot hold
            // leaves a plain ReLU (ppe_factory.cpp:170-178)
            if (param1 < 65504.0) {
                const int32_t lo = (int32_t)(int16_t)floatToHalfBits((float)param0), hi = (int32_t)(int16_t)floatToHalfBits((float)param1);
                ppe->clamp_high = (int32_t)(((uint32_t)lo << 16) + (uint32_t)hi);
                ppe->mode = VPX_PPE_LRELUX;
            } else {
                ppe->mode = VPX_PPE_LRELU;
            }
            return VPX_RESULT_SUCCESS;
        }
        // the clamp bounds in quantized steps around the zero point, cut to what the storage type holds; a range that
        // starts at the zero point and ends below the storage maximum is a ReLU-X
        const int64_t zp = out_type->zero_point;
        int64_t bound[2];
        const double real[2] = {param0, param1};
        for (int k = 0; k < 2; k++) bound[k] = zp + (int64_t)std::round(real[k] / out_type->scale);
        if (bound[0] < out_type->storage_min) bound[0] = out_type->storage_min;
        if (bound[1] > out_type->storage_max) bound[1] = out_type->storage_max;
        ppe->clamp_low = (int32_t)bound[0];
        ppe->clamp_high = (int32_t)bound[1];
        const bool from_zero = bound[0] == zp, below_max = bound[1] - zp < out_type->storage_max;
        if (from_zero && below_max) ppe->mode = VPX_PPE_LRELUX;
        return VPX_RESULT_SUCCESS;
    }
    case VPX_POSTOP_LEAKY_RELU: {
        ppe->mode = VPX_PPE_LPRELU;
        if (q) {
            ppe->clamp_low = (int32_t)out_type->storage_min;
            ppe->clamp_high = (int32_t)out_type->storage_max;
        }
        const double alpha = param0;
        if (isFloatEqual((float)alpha, 0.0f)) {
            ppe->lrelu_mult = 0;
        } else if (!isFloatEqual((float)alpha, 1.0f)) {
            const Approximation a = approximate(11, alpha);
            if (a.postShift != 0)
                return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT,
                            "%g approximates to multiplier %lld >> %lld with a further post-shift of %lld; this path has no post-shift stage",
                            alpha, (long long)a.mult, (long long)a.shift, (long long)a.postShift);
            ppe->lrelu_mult = (int32_t)a.mult;
            ppe->lrelu_shift = (int32_t)a.shift;
        }
        return VPX_RESULT_SUCCESS;
    }
    default: return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT, "post-op kind %d is not one of the VPX_POSTOP_* values", post_op);
    }
}

// Packed softmax parameters (update_sw_kernel_params.cpp:36-147): the tensor is reduced to the fewest (size, input
// stride, output stride) levels that still describe it, innermost first, and the kernel variant is chosen from them.
int vpx_generate_softmax_attr(uint32_t rank, const int64_t* dims, const int64_t* in_strides, const int64_t* out_strides,
                              int64_t axis, int64_t pad_size, uint64_t* words, uint32_t* n_words) {
    if (!dims || !in_strides || !out_strides || !words || !n_words)
        return fail(VPX_RESULT_ERROR_INVALID_NULL_HANDLE, "softmax parameters: null argument");
    if (rank < 1 || rank > VPX_MAX_ND_DIMS || axis < 0 || axis >= (int64_t)rank)
        return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT, "softmax parameters: axis %lld outside rank %u", (long long)axis, rank);
    struct Level {
        int64_t size, in_step, out_step;
        bool reduced;  // the softmax axis
    };
    // 1. levels of size one say nothing, except the axis itself
    std::vector<Level> kept;
    for (uint32_t d = 0; d < rank; d++)
        if (dims[d] != 1 || (int64_t)d == axis) kept.push_back(Level{dims[d], in_strides[d], out_strides[d], (int64_t)d == axis});
    // 2. above the axis, neighbours that both operands walk without a gap become one level
    size_t axis_at = 0;
    while (!kept[axis_at].reduced) axis_at++;
    std::vector<Level> levels(kept.begin(), kept.begin() + (std::ptrdiff_t)axis_at + 1);
    for (size_t d = axis_at + 1; d < kept.size(); d++) {
        const Level& below = kept[d - 1];
        const bool gapless = kept[d].in_step == below.in_step * below.size && kept[d].out_step == below.out_step * below.size;
        if (d >= axis_at + 2 && gapless)
            levels.back().size *= kept[d].size;
        else
            levels.push_back(kept[d]);
    }
    // 3. an innermost axis that is not unit-stride is served as an outer axis over an inner level of one element
    if (axis_at == 0 && (levels[0].in_step > 1 || levels[0].out_step > 1)) {
        levels.insert(levels.begin(), Level{1, levels[0].in_step, levels[0].out_step, false});
        axis_at = 1;
    }
    // 4. the kernel wants at least three levels: unit levels stacked on the outermost one
    const Level top = levels.back();
    while (levels.size() < 3) levels.push_back(Level{1, top.in_step * top.size, top.out_step * top.size, false});

    int64_t mode = VPX_SOFTMAX_OUTER;
    if (axis_at == 0) {
        const bool tiny_rows = (levels[0].size == 2 || levels[0].size == 4) && pad_size == 0 && levels[1].in_step == levels[0].size &&
                               levels[2].in_step == levels[2].out_step;
        mode = tiny_rows ? VPX_SOFTMAX_INNER_HARDCODED : VPX_SOFTMAX_INNER;
    }
    const auto two_i32 = [](int64_t lo, int64_t hi) { return ((uint64_t)(uint32_t)hi << 32) | (uint64_t)(uint32_t)lo; };
    uint32_t n = 0;
    words[n++] = two_i32((int64_t)axis_at, pad_size);
    words[n++] = two_i32(mode, (int64_t)levels.size());
    for (const Level& l : levels) {
        words[n++] = two_i32(l.size, l.size);
        words[n++] = two_i32(l.in_step, l.out_step);
    }
    *n_words = n;
    return VPX_RESULT_SUCCESS;
}

int vpx_get_quant_params_attr(const double* scales, const int64_t* zero_points, uint32_t n, uint32_t float_type,
                              uint64_t* words, uint32_t* n_words) {
    if (!scales || !zero_points || !words || !n_words) return fail(VPX_RESULT_ERROR_INVALID_NULL_HANDLE, "getQuantParamsAttr: null argument");
    if (float_type != VPX_NN_FP16 && float_type != VPX_NN_FP32)
        return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT, "a tensor that is not quantized must be FP16 or FP32 here");
    const uint32_t per = float_type == VPX_NN_FP16 ? 4 : 2, width = 64 / per;
    uint32_t w = 0;
    words[w++] = n;
    auto pack = [&](auto value_at) {
        for (uint32_t i = 0; i < n; i += per) {
            uint64_t word = 0;
            for (uint32_t k = 0; k < per && i + k < n; k++) {
                const float f = (float)value_at(i + k);
                uint64_t bits;
                if (float_type == VPX_NN_FP16) {
                    bits = floatToHalfBits(f);
                } else {
                    uint32_t b;
                    std::memcpy(&b, &f, 4);
                    bits = b;
                }
                word |= bits << (width * k);
            }
            words[w++] = word;
        }
    };
    pack([&](uint32_t i) { return scales[i]; });
    pack([&](uint32_t i) { return (double)zero_points[i]; });
    *n_words = w;
    return VPX_RESULT_SUCCESS;
}

namespace {

// computeReverseMemDim (sw_kernel.cpp:29-40): position of a logical dimension counted from the innermost memory
// dimension.  The order code holds one hex digit (logical index + 1) per memory dimension, the outermost in the
// lowest digit (NHWC = 0x2431: N, H, W, C).
int reverse_mem_dim(const vpx_tensor_desc_t& t, int64_t dim, int64_t* out) {
    const int64_t nd = t.num_dims;
    if (dim < 0) dim += nd;
    if (dim < 0 || dim >= nd) return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT, "axis %lld is outside a tensor of rank %lld", (long long)dim, (long long)nd);
    for (int64_t i = 0; i < nd; i++) {
        if ((int64_t)((t.dims_order >> (4 * i)) & 0xf) == dim + 1) {
            *out = nd - 1 - i;
            return VPX_RESULT_SUCCESS;
        }
    }
    return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT, "order 0x%llx does not name dimension %lld", (unsigned long long)t.dims_order, (long long)dim);
}

struct AttrWriter {
    std::vector<uint8_t> bytes;
    void i64(int64_t v) { const uint8_t* p = (const uint8_t*)&v; bytes.insert(bytes.end(), p, p + 8); }
    void boolean(int32_t v) { i64(v ? -1 : 0); }  // IntegerAttr of an i1 through getSExtValue()
    void f32(float v) { const uint8_t* p = (const uint8_t*)&v; bytes.insert(bytes.end(), p, p + 4); }
};

struct SimpleOp {
    const char* op;
    const char* entry;
    int n_float;  // float attributes taken from param0, param1
};
const SimpleOp kSimpleOps[] = {
    {"Convert", "convert", 0}, {"Add", "eltwise_add", 0}, {"Subtract", "eltwise_sub", 0}, {"Multiply", "eltwise_mul", 0},
    {"Divide", "eltwise_div", 0}, {"Minimum", "eltwise_min", 0}, {"Maximum", "eltwise_max", 0}, {"PRelu", "prelu_fp16", 0},
    {"DynamicQuantize", "dynamic_quantize", 0}, {"ReLU", "activation_relu", 0}, {"LeakyRelu", "leaky_relu_fp16", 1},
    {"Clamp", "activation_clamp", 2}, {"Negative", "activation_negative", 0}, {"Abs", "activation_abs", 0},
    {"HSwish", "activation_hswish", 0}, {"HSigmoid", "activation_hsigmoid", 0}, {"HardSigmoid", "activation_hardsigmoid", 2},
    {"Sigmoid", "activation_sigmoid", 0}, {"Tanh", "activation_tanh", 0}, {"Exp", "activation_exp", 0},
    {"Sqrt", "activation_sqrt", 0}, {"Log", "activation_log", 0}, {"Floor", "activation_floor", 0},
    {"Ceiling", "activation_ceil", 0}, {"Sign", "activation_sign", 0}, {"Elu", "activation_elu", 1},
    {"Selu", "activation_selu", 2}, {"Swish", "activation_swish", 1}, {"Mish", "activation_mish", 0},
    {"SoftPlus", "activation_softplus", 0}, {"Gelu", "activation_gelu", 0}, {"Erf", "activation_erf", 0},
};

}  // namespace

int vpx_get_kernel_info(const char* op, const vpx_op_attrs_t* a, const vpx_tensor_desc_t* input, char* entry,
                        size_t entry_capacity, void* attr_bytes, size_t* attr_size) {
    if (!op || !entry || !attr_size) return fail(VPX_RESULT_ERROR_INVALID_NULL_HANDLE, "vpx_get_kernel_info: null argument");
    const std::string name(op);
    std::string ent;
    AttrWriter w;
    const auto need = [&](bool ok, const char* what) {
        return ok ? VPX_RESULT_SUCCESS : fail(VPX_RESULT_ERROR_INVALID_NULL_HANDLE, "%s: %s is required", op, what);
    };
    int rc = VPX_RESULT_SUCCESS;
    bool found = false;
    for (const SimpleOp& s : kSimpleOps) {
        if (name != s.op) continue;
        if (s.n_float > 0 && (rc = need(a != nullptr, "attributes"))) return rc;
        if (s.n_float >= 1) w.f32(a->param0);
        if (s.n_float >= 2) w.f32(a->param1);
        ent = s.entry;
        found = true;
    }
    if (found) {
    } else if (name == "SoftMax") {
        if ((rc = need(a && input, "attributes and the input tensor"))) return rc;
        int64_t axis = 0;
        if ((rc = reverse_mem_dim(*input, a->axis_ind, &axis))) return rc;
        w.i64(axis);
        w.i64(a->pad_size);
        ent = input->data_type == VPX_NN_FP32 ? "softmaxFp32" : "softmax";
    } else if (name == "MVN") {
        if ((rc = need(a != nullptr, "attributes"))) return rc;
        w.boolean(a->across_channels);
        w.boolean(a->normalize_variance);
        w.f32(a->eps);
        ent = "mvn1";
    } else if (name == "MVN1Sum" || name == "MVN1Normalize") {
        if ((rc = need(a != nullptr, "attributes"))) return rc;
        w.boolean(a->across_channels);
        w.boolean(a->normalize_variance);
        ent = name == "MVN1Sum" ? "mvn1_sum" : "mvn1_norm";
    } else if (name == "MVN1MeanVar") {
        if ((rc = need(a && a->orig_shape, "attributes with orig_shape"))) return rc;
        for (int i = 0; i < 4; i++) w.i64(a->orig_shape[i]);
        w.boolean(a->across_channels);
        w.boolean(a->normalize_variance);
        w.i64(a->group_c);
        w.f32(a->eps);
        ent = "mvn1_mean_var";
    } else if (name == "MVN6") {
        if ((rc = need(a && input && (a->axes || a->num_axes == 0), "attributes with axes and the input tensor"))) return rc;
        // optionalIoAttr (sw_kernel.cpp:165-185): a marker after the MemRefData records, then a mask of present operands
        w.i64(INT64_MIN);
        w.i64(1 | (a->has_scale ? 2 : 0) | (a->has_bias ? 4 : 0) | 8);
        w.boolean(a->normalize_variance);
        w.i64(a->eps_mode);
        w.f32(a->eps);
        w.i64(a->num_axes);
        for (uint32_t i = 0; i < a->num_axes; i++) {
            int64_t axis = 0;
            if ((rc = reverse_mem_dim(*input, a->axes[i], &axis))) return rc;
            w.i64(axis);
        }
        ent = "mvn6";
    } else if (name == "FakeQuantize") {
        if ((rc = need(a != nullptr, "attributes"))) return rc;
        w.i64(a->levels);
        ent = "fake_quantize";
    } else if (name == "Quantize" || name == "Dequantize") {
        if ((rc = need(a && input && a->scales && a->zero_points && a->num_quant_params > 0, "quantization parameters and the float tensor"))) return rc;
        std::vector<uint64_t> words(1 + 2 * ((size_t)a->num_quant_params + 1));
        uint32_t n_words = 0;
        if ((rc = vpx_get_quant_params_attr(a->scales, a->zero_points, a->num_quant_params, input->data_type, words.data(), &n_words))) return rc;
        for (uint32_t i = 0; i < n_words; i++) w.i64((int64_t)words[i]);
        ent = name == "Quantize" ? "quantize" : "dequantize";
    } else if (name == "DynamicDequantize") {
        w.i64(INT64_MAX);  // delimiter: the zero point operand is optional (sw_kernel.cpp:1180-1183)
        ent = "dynamic_dequantize";
    } else {
        return fail(VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "vpx_get_kernel_info: operator '%s' has no kernel here", op);
    }
    if (ent.size() + 1 > entry_capacity) return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT, "vpx_get_kernel_info: entry buffer of %zu bytes is too small", entry_capacity);
    std::memcpy(entry, ent.c_str(), ent.size() + 1);
    if (attr_bytes) {
        if (*attr_size < w.bytes.size()) return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT, "vpx_get_kernel_info: attribute buffer holds %zu bytes, %zu are needed", *attr_size, w.bytes.size());
        if (!w.bytes.empty()) std::memcpy(attr_bytes, w.bytes.data(), w.bytes.size());
    }
    *attr_size = w.bytes.size();
    return VPX_RESULT_SUCCESS;
}

int vpx_create_kernel_params(const vpx_tensor_desc_t* inputs, uint32_t n_inputs, const vpx_tensor_desc_t* outputs,
                             uint32_t n_outputs, const void* attrs, size_t attrs_size, void* blob, size_t* blob_size) {
    if (!blob_size || (n_inputs && !inputs) || (n_outputs && !outputs) || (attrs_size && !attrs))
        return fail(VPX_RESULT_ERROR_INVALID_NULL_HANDLE, "createKernelParams: null argument");
    std::vector<uint8_t> v;
    auto append = [&](const void* p, size_t n) {
        const uint8_t* b = (const uint8_t*)p;
        v.insert(v.end(), b, b + n);
    };
    auto add_memref = [&](const vpx_tensor_desc_t& t) {
        vpx_memref_data_t m;
        std::memset(&m, 0, sizeof(m));
        m.numDims = t.num_dims;
        m.dimsOrder = t.dims_order;
        m.dataType = t.data_type;
        m.location = t.location;
        m.isStatic = t.dynamic_shape ? 0 : 1;
        append(&m, sizeof(m));
    };
    for (uint32_t i = 0; i < n_inputs; i++) add_memref(inputs[i]);
    for (uint32_t i = 0; i < n_outputs; i++) add_memref(outputs[i]);
    append(attrs, attrs_size);
    auto add_dims = [&](const vpx_tensor_desc_t* t, uint32_t n) {
        for (uint32_t i = 0; i < n; i++) append(t[i].dims, sizeof(int32_t) * t[i].num_dims);
    };
    auto add_strides = [&](const vpx_tensor_desc_t* t, uint32_t n) {
        for (uint32_t i = 0; i < n; i++) append(t[i].strides, sizeof(int64_t) * t[i].num_dims);
    };
    add_dims(inputs, n_inputs);
    add_strides(inputs, n_inputs);
    add_dims(outputs, n_outputs);
    add_strides(outputs, n_outputs);
    if (blob) {
        if (*blob_size < v.size()) {
            *blob_size = v.size();
            return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT, "createKernelParams: buffer too small, %zu bytes needed", v.size());
        }
        std::memcpy(blob, v.data(), v.size());
    }
    *blob_size = v.size();
    return VPX_RESULT_SUCCESS;
}

}  // extern "C"
