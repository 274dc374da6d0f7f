/*
 * CPU oracle for the vpux hot path -- TEST INFRASTRUCTURE ONLY (see vpx_oracle.h).
 * Build with -ffp-contract=off so that fp32 expressions round exactly as written.
 */
#include "vpx_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
void orc_set_num_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

/* ------------------------------------------------------------------ fp16 */

/* binary32 -> binary16 exactly as vpux::type::float16::float16(float) does it,
 * src/vpux_utils/src/core/type/float16.cpp:30-108: round to nearest even, gradual underflow,
 * overflow to infinity, NaN keeps its top 10 payload bits (forced non-zero), fp32 zero and
 * subnormals give signed zero.
 *
 * One deviation from IEEE is inherited on purpose.  The reference rounds the mantissa to 10 bits
 * first (:74-80) and, when that carries, bumps the exponent even if the result is subnormal; the
 * subnormal branch (:92-107) then re-reads the ORIGINAL mantissa with the bumped exponent.  For
 * |v| < 2^-15 with mantissa >= 0x7ff000 the result is therefore the rounding of 2*v. */
static uint16_t f32_to_f16_impl(float v, int reference_quirk) {
    uint32_t bits;
    memcpy(&bits, &v, 4);
    const uint16_t sign = (uint16_t)((bits >> 16) & 0x8000u);
    const uint32_t exp32 = (bits >> 23) & 0xffu;
    const uint32_t man = bits & 0x7fffffu;
    if (exp32 == 0xffu) {
        if (man == 0) return (uint16_t)(sign | 0x7c00u);
        uint32_t payload = man >> 13;
        if (payload == 0) payload = 1;
        return (uint16_t)(sign | 0x7c00u | payload);
    }
    if (exp32 == 0) return sign; /* fp32 zero and subnormals flush to signed zero (float16.cpp:69-72) */
    int e = (int)exp32 - 127 + 15;
    if (e > 0) {
        if (e > 30) return (uint16_t)(sign | 0x7c00u);
        uint32_t h = ((uint32_t)e << 10) | (man >> 13);
        const uint32_t rem = man & 0x1fffu;
        if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++; /* may carry into the exponent */
        if (h >= 0x7c00u) h = 0x7c00u;
        return (uint16_t)(sign | h);
    }
    if (reference_quirk && man >= 0x7ff000u) {
        e++; /* the carry of the first rounding, see above */
        if (e > 0) return (uint16_t)(sign | 0x0400u);
    }
    /* subnormal result: value = M * 2^(e-14) in units of 2^-24, M has the hidden bit */
    const uint32_t M = man | 0x800000u;
    const int sh = 14 - e;
    if (sh > 24) return sign; /* below half of the smallest subnormal */
    uint32_t h = M >> sh;
    const uint32_t rem = M & ((1u << sh) - 1u);
    const uint32_t half = 1u << (sh - 1);
    if (rem > half || (rem == half && (h & 1u))) h++;
    return (uint16_t)(sign | h);
}

uint16_t orc_f32_to_f16(float v) {
    return f32_to_f16_impl(v, 1);
}

/* Plain IEEE-754 round-to-nearest-even narrowing, without the deviation above.  Used for the
 * results of softmax and MVN, whose semantics come from the operator definitions rather than
 * from the reference's float16 class. */
uint16_t orc_f32_to_f16_ieee(float v) {
    return f32_to_f16_impl(v, 0);
}

/* exact widening, src/vpux_utils/src/core/type/float16.cpp:118-144 */
float orc_f16_to_f32(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp16 = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp16 == 0x1fu) {
        bits = sign | 0x7f800000u | (man << 13);
    } else if (exp16 != 0) {
        bits = sign | ((exp16 + 112u) << 23) | (man << 13);
    } else if (man == 0) {
        bits = sign;
    } else {
        int e = 113;
        while ((man & 0x400u) == 0) {
            man <<= 1;
            e--;
        }
        bits = sign | ((uint32_t)e << 23) | ((man & 0x3ffu) << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

void orc_convert_f32_to_f16(const float* in, uint16_t* out, size_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)n; i++) out[i] = orc_f32_to_f16(in[i]);
}
void orc_convert_f16_to_f32(const uint16_t* in, float* out, size_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)n; i++) out[i] = orc_f16_to_f32(in[i]);
}

/* ------------------------------------------------------------------ FakeQuantize */

/* vpux::fakeQuantize, src/vpux_compiler/src/utils/quantization.cpp:995-1003; fp32 throughout,
 * std::round = half away from zero. */
float orc_fake_quantize(float x, float in_lo, float in_hi, float out_lo, float out_hi, float levels) {
    if (x <= in_lo) return out_lo;
    if (x > in_hi) return out_hi;
    return roundf((x - in_lo) / (in_hi - in_lo) * (levels - 1.0f)) / (levels - 1.0f) * (out_hi - out_lo) + out_lo;
}

static int64_t bcast_offset(int rank, const int64_t* idx, const int64_t* bdims) {
    int64_t off = 0;
    for (int d = 0; d < rank; d++) {
        off = off * bdims[d] + (bdims[d] == 1 ? 0 : idx[d]);
    }
    return off;
}

static void unravel(int64_t lin, int rank, const int64_t* dims, int64_t* idx) {
    for (int d = rank - 1; d >= 0; d--) {
        idx[d] = lin % dims[d];
        lin /= dims[d];
    }
}

void orc_fake_quantize_f16(const uint16_t* x, uint16_t* y, int rank, const int64_t* dims, const uint16_t* const lims[4],
                           const int64_t* lim_dims, int64_t levels) {
    int64_t total = 1;
    for (int d = 0; d < rank; d++) total *= dims[d];
    const float fl = (float)levels;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < total; i++) {
        int64_t idx[16];
        unravel(i, rank, dims, idx);
        float l[4];
        for (int k = 0; k < 4; k++) l[k] = orc_f16_to_f32(lims[k][bcast_offset(rank, idx, lim_dims + k * rank)]);
        y[i] = orc_f32_to_f16(orc_fake_quantize(orc_f16_to_f32(x[i]), l[0], l[1], l[2], l[3], fl));
    }
}

/* ------------------------------------------------------------------ Quantize / Dequantize */

/* vpux::dequantize, include/vpux/compiler/utils/quantization.hpp:208-210: double product, then float */
float orc_dequantize_value(int64_t q, double scale, int64_t zp) {
    return (float)((double)(q - zp) * scale);
}

/* createQuantizeFn, src/vpux_compiler/src/dialect/const/attributes/quantize.cpp:91-106:
 * fakeQuantize from the dequantized storage range onto [qmin,qmax] with qmax-qmin+1 levels,
 * all arguments narrowed to float at the call, result truncated to integer. */
int64_t orc_quantize_value(double x, double scale, int64_t zp, int64_t qmin, int64_t qmax) {
    const float in_min = orc_dequantize_value(qmin, scale, zp);
    const float in_max = orc_dequantize_value(qmax, scale, zp);
    const float fq = orc_fake_quantize((float)x, in_min, in_max, (float)qmin, (float)qmax, (float)(qmax - qmin + 1));
    return (int64_t)fq;
}

#define QUANT_LOOP(LOAD)                                                                        \
    _Pragma("omp parallel for schedule(static)") for (int64_t o = 0; o < outer; o++) {          \
        for (int64_t a = 0; a < axis_size; a++) {                                               \
            for (int64_t i = 0; i < inner; i++) {                                               \
                const int64_t idx = (o * axis_size + a) * inner + i;                            \
                const int64_t v = orc_quantize_value((double)(LOAD), scales[a], zps[a], qmin, qmax); \
                if (out_is_signed)                                                              \
                    ((int8_t*)q)[idx] = (int8_t)v;                                              \
                else                                                                            \
                    ((uint8_t*)q)[idx] = (uint8_t)v;                                            \
            }                                                                                   \
        }                                                                                       \
    }

void orc_quantize_f16(const uint16_t* x, void* q, int out_is_signed, int64_t outer, int64_t axis_size, int64_t inner,
                      const double* scales, const int64_t* zps, int64_t qmin, int64_t qmax) {
    QUANT_LOOP(orc_f16_to_f32(x[idx]))
}
void orc_quantize_f32(const float* x, void* q, int out_is_signed, int64_t outer, int64_t axis_size, int64_t inner,
                      const double* scales, const int64_t* zps, int64_t qmin, int64_t qmax) {
    QUANT_LOOP(x[idx])
}

/* DequantizeAttr::transform loop, src/vpux_compiler/src/dialect/const/attributes/dequantize.cpp:42-107 */
void orc_dequantize_f32(const void* q, int in_is_signed, float* y, int64_t outer, int64_t axis_size, int64_t inner,
                        const double* scales, const int64_t* zps) {
#pragma omp parallel for schedule(static)
    for (int64_t o = 0; o < outer; o++)
        for (int64_t a = 0; a < axis_size; a++)
            for (int64_t i = 0; i < inner; i++) {
                const int64_t idx = (o * axis_size + a) * inner + i;
                const int64_t v = in_is_signed ? (int64_t)((const int8_t*)q)[idx] : (int64_t)((const uint8_t*)q)[idx];
                y[idx] = orc_dequantize_value(v, scales[a], zps[a]);
            }
}
void orc_dequantize_f16(const void* q, int in_is_signed, uint16_t* y, int64_t outer, int64_t axis_size, int64_t inner,
                        const double* scales, const int64_t* zps) {
#pragma omp parallel for schedule(static)
    for (int64_t o = 0; o < outer; o++)
        for (int64_t a = 0; a < axis_size; a++)
            for (int64_t i = 0; i < inner; i++) {
                const int64_t idx = (o * axis_size + a) * inner + i;
                const int64_t v = in_is_signed ? (int64_t)((const int8_t*)q)[idx] : (int64_t)((const uint8_t*)q)[idx];
                y[idx] = orc_f32_to_f16(orc_dequantize_value(v, scales[a], zps[a]));
            }
}

/* ------------------------------------------------------------------ Eltwise */

/* Minimum / Maximum (OpenVINO operator semantics; the kernel sources are absent, so parity unpinned): IEEE 754-2008
 * minNum / maxNum -- a NaN operand yields the other operand, NaN only when both are -- with -0 ordered below +0, so
 * that the result is one definite bit pattern for every pair of inputs. */
static float elt_min(float a, float b) {
    if (isnan(a)) return b;
    if (isnan(b)) return a;
    if (a == b) return signbit(a) ? a : b;
    return a < b ? a : b;
}
static float elt_max(float a, float b) {
    if (isnan(a)) return b;
    if (isnan(b)) return a;
    if (a == b) return signbit(a) ? b : a;
    return a > b ? a : b;
}

static float elt_apply(int op, float a, float b) {
    switch (op) {
    case ORC_ELT_ADD: return a + b;
    case ORC_ELT_SUB: return a - b;
    case ORC_ELT_MUL: return a * b;
    case ORC_ELT_MIN: return elt_min(a, b);
    case ORC_ELT_MAX: return elt_max(a, b);
    case ORC_ELT_DIV: return a / b;
    case ORC_ELT_PRELU: return a < 0.0f ? a * b : a;
    default: return 0.0f;
    }
}

/* float16 arithmetic = fp32 op then RNE, include/vpux/utils/core/type/float16.hpp:123-126 */
void orc_eltwise_f16(int op, const uint16_t* a, const uint16_t* b, uint16_t* y, int rank, const int64_t* dims,
                     const int64_t* a_dims, const int64_t* b_dims) {
    int64_t total = 1;
    for (int d = 0; d < rank; d++) total *= dims[d];
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < total; i++) {
        int64_t idx[16];
        unravel(i, rank, dims, idx);
        const float fa = orc_f16_to_f32(a[bcast_offset(rank, idx, a_dims)]);
        const float fb = orc_f16_to_f32(b[bcast_offset(rank, idx, b_dims)]);
        y[i] = orc_f32_to_f16(elt_apply(op, fa, fb));
    }
}

/* ------------------------------------------------------------------ Activations */

/* OpenVINO operator definitions of the unary VPU ops that lower to the activation kernels
 * (src/vpux_compiler/src/dialect/VPUIP/IR/ops/sw_kernel.cpp:650-941, 1266-1285, 1689-1845);
 * fp32 arithmetic, one rounding. */
float orc_activation(int op, float x, float p0, float p1) {
    switch (op) {
    case ORC_ACT_RELU: return x > 0.0f ? x : 0.0f;
    case ORC_ACT_LEAKY_RELU: return x < 0.0f ? x * p0 : x;
    case ORC_ACT_CLAMP: return x < p0 ? p0 : (x > p1 ? p1 : x);
    case ORC_ACT_NEGATIVE: return -x;
    case ORC_ACT_ABS: return fabsf(x);
    case ORC_ACT_HSWISH: return x * fminf(fmaxf(x + 3.0f, 0.0f), 6.0f) / 6.0f;
    case ORC_ACT_HSIGMOID: return fminf(fmaxf(x + 3.0f, 0.0f), 6.0f) / 6.0f;
    case ORC_ACT_HARDSIGMOID: return fmaxf(0.0f, fminf(1.0f, p0 * x + p1));
    case ORC_ACT_SIGMOID: return 1.0f / (1.0f + expf(-x));
    case ORC_ACT_TANH: return tanhf(x);
    case ORC_ACT_EXP: return expf(x);
    case ORC_ACT_SQRT: return sqrtf(x);
    case ORC_ACT_LOG: return logf(x);
    case ORC_ACT_FLOOR: return floorf(x);
    case ORC_ACT_CEIL: return ceilf(x);
    case ORC_ACT_SIGN: return x > 0.0f ? 1.0f : (x < 0.0f ? -1.0f : x);
    case ORC_ACT_ELU: return x < 0.0f ? p0 * (expf(x) - 1.0f) : x;
    case ORC_ACT_SELU: return x > 0.0f ? p1 * x : p0 * p1 * (expf(x) - 1.0f);
    case ORC_ACT_SWISH: return x / (1.0f + expf(-p0 * x));
    case ORC_ACT_MISH: return x * tanhf(x < 20.0f ? log1pf(expf(x)) : x);
    case ORC_ACT_SOFTPLUS: return x < 20.0f ? log1pf(expf(x)) : x;
    case ORC_ACT_GELU: return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
    case ORC_ACT_ERF: return erff(x);
    default: return 0.0f;
    }
}

void orc_activation_f16(int op, float p0, float p1, const uint16_t* x, uint16_t* y, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) y[i] = orc_f32_to_f16(orc_activation(op, orc_f16_to_f32(x[i]), p0, p1));
}

void orc_activation_f32(int op, float p0, float p1, const float* x, float* y, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) y[i] = orc_activation(op, x[i], p0, p1);
}

/* ------------------------------------------------------------------ Softmax */

/* y = exp(x - max) / sum(exp(x - max)) along the axis; fp32 exp, the running sum is
 * kept in double so the oracle does not favour one fp32 summation order. */
void orc_softmax_f32(const float* x, float* y, int64_t outer, int64_t axis, int64_t inner, int64_t pad) {
    const int64_t valid = axis - pad;
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t o = 0; o < outer; o++) {
        for (int64_t i = 0; i < inner; i++) {
            const float* px = x + o * axis * inner + i;
            float* py = y + o * axis * inner + i;
            float mx = -INFINITY;
            for (int64_t a = 0; a < valid; a++) mx = fmaxf(mx, px[a * inner]);
            double sum = 0.0;
            for (int64_t a = 0; a < valid; a++) sum += (double)expf(px[a * inner] - mx);
            for (int64_t a = 0; a < valid; a++) py[a * inner] = (float)((double)expf(px[a * inner] - mx) / sum);
            for (int64_t a = valid; a < axis; a++) py[a * inner] = 0.0f;
        }
    }
}

void orc_softmax_f16(const uint16_t* x, uint16_t* y, int64_t outer, int64_t axis, int64_t inner, int64_t pad) {
    const int64_t valid = axis - pad;
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t o = 0; o < outer; o++) {
        for (int64_t i = 0; i < inner; i++) {
            const uint16_t* px = x + o * axis * inner + i;
            uint16_t* py = y + o * axis * inner + i;
            float mx = -INFINITY;
            for (int64_t a = 0; a < valid; a++) mx = fmaxf(mx, orc_f16_to_f32(px[a * inner]));
            double sum = 0.0;
            for (int64_t a = 0; a < valid; a++) sum += (double)expf(orc_f16_to_f32(px[a * inner]) - mx);
            for (int64_t a = 0; a < valid; a++) {
                const double e = (double)expf(orc_f16_to_f32(px[a * inner]) - mx);
                py[a * inner] = orc_f32_to_f16_ieee((float)(e / sum));
            }
            for (int64_t a = valid; a < axis; a++) py[a * inner] = 0;
        }
    }
}

/* ------------------------------------------------------------------ MVN-1 */

/* mean and biased variance over (C,S) per n when across_channels, else over S per (n,c);
 * y = (x-mean)/sqrt(var+eps) (eps inside the sqrt) or x-mean.  Two-pass, double accumulators. */
void orc_mvn_f16(const uint16_t* x, uint16_t* y, int64_t N, int64_t C, int64_t S, int64_t stride_n, int64_t stride_c,
                 int64_t stride_s, int across_channels, int normalize_variance, float eps) {
    const int64_t groups = across_channels ? N : N * C;
    const int64_t gc = across_channels ? C : 1;
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t g = 0; g < groups; g++) {
        const int64_t n = across_channels ? g : g / C;
        const int64_t c0 = across_channels ? 0 : g % C;
        const int64_t base = n * stride_n + c0 * stride_c;
        const double cnt = (double)(gc * S);
        double sum = 0.0;
        for (int64_t c = 0; c < gc; c++)
            for (int64_t s = 0; s < S; s++) sum += (double)orc_f16_to_f32(x[base + c * stride_c + s * stride_s]);
        const double mean = sum / cnt;
        double sq = 0.0;
        for (int64_t c = 0; c < gc; c++)
            for (int64_t s = 0; s < S; s++) {
                const double d = (double)orc_f16_to_f32(x[base + c * stride_c + s * stride_s]) - mean;
                sq += d * d;
            }
        const double var = sq / cnt;
        const double inv = normalize_variance ? 1.0 / sqrt(var + (double)eps) : 1.0;
        for (int64_t c = 0; c < gc; c++)
            for (int64_t s = 0; s < S; s++) {
                const int64_t off = base + c * stride_c + s * stride_s;
                y[off] = orc_f32_to_f16_ieee((float)(((double)orc_f16_to_f32(x[off]) - mean) * inv));
            }
    }
}

/* ------------------------------------------------------------------ scale approximation */

/* approximate<>, include/vpux/compiler/utils/quantization.hpp:65-78 */
int orc_approximate(int bits, double target, int64_t* mult, int64_t* shift, int64_t* post_shift) {
    int exponent = 0;
    const double mantissa = frexp(target, &exponent);
    const double m = floor(mantissa * pow(2.0, bits));
    if (m > 2147483647.0 || m < -2147483648.0) return -1;
    *mult = (int64_t)m;
    *shift = exponent > bits ? 0 : bits - exponent;
    *post_shift = exponent > bits ? bits - exponent : 0;
    return 0;
}

/* arch37xx::getScale for quantized input, nce_sparsity_converters.cpp:22-29 */
int32_t orc_wt_pack_scale(uint8_t shift, int16_t mult) {
    return (int32_t)(((uint32_t)shift << 8) | ((uint32_t)(int32_t)mult << 16));
}
void orc_wt_unpack_scale(int32_t word, int32_t* mult, int32_t* shift) {
    *mult = (int32_t)(int16_t)((uint32_t)word >> 16);
    *shift = (int32_t)(((uint32_t)word >> 8) & 0xffu);
}

/* ------------------------------------------------------------------ integer PPE */

/* Order of operations as emitted by buildIntPPEConfig
 * (expand_dpu_config_invariant_ppe.cpp:322-380): bias add, scale multiply, scale shift,
 * prelu multiply and prelu shift on negative values, a single round-to-nearest-even over
 * the combined shift (round mode RNE, :51-53), zero-point offset, clamp, convert. */
static int64_t shift_round_half_even(int64_t t, int s) {
    if (s <= 0) return t;
    if (s >= 64) return 0; /* |t| < 2^63 so |t / 2^s| < 1/2 */
    const int64_t q = t >> s; /* floor */
    const uint64_t mask = (1ull << s) - 1ull;
    const uint64_t rem = (uint64_t)t & mask;
    const uint64_t half = 1ull << (s - 1);
    if (rem > half || (rem == half && (q & 1))) return q + 1;
    return q;
}

int32_t orc_ppe_requant(int32_t acc, int32_t bias, int32_t mult, int32_t shift, const orc_ppe_t* ppe) {
    const int32_t biased = (int32_t)((uint32_t)acc + (uint32_t)bias); /* 32-bit accumulator wraps */
    int64_t t = (int64_t)biased * (int64_t)mult;
    int s = shift;
    if (t < 0) {
        t *= (int64_t)ppe->prelu_mult;
        s += ppe->prelu_shift;
    }
    int64_t r = shift_round_half_even(t, s);
    r += ppe->zp_out;
    if (r < ppe->clamp_low) r = ppe->clamp_low;
    if (r > ppe->clamp_high) r = ppe->clamp_high;
    return (int32_t)r;
}

/* fp16 output of an integer convolution: "INT32 s17.15 fixed-point convert to FP16"
 * (runtime_dpu_parser_imports.cpp.inc:546-552, ppe_i32_convert = 1).  The pipeline is the same up to
 * the round stage, which here keeps 15 fractional bits: fx = round_half_even(t / 2^(s - 15)) saturated
 * to 32 bits is the s17.15 number, fx * 2^-15 is narrowed to fp16 with one round-to-nearest-even
 * (65520 and above become infinity), and the clamp is the pair of fp16 bounds the compiler packs into
 * clamp_high as 0xllllhhhh (dialect/VPU/utils/ppe_utils.hpp:36-87; clamp_low is ignored by that
 * convention and 0x7fffffff, whose halves are not numbers, means no clamp).  No zero point is added
 * (setupQuantInFloatOut programs none).  "parity unpinned" against silicon like orc_ppe_requant. */
static uint16_t s1715_to_f16(int64_t fx) {
    const uint16_t sign = fx < 0 ? 0x8000u : 0u;
    uint64_t a = (uint64_t)(fx < 0 ? -fx : fx); /* value = a * 2^-15 */
    if (a == 0) return sign;
    int top = 63;
    while (!((a >> top) & 1u)) top--; /* a in [2^top, 2^(top+1)) : value in [2^(top-15), ...) */
    int e = top - 15;                 /* unbiased exponent of the value */
    int drop;                         /* low bits of a that do not fit the significand */
    if (e < -14) {                    /* subnormal half: quantum 2^-24 = a-units of 2^-9; nothing is dropped */
        return (uint16_t)(sign | (uint16_t)(a << 9));
    }
    drop = top - 10;
    uint64_t q = a, rem = 0, half = 0;
    if (drop > 0) {
        q = a >> drop;
        rem = a & ((1ull << drop) - 1ull);
        half = 1ull << (drop - 1);
        if (rem > half || (rem == half && (q & 1ull))) q++;
        if (q == (1ull << 11)) { /* carried into the next binade */
            q >>= 1;
            e++;
        }
    } else {
        q = a << (-drop);
    }
    if (e > 15) return (uint16_t)(sign | 0x7c00u);
    return (uint16_t)(sign | (uint16_t)((e + 15) << 10) | (uint16_t)(q & 0x3ffu));
}

uint16_t orc_ppe_requant_f16(int32_t acc, int32_t bias, int32_t mult, int32_t shift, const orc_ppe_t* ppe) {
    const int32_t biased = (int32_t)((uint32_t)acc + (uint32_t)bias);
    int64_t t = (int64_t)biased * (int64_t)mult;
    int s = shift;
    if (t < 0) {
        t *= (int64_t)ppe->prelu_mult;
        s += ppe->prelu_shift;
    }
    s -= 15;
    int64_t fx;
    if (s >= 0) {
        fx = shift_round_half_even(t, s);
    } else {
        const int up = -s; /* at most 15: |t| < 2^58 may overflow 64 bits only when it saturates anyway */
        if (t > (INT64_MAX >> up)) fx = INT64_MAX;
        else if (t < -(INT64_MAX >> up)) fx = -INT64_MAX;
        else fx = t * ((int64_t)1 << up);
    }
    if (fx > INT32_MAX) fx = INT32_MAX;
    if (fx < INT32_MIN) fx = INT32_MIN;
    uint16_t h = s1715_to_f16(fx);
    if (ppe->clamp_high != INT32_MAX) {
        const uint16_t hi = (uint16_t)((uint32_t)ppe->clamp_high & 0xffffu);
        const uint16_t lo = (uint16_t)(((uint32_t)ppe->clamp_high >> 16) & 0xffffu);
        const float v = orc_f16_to_f32(h);
        if ((lo & 0x7fffu) <= 0x7c00u && v < orc_f16_to_f32(lo)) h = lo;
        if ((hi & 0x7fffu) <= 0x7c00u && v > orc_f16_to_f32(hi)) h = hi;
    }
    return h;
}

/* ------------------------------------------------------------------ NCE conv / matmul */

static inline int32_t load8(const void* p, int64_t i, int is_signed) {
    return is_signed ? (int32_t)((const int8_t*)p)[i] : (int32_t)((const uint8_t*)p)[i];
}

/* acc[n,oy,ox,oc] = sum over valid taps of (in - zp_in) * (w - zp_w); padded taps add 0
 * (MPE zero points: runtime_dpu_parser_imports.cpp.inc:872-875,940-945; no pad value :877-879). */
void orc_nce_conv_rows(const orc_conv_t* d, const void* in, const void* w, const int32_t* wt, void* out,
                       int32_t* acc_out, int64_t row0, int64_t nrows) {
    const int64_t OH = (d->H + d->pad_top + d->pad_bottom - d->KY) / d->stride_y + 1;
    const int64_t OW = (d->W + d->pad_left + d->pad_right - d->KX) / d->stride_x + 1;
    const int64_t IC = d->IC, OC = d->OC;
    const int fast = d->in_signed == 0 && d->w_signed == 1;
    /* dense unless strides are given */
    const int in_view = (d->in_strides[0] | d->in_strides[1] | d->in_strides[2]) != 0;
    const int out_view = (d->out_strides[0] | d->out_strides[1] | d->out_strides[2]) != 0;
    const int64_t isw = in_view ? d->in_strides[2] : IC, ish = in_view ? d->in_strides[1] : d->W * IC,
                  isn = in_view ? d->in_strides[0] : d->H * d->W * IC;
    const int64_t osw = out_view ? d->out_strides[2] : OC, osh = out_view ? d->out_strides[1] : OW * OC,
                  osn = out_view ? d->out_strides[0] : OH * OW * OC;
#pragma omp parallel for schedule(dynamic, 16)
    for (int64_t row = row0; row < row0 + nrows; row++) {
        const int64_t n = row / (OH * OW);
        const int64_t oy = (row / OW) % OH;
        const int64_t ox = row % OW;
        const int64_t obase = n * osn + oy * osh + ox * osw;
        for (int64_t oc = 0; oc < OC; oc++) {
            int32_t acc = 0;
            for (int64_t ky = 0; ky < d->KY; ky++) {
                const int64_t iy = oy * d->stride_y + ky - d->pad_top;
                if (iy < 0 || iy >= d->H) continue;
                for (int64_t kx = 0; kx < d->KX; kx++) {
                    const int64_t ix = ox * d->stride_x + kx - d->pad_left;
                    if (ix < 0 || ix >= d->W) continue;
                    const int64_t ibase = n * isn + iy * ish + ix * isw;
                    const int64_t wbase = ((oc * d->KY + ky) * d->KX + kx) * IC;
                    int32_t part = 0;
                    if (fast) {
                        const uint8_t* pi = (const uint8_t*)in + ibase;
                        const int8_t* pw = (const int8_t*)w + wbase;
                        for (int64_t ic = 0; ic < IC; ic++)
                            part += ((int32_t)pi[ic] - d->zp_in) * ((int32_t)pw[ic] - d->zp_w);
                    } else if (d->in_signed && d->w_signed) {
                        const int8_t* pi = (const int8_t*)in + ibase;
                        const int8_t* pw = (const int8_t*)w + wbase;
                        for (int64_t ic = 0; ic < IC; ic++)
                            part += ((int32_t)pi[ic] - d->zp_in) * ((int32_t)pw[ic] - d->zp_w);
                    } else {
                        for (int64_t ic = 0; ic < IC; ic++)
                            part += (load8(in, ibase + ic, d->in_signed) - d->zp_in) *
                                    (load8(w, wbase + ic, d->w_signed) - d->zp_w);
                    }
                    acc += part;
                }
            }
            int32_t mult, shift;
            orc_wt_unpack_scale(wt[oc * 4 + 2], &mult, &shift);
            if (acc_out) acc_out[row * OC + oc] = acc;
            if (d->out_signed == 2) { /* fp16 output */
                ((uint16_t*)out)[obase + oc] = orc_ppe_requant_f16(acc, wt[oc * 4 + 3], mult, shift, &d->ppe);
                continue;
            }
            const int32_t r = orc_ppe_requant(acc, wt[oc * 4 + 3], mult, shift, &d->ppe);
            /* convert: saturate to the storage type */
            if (d->out_signed)
                ((int8_t*)out)[obase + oc] = (int8_t)(r < -128 ? -128 : (r > 127 ? 127 : r));
            else
                ((uint8_t*)out)[obase + oc] = (uint8_t)(r < 0 ? 0 : (r > 255 ? 255 : r));
        }
    }
}

void orc_nce_conv(const orc_conv_t* d, const void* in, const void* w, const int32_t* wt, void* out, int32_t* acc_out) {
    const int64_t OH = (d->H + d->pad_top + d->pad_bottom - d->KY) / d->stride_y + 1;
    const int64_t OW = (d->W + d->pad_left + d->pad_right - d->KX) / d->stride_x + 1;
    orc_nce_conv_rows(d, in, w, wt, out, acc_out, 0, d->N * OH * OW);
}

void orc_nce_eltwise(const void* a, int a_signed, const void* b, int b_signed, void* out, int out_signed, int64_t n,
                     int32_t zp_a, int32_t zp_b, int32_t mult_a, int32_t mult_b, int subtract, int32_t out_mult,
                     int32_t out_shift, const orc_ppe_t* ppe) {
    const uint8_t* pa = (const uint8_t*)a;
    const uint8_t* pb = (const uint8_t*)b;
    uint8_t* po = (uint8_t*)out;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        const int32_t va = (a_signed ? (int32_t)(int8_t)pa[i] : (int32_t)pa[i]) - zp_a;
        const int32_t vb = (b_signed ? (int32_t)(int8_t)pb[i] : (int32_t)pb[i]) - zp_b;
        const int32_t acc = va * mult_a + (subtract ? -1 : 1) * vb * mult_b;
        int32_t r = orc_ppe_requant(acc, 0, out_mult, out_shift, ppe);
        if (out_signed) r = r < -128 ? -128 : (r > 127 ? 127 : r);
        else r = r < 0 ? 0 : (r > 255 ? 255 : r);
        po[i] = (uint8_t)r;
    }
}

/* The same task with an fp16 output: the sum goes through the fixed-point PPE of orc_ppe_requant_f16 (no output zero
 * point).  "parity unpinned" against silicon like that function. */
void orc_nce_eltwise_f16(const void* a, int a_signed, const void* b, int b_signed, uint16_t* out, int64_t n, int32_t zp_a,
                         int32_t zp_b, int32_t mult_a, int32_t mult_b, int subtract, int32_t out_mult, int32_t out_shift,
                         const orc_ppe_t* ppe) {
    const uint8_t* pa = (const uint8_t*)a;
    const uint8_t* pb = (const uint8_t*)b;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        const int32_t va = (a_signed ? (int32_t)(int8_t)pa[i] : (int32_t)pa[i]) - zp_a;
        const int32_t vb = (b_signed ? (int32_t)(int8_t)pb[i] : (int32_t)pb[i]) - zp_b;
        const int32_t acc = va * mult_a + (subtract ? -1 : 1) * vb * mult_b;
        out[i] = orc_ppe_requant_f16(acc, 0, out_mult, out_shift, ppe);
    }
}

/* The two eltwise functions above on views of larger tensors: one pixel's channels at a time, through the same
 * per-value functions. */
void orc_nce_eltwise_views(const void* a, int a_signed, const void* b, int b_signed, void* out, int out_kind,
                           const int64_t dims[4], const int64_t a_strides[3], const int64_t b_strides[3],
                           const int64_t out_strides[3], int32_t zp_a, int32_t zp_b, int32_t mult_a, int32_t mult_b,
                           int subtract, int32_t out_mult, int32_t out_shift, const orc_ppe_t* ppe) {
    const int64_t N = dims[0], H = dims[1], W = dims[2], Cn = dims[3];
#pragma omp parallel for schedule(static)
    for (int64_t pixel = 0; pixel < N * H * W; pixel++) {
        const int64_t n = pixel / (H * W), y = (pixel / W) % H, x = pixel % W;
        const uint8_t* pa = (const uint8_t*)a + n * a_strides[0] + y * a_strides[1] + x * a_strides[2];
        const uint8_t* pb = (const uint8_t*)b + n * b_strides[0] + y * b_strides[1] + x * b_strides[2];
        const int64_t o = n * out_strides[0] + y * out_strides[1] + x * out_strides[2];
        if (out_kind == 2)
            orc_nce_eltwise_f16(pa, a_signed, pb, b_signed, (uint16_t*)out + o, Cn, zp_a, zp_b, mult_a, mult_b, subtract, out_mult,
                                out_shift, ppe);
        else
            orc_nce_eltwise(pa, a_signed, pb, b_signed, (uint8_t*)out + o, out_kind, Cn, zp_a, zp_b, mult_a, mult_b, subtract,
                            out_mult, out_shift, ppe);
    }
}
