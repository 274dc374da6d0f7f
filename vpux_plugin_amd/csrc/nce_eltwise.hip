// Task type ELTWISE of the NCE task: the quantized add / subtract of two 8-bit tensors.
#include "nce_common.h"

namespace vpx {
namespace nce {
namespace {

// ---------------------------------------------------------------- NCE eltwise (quantized add / subtract)
// out = PPE((a - zp_a) * m1 +/- (b - zp_b) * m2): a streaming kernel, 16 bytes of each operand per
// lane.  The zero points are folded into the bias (acc = a * m1 +/- b * m2 - (zp_a * m1 +/- zp_b * m2)),
// which leaves two 24-bit multiply-adds per value in front of the shared PPE tail.
struct EltParams {
    int m1, m2;  // m2 negated for a subtraction
    ChanPrep cp;
    PpePack pk;
    int general;
    ChanPrep cp16;         // fp16 output: the factors with 15 fractional bits kept, plain form (see ppe_fast_f16)
    float f16_lo, f16_hi;  // and its clamp bounds
};

// OUT_F16: sixteen sums leave as sixteen fp16 values (two 16-byte stores per lane).
template <bool A_SIGNED, bool B_SIGNED, bool SAME_F, bool OUT_F16 = false>
__global__ __launch_bounds__(256) void nce_eltwise_kernel(const uint8_t* __restrict__ a, const uint8_t* __restrict__ b,
                                                          uint8_t* __restrict__ out, int64_t n_vec, int64_t n,
                                                          EltParams e) {
    auto val = [](unsigned word, int k, bool sgn) {
        return sgn ? (int)(int8_t)(word >> (8 * k)) : (int)((word >> (8 * k)) & 0xffu);
    };
    if constexpr (OUT_F16) {
        uint16_t* out16 = reinterpret_cast<uint16_t*>(out);
        const int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
        if (v < n_vec) {
            const i32x4 qa = reinterpret_cast<const i32x4*>(a)[v];
            const i32x4 qb = reinterpret_cast<const i32x4*>(b)[v];
            i32x4 r[2] = {i32x4{0, 0, 0, 0}, i32x4{0, 0, 0, 0}};
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const int acc = val((unsigned)qa[j], k, A_SIGNED) * e.m1 + val((unsigned)qb[j], k, B_SIGNED) * e.m2;
                    const int idx = 4 * j + k;  // value idx of the sixteen: half (idx % 2) of dword idx / 2
                    r[idx >> 3][(idx >> 1) & 3] |= (int)ppe_fast_f16(acc, e.cp16, e.f16_lo, e.f16_hi) << (16 * (idx & 1));
                }
            __builtin_nontemporal_store(r[0], reinterpret_cast<i32x4*>(out16) + 2 * v);
            __builtin_nontemporal_store(r[1], reinterpret_cast<i32x4*>(out16) + 2 * v + 1);
        }
        if (blockIdx.x == gridDim.x - 1) {
            for (int64_t i = n_vec * 16 + threadIdx.x; i < n; i += 256) {
                const int acc = val(a[i], 0, A_SIGNED) * e.m1 + val(b[i], 0, B_SIGNED) * e.m2;
                out16[i] = ppe_fast_f16(acc, e.cp16, e.f16_lo, e.f16_hi);
            }
        }
        return;
    }
    auto four = [&](unsigned wa, unsigned wb, auto general_c) {
        int acc[4];
#pragma unroll
        for (int k = 0; k < 4; k++) acc[k] = val(wa, k, A_SIGNED) * e.m1 + val(wb, k, B_SIGNED) * e.m2;
        return ppe_pack4<SAME_F, decltype(general_c)::value>(acc[0], acc[1], acc[2], acc[3], e.cp, e.pk);
    };
    const int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (v < n_vec) {
        const i32x4 qa = reinterpret_cast<const i32x4*>(a)[v];
        const i32x4 qb = reinterpret_cast<const i32x4*>(b)[v];
        i32x4 r;
        if (e.general) {
#pragma unroll
            for (int j = 0; j < 4; j++) r[j] = (int)four((unsigned)qa[j], (unsigned)qb[j], std::true_type{});
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) r[j] = (int)four((unsigned)qa[j], (unsigned)qb[j], std::false_type{});
        }
        __builtin_nontemporal_store(r, reinterpret_cast<i32x4*>(out) + v);
    }
    // ragged tail (fewer than 16 bytes) and unaligned tensors: one value per lane
    if (blockIdx.x == gridDim.x - 1) {
        for (int64_t i = n_vec * 16 + threadIdx.x; i < n; i += 256) {
            const int acc = val(a[i], 0, A_SIGNED) * e.m1 + val(b[i], 0, B_SIGNED) * e.m2;
            out[i] = (uint8_t)ppe_pack4<SAME_F, true>(acc, 0, 0, 0, e.cp, e.pk);
        }
    }
}

// The same task on operands that are views of larger tensors (strides per image, row and pixel; a pixel's channels
// are contiguous): a lane takes up to sixteen channels of one pixel, in 16-byte accesses where the operand's base and
// strides allow, else byte by byte.
struct EltViews {
    int64_t H, W, C;
    int64_t asn, ash, asw, bsn, bsh, bsw, osn, osh, osw;  // a and b in bytes, the output in elements
    int cpp;            // sixteen-channel chunks per pixel
    int in_vec;         // both inputs: base and strides are multiples of 16 bytes
    unsigned out_bits;  // the output's base address and strides in bytes, or-ed
};

template <bool A_SIGNED, bool B_SIGNED, bool SAME_F, bool OUT_F16>
__global__ __launch_bounds__(256) void nce_eltwise_views_kernel(const uint8_t* __restrict__ a, const uint8_t* __restrict__ b,
                                                                uint8_t* __restrict__ out, int64_t chunks, EltViews ev, EltParams e) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= chunks) return;
    const int64_t pixel = t / ev.cpp;
    const int c0 = (int)(t - pixel * ev.cpp) * 16;
    const int64_t hw = ev.H * ev.W, n = pixel / hw, rem = pixel - n * hw, y = rem / ev.W, x = rem - y * ev.W;
    const uint8_t* pa = a + (n * ev.asn + y * ev.ash + x * ev.asw + c0);
    const uint8_t* pb = b + (n * ev.bsn + y * ev.bsh + x * ev.bsw + c0);
    const int64_t o = n * ev.osn + y * ev.osh + x * ev.osw + c0;
    const int count = ev.C - c0 < 16 ? (int)(ev.C - c0) : 16;
    i32x4 qa = i32x4{0, 0, 0, 0}, qb = i32x4{0, 0, 0, 0};
    if (ev.in_vec && count == 16) {
        qa = *reinterpret_cast<const i32x4*>(pa);
        qb = *reinterpret_cast<const i32x4*>(pb);
    } else {
        for (int k = 0; k < count; k++) {
            qa[k >> 2] |= (int)pa[k] << (8 * (k & 3));
            qb[k >> 2] |= (int)pb[k] << (8 * (k & 3));
        }
    }
    auto val = [](unsigned word, int k, bool sgn) {
        return sgn ? (int)(int8_t)(word >> (8 * k)) : (int)((word >> (8 * k)) & 0xffu);
    };
    if constexpr (OUT_F16) {
        uint16_t* const po = reinterpret_cast<uint16_t*>(out) + o;
        i32x4 r[2] = {i32x4{0, 0, 0, 0}, i32x4{0, 0, 0, 0}};
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int acc = val((unsigned)qa[j], k, A_SIGNED) * e.m1 + val((unsigned)qb[j], k, B_SIGNED) * e.m2;
                const int idx = 4 * j + k;
                r[idx >> 3][(idx >> 1) & 3] |= (int)ppe_fast_f16(acc, e.cp16, e.f16_lo, e.f16_hi) << (16 * (idx & 1));
            }
        if ((ev.out_bits & 15) == 0 && count == 16) {
            __builtin_nontemporal_store(r[0], reinterpret_cast<i32x4*>(po));
            __builtin_nontemporal_store(r[1], reinterpret_cast<i32x4*>(po) + 1);
        } else {
            const int al = out_align(ev.out_bits);
            store_tail16(reinterpret_cast<uint8_t*>(po), r[0], (count < 8 ? count : 8) * 2, al);
            if (count > 8) store_tail16(reinterpret_cast<uint8_t*>(po + 8), r[1], (count - 8) * 2, al);
        }
    } else {
        i32x4 r;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            int acc[4];
#pragma unroll
            for (int k = 0; k < 4; k++) acc[k] = val((unsigned)qa[j], k, A_SIGNED) * e.m1 + val((unsigned)qb[j], k, B_SIGNED) * e.m2;
            r[j] = (int)ppe_pack4<SAME_F, true>(acc[0], acc[1], acc[2], acc[3], e.cp, e.pk);
        }
        if ((ev.out_bits & 15) == 0 && count == 16) __builtin_nontemporal_store(r, reinterpret_cast<i32x4*>(out + o));
        else store_tail16(out + o, r, count, out_align(ev.out_bits));
    }
}

}  // namespace

// PPE of one eltwise value on the host: decides which device variant is needed
int launch_nce_eltwise(const vpx_nce_task_t& t, const Ppe& ppe, hipStream_t s, const char** kernel_name) {
    const bool a_signed = t.input_type == VPX_NN_I8, b_signed = t.weights_type == VPX_NN_I8, out_signed = t.output_type == VPX_NN_I8;
    const bool out_f16 = t.output_type == VPX_NN_FP16;
    const int64_t n = t.N * t.H * t.W * t.IC;
    *kernel_name = "nce_eltwise_kernel";
    if (n == 0) return VPX_RESULT_SUCCESS;
    const int sign = t.eltwise_type == VPX_ELTWISE_SUBTRACT ? -1 : 1;
    const long long bias = -((long long)t.zp_in * t.ppe.in1_quant_mult + (long long)sign * t.zp_w * t.ppe.in2_quant_mult);
    VPX_REQUIRE(bias > -(1ll << 30) && bias < (1ll << 30), VPX_RESULT_ERROR_INVALID_ARGUMENT,
                "NCE eltwise: zero points and input multipliers do not fit the 32-bit accumulator");
    const int tmin = out_signed ? -128 : 0, tmax = out_signed ? 127 : 255;
    int lo = ppe.clamp_lo > tmin ? ppe.clamp_lo : tmin, hi = ppe.clamp_hi < tmax ? ppe.clamp_hi : tmax;
    if (lo > tmax) lo = tmax;
    if (hi < tmin) hi = tmin;
    if (lo > hi) lo = hi;
    EltParams e{};
    e.m1 = t.ppe.in1_quant_mult;
    e.m2 = sign * t.ppe.in2_quant_mult;
    // host copy of ppe_prepare_packed / make_ppe_pack
    const double f_pos = std::ldexp((double)t.ppe.quant_mult, -t.ppe.quant_shift);
    const double f_neg = std::ldexp((double)((long long)t.ppe.quant_mult * (long long)ppe.prelu_mult), -(t.ppe.quant_shift + ppe.prelu_shift));
    auto bmax = [](double f) {
        const float a = std::fabs((float)f);
        return a <= 0.5f ? 0x7fffffff : (int)(1.0e9f / a);
    };
    const bool swap = t.ppe.quant_mult < 0;  // as ppe_prepare_packed does
    e.cp.f_pos = swap ? f_neg : f_pos;
    e.cp.f_neg = swap ? f_pos : f_neg;
    e.cp.bias = (int)((unsigned)(int)bias + 0x80000000u);
    e.cp.sgn = swap ? -1 : 0;
    e.cp.bmax_pos = bmax(e.cp.f_pos);
    e.cp.bmax_neg = bmax(e.cp.f_neg);
    const int off = out_signed ? 128 : 0, z = t.zp_out + off;
    e.pk = PpePack{6755399441055744.0 + (double)(z & ~1), z & 1, lo + off, hi + off, out_signed ? 0x80808080u : 0u};
    e.general = (e.cp.bmax_pos != 0x7fffffff || e.cp.bmax_neg != 0x7fffffff || (z & 1)) ? 1 : 0;
    // host copy of ppe_prepare with shift - 15 (an fp16 output keeps 15 fractional bits of the scaled value)
    e.cp16.f_pos = std::ldexp((double)t.ppe.quant_mult, -(t.ppe.quant_shift - 15));
    e.cp16.f_neg = std::ldexp((double)((long long)t.ppe.quant_mult * (long long)ppe.prelu_mult), -(t.ppe.quant_shift - 15 + ppe.prelu_shift));
    e.cp16.bias = (int)bias;
    e.cp16.sgn = t.ppe.quant_mult < 0 ? -1 : 0;
    e.cp16.bmax_pos = e.cp16.bmax_neg = 0x7fffffff;
    e.f16_lo = ppe.f16_lo;
    e.f16_hi = ppe.f16_hi;
    const bool same_f = ppe.prelu_mult == 1 && ppe.prelu_shift == 0;
    View va, vb, vo;
    int vrc = operand_view(t.input_strides, t.N, t.H, t.W, t.IC, "first input", &va);
    if (!vrc) vrc = operand_view(t.weights_strides, t.N, t.H, t.W, t.IC, "second input", &vb);
    if (!vrc) vrc = operand_view(t.output_strides, t.N, t.H, t.W, t.IC, "output", &vo);
    if (vrc) return vrc;
    if (!(va.dense && vb.dense && vo.dense)) {
        // views of larger tensors: up to sixteen channels of a pixel per lane
        EltViews ev{};
        ev.H = t.H; ev.W = t.W; ev.C = t.IC;
        ev.asn = va.sn; ev.ash = va.sh; ev.asw = va.sw;
        ev.bsn = vb.sn; ev.bsh = vb.sh; ev.bsw = vb.sw;
        ev.osn = vo.sn; ev.osh = vo.sh; ev.osw = vo.sw;
        ev.cpp = (int)((t.IC + 15) / 16);
        ev.in_vec = ((reinterpret_cast<uintptr_t>(t.input) | reinterpret_cast<uintptr_t>(t.weights) | (uintptr_t)(va.sn | va.sh | va.sw) |
                      (uintptr_t)(vb.sn | vb.sh | vb.sw)) & 15) == 0 ? 1 : 0;
        const int ob = out_f16 ? 2 : 1;
        ev.out_bits = (unsigned)(reinterpret_cast<uintptr_t>(t.output) | (uintptr_t)((vo.sn | vo.sh | vo.sw) * ob));
        VPX_REQUIRE(t.IC < (1ll << 31) - 16, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "NCE eltwise: %lld channels are too many", (long long)t.IC);
        const int64_t chunks = t.N * t.H * t.W * ev.cpp;
        const int64_t blocks = (chunks + 255) / 256;
        VPX_REQUIRE(blocks < (1ll << 31), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "NCE eltwise: tensor of %lld elements is too large", (long long)n);
#define VPX_ELTV(AS, BS, SF, F16)                                                                                      \
    hipLaunchKernelGGL((nce_eltwise_views_kernel<AS, BS, SF, F16>), dim3((unsigned)blocks), dim3(256), 0, s,          \
                       (const uint8_t*)t.input, (const uint8_t*)t.weights, (uint8_t*)t.output, chunks, ev, e)
#define VPX_ELTV_S(AS, BS)                                                                                             \
    do {                                                                                                               \
        if (out_f16) VPX_ELTV(AS, BS, false, true);                                                                    \
        else if (same_f) VPX_ELTV(AS, BS, true, false);                                                                \
        else VPX_ELTV(AS, BS, false, false);                                                                           \
    } while (0)
        if (a_signed && b_signed) VPX_ELTV_S(true, true);
        else if (a_signed) VPX_ELTV_S(true, false);
        else if (b_signed) VPX_ELTV_S(false, true);
        else VPX_ELTV_S(false, false);
#undef VPX_ELTV_S
#undef VPX_ELTV
        VPX_HIP_CHECK(hipGetLastError());
        *kernel_name = "nce_eltwise_views_kernel";
        return VPX_RESULT_SUCCESS;
    }
    const bool aligned = ((reinterpret_cast<uintptr_t>(t.input) | reinterpret_cast<uintptr_t>(t.weights) |
                           reinterpret_cast<uintptr_t>(t.output)) & 15) == 0;
    const int64_t n_vec = aligned ? n / 16 : 0;
    const int64_t blocks64 = n_vec > 0 ? (n_vec + 255) / 256 : 1;
    VPX_REQUIRE(blocks64 < (1ll << 31), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "NCE eltwise: tensor of %lld elements is too large", (long long)n);
    const dim3 grid((unsigned)blocks64), block(256);
#define VPX_ELT(AS, BS, SF)                                                                                            \
    hipLaunchKernelGGL((nce_eltwise_kernel<AS, BS, SF>), grid, block, 0, s, (const uint8_t*)t.input,                   \
                       (const uint8_t*)t.weights, (uint8_t*)t.output, n_vec, n, e)
#define VPX_ELT16(AS, BS)                                                                                              \
    hipLaunchKernelGGL((nce_eltwise_kernel<AS, BS, false, true>), grid, block, 0, s, (const uint8_t*)t.input,          \
                       (const uint8_t*)t.weights, (uint8_t*)t.output, n_vec, n, e)
    if (out_f16) {
        if (a_signed && b_signed) VPX_ELT16(true, true);
        else if (a_signed) VPX_ELT16(true, false);
        else if (b_signed) VPX_ELT16(false, true);
        else VPX_ELT16(false, false);
#undef VPX_ELT16
        VPX_HIP_CHECK(hipGetLastError());
        return VPX_RESULT_SUCCESS;
    }
    const int sel = (a_signed ? 4 : 0) | (b_signed ? 2 : 0) | (same_f ? 1 : 0);
    switch (sel) {
    case 0: VPX_ELT(false, false, false); break;
    case 1: VPX_ELT(false, false, true); break;
    case 2: VPX_ELT(false, true, false); break;
    case 3: VPX_ELT(false, true, true); break;
    case 4: VPX_ELT(true, false, false); break;
    case 5: VPX_ELT(true, false, true); break;
    case 6: VPX_ELT(true, true, false); break;
    default: VPX_ELT(true, true, true); break;
    }
#undef VPX_ELT
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

}  // namespace nce
}  // namespace vpx
