// Streaming ACT-SHAVE kernels: convert, eltwise_*, fake_quantize, quantize, dequantize.
//
// All of them are HBM-bound maps.  The fast path views compact operands as flat arrays and moves
// 128 bits per lane per access, several independent accesses in flight per lane; a strided /
// broadcasting path covers sub-views and NUMPY broadcast one element per lane.
#include <type_traits>
#include <vector>

#include "vpx_common.h"

#include <cstring>
#include <mutex>
#include <unordered_map>
#include <vector>

namespace vpx {

namespace {

typedef _Float16 half_t;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <int BYTES>
struct Words;
template <>
struct Words<1> {
    typedef uint8_t type;
};
template <>
struct Words<2> {
    typedef uint16_t type;
};
template <>
struct Words<4> {
    typedef uint32_t type;
};
template <>
struct Words<8> {
    typedef u32x2 type;
};
template <>
struct Words<16> {
    typedef u32x4 type;
};
typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));
template <>
struct Words<32> {
    typedef u32x8 type;  // two 128-bit accesses
};

// N elements of T moved by one 8...128-bit access per lane.  Adjacent lanes touch adjacent
// words, so a wavefront's access is one contiguous run; the wider operand of a kernel gets the
// 128-bit form.  Stores are non-temporal (results are not re-read); loads are ordinary, which
// measures faster than non-temporal loads on this memory system.
template <typename T, int N>
struct Pack {
    typedef typename Words<sizeof(T) * N>::type W;
    W q;
    __device__ __forceinline__ T get(int k) const { return reinterpret_cast<const T*>(&q)[k]; }
    __device__ __forceinline__ void set(int k, T v) { reinterpret_cast<T*>(&q)[k] = v; }
    __device__ __forceinline__ void load(const T* base, int64_t v) { q = reinterpret_cast<const W*>(base)[v]; }
    // The flat streaming maps: the large-tensor form of the kernel (ONCE: 2 M vectors and more, 32 MB per operand) marks
    // its words as read once for the caches, which tensors beyond the caches repay (a plain copy 0.715 -> 0.742 of the
    // HBM peak, the fp16 add of [4096,11008] 0.73 -> 0.80); smaller tensors keep the plain load, which finds what the
    // previous kernel left in the caches.
    template <bool ONCE>
    __device__ __forceinline__ void load_stream(const T* base, int64_t v) {
        if constexpr (ONCE) q = __builtin_nontemporal_load(reinterpret_cast<const W*>(base) + v);
        else q = reinterpret_cast<const W*>(base)[v];
    }
    __device__ __forceinline__ void store(T* base, int64_t v) const {
        __builtin_nontemporal_store(q, reinterpret_cast<W*>(base) + v);
    }
};

constexpr int kBlock = 256;
constexpr unsigned kRowsPerGridY = 65535;  // rows one grid.y covers in the kernels that take the row from the grid
constexpr int kUnroll = 4;

// fp32 -> fp16 with the exact behaviour of vpux::type::float16
// (src/vpux_utils/src/core/type/float16.cpp:30-108): round to nearest even; a NaN keeps its sign
// and top ten payload bits (at least one set); and a value below 2^-15 whose mantissa is at least
// 0x7ff000 rounds as if it were doubled (the exponent bump of the reference's first rounding step
// leaks into its subnormal branch, :74-107).
__device__ __forceinline__ half_t f32_to_f16(float f) {
    const uint32_t bits = __builtin_bit_cast(uint32_t, f);
    const uint32_t e = bits & 0x7f800000u;
    const bool doubled = e != 0 && e <= (111u << 23) && (bits & 0x7fffffu) >= 0x7ff000u;
    half_t h = (half_t)(doubled ? f * 2.0f : f);
    if (__builtin_isnan(f)) {
        uint32_t payload = (bits & 0x7fffffu) >> 13;
        payload = payload ? payload : 1u;
        const uint16_t hb = (uint16_t)(((bits >> 16) & 0x8000u) | 0x7c00u | payload);
        h = __builtin_bit_cast(half_t, hb);
    }
    return h;
}

// vpux::fakeQuantize, src/vpux_compiler/src/utils/quantization.cpp:995-1003 (fp32, round half away)
__device__ __forceinline__ float fq_f32(float x, float ilo, float ihi, float olo, float ohi, float lm1) {
    const float q = roundf((x - ilo) / (ihi - ilo) * lm1) / lm1 * (ohi - olo) + olo;
    return x <= ilo ? olo : (x > ihi ? ohi : q);
}

// a / c, correctly rounded, from r = RN(1 / c): q = RN(a r) is within an ulp, the residual
// a - q c is exact in one fma, and the corrected q + residual * r rounds to the true quotient
// (Markstein).  Three operations instead of the dozen of an IEEE division; valid away from
// overflow and underflow, where the operands of a FakeQuantize live.
__device__ __forceinline__ float div_const(float a, float c, float r) {
    const float q = a * r;
    const float rem = __builtin_fmaf(-q, c, a);
    return __builtin_fmaf(rem, r, q);
}

// Per-tensor FakeQuantize prepared on the host: ranges and their correctly rounded reciprocals.
struct FqConst {
    float ilo, ihi, olo, ohi, lm1;
    float irange, r_irange;  // ihi - ilo and RN(1 / (ihi - ilo))
    float r_lm1;             // RN(1 / lm1)
    float orange;            // ohi - olo
};
// round half away from zero for t >= 0: nearest-even, then a tie that went down to the even neighbour goes up
// (two instructions fewer than the general roundf; negative arguments only occur where the caller discards the result)
__device__ __forceinline__ float round_half_up_nonneg(float t) {
    const float r = __builtin_rintf(t);
    return t - r == 0.5f ? r + 1.0f : r;
}
__device__ __forceinline__ float fq_f32_const(float x, const FqConst& c) {
    // the level is only used for ilo < x <= ihi, where it is not negative
    const float level = round_half_up_nonneg(div_const(x - c.ilo, c.irange, c.r_irange) * c.lm1);
    const float q = div_const(level, c.lm1, c.r_lm1) * c.orange + c.olo;
    return x <= c.ilo ? c.olo : (x > c.ihi ? c.ohi : q);
}

template <typename T>
__device__ __forceinline__ T narrow(float r);
template <>
__device__ __forceinline__ half_t narrow<half_t>(float r) {
    return f32_to_f16(r);
}
template <>
__device__ __forceinline__ float narrow<float>(float r) {
    return r;
}

// Narrows N fp32 results to fp16 as vpux::type::float16 would.  The reference deviates from IEEE
// only for nonzero magnitudes below 2^-15; a wave that holds no such value -- nearly always --
// takes the plain conversion instruction, the others the exact emulation.
template <int N>
__device__ __forceinline__ void narrow_vec(const float (&r)[N], half_t (&h)[N]) {
    // (bits << 1) - 2 drops the sign and sends zero to the top of the range: the nonzero magnitudes below 2^-15
    // are the values under 0x6ffffffe, so one running minimum finds them.  NaNs (payload rule) are found two
    // values per comparison; the votes are combined as wave masks.
    uint32_t lo = 0xffffffffu;
#pragma unroll
    for (int k = 0; k < N; k++) {
        const uint32_t w = (__builtin_bit_cast(uint32_t, r[k]) << 1) - 2u;
        lo = w < lo ? w : lo;
    }
    uint64_t zone = 0;  // lanes that need the exact emulation
#pragma unroll
    for (int k = 0; k + 1 < N; k += 2) zone |= __builtin_amdgcn_ballot_w64(__builtin_isunordered(r[k], r[k + 1]));
    if (N & 1) zone |= __builtin_amdgcn_ballot_w64(__builtin_isnan(r[N - 1]));
    if (__builtin_amdgcn_ballot_w64(lo < 0x6ffffffeu) != 0) {
        // Some value lies below 2^-15 (the negative tail of GELU or Swish does in every wave): only those whose top
        // eleven mantissa bits are all set round differently, one in 2048.  Look again before leaving the fast path.
#pragma unroll
        for (int k = 0; k < N; k++)
            zone |= __builtin_amdgcn_ballot_w64(__builtin_fabsf(r[k]) < 0x1p-15f &&
                                                (__builtin_bit_cast(uint32_t, r[k]) & 0x7ff000u) == 0x7ff000u);
    }
    if (zone != 0) {
#pragma unroll
        for (int k = 0; k < N; k++) h[k] = f32_to_f16(r[k]);
    } else {
#pragma unroll
        for (int k = 0; k < N; k++) h[k] = (half_t)r[k];
    }
}

// A functor may expose `f32(...)`, the fp32 value that still has to be narrowed to fp16; the maps
// then narrow a whole vector at once (narrow_vec) instead of value by value.
template <class Fn, class = void>
struct HasF32 : std::false_type {};
template <class Fn>
struct HasF32<Fn, std::void_t<decltype(Fn::kF32)>> : std::true_type {};

// ---------------------------------------------------------------- flat streaming skeleton
// F provides: static constexpr int VEC; void vec(int64_t v) (elements [v*VEC, v*VEC+VEC)); void one(int64_t i).
template <class F, int BLOCK, int UNROLL>
__global__ __launch_bounds__(BLOCK) void stream_kernel(F f, int64_t n_vec, int64_t n) {
    const int64_t block0 = (int64_t)blockIdx.x * (BLOCK * UNROLL);
    if (block0 + BLOCK * UNROLL <= n_vec) {
        f.template vecs<UNROLL>(block0 + threadIdx.x, BLOCK);
    } else {
        for (int u = 0; u < UNROLL; u++) {
            const int64_t v = block0 + u * BLOCK + threadIdx.x;
            if (v < n_vec) f.template vecs<1>(v, 0);
        }
    }
    // ragged tail, fewer than VEC elements
    if (blockIdx.x == gridDim.x - 1) {
        const int64_t i = n_vec * F::VEC + threadIdx.x;
        if (i < n) f.one(i);
    }
}

template <class F>
int launch_stream(const F& f, int64_t n, hipStream_t s) {
    if (n <= 0) return VPX_RESULT_SUCCESS;
    const int64_t n_vec = n / F::VEC;
    // A tensor too small to give every compute unit several full-size workgroups is latency-bound:
    // fewer vectors per lane, and in the end single-wave workgroups, spread it over more units.
    const int tier = n_vec >= (int64_t)kBlock * kUnroll * 2048 ? 2 : (n_vec >= (int64_t)kBlock * 1024 ? 1 : 0);
    const int64_t per_block = tier == 2 ? kBlock * kUnroll : (tier == 1 ? kBlock : 64);
    int64_t blocks = (n_vec + per_block - 1) / per_block;
    if (blocks < 1) blocks = 1;
    VPX_REQUIRE(blocks < (1ll << 31), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "tensor of %lld elements is too large",
                (long long)n);
    const dim3 grid((unsigned)blocks);
    if (tier == 2) hipLaunchKernelGGL((stream_kernel<F, kBlock, kUnroll>), grid, dim3(kBlock), 0, s, f, n_vec, n);
    else if (tier == 1) hipLaunchKernelGGL((stream_kernel<F, kBlock, 1>), grid, dim3(kBlock), 0, s, f, n_vec, n);
    else hipLaunchKernelGGL((stream_kernel<F, 64, 1>), grid, dim3(64), 0, s, f, n_vec, n);
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

// A unary map from TI to TO; Fn is a stateless-or-small functor applied per element in fp32.
template <typename TI, typename TO, int VEC_, class Fn>
struct UnaryMap {
    static constexpr int VEC = VEC_;
    const TI* __restrict__ in;
    TO* __restrict__ out;
    Fn fn;
    template <int U>
    __device__ __forceinline__ void vecs(int64_t v0, int64_t step) const {
        Pack<TI, VEC> x[U];
#pragma unroll
        for (int u = 0; u < U; u++) x[u].template load_stream<(U == kUnroll)>(in, v0 + u * step);
#pragma unroll
        for (int u = 0; u < U; u++) {
            Pack<TO, VEC> y;
            if constexpr (HasF32<Fn>::value && std::is_same<TO, half_t>::value) {
                float r[VEC];
                half_t h[VEC];
#pragma unroll
                for (int k = 0; k < VEC; k++) r[k] = fn.f32(x[u].get(k));
                narrow_vec(r, h);
#pragma unroll
                for (int k = 0; k < VEC; k++) y.set(k, h[k]);
            } else {
#pragma unroll
                for (int k = 0; k < VEC; k++) y.set(k, fn(x[u].get(k)));
            }
            y.store(out, v0 + u * step);
        }
    }
    __device__ __forceinline__ void one(int64_t i) const {
        out[i] = fn(in[i]);
    }
};

template <typename T, int VEC_, class Fn>
struct BinaryMap {
    static constexpr int VEC = VEC_;
    const T* __restrict__ a;
    const T* __restrict__ b;
    T* __restrict__ out;
    Fn fn;
    template <int U>
    __device__ __forceinline__ void vecs(int64_t v0, int64_t step) const {
        Pack<T, VEC> x[U], y[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            x[u].template load_stream<(U == kUnroll)>(a, v0 + u * step);
            y[u].template load_stream<(U == kUnroll)>(b, v0 + u * step);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            Pack<T, VEC> r;
            if constexpr (HasF32<Fn>::value && std::is_same<T, half_t>::value) {
                float f[VEC];
                half_t h[VEC];
#pragma unroll
                for (int k = 0; k < VEC; k++) f[k] = fn.f32(x[u].get(k), y[u].get(k));
                narrow_vec(f, h);
#pragma unroll
                for (int k = 0; k < VEC; k++) r.set(k, h[k]);
            } else {
#pragma unroll
                for (int k = 0; k < VEC; k++) r.set(k, fn(x[u].get(k), y[u].get(k)));
            }
            r.store(out, v0 + u * step);
        }
    }
    __device__ __forceinline__ void one(int64_t i) const {
        out[i] = fn(a[i], b[i]);
    }
};

// ---------------------------------------------------------------- element functors
struct CvtF16F32 {
    __device__ __forceinline__ float operator()(half_t h) const { return (float)h; }
};
struct CvtF32F16 {
    static constexpr bool kF32 = true;
    __device__ __forceinline__ float f32(float f) const { return f; }
    __device__ __forceinline__ half_t operator()(float f) const { return f32_to_f16(f); }
};
template <typename T>
struct Copy {
    __device__ __forceinline__ T operator()(T v) const { return v; }
};

// float16 arithmetic = fp32 operation, then one rounding (include/vpux/utils/core/type/float16.hpp:123-150)
template <typename T, int OP>
struct EltFn {
    static constexpr bool kF32 = true;
    __device__ __forceinline__ float f32(T x, T y) const {
        const float a = (float)x, b = (float)y;
        if (OP == ELT_ADD) return a + b;
        if (OP == ELT_SUB) return a - b;
        if (OP == ELT_MUL) return a * b;
        if (OP == ELT_MIN) return fminf(a, b);
        if (OP == ELT_MAX) return fmaxf(a, b);
        if (OP == ELT_PRELU) return a < 0.f ? a * b : a;
        return a / b;
    }
    __device__ __forceinline__ T operator()(T x, T y) const { return narrow<T>(f32(x, y)); }
};

// Unary activations with the OpenVINO operator definitions the VPU ops carry over (operator list:
// src/vpux_compiler/src/dialect/VPUIP/IR/ops/sw_kernel.cpp:650-941,1266-1285,1689-1845): fp32 arithmetic,
// one rounding to the storage type.
// Building blocks for fp16 tensors, where the result is rounded to 11 bits: hardware exp2 / log2 /
// reciprocal (about 1 ulp of fp32 each) instead of the correctly rounded library routines.
__device__ __forceinline__ float fast_exp(float x) {
    return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f);
}
__device__ __forceinline__ float fast_rcp(float x) {
    return __builtin_amdgcn_rcpf(x);
}
// log(1 + t) for 0 <= t <= 1: two terms of the series where 1 + t would lose the low bits of t
__device__ __forceinline__ float fast_log1p_unit(float t) {
    const float series = t * __builtin_fmaf(t, -0.5f, 1.f);
    const float direct = __builtin_amdgcn_logf(1.f + t) * 0.69314718055994530942f;
    return t < 0.0009765625f ? series : direct;
}
__device__ __forceinline__ float fast_softplus(float x) {
    return fmaxf(x, 0.f) + fast_log1p_unit(fast_exp(-fabsf(x)));
}
// tanh(x) = 1 - 2 / (1 + e^2x) holds for both signs and saturates by itself; below 2^-6 the
// subtraction would cancel and x (1 - x^2 / 3) is exact to fp32.
__device__ __forceinline__ float fast_tanh(float x) {
    const float small = x * __builtin_fmaf(x * x, -0.33333334f, 1.f);
    const float big = __builtin_fmaf(-2.f, fast_rcp(1.f + __builtin_amdgcn_exp2f(x * 2.88539008177792681472f)), 1.f);
    return fabsf(x) < 0.015625f ? small : big;
}
// e^x - 1 for x <= 0: four terms of the series above -1/16, where the subtraction would cancel
__device__ __forceinline__ float fast_expm1_neg(float x) {
    float p = __builtin_fmaf(x, 0.041666668f, 0.16666667f);
    p = __builtin_fmaf(p, x, 0.5f);
    p = __builtin_fmaf(p, x, 1.f);
    return x > -0.0625f ? p * x : fast_exp(x) - 1.f;
}
// erfc(a) = 2^P(a) for a >= 0, P a polynomial of degree 8 fitted here to log2 erfc: one exp2 and eight fmas, with
// a relative error of erfc below 3e-6 up to a = 3.15 (beyond, fp16 results have long saturated; at the clamp 1 - erfc
// is 1 in fp32).  The relative error is what counts: GELU multiplies x by 1 + erf, which is erfc on the negative side.
// erf(v) = sign(v) (1 - erfc|v|); below 1/16 the subtraction cancels and three terms of the series are exact to fp32.
__device__ __forceinline__ float fast_erf(float v) {
    const float a = fminf(fabsf(v), 4.1f);
    float p = __builtin_fmaf(a, -3.72667832e-06f, 3.3506035e-05f);
    p = __builtin_fmaf(p, a, 0.000174893775f);
    p = __builtin_fmaf(p, a, -0.00430425219f);
    p = __builtin_fmaf(p, a, 0.0324461259f);
    p = __builtin_fmaf(p, a, -0.151220308f);
    p = __builtin_fmaf(p, a, -0.917526312f);
    p = __builtin_fmaf(p, a, -1.62802012f);
    p = __builtin_fmaf(p, a, 2.31981246e-06f);
    const float big = __builtin_copysignf(1.f - __builtin_amdgcn_exp2f(p), v);
    const float m = v * v;
    const float small = v * __builtin_fmaf(m, __builtin_fmaf(m, 0.11283791670955126f, -0.37612638903183754f), 1.1283791670955126f);
    return fabsf(v) >= 0.0625f ? big : small;  // a NaN takes the series, which keeps it
}
// GELU 0.5 x (1 + erf(x / sqrt 2)) with the same form in |x| directly: c = erfc(|x| / sqrt 2) = 2^P(|x|).  1 - c
// is rounded to fp32 before it is added to 1, as erf is in the defining formula: on the negative side that decides
// the last bits of 1 + erf.  0.5 + 0.5 s in one fma equals 0.5 (1 + s) rounded; no series is needed near 0, where
// 1 + erf is 1.
__device__ __forceinline__ float fast_gelu(float x) {
    const float a = fminf(fabsf(x), 5.8f);
    float p = __builtin_fmaf(a, -2.34842093e-07f, 2.9970647e-06f);
    p = __builtin_fmaf(p, a, 2.16017165e-05f);
    p = __builtin_fmaf(p, a, -0.000759922737f);
    p = __builtin_fmaf(p, a, 0.00810957688f);
    p = __builtin_fmaf(p, a, -0.0534623619f);
    p = __builtin_fmaf(p, a, -0.458764225f);
    p = __builtin_fmaf(p, a, -1.15118387f);
    p = __builtin_fmaf(p, a, 2.31379299e-06f);
    const float s = __builtin_copysignf(1.f - __builtin_amdgcn_exp2f(p), x);
    return x * __builtin_fmaf(s, 0.5f, 0.5f);
}
// sqrt of a value that came from fp16 (so never an fp32 subnormal), correctly rounded: the hardware root and
// reciprocal root are good to an ulp, the residual x - y^2 is exact in one fma, and y + residual / (2 y)
// rounds to the nearest fp32.  Zero and infinity keep the hardware result (their residual is not a number).
__device__ __forceinline__ float fast_sqrt(float x) {
    const float y = __builtin_amdgcn_sqrtf(x);
    const float h = 0.5f * __builtin_amdgcn_rsqf(x);
    const float fixed = __builtin_fmaf(__builtin_fmaf(-y, y, x), h, y);
    return __builtin_amdgcn_classf(x, 0x260) ? y : fixed;  // +-0, +inf
}

template <typename T, int OP>
struct ActFn {
    static constexpr bool kF32 = true;
    static constexpr bool kFast = std::is_same<T, half_t>::value;
    float p0, p1;
    __device__ __forceinline__ float f32(T v) const {
        const float x = (float)v;
        constexpr float kSixth = 0.16666667163372039794921875f;  // RN(1/6)
        if (OP == ACT_RELU) return x > 0.f ? x : 0.f;
        if (OP == ACT_LEAKY_RELU) return x < 0.f ? x * p0 : x;
        if (OP == ACT_CLAMP) return x < p0 ? p0 : (x > p1 ? p1 : x);
        if (OP == ACT_NEGATIVE) return -x;
        if (OP == ACT_ABS) return fabsf(x);
        if (OP == ACT_HSWISH) {
            // x * relu6(x + 3) / 6 with the exact quotient of div_const; an infinite product stays infinite
            const float a = x * fminf(fmaxf(x + 3.f, 0.f), 6.f);
            return fabsf(a) == INFINITY ? a : div_const(a, 6.f, kSixth);
        }
        if (OP == ACT_HSIGMOID) return div_const(fminf(fmaxf(x + 3.f, 0.f), 6.f), 6.f, kSixth);
        if (OP == ACT_HARDSIGMOID) return fmaxf(0.f, fminf(1.f, p0 * x + p1));
        if (OP == ACT_SIGMOID) return kFast ? fast_rcp(1.f + fast_exp(-x)) : 1.f / (1.f + expf(-x));
        if (OP == ACT_TANH) return kFast ? fast_tanh(x) : tanhf(x);
        if (OP == ACT_EXP) return kFast ? fast_exp(x) : expf(x);
        if (OP == ACT_SQRT) return kFast ? fast_sqrt(x) : sqrtf(x);
        if (OP == ACT_LOG) return logf(x);
        if (OP == ACT_FLOOR) return floorf(x);
        if (OP == ACT_CEIL) return ceilf(x);
        if (OP == ACT_SIGN) return x > 0.f ? 1.f : (x < 0.f ? -1.f : x);
        if (OP == ACT_ELU) return x < 0.f ? p0 * (kFast ? fast_expm1_neg(x) : expf(x) - 1.f) : x;
        if (OP == ACT_SELU) return x > 0.f ? p1 * x : p0 * p1 * (kFast ? fast_expm1_neg(x) : expf(x) - 1.f);
        if (OP == ACT_SWISH) return kFast ? x * fast_rcp(1.f + fast_exp(-p0 * x)) : x / (1.f + expf(-p0 * x));
        if (OP == ACT_MISH) {
            if (!kFast) return x * tanhf(x < 20.f ? log1pf(expf(x)) : x);
            // tanh(log(1 + e^x)) = n / (n + 2) with n = e^x (e^x + 2): no cancellation at either end
            const float e = fast_exp(fminf(x, 20.f));
            const float n = e * (e + 2.f);
            return x * (n * fast_rcp(n + 2.f));
        }
        if (OP == ACT_SOFTPLUS) return kFast ? fast_softplus(x) : (x < 20.f ? log1pf(expf(x)) : x);
        if (OP == ACT_GELU) return kFast ? fast_gelu(x) : 0.5f * x * (1.f + erff(x * 0.70710678118654752440f));
        return kFast ? fast_erf(x) : erff(x);
    }
    __device__ __forceinline__ T operator()(T v) const { return narrow<T>(f32(v)); }
};

// Per-tensor FakeQuantize as a flat streaming map.  The four limits are device tensors of one
// element; every lane turns them into the constants of fq_f32_const once (two IEEE divisions per
// lane instead of two per value).
struct FqMap {
    static constexpr int VEC = 8;
    const half_t* __restrict__ in;
    half_t* __restrict__ out;
    const half_t* ilo;
    const half_t* ihi;
    const half_t* olo;
    const half_t* ohi;
    float lm1;
    __device__ __forceinline__ FqConst prep() const {
        FqConst c;
        c.ilo = (float)*ilo;
        c.ihi = (float)*ihi;
        c.olo = (float)*olo;
        c.ohi = (float)*ohi;
        c.lm1 = lm1;
        c.irange = c.ihi - c.ilo;
        c.r_irange = 1.0f / c.irange;
        c.r_lm1 = 1.0f / lm1;
        c.orange = c.ohi - c.olo;
        return c;
    }
    template <int U>
    __device__ __forceinline__ void vecs(int64_t v0, int64_t step) const {
        const FqConst c = prep();
        Pack<half_t, VEC> x[U];
#pragma unroll
        for (int u = 0; u < U; u++) x[u].template load_stream<(U == kUnroll)>(in, v0 + u * step);
#pragma unroll
        for (int u = 0; u < U; u++) {
            float r[VEC];
            half_t h[VEC];
#pragma unroll
            for (int k = 0; k < VEC; k++) r[k] = fq_f32_const((float)x[u].get(k), c);
            narrow_vec(r, h);
            Pack<half_t, VEC> y;
#pragma unroll
            for (int k = 0; k < VEC; k++) y.set(k, h[k]);
            y.store(out, v0 + u * step);
        }
    }
    __device__ __forceinline__ void one(int64_t i) const {
        out[i] = f32_to_f16(fq_f32_const((float)in[i], prep()));
    }
};

// FakeQuantize with limits that vary between values (vnd_kernel functor).  Both divisions of the formula are by
// constants of a channel: the level count's reciprocal comes from the host, the input range's is one IEEE division
// per vector when the limits are constant along the innermost run (SCALAR: per-channel limits of a channel-major
// tensor, per-row limits of a weight matrix), else one per value; the quotients themselves are div_const's.
template <bool SCALAR>
struct FqVecFn {
    float lm1, r_lm1;
    __device__ __forceinline__ void operator()(const Pack<half_t, 8> (&x)[5], Pack<half_t, 8>& y) const {
        float r[8];
        half_t h[8];
        FqConst c;
        c.lm1 = lm1;
        c.r_lm1 = r_lm1;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            if (!SCALAR || k == 0) {
                c.ilo = (float)x[1].get(k);
                c.ihi = (float)x[2].get(k);
                c.olo = (float)x[3].get(k);
                c.ohi = (float)x[4].get(k);
                c.irange = c.ihi - c.ilo;
                c.r_irange = 1.0f / c.irange;
                c.orange = c.ohi - c.olo;
            }
            r[k] = fq_f32_const((float)x[0].get(k), c);
        }
        narrow_vec(r, h);
#pragma unroll
        for (int k = 0; k < 8; k++) y.set(k, h[k]);
    }
};

// createQuantizeFn, src/vpux_compiler/src/dialect/const/attributes/quantize.cpp:91-106: the FakeQuantize onto
// [qmin, qmax] with the limits of a launch prepared on the host (both divisions by constants, see div_const)
// SIMPLE: the host has checked that level / lm1 * (ohi - olo) + olo gives back level + olo for every level (it
// does for the 8-bit ranges), so the second division of the FakeQuantize formula is skipped; the input is
// limited to [ilo, ihi] first, which stands for the formula's two comparisons (the level is monotone in x).
// One value of the SIMPLE form below: `c` needs ilo, ihi, irange, r_irange, lm1 and olo.
__device__ __forceinline__ int quantize_simple(float x, const FqConst& c) {
    const float m = div_const(__builtin_amdgcn_fmed3f(x, c.ilo, c.ihi) - c.ilo, c.irange, c.r_irange) * c.lm1;  // >= 0
    // round half away from zero: nearest-even, then a tie that went down to the even neighbour goes up
    const float r = __builtin_rintf(m);
    return (int)r + (int)c.olo + (m - r == 0.5f ? 1 : 0);
}
// Whether level / lm1 * (qmax - qmin) + qmin gives back level + qmin for every level, in float arithmetic (host).
static bool levels_are_identity(float qmin, float qmax, float lm1) {
    bool same = lm1 >= 1.0f && lm1 <= 65535.0f;
    for (int level = 0; same && level <= (int)lm1; level++) same = (float)level / lm1 * (qmax - qmin) + qmin == (float)(level + (int)qmin);
    return same;
}

template <typename TI, typename TQ, bool SIMPLE>
struct QuantFn {
    FqConst c;
    __device__ __forceinline__ TQ operator()(TI x) const {
        if (SIMPLE) return (TQ)quantize_simple((float)x, c);
        return (TQ)(int)fq_f32_const((float)x, c);
    }
};


// vpux::dequantize, include/vpux/compiler/utils/quantization.hpp:208-210: double product -> float
// PLAIN: every nonzero result is at least 2^-14 in magnitude and finite, where the reference's
// float16 rounding is plain round-to-nearest-even, one conversion instruction.
template <typename TQ, typename TO, bool PLAIN>
struct DequantFn {
    double scale;
    int zp;
    __device__ __forceinline__ TO operator()(TQ q) const {
        const float r = (float)((double)((int)q - zp) * scale);
        if (PLAIN) return (TO)r;
        return narrow<TO>(r);
    }
};

// The same product with a scale that is a float (the per-axis tables hold what the blob shipped as fp16 or fp32):
// an 8-bit difference times 24 bits is exact in double, so the double product rounded to float is the float
// product rounded once.
__device__ __forceinline__ float dequant_f32(int diff, float scale) {
    return (float)diff * scale;
}

// ---------------------------------------------------------------- strided / broadcast path
template <int NOPS>
__device__ __forceinline__ void nd_offsets(const NdIndex& ix, int64_t lin, int64_t off[NOPS]) {
#pragma unroll
    for (int o = 0; o < NOPS; o++) off[o] = 0;
    for (int d = 0; d < ix.nd; d++) {
        const int64_t q = lin / ix.dims[d];
        const int64_t r = lin - q * ix.dims[d];
        lin = q;
#pragma unroll
        for (int o = 0; o < NOPS; o++) off[o] += r * ix.stride[o][d];
    }
}

template <typename TI, typename TO, class Fn>
__global__ __launch_bounds__(kBlock) void nd_unary_kernel(const TI* in, TO* out, Fn fn, NdIndex ix, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    int64_t off[2];
    nd_offsets<2>(ix, i, off);
    out[off[1]] = fn(in[off[0]]);
}

// dynamic_quantize (VPU.DynamicQuantize, src/vpux_compiler/tblgen/vpux/compiler/dialect/VPU/ops.td:6646-6660: f32 in,
// u8 out, one f32 scale, one u8 zero point).  The reference holds only the signature; the arithmetic is that of the
// ONNX operator the op is imported from (DynamicQuantizeLinear): the range [min(0, min x), max(0, max x)] maps onto
// 0..255, scale = range / 255 (1 for an all-zero tensor), zero point = rne(clamp(-min / scale)),
// y = clamp(rne(x / scale) + zero point); NaNs do not take part in the range.
struct MinMax {
    float lo, hi;
};
__device__ __forceinline__ MinMax mm_merge(MinMax a, MinMax b) {
    return MinMax{fminf(a.lo, b.lo), fmaxf(a.hi, b.hi)};
}
__device__ __forceinline__ MinMax mm_block(MinMax m, MinMax* smem) {
    smem[threadIdx.x] = m;
    __syncthreads();
    for (int step = kBlock / 2; step > 0; step >>= 1) {
        if ((int)threadIdx.x < step) smem[threadIdx.x] = mm_merge(smem[threadIdx.x], smem[threadIdx.x + step]);
        __syncthreads();
    }
    return smem[0];
}
__global__ __launch_bounds__(kBlock) void dynq_range_kernel(const float* __restrict__ x, int64_t n, MinMax* __restrict__ partial) {
    __shared__ MinMax smem[kBlock];
    MinMax m{0.f, 0.f};
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
        const float v = x[i];
        m.lo = fminf(m.lo, v);  // fminf / fmaxf return the other operand for a NaN
        m.hi = fmaxf(m.hi, v);
    }
    m = mm_block(m, smem);
    if (threadIdx.x == 0) partial[blockIdx.x] = m;
}
__global__ __launch_bounds__(kBlock) void dynq_params_kernel(const MinMax* __restrict__ partial, int count, float* __restrict__ scale,
                                                             uint8_t* __restrict__ zp) {
    __shared__ MinMax smem[kBlock];
    MinMax m{0.f, 0.f};
    for (int i = threadIdx.x; i < count; i += kBlock) m = mm_merge(m, partial[i]);
    m = mm_block(m, smem);
    if (threadIdx.x == 0) {
        const float sc = m.hi == m.lo ? 1.0f : (m.hi - m.lo) / 255.0f;
        const float z = fminf(fmaxf(0.0f - m.lo / sc, 0.0f), 255.0f);
        *scale = sc;
        *zp = (uint8_t)rintf(z);
    }
}
struct DynQuantMap {
    static constexpr int VEC = 4;
    const float* __restrict__ in;
    uint8_t* __restrict__ out;
    const float* __restrict__ scale;
    const uint8_t* __restrict__ zp;
    __device__ __forceinline__ uint8_t q(float x, float sc, float z) const {
        const float v = rintf(x / sc) + z;
        return (uint8_t)fminf(fmaxf(v, 0.f), 255.f);  // NaN -> 0
    }
    template <int U>
    __device__ __forceinline__ void vecs(int64_t v0, int64_t step) const {
        const float sc = *scale, z = (float)*zp;
        Pack<float, VEC> x[U];
#pragma unroll
        for (int u = 0; u < U; u++) x[u].template load_stream<(U == kUnroll)>(in, v0 + u * step);
#pragma unroll
        for (int u = 0; u < U; u++) {
            Pack<uint8_t, VEC> y;
#pragma unroll
            for (int k = 0; k < VEC; k++) y.set(k, q(x[u].get(k), sc, z));
            y.store(out, v0 + u * step);
        }
    }
    __device__ __forceinline__ void one(int64_t i) const {
        out[i] = q(in[i], *scale, (float)*zp);
    }
};

__global__ __launch_bounds__(kBlock) void dynq_scalar_kernel(DynQuantMap f, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) f.one(i);
}

// dynamic_dequantize: y = (q - zp) * scale with scale and zero point read from tensors that broadcast onto
// the input (VPU.DynamicDequantize, src/vpux_compiler/tblgen/vpux/compiler/dialect/VPU/ops.td:7780-7819).
// A lane takes VEC values along the innermost dimension; with VEC > 1 scale and zero point are constant along it
// (per-row or per-group scales of a weight matrix) and `ix` counts the innermost dimension in vectors.
// PER_VALUE: scale and zero point run along the innermost dimension with the values (per-column parameters): a lane
// reads VEC of each, contiguous like its values.
template <typename TQ, typename TS, typename TO, int VEC, bool PER_VALUE = false, bool GRID2D = false>
__global__ __launch_bounds__(kBlock) void dyn_dequant_kernel(const TQ* __restrict__ in, const TS* __restrict__ scale,
                                                             const uint8_t* __restrict__ zp, int zp_signed, TO* __restrict__ out,
                                                             NdIndex ix, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    int64_t off[4] = {0, 0, 0, 0};
    if (GRID2D) {  // at most two dimensions: the position in the row from grid x, the row from grid y and z
        const uint32_t row = blockIdx.y + blockIdx.z * kRowsPerGridY;
        if (i >= ix.dims[0] || (ix.nd == 2 && row >= (uint32_t)ix.dims[1])) return;
#pragma unroll
        for (int o = 0; o < 4; o++) off[o] = i * ix.stride[o][0] + (ix.nd == 2 ? (int64_t)row * ix.stride[o][1] : 0);
    } else if (i >= n) {
        return;
    } else if (n < (1ll << 32)) {  // 32-bit divisions: a quarter of the instructions of the 64-bit ones
        uint32_t lin = (uint32_t)i;
        for (int d = 0; d < ix.nd; d++) {
            const uint32_t q = lin / (uint32_t)ix.dims[d];
            const uint32_t r = lin - q * (uint32_t)ix.dims[d];
            lin = q;
#pragma unroll
            for (int o = 0; o < 4; o++) off[o] += (int64_t)r * ix.stride[o][d];
        }
    } else {
        nd_offsets<4>(ix, i, off);
    }
    Pack<TQ, VEC> x;
    x.load(in + off[0], 0);
    float r[VEC];
    if (PER_VALUE) {
        Pack<TS, VEC> sc;
        sc.load(scale + off[1], 0);
        Pack<uint8_t, VEC> z;
        if (zp) z.load(zp + off[2], 0);
#pragma unroll
        for (int k = 0; k < VEC; k++) {
            const int zk = zp ? (zp_signed ? (int)(int8_t)z.get(k) : (int)z.get(k)) : 0;
            r[k] = (float)((int)x.get(k) - zk) * (float)sc.get(k);
        }
    } else {
        const float sc = (float)scale[off[1]];
        int z = 0;
        if (zp) z = zp_signed ? (int)(int8_t)zp[off[2]] : (int)zp[off[2]];
#pragma unroll
        for (int k = 0; k < VEC; k++) r[k] = (float)((int)x.get(k) - z) * sc;
    }
    Pack<TO, VEC> y;
    if constexpr (std::is_same<TO, half_t>::value) {
        half_t h[VEC];
        narrow_vec(r, h);
#pragma unroll
        for (int k = 0; k < VEC; k++) y.set(k, h[k]);
    } else {
#pragma unroll
        for (int k = 0; k < VEC; k++) y.set(k, r[k]);
    }
    y.store(out + off[3], 0);
}

template <typename T, class Fn>
__global__ __launch_bounds__(kBlock) void nd_binary_kernel(const T* a, const T* b, T* out, Fn fn, NdIndex ix,
                                                           int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    int64_t off[3];
    nd_offsets<3>(ix, i, off);
    out[off[2]] = fn(a[off[0]], b[off[1]]);
}

// fake_quantize with limits that broadcast along some dimensions (per-channel and the like)
__global__ __launch_bounds__(kBlock) void nd_fq_kernel(const half_t* in, half_t* out, const half_t* ilo,
                                                       const half_t* ihi, const half_t* olo, const half_t* ohi,
                                                       NdIndex io, NdIndex lim, float lm1, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    int64_t off[2], lo[4];
    nd_offsets<2>(io, i, off);
    nd_offsets<4>(lim, i, lo);
    out[off[1]] = f32_to_f16(fq_f32((float)in[off[0]], (float)ilo[lo[0]], (float)ihi[lo[1]], (float)olo[lo[2]],
                                    (float)ohi[lo[3]], lm1));
}

// ---------------------------------------------------------------- vectorised broadcast path
// Same-type maps over operands that broadcast or are strided in the outer dimensions but are, along
// the innermost (merged) dimension, either contiguous or constant.  Work is dealt out in vectors of
// VEC elements of the innermost dimension; a lane finds its row by divisions with reciprocals
// prepared on the host, loads a vector from each contiguous operand and one element from each
// constant one.  NOPS operands, the last one is the output.
struct VndIndex {
    int nd;                          // row dimensions (all but the innermost)
    uint32_t vec_per_row;            // vectors along the innermost dimension
    uint64_t m_vec_per_row;          // ceil(2^64 / vec_per_row)
    uint32_t dims[kMaxDims];         // row dimensions, innermost first
    uint64_t m_dims[kMaxDims];
    int64_t stride[6][kMaxDims];     // element strides of the row dimensions
    int inner_stride[6];             // 1 or 0
};

__device__ __forceinline__ uint32_t fdiv64(uint32_t a, uint32_t d, uint64_t m) {
    return d == 1 ? a : (uint32_t)__umul64hi((uint64_t)a, m);
}

// One vector of the output from one vector (or one broadcast value) of every input.
template <typename T, int NOPS, class Fn>
__device__ __forceinline__ void vnd_apply(const T* const (&src)[5], T* pout, const Fn& fn, const int64_t (&off)[NOPS],
                                          const int (&inner_stride)[6]) {
    constexpr int VEC = 16 / sizeof(T);
    Pack<T, VEC> x[NOPS - 1];
#pragma unroll
    for (int o = 0; o < NOPS - 1; o++) {
        if (inner_stride[o]) {
            x[o].load(src[o] + off[o], 0);
        } else {
            const T e = src[o][off[o]];
#pragma unroll
            for (int k = 0; k < VEC; k++) x[o].set(k, e);
        }
    }
    Pack<T, VEC> y;
    fn(x, y);
    y.store(pout + off[NOPS - 1], 0);
}

template <typename T, int NOPS, class Fn>
__global__ __launch_bounds__(kBlock) void vnd_kernel(const T* p0, const T* p1, const T* p2, const T* p3, const T* p4, T* pout,
                                                     Fn fn, VndIndex ix, uint32_t total_vec) {
    constexpr int VEC = 16 / sizeof(T);
    const uint32_t v = blockIdx.x * kBlock + threadIdx.x;
    if (v >= total_vec) return;
    uint32_t row = fdiv64(v, ix.vec_per_row, ix.m_vec_per_row);
    const uint32_t iv = v - row * ix.vec_per_row;
    int64_t off[NOPS];
#pragma unroll
    for (int o = 0; o < NOPS; o++) off[o] = (int64_t)iv * VEC * ix.inner_stride[o];
    for (int d = 0; d < ix.nd; d++) {
        const uint32_t q = fdiv64(row, ix.dims[d], ix.m_dims[d]);
        const uint32_t r = row - q * ix.dims[d];
        row = q;
#pragma unroll
        for (int o = 0; o < NOPS; o++) off[o] += (int64_t)r * ix.stride[o][d];
    }
    const T* const src[5] = {p0, p1, p2, p3, p4};
    vnd_apply<T, NOPS, Fn>(src, pout, fn, off, ix.inner_stride);
}

// The same for tensors that merge into rows x one inner run (a bias or slope per column, a scale per row): the
// row comes from the grid, so its offsets are scalar arithmetic and a lane only scales its position in the row.
// TWO: two row dimensions (channels and batch of a channel-major tensor with per-channel operands), grid y and z.
// BCAST: bit o set = input o is constant along the row (one value per row), known at compile time so that the
// loads of all operands are issued together instead of one branch, and one wait, per operand; -1 = read the
// pattern from the index at run time.
template <typename T, int NOPS, class Fn, bool TWO, int BCAST>
__global__ __launch_bounds__(kBlock) void vrow_kernel(const T* __restrict__ p0, const T* __restrict__ p1, const T* __restrict__ p2,
                                                      const T* __restrict__ p3, const T* __restrict__ p4, T* __restrict__ pout,
                                                      Fn fn, VndIndex ix, uint32_t rows) {
    constexpr int VEC = 16 / sizeof(T);
    const uint32_t iv = blockIdx.x * kBlock + threadIdx.x;
    const uint32_t row = TWO ? blockIdx.y : blockIdx.y + blockIdx.z * kRowsPerGridY;
    if (iv >= ix.vec_per_row || row >= rows) return;
    // the row's part of every address is the same for the whole workgroup (scalar registers); a lane adds a
    // 32-bit position in the row, or nothing where the operand is constant along it
    const T* const src[5] = {p0, p1, p2, p3, p4};
    Pack<T, VEC> x[NOPS - 1];
#pragma unroll
    for (int o = 0; o < NOPS - 1; o++) {
        const T* base = src[o] + ((int64_t)row * ix.stride[o][0] + (TWO ? (int64_t)blockIdx.z * ix.stride[o][1] : 0));
        if (BCAST < 0 ? ix.inner_stride[o] != 0 : !((BCAST >> o) & 1)) {
            x[o].load(base, iv);
        } else {
            const T e = *base;
#pragma unroll
            for (int k = 0; k < VEC; k++) x[o].set(k, e);
        }
    }
    Pack<T, VEC> y;
    fn(x, y);
    T* obase = pout + ((int64_t)row * ix.stride[NOPS - 1][0] + (TWO ? (int64_t)blockIdx.z * ix.stride[NOPS - 1][1] : 0));
    y.store(obase, iv);
}

// Host side: merges dimensions that every operand walks contiguously or not at all, then checks
// what vnd_kernel needs.  `ops` are NOPS memrefs broadcastable to the last one.  Returns false when
// the shape does not qualify (the caller falls back to the one-element-per-lane kernels).
template <typename T, int NOPS>
bool make_vnd(const MemRef* const (&ops)[NOPS], VndIndex& ix, uint32_t& total_vec) {
    constexpr int VEC = 16 / sizeof(T);
    const MemRef& out = *ops[NOPS - 1];
    if (out.nd > kMaxDims || out.nd < 1) return false;
    int64_t dims[kMaxDims], st[NOPS][kMaxDims];
    int nd = 0;
    for (int d = 0; d < out.nd; d++) {
        if (out.dims[d] == 1) continue;
        int64_t cur[NOPS];
        for (int o = 0; o < NOPS; o++) {
            const MemRef& m = *ops[o];
            const bool scalar = m.numel() == 1;
            if (!scalar && m.nd != out.nd) return false;
            cur[o] = scalar || m.dims[d] == 1 ? 0 : m.strides[d];
            if (!scalar && m.dims[d] != 1 && m.dims[d] != out.dims[d]) return false;
        }
        bool merge = nd > 0;
        for (int o = 0; o < NOPS && merge; o++) merge = cur[o] == st[o][nd - 1] * dims[nd - 1];
        if (merge) {
            dims[nd - 1] *= out.dims[d];
        } else {
            dims[nd] = out.dims[d];
            for (int o = 0; o < NOPS; o++) st[o][nd] = cur[o];
            nd++;
        }
    }
    if (nd == 0) return false;  // a single element: not worth a vector path
    if (dims[0] % VEC != 0 || dims[0] / VEC >= (1ll << 32)) return false;
    ix = VndIndex{};
    for (int o = 0; o < NOPS; o++) {
        if (st[o][0] != 0 && st[o][0] != 1) return false;
        if (o == NOPS - 1 && st[o][0] != 1) return false;
        ix.inner_stride[o] = (int)st[o][0];
        if ((reinterpret_cast<uintptr_t>(ops[o]->data) & 15) != 0 && st[o][0] == 1) return false;
        for (int d = 1; d < nd; d++)
            if (st[o][0] == 1 && st[o][d] % VEC != 0) return false;
    }
    auto magic = [](uint64_t d) { return d == 1 ? 0ull : (~0ull) / d + 1ull; };
    ix.vec_per_row = (uint32_t)(dims[0] / VEC);
    ix.m_vec_per_row = magic(ix.vec_per_row);
    ix.nd = nd - 1;
    int64_t total = dims[0] / VEC;
    for (int d = 1; d < nd; d++) {
        if (dims[d] >= (1ll << 32)) return false;
        ix.dims[d - 1] = (uint32_t)dims[d];
        ix.m_dims[d - 1] = magic((uint64_t)dims[d]);
        for (int o = 0; o < NOPS; o++) ix.stride[o][d - 1] = st[o][d];
        total *= dims[d];
        if (total >= (1ll << 32)) return false;
    }
    total_vec = (uint32_t)total;
    return total > 0;
}

template <typename T, int NOPS, class Fn, bool TWO, int BCAST>
int launch_vrow_as(const dim3& grid, const T* p0, const T* p1, const T* p2, const T* p3, const T* p4, T* pout, const Fn& fn,
                   const VndIndex& vx, uint32_t rows, hipStream_t s) {
    hipLaunchKernelGGL((vrow_kernel<T, NOPS, Fn, TWO, BCAST>), grid, dim3(kBlock), 0, s, p0, p1, p2, p3, p4, pout, fn, vx, rows);
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

// The broadcast patterns that have a kernel: any for two inputs; for five (FakeQuantize), limits that all run along
// the row or are all constant along it.  Returns -1 when there is none.
template <typename T, int NOPS, class Fn, bool TWO>
int launch_vrow(int mask, const dim3& grid, const T* p0, const T* p1, const T* p2, const T* p3, const T* p4, T* pout, const Fn& fn,
                const VndIndex& vx, uint32_t rows, hipStream_t s) {
#define VPX_VROW(M) \
    if (mask == M) return launch_vrow_as<T, NOPS, Fn, TWO, M>(grid, p0, p1, p2, p3, p4, pout, fn, vx, rows, s)
    if constexpr (NOPS == 3) {
        // two inputs: decided at run time (measured faster than the compile-time form: 27.5 against 29.2 us for a
        // per-column operand on a [4096, 11008] tensor)
        return launch_vrow_as<T, NOPS, Fn, TWO, -1>(grid, p0, p1, p2, p3, p4, pout, fn, vx, rows, s);
    } else {
        VPX_VROW(0);
        VPX_VROW(30);
    }
#undef VPX_VROW
    return -1;
}

template <typename T, int NOPS, class Fn>
int launch_vnd(const T* p0, const T* p1, const T* p2, const T* p3, const T* p4, T* pout, const Fn& fn, const VndIndex& vx,
               uint32_t total_vec, hipStream_t s) {
    int mask = 0;
    for (int o = 0; o < NOPS - 1; o++) mask |= vx.inner_stride[o] ? 0 : 1 << o;
    if (vx.nd <= 1 && vx.vec_per_row >= 64) {
        const uint32_t rows = vx.nd == 1 ? vx.dims[0] : 1;
        const dim3 grid((vx.vec_per_row + kBlock - 1) / kBlock, rows < kRowsPerGridY ? rows : kRowsPerGridY,
                        (rows + kRowsPerGridY - 1) / kRowsPerGridY);
        if (grid.z <= 65535) {
            const int rc = launch_vrow<T, NOPS, Fn, false>(mask, grid, p0, p1, p2, p3, p4, pout, fn, vx, rows, s);
            if (rc >= 0) return rc;
        }
    }
    if (vx.nd == 2 && vx.vec_per_row >= 64 && vx.dims[0] <= 65535 && vx.dims[1] <= 65535) {
        const dim3 grid((vx.vec_per_row + kBlock - 1) / kBlock, vx.dims[0], vx.dims[1]);
        const int rc = launch_vrow<T, NOPS, Fn, true>(mask, grid, p0, p1, p2, p3, p4, pout, fn, vx, vx.dims[0], s);
        if (rc >= 0) return rc;
    }
    hipLaunchKernelGGL((vnd_kernel<T, NOPS, Fn>), dim3((total_vec + kBlock - 1) / kBlock), dim3(kBlock), 0, s, p0, p1, p2, p3, p4,
                       pout, fn, vx, total_vec);
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

int grid_1d(int64_t n, unsigned* blocks) {
    const int64_t b = (n + kBlock - 1) / kBlock;
    VPX_REQUIRE(b < (1ll << 31), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "tensor of %lld elements is too large",
                (long long)n);
    *blocks = (unsigned)(b < 1 ? 1 : b);
    return VPX_RESULT_SUCCESS;
}

// Fill operand `slot` of an NdIndex from a memref that must broadcast onto `out`.
int fill_index(NdIndex& ix, int slot, const MemRef& m, const MemRef& out, const char* what) {
    VPX_REQUIRE(out.nd <= kMaxDims, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                "%s: rank %d exceeds the %d dimensions the strided path handles", what, out.nd, kMaxDims);
    VPX_REQUIRE(m.nd == out.nd || m.numel() == 1, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                "%s: rank %d does not match the output rank %d", what, m.nd, out.nd);
    ix.nd = out.nd;
    for (int d = 0; d < out.nd; d++) {
        ix.dims[d] = (int32_t)out.dims[d];
        if (m.numel() == 1) {
            ix.stride[slot][d] = 0;
            continue;
        }
        VPX_REQUIRE(m.dims[d] == out.dims[d] || m.dims[d] == 1, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                    "%s: dimension %d of size %lld cannot broadcast to %lld", what, d, (long long)m.dims[d],
                    (long long)out.dims[d]);
        ix.stride[slot][d] = m.dims[d] == 1 ? 0 : m.strides[d];
    }
    return VPX_RESULT_SUCCESS;
}

bool same_shape(const MemRef& a, const MemRef& b) {
    if (a.nd != b.nd) return false;
    for (int d = 0; d < a.nd; d++)
        if (a.dims[d] != b.dims[d]) return false;
    return true;
}

bool aligned16(const void* p) {
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

}  // namespace

// ---------------------------------------------------------------- convert
template <typename TI, typename TO, class Fn>
static int convert_impl(const MemRef& in, const MemRef& out, Fn fn, hipStream_t s) {
    const int64_t n = out.numel();
    if (in.compact && out.compact && aligned16(in.data) && aligned16(out.data)) {
        constexpr int VEC = 16 / (sizeof(TI) > sizeof(TO) ? sizeof(TI) : sizeof(TO));
        UnaryMap<TI, TO, VEC, Fn> f{(const TI*)in.data, (TO*)out.data, fn};
        return launch_stream(f, n, s);
    }
    NdIndex ix{};
    int rc = fill_index(ix, 0, in, out, "convert input");
    if (rc) return rc;
    rc = fill_index(ix, 1, out, out, "convert output");
    if (rc) return rc;
    unsigned blocks;
    rc = grid_1d(n, &blocks);
    if (rc) return rc;
    if (n == 0) return VPX_RESULT_SUCCESS;
    hipLaunchKernelGGL((nd_unary_kernel<TI, TO, Fn>), dim3(blocks), dim3(kBlock), 0, s, (const TI*)in.data,
                       (TO*)out.data, fn, ix, n);
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

int launch_convert(const MemRef& in, const MemRef& out, hipStream_t s) {
    VPX_REQUIRE(same_shape(in, out), VPX_RESULT_ERROR_INVALID_ARGUMENT, "convert: input and output shapes differ");
    if (in.dtype == VPX_NN_FP16 && out.dtype == VPX_NN_FP32) return convert_impl<half_t, float>(in, out, CvtF16F32{}, s);
    if (in.dtype == VPX_NN_FP32 && out.dtype == VPX_NN_FP16) return convert_impl<float, half_t>(in, out, CvtF32F16{}, s);
    if (in.dtype == out.dtype && in.elem_bits == 16) return convert_impl<uint16_t, uint16_t>(in, out, Copy<uint16_t>{}, s);
    if (in.dtype == out.dtype && in.elem_bits == 32) return convert_impl<uint32_t, uint32_t>(in, out, Copy<uint32_t>{}, s);
    if (in.dtype == out.dtype && in.elem_bits == 8) return convert_impl<uint8_t, uint8_t>(in, out, Copy<uint8_t>{}, s);
    return fail(VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "convert: %s -> %s is not implemented", dtype_name(in.dtype),
                dtype_name(out.dtype));
}

// ---------------------------------------------------------------- activations
template <typename T, int OP>
static int activation_impl(int op, float p0, float p1, const MemRef& in, const MemRef& out, hipStream_t s) {
    if (op == OP) return convert_impl<T, T>(in, out, ActFn<T, OP>{p0, p1}, s);
    if constexpr (OP + 1 < ACT_COUNT) return activation_impl<T, OP + 1>(op, p0, p1, in, out, s);
    return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT, "activation: unknown operation %d", op);
}

int launch_activation(int op, float p0, float p1, const MemRef& in, const MemRef& out, hipStream_t s) {
    VPX_REQUIRE(same_shape(in, out), VPX_RESULT_ERROR_INVALID_ARGUMENT, "activation: input and output shapes differ");
    VPX_REQUIRE(in.dtype == out.dtype, VPX_RESULT_ERROR_INVALID_ARGUMENT, "activation: input %s and output %s types differ",
                dtype_name(in.dtype), dtype_name(out.dtype));
    if (op == ACT_CLAMP)
        VPX_REQUIRE(p0 <= p1, VPX_RESULT_ERROR_INVALID_ARGUMENT, "activation_clamp: min %g exceeds max %g", (double)p0, (double)p1);
    if (in.dtype == VPX_NN_FP16) return activation_impl<half_t, 0>(op, p0, p1, in, out, s);
    if (in.dtype == VPX_NN_FP32) return activation_impl<float, 0>(op, p0, p1, in, out, s);
    return fail(VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "activation: element type %s is not implemented", dtype_name(in.dtype));
}

// ---------------------------------------------------------------- eltwise
template <typename T, int OP>
static int eltwise_impl(const MemRef& a, const MemRef& b, const MemRef& out, hipStream_t s) {
    const int64_t n = out.numel();
    typedef EltFn<T, OP> Fn;
    if (a.compact && b.compact && out.compact && same_shape(a, out) && same_shape(b, out) && aligned16(a.data) &&
        aligned16(b.data) && aligned16(out.data)) {
        BinaryMap<T, 16 / sizeof(T), Fn> f{(const T*)a.data, (const T*)b.data, (T*)out.data, Fn{}};
        return launch_stream(f, n, s);
    }
    {
        struct VecFn {
            __device__ __forceinline__ void operator()(const Pack<T, 16 / sizeof(T)> (&x)[2], Pack<T, 16 / sizeof(T)>& y) const {
                Fn f;
                constexpr int V = (int)(16 / sizeof(T));
                if constexpr (std::is_same<T, half_t>::value) {
                    float r[V];
                    half_t h[V];
#pragma unroll
                    for (int k = 0; k < V; k++) r[k] = f.f32(x[0].get(k), x[1].get(k));
                    narrow_vec(r, h);
#pragma unroll
                    for (int k = 0; k < V; k++) y.set(k, h[k]);
                } else {
#pragma unroll
                    for (int k = 0; k < V; k++) y.set(k, f(x[0].get(k), x[1].get(k)));
                }
            }
        };
        const MemRef* const ops[3] = {&a, &b, &out};
        VndIndex vx;
        uint32_t total_vec = 0;
        if (make_vnd<T, 3>(ops, vx, total_vec)) {
            return launch_vnd<T, 3, VecFn>((const T*)a.data, (const T*)b.data, (const T*)nullptr, (const T*)nullptr, (const T*)nullptr,
                                           (T*)out.data, VecFn{}, vx, total_vec, s);
        }
    }
    NdIndex ix{};
    int rc = fill_index(ix, 0, a, out, "eltwise input 1");
    if (rc) return rc;
    rc = fill_index(ix, 1, b, out, "eltwise input 2");
    if (rc) return rc;
    rc = fill_index(ix, 2, out, out, "eltwise output");
    if (rc) return rc;
    unsigned blocks;
    rc = grid_1d(n, &blocks);
    if (rc) return rc;
    if (n == 0) return VPX_RESULT_SUCCESS;
    hipLaunchKernelGGL((nd_binary_kernel<T, Fn>), dim3(blocks), dim3(kBlock), 0, s, (const T*)a.data, (const T*)b.data,
                       (T*)out.data, Fn{}, ix, n);
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

template <typename T>
static int eltwise_dispatch(int op, const MemRef& a, const MemRef& b, const MemRef& out, hipStream_t s) {
    switch (op) {
    case ELT_ADD: return eltwise_impl<T, ELT_ADD>(a, b, out, s);
    case ELT_SUB: return eltwise_impl<T, ELT_SUB>(a, b, out, s);
    case ELT_MUL: return eltwise_impl<T, ELT_MUL>(a, b, out, s);
    case ELT_MIN: return eltwise_impl<T, ELT_MIN>(a, b, out, s);
    case ELT_MAX: return eltwise_impl<T, ELT_MAX>(a, b, out, s);
    case ELT_DIV: return eltwise_impl<T, ELT_DIV>(a, b, out, s);
    case ELT_PRELU: return eltwise_impl<T, ELT_PRELU>(a, b, out, s);
    default: return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT, "eltwise: unknown operation %d", op);
    }
}

int launch_eltwise(int op, const MemRef& a, const MemRef& b, const MemRef& out, hipStream_t s) {
    VPX_REQUIRE(a.dtype == b.dtype && a.dtype == out.dtype, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                "eltwise: operand types differ (%s, %s -> %s)", dtype_name(a.dtype), dtype_name(b.dtype),
                dtype_name(out.dtype));
    if (out.dtype == VPX_NN_FP16) return eltwise_dispatch<half_t>(op, a, b, out, s);
    if (out.dtype == VPX_NN_FP32) return eltwise_dispatch<float>(op, a, b, out, s);
    return fail(VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "eltwise: element type %s is not implemented",
                dtype_name(out.dtype));
}

// ---------------------------------------------------------------- fake_quantize
// FakeQuantize of a packed tensor whose limits hold one value per innermost channel (or one value): a lane owns
// eight adjacent channels, prepares their constants once (the one IEEE division per channel) and walks kFqInnerRows
// rows.  Lanes are dealt along the rows' 128-bit words first, so short channel runs leave no lane idle.
constexpr int kFqInnerRows = 8;
// How the channel-minor kernels deal the 128-bit words of a [rows x cvecs] tensor: a lane visits words
// first + k * step (k < R, below end) that all hold the same eight channels `cv`.  When a workgroup's lanes cover
// whole rows (cvecs divides the workgroup) the R visits of a workgroup are R adjacent runs of kBlock words, else a
// lane walks R consecutive rows of its column of words.
struct InnerDeal {
    uint32_t cv;
    int64_t first, step, end;
};
__device__ __forceinline__ InnerDeal inner_deal(uint32_t cvecs, int64_t rows, int R) {
    InnerDeal d;
    d.end = rows * cvecs;
    if (kBlock % cvecs == 0) {
        d.cv = threadIdx.x % cvecs;
        d.first = (int64_t)blockIdx.x * kBlock * R + threadIdx.x;
        d.step = kBlock;
    } else {
        const int64_t lane = (int64_t)blockIdx.x * kBlock + threadIdx.x;
        d.cv = (uint32_t)(lane % cvecs);
        d.first = lane / cvecs * R * cvecs + d.cv;
        d.step = cvecs;
    }
    return d;
}
static inline unsigned inner_deal_blocks(uint32_t cvecs, int64_t rows, int R) {
    if (kBlock % cvecs == 0) return (unsigned)((rows * cvecs + (int64_t)kBlock * R - 1) / ((int64_t)kBlock * R));
    return (unsigned)(((rows + R - 1) / R * cvecs + kBlock - 1) / kBlock);
}
__global__ __launch_bounds__(kBlock) void fq_inner8_kernel(const half_t* __restrict__ in, half_t* __restrict__ out,
                                                           const half_t* __restrict__ l0, const half_t* __restrict__ l1,
                                                           const half_t* __restrict__ l2, const half_t* __restrict__ l3,
                                                           uint32_t per_channel,  // bit k: limit k has a value per channel
                                                           uint32_t cvecs, int64_t rows, float lm1, float r_lm1) {
    const InnerDeal d = inner_deal(cvecs, rows, kFqInnerRows);  // lanes past the end compute on word cv and store nothing
    const uint32_t cv = d.cv;
    const half_t* lim[4] = {l0, l1, l2, l3};
    float c[4][8];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        if (per_channel >> k & 1) {
            Pack<half_t, 8> v;
            v.load(lim[k], cv);
#pragma unroll
            for (int e = 0; e < 8; e++) c[k][e] = (float)v.get(e);
        } else {
            const float f = (float)lim[k][0];
#pragma unroll
            for (int e = 0; e < 8; e++) c[k][e] = f;
        }
    }
    float r_irange[8];
#pragma unroll
    for (int e = 0; e < 8; e++) r_irange[e] = 1.0f / (c[1][e] - c[0][e]);
    Pack<half_t, 8> xs[kFqInnerRows];
#pragma unroll
    for (int r = 0; r < kFqInnerRows; r++) {
        const int64_t v = d.first + r * d.step;
        xs[r].load(in, v < d.end ? v : cv);
    }
#pragma unroll
    for (int r = 0; r < kFqInnerRows; r++) {
        float f[8];
        half_t h[8];
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const FqConst cst{c[0][e], c[1][e], c[2][e], c[3][e], lm1, c[1][e] - c[0][e], r_irange[e], r_lm1, c[3][e] - c[2][e]};
            f[e] = fq_f32_const((float)xs[r].get(e), cst);
        }
        narrow_vec(f, h);  // every lane of the wavefront votes, also those without a row
        Pack<half_t, 8> y;
#pragma unroll
        for (int e = 0; e < 8; e++) y.set(e, h[e]);
        if (d.first + r * d.step < d.end) y.store(out, d.first + r * d.step);
    }
}

int launch_fake_quantize(const MemRef& in, const MemRef lims[4], const MemRef& out, int64_t levels, hipStream_t s) {
    // Only FP16 in/out, like the reference kernel (sw_kernel.cpp:1156-1157).
    VPX_REQUIRE(in.dtype == VPX_NN_FP16 && out.dtype == VPX_NN_FP16, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                "fake_quantize: only FP16 input/output is supported, got %s -> %s", dtype_name(in.dtype),
                dtype_name(out.dtype));
    for (int k = 0; k < 4; k++)
        VPX_REQUIRE(lims[k].dtype == VPX_NN_FP16, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                    "fake_quantize: limit %d must be FP16, got %s", k, dtype_name(lims[k].dtype));
    VPX_REQUIRE(levels >= 2, VPX_RESULT_ERROR_INVALID_ARGUMENT, "fake_quantize: levels must be at least 2, got %lld",
                (long long)levels);
    VPX_REQUIRE(same_shape(in, out), VPX_RESULT_ERROR_INVALID_ARGUMENT, "fake_quantize: input and output shapes differ");
    const int64_t n = out.numel();
    const float lm1 = (float)levels - 1.0f;
    const bool per_tensor =
            lims[0].numel() == 1 && lims[1].numel() == 1 && lims[2].numel() == 1 && lims[3].numel() == 1;
    if (per_tensor && in.compact && out.compact && aligned16(in.data) && aligned16(out.data)) {
        FqMap f{(const half_t*)in.data, (half_t*)out.data, (const half_t*)lims[0].data, (const half_t*)lims[1].data,
                (const half_t*)lims[2].data, (const half_t*)lims[3].data, lm1};
        return launch_stream(f, n, s);
    }
    if (in.compact && out.compact && aligned16(in.data) && aligned16(out.data) && in.nd >= 1 && in.dims[0] % 8 == 0) {
        // limits per innermost channel (channel-minor activations): constants per lane, kept across rows
        const int64_t ch = in.dims[0];
        uint32_t per_channel = 0;
        const int64_t rows = n / ch, lanes = (rows + kFqInnerRows - 1) / kFqInnerRows * (ch / 8);
        bool ok = n > 0 && lanes / kBlock < (1ll << 31) - 1;
        for (int k = 0; k < 4 && ok; k++) {
            if (lims[k].numel() == 1) continue;
            ok = lims[k].numel() == ch && lims[k].dims[0] == ch && lims[k].strides[0] == 1 && aligned16(lims[k].data);
            per_channel |= 1u << k;
        }
        if (ok) {
            hipLaunchKernelGGL(fq_inner8_kernel, dim3(inner_deal_blocks((uint32_t)(ch / 8), rows, kFqInnerRows)), dim3(kBlock), 0, s, (const half_t*)in.data,
                               (half_t*)out.data, (const half_t*)lims[0].data, (const half_t*)lims[1].data, (const half_t*)lims[2].data,
                               (const half_t*)lims[3].data, per_channel, (uint32_t)(ch / 8), rows, lm1, 1.0f / lm1);
            VPX_HIP_CHECK(hipGetLastError());
            return VPX_RESULT_SUCCESS;
        }
    }
    {
        // limits that broadcast (per channel and the like): five inputs, vectors along the innermost run
        const MemRef* const ops[6] = {&in, &lims[0], &lims[1], &lims[2], &lims[3], &out};
        VndIndex vx;
        uint32_t total_vec = 0;
        if (make_vnd<half_t, 6>(ops, vx, total_vec)) {
            const bool scalar = !vx.inner_stride[1] && !vx.inner_stride[2] && !vx.inner_stride[3] && !vx.inner_stride[4];
            if (scalar)
                return launch_vnd<half_t, 6, FqVecFn<true>>((const half_t*)in.data, (const half_t*)lims[0].data, (const half_t*)lims[1].data,
                                                            (const half_t*)lims[2].data, (const half_t*)lims[3].data, (half_t*)out.data,
                                                            FqVecFn<true>{lm1, 1.0f / lm1}, vx, total_vec, s);
            return launch_vnd<half_t, 6, FqVecFn<false>>((const half_t*)in.data, (const half_t*)lims[0].data, (const half_t*)lims[1].data,
                                                         (const half_t*)lims[2].data, (const half_t*)lims[3].data, (half_t*)out.data,
                                                         FqVecFn<false>{lm1, 1.0f / lm1}, vx, total_vec, s);
        }
    }
    NdIndex io{}, lim{};
    int rc = fill_index(io, 0, in, out, "fake_quantize input");
    if (rc) return rc;
    rc = fill_index(io, 1, out, out, "fake_quantize output");
    if (rc) return rc;
    for (int k = 0; k < 4; k++) {
        rc = fill_index(lim, k, lims[k], out, "fake_quantize limit");
        if (rc) return rc;
    }
    unsigned blocks;
    rc = grid_1d(n, &blocks);
    if (rc) return rc;
    if (n == 0) return VPX_RESULT_SUCCESS;
    hipLaunchKernelGGL(nd_fq_kernel, dim3(blocks), dim3(kBlock), 0, s, (const half_t*)in.data, (half_t*)out.data,
                       (const half_t*)lims[0].data, (const half_t*)lims[1].data, (const half_t*)lims[2].data,
                       (const half_t*)lims[3].data, io, lim, lm1, n);
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

// ---------------------------------------------------------------- quantize / dequantize
template <typename TI, typename TQ>
static int quantize_impl(const MemRef& in, const MemRef& out, double scale, int64_t zp, int64_t qmin, int64_t qmax,
                         hipStream_t s) {
    // Limits of the FakeQuantize the reference quantizer is built from (quantize.cpp:91-96); the same float
    // operations as the device's own preparation of a FakeQuantize (FqMap::prep).
    FqConst c;
    c.ilo = (float)((double)(qmin - zp) * scale);
    c.ihi = (float)((double)(qmax - zp) * scale);
    c.olo = (float)qmin;
    c.ohi = (float)qmax;
    c.lm1 = (float)(qmax - qmin + 1) - 1.0f;
    c.irange = c.ihi - c.ilo;
    c.r_irange = 1.0f / c.irange;
    c.r_lm1 = 1.0f / c.lm1;
    c.orange = c.ohi - c.olo;
    if (c.irange > 0.0f && levels_are_identity(c.olo, c.ohi, c.lm1)) return convert_impl<TI, TQ>(in, out, QuantFn<TI, TQ, true>{c}, s);
    return convert_impl<TI, TQ>(in, out, QuantFn<TI, TQ, false>{c}, s);
}

int launch_quantize(const MemRef& in, const MemRef& out, double scale, int64_t zp, hipStream_t s) {
    VPX_REQUIRE(same_shape(in, out), VPX_RESULT_ERROR_INVALID_ARGUMENT, "quantize: input and output shapes differ");
    VPX_REQUIRE(scale > 0.0, VPX_RESULT_ERROR_INVALID_ARGUMENT, "quantize: scale must be positive, got %g", scale);
    if (in.dtype == VPX_NN_FP16 && out.dtype == VPX_NN_U8) return quantize_impl<half_t, uint8_t>(in, out, scale, zp, 0, 255, s);
    if (in.dtype == VPX_NN_FP16 && out.dtype == VPX_NN_I8) return quantize_impl<half_t, int8_t>(in, out, scale, zp, -128, 127, s);
    if (in.dtype == VPX_NN_FP32 && out.dtype == VPX_NN_U8) return quantize_impl<float, uint8_t>(in, out, scale, zp, 0, 255, s);
    if (in.dtype == VPX_NN_FP32 && out.dtype == VPX_NN_I8) return quantize_impl<float, int8_t>(in, out, scale, zp, -128, 127, s);
    return fail(VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "quantize: %s -> %s is not implemented", dtype_name(in.dtype),
                dtype_name(out.dtype));
}

int launch_dequantize(const MemRef& in, const MemRef& out, double scale, int64_t zp, hipStream_t s) {
    VPX_REQUIRE(same_shape(in, out), VPX_RESULT_ERROR_INVALID_ARGUMENT, "dequantize: input and output shapes differ");
    const int z = (int)zp;
    const bool plain = __builtin_isfinite(scale) && __builtin_fabs(scale) >= 0x1p-14 && __builtin_fabs(scale) < 64.0;
    if (in.dtype == VPX_NN_U8 && out.dtype == VPX_NN_FP16)
        return plain ? convert_impl<uint8_t, half_t>(in, out, DequantFn<uint8_t, half_t, true>{scale, z}, s)
                     : convert_impl<uint8_t, half_t>(in, out, DequantFn<uint8_t, half_t, false>{scale, z}, s);
    if (in.dtype == VPX_NN_I8 && out.dtype == VPX_NN_FP16)
        return plain ? convert_impl<int8_t, half_t>(in, out, DequantFn<int8_t, half_t, true>{scale, z}, s)
                     : convert_impl<int8_t, half_t>(in, out, DequantFn<int8_t, half_t, false>{scale, z}, s);
    if (in.dtype == VPX_NN_U8 && out.dtype == VPX_NN_FP32)
        return convert_impl<uint8_t, float>(in, out, DequantFn<uint8_t, float, true>{scale, z}, s);
    if (in.dtype == VPX_NN_I8 && out.dtype == VPX_NN_FP32)
        return convert_impl<int8_t, float>(in, out, DequantFn<int8_t, float, true>{scale, z}, s);
    return fail(VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "dequantize: %s -> %s is not implemented", dtype_name(in.dtype),
                dtype_name(out.dtype));
}


// ---------------------------------------------------------------- dynamic_quantize
int launch_dynamic_quantize(const MemRef& in, const MemRef& out, const MemRef& scale, const MemRef& zp, hipStream_t s) {
    VPX_REQUIRE(in.dtype == VPX_NN_FP32 && out.dtype == VPX_NN_U8 && scale.dtype == VPX_NN_FP32 && zp.dtype == VPX_NN_U8,
                VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "dynamic_quantize: expects FP32 -> U8 with an FP32 scale and a U8 zero point, got %s -> %s, %s, %s",
                dtype_name(in.dtype), dtype_name(out.dtype), dtype_name(scale.dtype), dtype_name(zp.dtype));
    VPX_REQUIRE(same_shape(in, out), VPX_RESULT_ERROR_INVALID_ARGUMENT, "dynamic_quantize: input and output shapes differ");
    VPX_REQUIRE(scale.numel() == 1 && zp.numel() == 1, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                "dynamic_quantize: scale and zero point are single values");
    const int64_t n = in.numel();
    VPX_REQUIRE(n == 0 || (in.compact && out.compact), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                "dynamic_quantize: only compact tensors are supported");
    int64_t blocks = (n + kBlock * 16 - 1) / (kBlock * 16);
    if (blocks > 2048) blocks = 2048;
    if (blocks < 1) blocks = 1;
    void* ws = nullptr;
    int rc = get_workspace(s, sizeof(MinMax) * (size_t)blocks, &ws);
    if (rc) return rc;
    hipLaunchKernelGGL(dynq_range_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, s, (const float*)in.data, n, (MinMax*)ws);
    VPX_HIP_CHECK(hipGetLastError());
    hipLaunchKernelGGL(dynq_params_kernel, dim3(1), dim3(kBlock), 0, s, (const MinMax*)ws, (int)blocks, (float*)scale.data,
                       (uint8_t*)zp.data);
    VPX_HIP_CHECK(hipGetLastError());
    if (n == 0) return VPX_RESULT_SUCCESS;
    DynQuantMap f{(const float*)in.data, (uint8_t*)out.data, (const float*)scale.data, (const uint8_t*)zp.data};
    if (aligned16(in.data) && (reinterpret_cast<uintptr_t>(out.data) & 3) == 0) return launch_stream(f, n, s);
    unsigned g;
    rc = grid_1d(n, &g);
    if (rc) return rc;
    hipLaunchKernelGGL(dynq_scalar_kernel, dim3(g), dim3(kBlock), 0, s, f, n);
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

// Drops unit dimensions and merges neighbours that every operand walks as one run (or not at all).
static void merge_index(NdIndex& ix, int slots) {
    int nd = 0;
    for (int d = 0; d < ix.nd; d++) {
        if (ix.dims[d] == 1) continue;
        bool merge = nd > 0 && (int64_t)ix.dims[nd - 1] * ix.dims[d] < (1ll << 31);
        for (int o = 0; o < slots && merge; o++) merge = ix.stride[o][d] == ix.stride[o][nd - 1] * ix.dims[nd - 1];
        if (merge) {
            ix.dims[nd - 1] *= ix.dims[d];
        } else {
            ix.dims[nd] = ix.dims[d];
            for (int o = 0; o < slots; o++) ix.stride[o][nd] = ix.stride[o][d];
            nd++;
        }
    }
    if (nd == 0) {
        ix.dims[0] = 1;
        for (int o = 0; o < slots; o++) ix.stride[o][0] = 0;
        nd = 1;
    }
    ix.nd = nd;
}

// ---------------------------------------------------------------- dynamic_dequantize
template <typename TQ, typename TS, typename TO>
static int dyn_dequant_impl(const MemRef& in, const MemRef& scale, const MemRef* zp, const MemRef& out, hipStream_t s) {
    NdIndex ix{};
    int rc = fill_index(ix, 0, in, out, "dynamic_dequantize input");
    if (rc) return rc;
    rc = fill_index(ix, 1, scale, out, "dynamic_dequantize scale");
    if (rc) return rc;
    if (zp) {
        rc = fill_index(ix, 2, *zp, out, "dynamic_dequantize zero point");
        if (rc) return rc;
    }
    rc = fill_index(ix, 3, out, out, "dynamic_dequantize output");
    if (rc) return rc;
    int64_t n = out.numel();
    if (n == 0) return VPX_RESULT_SUCCESS;
    if (!zp)
        for (int d = 0; d < ix.nd; d++) ix.stride[2][d] = ix.stride[1][d];  // an absent operand must not block a merge
    merge_index(ix, 4);
    const uint8_t* pz = zp ? (const uint8_t*)zp->data : nullptr;
    const int zp_signed = zp && zp->dtype == VPX_NN_I8 ? 1 : 0;
    constexpr int VEC = 16 / (int)sizeof(TO);
    bool vec = ix.dims[0] % VEC == 0 && ix.stride[0][0] == 1 && ix.stride[3][0] == 1 &&
               (reinterpret_cast<uintptr_t>(in.data) % (VEC * sizeof(TQ))) == 0 && aligned16(out.data);
    for (int d = 1; d < ix.nd && vec; d++) vec = ix.stride[0][d] % VEC == 0 && ix.stride[3][d] % VEC == 0;
    // parameters constant along the innermost dimension (per row / per group), or running along it with the values
    const bool per_row = ix.stride[1][0] == 0 && ix.stride[2][0] == 0;
    bool per_value = ix.stride[1][0] == 1 && (!zp || ix.stride[2][0] == 1) &&
                     (reinterpret_cast<uintptr_t>(scale.data) % (VEC * sizeof(TS))) == 0 && (!zp || reinterpret_cast<uintptr_t>(pz) % VEC == 0);
    for (int d = 1; d < ix.nd && per_value; d++) per_value = ix.stride[1][d] % VEC == 0 && ix.stride[2][d] % VEC == 0;
    vec = vec && (per_row || per_value);
    unsigned blocks;
    if (vec) {
        ix.dims[0] /= VEC;
        ix.stride[0][0] = VEC;
        ix.stride[3][0] = VEC;
        if (!per_row) {
            ix.stride[1][0] = VEC;
            if (zp) ix.stride[2][0] = VEC;
        }
        n /= VEC;
        const uint32_t rows = ix.nd == 2 ? (uint32_t)ix.dims[1] : 1;
        if (ix.nd <= 2 && ix.dims[0] >= 64 && (rows + kRowsPerGridY - 1) / kRowsPerGridY <= 65535) {
            const dim3 grid(((unsigned)ix.dims[0] + kBlock - 1) / kBlock, rows < kRowsPerGridY ? rows : kRowsPerGridY,
                            (rows + kRowsPerGridY - 1) / kRowsPerGridY);
            if (per_row)
                hipLaunchKernelGGL((dyn_dequant_kernel<TQ, TS, TO, VEC, false, true>), grid, dim3(kBlock), 0, s, (const TQ*)in.data,
                                   (const TS*)scale.data, pz, zp_signed, (TO*)out.data, ix, n);
            else
                hipLaunchKernelGGL((dyn_dequant_kernel<TQ, TS, TO, VEC, true, true>), grid, dim3(kBlock), 0, s, (const TQ*)in.data,
                                   (const TS*)scale.data, pz, zp_signed, (TO*)out.data, ix, n);
            VPX_HIP_CHECK(hipGetLastError());
            return VPX_RESULT_SUCCESS;
        }
        rc = grid_1d(n, &blocks);
        if (rc) return rc;
        if (per_row)
            hipLaunchKernelGGL((dyn_dequant_kernel<TQ, TS, TO, VEC, false>), dim3(blocks), dim3(kBlock), 0, s, (const TQ*)in.data,
                               (const TS*)scale.data, pz, zp_signed, (TO*)out.data, ix, n);
        else
            hipLaunchKernelGGL((dyn_dequant_kernel<TQ, TS, TO, VEC, true>), dim3(blocks), dim3(kBlock), 0, s, (const TQ*)in.data,
                               (const TS*)scale.data, pz, zp_signed, (TO*)out.data, ix, n);
    } else {
        rc = grid_1d(n, &blocks);
        if (rc) return rc;
        hipLaunchKernelGGL((dyn_dequant_kernel<TQ, TS, TO, 1>), dim3(blocks), dim3(kBlock), 0, s, (const TQ*)in.data,
                           (const TS*)scale.data, pz, zp_signed, (TO*)out.data, ix, n);
    }
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

template <typename TQ, typename TS>
static int dyn_dequant_out(const MemRef& in, const MemRef& scale, const MemRef* zp, const MemRef& out, hipStream_t s) {
    if (out.dtype == VPX_NN_FP16) return dyn_dequant_impl<TQ, TS, half_t>(in, scale, zp, out, s);
    return dyn_dequant_impl<TQ, TS, float>(in, scale, zp, out, s);
}

int launch_dynamic_dequantize(const MemRef& in, const MemRef& scale, const MemRef* zp, const MemRef& out, hipStream_t s) {
    VPX_REQUIRE(in.dtype == VPX_NN_I8 || in.dtype == VPX_NN_U8, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                "dynamic_dequantize: only I8 / U8 input is implemented, got %s", dtype_name(in.dtype));
    VPX_REQUIRE(scale.dtype == VPX_NN_FP16 || scale.dtype == VPX_NN_FP32, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                "dynamic_dequantize: scale must be FP16 or FP32, got %s", dtype_name(scale.dtype));
    VPX_REQUIRE(out.dtype == VPX_NN_FP16 || out.dtype == VPX_NN_FP32, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                "dynamic_dequantize: output must be FP16 or FP32, got %s", dtype_name(out.dtype));
    if (zp)
        VPX_REQUIRE(zp->dtype == VPX_NN_I8 || zp->dtype == VPX_NN_U8, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                    "dynamic_dequantize: only I8 / U8 zero points are implemented, got %s", dtype_name(zp->dtype));
    VPX_REQUIRE(same_shape(in, out), VPX_RESULT_ERROR_INVALID_ARGUMENT, "dynamic_dequantize: input and output shapes differ");
    const bool s16 = scale.dtype == VPX_NN_FP16;
    if (in.dtype == VPX_NN_I8)
        return s16 ? dyn_dequant_out<int8_t, half_t>(in, scale, zp, out, s) : dyn_dequant_out<int8_t, float>(in, scale, zp, out, s);
    return s16 ? dyn_dequant_out<uint8_t, half_t>(in, scale, zp, out, s) : dyn_dequant_out<uint8_t, float>(in, scale, zp, out, s);
}

// ---------------------------------------------------------------- per-axis quantize / dequantize
// The params blob ships n scales and zero points but not the axis they run along
// (getQuantParamsAttr, sw_kernel.cpp:130-163), so it is taken to be the one dimension of size n;
// when several dimensions have that size, the channel dimension (logical dimension 1 of the
// memref's order) if it is among them.  Operands must be compact.
namespace {

struct AxisChunk {
    float a[256];
    float b[256];
};

// Kernel arguments are the one path from host to device memory that a caller's graph capture can
// record: the per-channel table goes to the workspace 256 entries per launch.
__global__ __launch_bounds__(256) void fill_axis_table(float4* table, float* planes, int64_t n, AxisChunk c, int count) {
    // {a, b, b - a, 1 / (b - a)}: the last two are the constants of a channel's FakeQuantize (unused by dequantize).
    // Behind the table the same four values lie as four planes of n floats, for the kernels in which a lane
    // takes eight adjacent channels and reads each constant of the eight as two 128-bit words.
    const float lo = c.a[threadIdx.x], hi = c.b[threadIdx.x];
    if ((int)threadIdx.x < count) {
        const float4 e{lo, hi, hi - lo, 1.0f / (hi - lo)};
        table[threadIdx.x] = e;
        planes[threadIdx.x] = e.x;
        planes[n + threadIdx.x] = e.y;
        planes[2 * n + threadIdx.x] = e.z;
        planes[3 * n + threadIdx.x] = e.w;
    }
}

struct AxisGeom {
    uint32_t inner, count;
    uint64_t m_inner, m_count;
};
__device__ __forceinline__ uint32_t axis_channel(uint32_t i, const AxisGeom& g) {
    const uint32_t q = fdiv64(i, g.inner, g.m_inner);
    return q - fdiv64(q, g.count, g.m_count) * g.count;
}

// table entry: {in_min, in_max} of the channel's quantizer (quantize.cpp:91-96)
template <typename TI, typename TQ>
__global__ __launch_bounds__(kBlock) void quantize_axis_kernel(const TI* __restrict__ in, TQ* __restrict__ out,
                                                               const float4* __restrict__ table, AxisGeom g, uint32_t n,
                                                               float qmin, float qmax, float lm1) {
    const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const float4 p = table[axis_channel(i, g)];
    out[i] = (TQ)(int)fq_f32((float)in[i], p.x, p.y, qmin, qmax, lm1);
}

// table entry: {scale, zero point as a float (an integer of at most 9 bits)}
template <typename TQ, typename TO>
__global__ __launch_bounds__(kBlock) void dequantize_axis_kernel(const TQ* __restrict__ in, TO* __restrict__ out,
                                                                 const float4* __restrict__ table, AxisGeom g, uint32_t n) {
    const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const float4 p = table[axis_channel(i, g)];
    out[i] = narrow<TO>(dequant_f32((int)in[i] - (int)p.y, p.x));
}

// One 128-bit access of the wider operand per lane: the axis is not the innermost dimension and the run below it is
// a multiple of the vector, so a lane's values share a channel, whose FakeQuantize constants come from its table entry.
template <typename TI, typename TQ, bool SIMPLE>
__global__ __launch_bounds__(kBlock) void quantize_axis_vec_kernel(const TI* __restrict__ in, TQ* __restrict__ out,
                                                                   const float4* __restrict__ table, AxisGeom g, uint32_t n_vec,
                                                                   float qmin, float qmax, float lm1) {
    constexpr int V = 16 / (int)sizeof(TI);
    const uint32_t v = blockIdx.x * kBlock + threadIdx.x;
    if (v >= n_vec) return;
    Pack<TI, V> x;
    x.load(in, v);
    Pack<TQ, V> y;
    const float4 p = table[axis_channel(v * V, g)];
    const FqConst c{p.x, p.y, qmin, qmax, lm1, p.z, p.w, 1.0f / lm1, qmax - qmin};
#pragma unroll
    for (int k = 0; k < V; k++) y.set(k, SIMPLE ? (TQ)quantize_simple((float)x.get(k), c) : (TQ)(int)fq_f32_const((float)x.get(k), c));
    y.store(out, v);
}

template <typename TQ, typename TO>
__global__ __launch_bounds__(kBlock) void dequantize_axis_vec_kernel(const TQ* __restrict__ in, TO* __restrict__ out,
                                                                     const float4* __restrict__ table, AxisGeom g, uint32_t n_vec) {
    constexpr int V = 16 / (int)sizeof(TO);
    const uint32_t v = blockIdx.x * kBlock + threadIdx.x;
    if (v >= n_vec) return;
    Pack<TQ, V> x;
    x.load(in, v);
    const float4 p = table[axis_channel(v * V, g)];
    float r[V];
#pragma unroll
    for (int k = 0; k < V; k++) r[k] = dequant_f32((int)x.get(k) - (int)p.y, p.x);
    Pack<TO, V> y;
    if constexpr (std::is_same<TO, half_t>::value) {
        half_t h[V];
        narrow_vec(r, h);
#pragma unroll
        for (int k = 0; k < V; k++) y.set(k, h[k]);
    } else {
#pragma unroll
        for (int k = 0; k < V; k++) y.set(k, r[k]);
    }
    y.store(out, v);
}

// The axis is the innermost dimension: a lane takes one channel (its table entry is read, and its FakeQuantize
// constants prepared, once) and walks kAxisRows rows; the 64 lanes of a wavefront touch 64 adjacent values of a row.
constexpr int kAxisRows = 16;
template <typename TI, typename TQ>
__global__ __launch_bounds__(kBlock) void quantize_axis_inner_kernel(const TI* __restrict__ in, TQ* __restrict__ out,
                                                                     const float4* __restrict__ table, uint32_t count, uint32_t rows,
                                                                     float qmin, float qmax, float lm1) {
    const uint32_t ctiles = (count + kBlock - 1) / kBlock;
    const uint32_t c = (blockIdx.x % ctiles) * kBlock + threadIdx.x;
    const uint32_t r0 = (blockIdx.x / ctiles) * kAxisRows;
    if (c >= count) return;
    const float4 p = table[c];
    const FqConst cst{p.x, p.y, qmin, qmax, lm1, p.z, p.w, 1.0f / lm1, qmax - qmin};
    TI x[kAxisRows];
#pragma unroll
    for (int r = 0; r < kAxisRows; r++) x[r] = r0 + r < rows ? in[(r0 + r) * count + c] : (TI)0;
#pragma unroll
    for (int r = 0; r < kAxisRows; r++)
        if (r0 + r < rows) out[(r0 + r) * count + c] = (TQ)(int)fq_f32_const((float)x[r], cst);
}

template <typename TQ, typename TO>
__global__ __launch_bounds__(kBlock) void dequantize_axis_inner_kernel(const TQ* __restrict__ in, TO* __restrict__ out,
                                                                       const float4* __restrict__ table, uint32_t count, uint32_t rows) {
    const uint32_t ctiles = (count + kBlock - 1) / kBlock;
    const uint32_t c = (blockIdx.x % ctiles) * kBlock + threadIdx.x;
    const uint32_t r0 = (blockIdx.x / ctiles) * kAxisRows;
    const bool live = c < count;
    const float4 p = live ? table[c] : float4{0.f, 0.f, 0.f, 0.f};
    float v[kAxisRows];
#pragma unroll
    for (int r = 0; r < kAxisRows; r++) {
        const int q = live && r0 + r < rows ? (int)in[(r0 + r) * count + c] : 0;
        v[r] = dequant_f32(q - (int)p.y, p.x);
    }
    if constexpr (std::is_same<TO, half_t>::value) {
        half_t h[kAxisRows];
        narrow_vec(v, h);  // every lane of the wavefront takes part in the vote
#pragma unroll
        for (int r = 0; r < kAxisRows; r++)
            if (live && r0 + r < rows) out[(r0 + r) * count + c] = h[r];
    } else {
#pragma unroll
        for (int r = 0; r < kAxisRows; r++)
            if (live && r0 + r < rows) out[(r0 + r) * count + c] = v[r];
    }
}

// Tables already on the device, by content: the parameters of a layer are constants, so after the first call a
// per-axis launch is one kernel.  Entries belong to a (device, stream) like the workspace and are found through a
// 64-bit hash of the parameter bytes (a hit is confirmed by comparing them); vpx_workspace_release frees them.
struct AxisTableEntry {
    int dev;
    hipStream_t stream;
    std::vector<float> a, b;
    float4* table;
};
std::mutex g_axis_mutex;
std::unordered_multimap<uint64_t, AxisTableEntry> g_axis_tables;
constexpr size_t kMaxAxisTables = 64;

uint64_t axis_key(int dev, hipStream_t s, const float* a, const float* b, int64_t n) {
    uint64_t h = 0xcbf29ce484222325ull ^ (uint64_t)(uint32_t)dev ^ ((uint64_t)(uintptr_t)s << 7);
    auto mix = [&h](const float* v, int64_t cnt) {
        for (int64_t i = 0; i < cnt; i++) {
            uint32_t w;
            memcpy(&w, v + i, 4);
            h = (h ^ w) * 0x100000001b3ull;
            h ^= h >> 29;
        }
    };
    mix(a, n);
    mix(b, n);
    return h;
}

int axis_setup(const char* what, const MemRef& ref, const MemRef& other, int64_t n, const float* a, const float* b, hipStream_t s,
               AxisGeom& g, float4** table) {
    VPX_REQUIRE(ref.compact && other.compact, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "%s: per-axis form needs compact operands", what);
    VPX_REQUIRE(ref.numel() < (1ll << 32), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "%s: tensor of %lld elements is too large", what,
                (long long)ref.numel());
    int axis = -1, hits = 0;
    for (int d = 0; d < ref.nd; d++)
        if (ref.dims[d] == n) {
            axis = d;
            hits++;
        }
    VPX_REQUIRE(hits >= 1, VPX_RESULT_ERROR_INVALID_ARGUMENT, "%s: no dimension has the size of the %lld quantization parameters", what,
                (long long)n);
    if (hits > 1) {
        // memory position (innermost = 0) of logical dimension 1
        int pc = -1;
        for (int i = 0; i < ref.nd; i++)
            if ((int)((ref.order >> (4 * i)) & 0xf) == 2) pc = ref.nd - 1 - i;
        VPX_REQUIRE(pc >= 0 && ref.dims[pc] == n, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                    "%s: %d dimensions have size %lld and the channel dimension is not one of them: the axis is ambiguous", what, hits,
                    (long long)n);
        axis = pc;
    }
    int64_t inner = 1;
    for (int d = 0; d < axis; d++) inner *= ref.dims[d];
    auto magic = [](uint64_t d) { return d == 1 ? 0ull : (~0ull) / d + 1ull; };
    g.inner = (uint32_t)inner;
    g.count = (uint32_t)n;
    g.m_inner = magic((uint64_t)inner);
    g.m_count = magic((uint64_t)n);
    int dev = 0;
    VPX_HIP_CHECK(hipGetDevice(&dev));
    bool keep = false;
    const uint64_t key = axis_key(dev, s, a, b, n);
    {
        std::lock_guard<std::mutex> lock(g_axis_mutex);
        const auto range = g_axis_tables.equal_range(key);
        for (auto it = range.first; it != range.second; ++it) {
            const AxisTableEntry& e = it->second;
            if (e.dev == dev && e.stream == s && (int64_t)e.a.size() == n && memcmp(e.a.data(), a, sizeof(float) * (size_t)n) == 0 &&
                memcmp(e.b.data(), b, sizeof(float) * (size_t)n) == 0) {
                *table = e.table;
                return VPX_RESULT_SUCCESS;
            }
        }
        keep = g_axis_tables.size() < kMaxAxisTables && !noalloc_call();
    }
    // a table built under stream capture would need a hipMalloc inside the capture: take the workspace instead
    if (keep) {
        hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &st) != hipSuccess) (void)hipGetLastError();
        else if (st != hipStreamCaptureStatusNone) keep = false;
    }
    void* mem = nullptr;
    if (keep) {
        VPX_HIP_CHECK(hipMalloc(&mem, 2 * sizeof(float4) * (size_t)n));
    } else {
        const int rc = get_workspace(s, 2 * sizeof(float4) * (size_t)n, &mem);
        if (rc) return rc;
    }
    *table = (float4*)mem;
    for (int64_t c0 = 0; c0 < n; c0 += 256) {
        AxisChunk ch;
        const int cnt = (int)(n - c0 < 256 ? n - c0 : 256);
        for (int k = 0; k < cnt; k++) {
            ch.a[k] = a[c0 + k];
            ch.b[k] = b[c0 + k];
        }
        for (int k = cnt; k < 256; k++) ch.a[k] = ch.b[k] = 0.f;
        hipLaunchKernelGGL(fill_axis_table, dim3(1), dim3(256), 0, s, *table + c0, (float*)(*table + n) + c0, n, ch, cnt);
        VPX_HIP_CHECK(hipGetLastError());
    }
    if (keep) {
        std::lock_guard<std::mutex> lock(g_axis_mutex);
        g_axis_tables.emplace(key, AxisTableEntry{dev, s, std::vector<float>(a, a + n), std::vector<float>(b, b + n), *table});
    }
    return VPX_RESULT_SUCCESS;
}

// The same with eight adjacent channels per lane, for channel counts that are a multiple of eight: one 128-bit
// access per lane and row for the 16-bit side, the eight channels' constants kept in registers across the rows.
template <typename TI, typename TQ, bool SIMPLE>
__global__ __launch_bounds__(kBlock) void quantize_axis_inner8_kernel(const TI* __restrict__ in, TQ* __restrict__ out,
                                                                      const float4* __restrict__ table, uint32_t count, uint32_t rows,
                                                                      float qmin, float qmax, float lm1) {
    // lanes are dealt along a row's 128-bit words first, then over runs of kAxisRows rows: short channel runs idle no lane
    const uint32_t cvecs = count / 8;
    const InnerDeal d = inner_deal(cvecs, rows, kAxisRows);
    const uint32_t cv = d.cv;
    if (d.first >= d.end) return;
    float4 p[8];
    {
        const float4* planes = reinterpret_cast<const float4*>(table + count);  // four planes of count floats
        const uint32_t pv = count / 4;                                         // float4 words per plane
        float4 q[4][2];
#pragma unroll
        for (int c = 0; c < 4; c++) {
            q[c][0] = planes[c * pv + cv * 2];
            q[c][1] = planes[c * pv + cv * 2 + 1];
        }
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const int h = k >> 2, e = k & 3;
            auto pick = [&](const float4& v) { return e == 0 ? v.x : (e == 1 ? v.y : (e == 2 ? v.z : v.w)); };
            p[k] = float4{pick(q[0][h]), pick(q[1][h]), pick(q[2][h]), pick(q[3][h])};
        }
    }
    const float r_lm1 = 1.0f / lm1, orange = qmax - qmin;
    constexpr int kBatch = 8;  // rows whose loads are issued together
#pragma unroll
    for (int rb = 0; rb < kAxisRows; rb += kBatch) {
        Pack<TI, 8> xs[kBatch];
#pragma unroll
        for (int r = 0; r < kBatch; r++)
            if (d.first + (rb + r) * d.step < d.end) xs[r].load(in, d.first + (rb + r) * d.step);
#pragma unroll
        for (int r = 0; r < kBatch; r++) {
        const int64_t v = d.first + (rb + r) * d.step;
        if (v >= d.end) break;
        const Pack<TI, 8>& x = xs[r];
        Pack<TQ, 8> y;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const float f = (float)x.get(k);
            const FqConst cst{p[k].x, p[k].y, qmin, qmax, lm1, p[k].z, p[k].w, r_lm1, orange};
            y.set(k, SIMPLE ? (TQ)quantize_simple(f, cst) : (TQ)(int)fq_f32_const(f, cst));
        }
        y.store(out, v);
        }
    }
}
template <typename TQ, typename TO>
__global__ __launch_bounds__(kBlock) void dequantize_axis_inner8_kernel(const TQ* __restrict__ in, TO* __restrict__ out,
                                                                        const float4* __restrict__ table, uint32_t count, uint32_t rows) {
    const uint32_t cvecs = count / 8;
    const InnerDeal d = inner_deal(cvecs, rows, kAxisRows);  // lanes past the end read word cv and store nothing: every
    const uint32_t cv = d.cv;                                // lane takes part in the votes of narrow_vec
    float sc[8];
    int zp[8];
    {
        const float4* planes = reinterpret_cast<const float4*>(table + count);  // plane 0: scales, plane 1: zero points
        const uint32_t pv = count / 4, at = cv * 2;
        const float4 s0 = planes[at], s1 = planes[at + 1], z0 = planes[pv + at], z1 = planes[pv + at + 1];
        const float sv[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
        const float zv[8] = {z0.x, z0.y, z0.z, z0.w, z1.x, z1.y, z1.z, z1.w};
#pragma unroll
        for (int k = 0; k < 8; k++) {
            sc[k] = sv[k];
            zp[k] = (int)zv[k];
        }
    }
    Pack<TQ, 8> xs[kAxisRows];  // every row's load is issued before the first result is needed
#pragma unroll
    for (int r = 0; r < kAxisRows; r++) xs[r].load(in, d.first + r * d.step < d.end ? d.first + r * d.step : cv);
#pragma unroll
    for (int r = 0; r < kAxisRows; r++) {
        const int64_t v = d.first + r * d.step;
        const Pack<TQ, 8>& x = xs[r];
        float f[8];
#pragma unroll
        for (int k = 0; k < 8; k++) f[k] = dequant_f32((int)x.get(k) - zp[k], sc[k]);
        Pack<TO, 8> y;
        if constexpr (std::is_same<TO, half_t>::value) {
            half_t h[8];
            narrow_vec(f, h);
#pragma unroll
            for (int k = 0; k < 8; k++) y.set(k, h[k]);
        } else {
#pragma unroll
            for (int k = 0; k < 8; k++) y.set(k, f[k]);
        }
        if (v < d.end) y.store(out, v);
    }
}

template <typename TI, typename TQ>
int quantize_axis_impl(const MemRef& in, const MemRef& out, const double* scales, const int64_t* zps, int64_t n, int64_t qmin,
                       int64_t qmax, hipStream_t s) {
    std::vector<float> lo((size_t)n), hi((size_t)n);
    for (int64_t c = 0; c < n; c++) {
        VPX_REQUIRE(scales[c] > 0.0, VPX_RESULT_ERROR_INVALID_ARGUMENT, "quantize: scale %lld must be positive, got %g", (long long)c,
                    scales[c]);
        lo[(size_t)c] = (float)((double)(qmin - zps[c]) * scales[c]);
        hi[(size_t)c] = (float)((double)(qmax - zps[c]) * scales[c]);
    }
    AxisGeom g;
    float4* table = nullptr;
    int rc = axis_setup("quantize", in, out, n, lo.data(), hi.data(), s, g, &table);
    if (rc) return rc;
    const uint32_t total = (uint32_t)in.numel();
    if (total == 0) return VPX_RESULT_SUCCESS;
    const float fmin_ = (float)qmin, fmax_ = (float)qmax, lm1 = (float)(qmax - qmin + 1) - 1.0f;
    constexpr uint32_t V = 16 / sizeof(TI);
    const bool al = (reinterpret_cast<uintptr_t>(in.data) & 15) == 0 && (reinterpret_cast<uintptr_t>(out.data) % V) == 0;
    const dim3 vgrid((total / V + kBlock - 1) / kBlock);
    const bool simple = levels_are_identity(fmin_, fmax_, lm1);
    if (al && g.inner % V == 0) {
        if (simple)
            hipLaunchKernelGGL((quantize_axis_vec_kernel<TI, TQ, true>), vgrid, dim3(kBlock), 0, s, (const TI*)in.data, (TQ*)out.data, table,
                               g, total / V, fmin_, fmax_, lm1);
        else
            hipLaunchKernelGGL((quantize_axis_vec_kernel<TI, TQ, false>), vgrid, dim3(kBlock), 0, s, (const TI*)in.data, (TQ*)out.data, table,
                               g, total / V, fmin_, fmax_, lm1);
    }
    else if (g.inner == 1) {
        const uint32_t rows = total / g.count;
        if (g.count % 8 == 0 && (reinterpret_cast<uintptr_t>(in.data) % (8 * sizeof(TI))) == 0 && (reinterpret_cast<uintptr_t>(out.data) & 7) == 0) {
            const dim3 igrid(inner_deal_blocks(g.count / 8, rows, kAxisRows));
            if (simple)
                hipLaunchKernelGGL((quantize_axis_inner8_kernel<TI, TQ, true>), igrid, dim3(kBlock), 0, s, (const TI*)in.data, (TQ*)out.data,
                                   table, g.count, rows, fmin_, fmax_, lm1);
            else
                hipLaunchKernelGGL((quantize_axis_inner8_kernel<TI, TQ, false>), igrid, dim3(kBlock), 0, s, (const TI*)in.data, (TQ*)out.data,
                                   table, g.count, rows, fmin_, fmax_, lm1);
        } else {
            const dim3 igrid(((g.count + kBlock - 1) / kBlock) * ((rows + kAxisRows - 1) / kAxisRows));
            hipLaunchKernelGGL((quantize_axis_inner_kernel<TI, TQ>), igrid, dim3(kBlock), 0, s, (const TI*)in.data, (TQ*)out.data, table,
                               g.count, rows, fmin_, fmax_, lm1);
        }
    }
    else
        hipLaunchKernelGGL((quantize_axis_kernel<TI, TQ>), dim3((total + kBlock - 1) / kBlock), dim3(kBlock), 0, s, (const TI*)in.data,
                           (TQ*)out.data, table, g, total, fmin_, fmax_, lm1);
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

template <typename TQ, typename TO>
int dequantize_axis_impl(const MemRef& in, const MemRef& out, const double* scales, const int64_t* zps, int64_t n, hipStream_t s) {
    std::vector<float> sc((size_t)n), zp((size_t)n);
    for (int64_t c = 0; c < n; c++) {
        sc[(size_t)c] = (float)scales[c];  // exact: the blob ships scales as fp16 or fp32
        zp[(size_t)c] = (float)zps[c];
    }
    AxisGeom g;
    float4* table = nullptr;
    int rc = axis_setup("dequantize", out, in, n, sc.data(), zp.data(), s, g, &table);
    if (rc) return rc;
    const uint32_t total = (uint32_t)in.numel();
    if (total == 0) return VPX_RESULT_SUCCESS;
    constexpr uint32_t V = 16 / sizeof(TO);
    const bool al = (reinterpret_cast<uintptr_t>(in.data) % V) == 0 && (reinterpret_cast<uintptr_t>(out.data) & 15) == 0;
    const dim3 vgrid((total / V + kBlock - 1) / kBlock);
    if (al && g.inner % V == 0)
        hipLaunchKernelGGL((dequantize_axis_vec_kernel<TQ, TO>), vgrid, dim3(kBlock), 0, s, (const TQ*)in.data, (TO*)out.data,
                           table, g, total / V);
    else if (g.inner == 1) {
        const uint32_t rows = total / g.count;
        if (g.count % 8 == 0 && (reinterpret_cast<uintptr_t>(in.data) & 7) == 0 && (reinterpret_cast<uintptr_t>(out.data) % (8 * sizeof(TO))) == 0) {
            const dim3 igrid(inner_deal_blocks(g.count / 8, rows, kAxisRows));
            hipLaunchKernelGGL((dequantize_axis_inner8_kernel<TQ, TO>), igrid, dim3(kBlock), 0, s, (const TQ*)in.data, (TO*)out.data, table,
                               g.count, rows);
        } else {
            const dim3 igrid(((g.count + kBlock - 1) / kBlock) * ((rows + kAxisRows - 1) / kAxisRows));
            hipLaunchKernelGGL((dequantize_axis_inner_kernel<TQ, TO>), igrid, dim3(kBlock), 0, s, (const TQ*)in.data, (TO*)out.data, table,
                               g.count, rows);
        }
    }
    else
        hipLaunchKernelGGL((dequantize_axis_kernel<TQ, TO>), dim3((total + kBlock - 1) / kBlock), dim3(kBlock), 0, s, (const TQ*)in.data,
                           (TO*)out.data, table, g, total);
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

}  // namespace

int release_axis_tables(int dev, hipStream_t s) {
    // every table of the stream leaves the cache and is freed; the first failure, if any, is what the call returns
    std::lock_guard<std::mutex> lock(g_axis_mutex);
    hipError_t first = hipSuccess;
    for (auto it = g_axis_tables.begin(); it != g_axis_tables.end();) {
        if (it->second.dev == dev && it->second.stream == s) {
            const hipError_t e = hipFree(it->second.table);
            if (e != hipSuccess && first == hipSuccess) first = e;
            it = g_axis_tables.erase(it);
        } else {
            ++it;
        }
    }
    VPX_HIP_CHECK(first);
    return VPX_RESULT_SUCCESS;
}

int launch_quantize_per_axis(const MemRef& in, const MemRef& out, const double* scales, const int64_t* zps, int64_t n,
                             hipStream_t s) {
    VPX_REQUIRE(same_shape(in, out), VPX_RESULT_ERROR_INVALID_ARGUMENT, "quantize: input and output shapes differ");
    if (in.dtype == VPX_NN_FP16 && out.dtype == VPX_NN_U8) return quantize_axis_impl<half_t, uint8_t>(in, out, scales, zps, n, 0, 255, s);
    if (in.dtype == VPX_NN_FP16 && out.dtype == VPX_NN_I8) return quantize_axis_impl<half_t, int8_t>(in, out, scales, zps, n, -128, 127, s);
    if (in.dtype == VPX_NN_FP32 && out.dtype == VPX_NN_U8) return quantize_axis_impl<float, uint8_t>(in, out, scales, zps, n, 0, 255, s);
    if (in.dtype == VPX_NN_FP32 && out.dtype == VPX_NN_I8) return quantize_axis_impl<float, int8_t>(in, out, scales, zps, n, -128, 127, s);
    return fail(VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "quantize: %s -> %s is not implemented", dtype_name(in.dtype),
                dtype_name(out.dtype));
}

int launch_dequantize_per_axis(const MemRef& in, const MemRef& out, const double* scales, const int64_t* zps, int64_t n,
                               hipStream_t s) {
    VPX_REQUIRE(same_shape(in, out), VPX_RESULT_ERROR_INVALID_ARGUMENT, "dequantize: input and output shapes differ");
    if (in.dtype == VPX_NN_U8 && out.dtype == VPX_NN_FP16) return dequantize_axis_impl<uint8_t, half_t>(in, out, scales, zps, n, s);
    if (in.dtype == VPX_NN_I8 && out.dtype == VPX_NN_FP16) return dequantize_axis_impl<int8_t, half_t>(in, out, scales, zps, n, s);
    if (in.dtype == VPX_NN_U8 && out.dtype == VPX_NN_FP32) return dequantize_axis_impl<uint8_t, float>(in, out, scales, zps, n, s);
    if (in.dtype == VPX_NN_I8 && out.dtype == VPX_NN_FP32) return dequantize_axis_impl<int8_t, float>(in, out, scales, zps, n, s);
    return fail(VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "dequantize: %s -> %s is not implemented", dtype_name(in.dtype),
                dtype_name(out.dtype));
}

}  // namespace vpx
