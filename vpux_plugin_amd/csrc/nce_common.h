// Shared pieces of the NCE cluster task on CDNA4 (8-bit convolution / matmul with int32 accumulation on the i8 MFMA
// units and the integer PPE fused into the epilogue): the PPE arithmetic, the descriptors the host hands to the kernels,
// the LDS and store helpers, and the launchers each kernel family's translation unit exports.
//
//   nce.hip             the dispatcher (vpx_nce_task -> kernel), tuning knobs, operand views, preparation kernels
//   nce_gemm.hip        nce_gemm_mfma: 1x1 layers and NCE.MatMul
//   nce_gemm_regb.hip   nce_gemm_regb: the same with a short K and many rows, weights in registers
//   nce_conv_patch.hip  nce_conv_regw / nce_conv_tile / nce_conv_stream: input rows of a tile in LDS
//   nce_conv_rows.hip   nce_conv_rows16: channel counts that are a multiple of 16 only
//   nce_conv_gather.hip nce_conv_mfma / nce_conv_mfma16 / nce_conv_naive: the general fallbacks
//   nce_eltwise.hip     task type ELTWISE
//
// Zero points: the MFMA paths multiply raw bytes (u8 activations are re-biased to s8 by flipping
// the top bit) and add the missing term to the bias: acc_true = acc_raw + k * sum_k w[oc][k] with
// k = 128 - zp_in (u8) or -zp_in (i8); padded taps are filled with the byte that stands for the
// zero point so they contribute exactly 0, as the MPE does (runtime_dpu_parser_imports.cpp.inc:872-879).
// A weight zero point (mpe_wtbias, :940-945) adds one term per output position, prepared by two small
// kernels and added to the accumulators before the PPE (see nce_pixel_sum_kernel).
#pragma once

#include <atomic>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <type_traits>
#include <utility>

#include "vpx_common.h"

namespace vpx {
namespace nce {

typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
typedef int32_t i32x16 __attribute__((ext_vector_type(16)));

struct Ppe {
    int prelu_mult, prelu_shift, zp_out, clamp_lo, clamp_hi;
    float f16_lo, f16_hi;  // fp16 output only: the clamp bounds unpacked from clamp_high (infinite when absent)
};

enum OutKind { OUT_U8 = 0, OUT_I8 = 1, OUT_F16 = 2 };

// Raw per-channel PPE parameters, unpacked from weight-table words 2 and 3.
struct ChanParams {
    int bias, mult, shift;
};

// Integer PPE in the order the compiler programs it (expand_dpu_config_invariant_ppe.cpp:322-380):
// bias add, scale multiply, [prelu multiply on negatives], one round-half-even over the combined
// right shift, zero point, clamp.  64-bit integer arithmetic; the general, slow form.
__device__ __forceinline__ int ppe_requant(int acc, ChanParams c, Ppe p) {
    const int biased = (int)((unsigned)acc + (unsigned)c.bias);
    long long t = (long long)biased * (long long)c.mult;
    int s = c.shift;
    if (t < 0) {
        t *= (long long)p.prelu_mult;
        s += p.prelu_shift;
    }
    long long r;
    if (s <= 0) {
        r = t;
    } else if (s >= 64) {
        r = 0;
    } else {
        const long long q = t >> s;
        const unsigned long long rem = (unsigned long long)t & ((1ull << s) - 1ull);
        const unsigned long long half = 1ull << (s - 1);
        r = q + ((rem > half || (rem == half && (q & 1))) ? 1 : 0);
    }
    r += p.zp_out;
    r = r < p.clamp_lo ? p.clamp_lo : r;
    r = r > p.clamp_hi ? p.clamp_hi : r;
    return (int)r;
}

// fp16 output ("INT32 s17.15 fixed-point convert to FP16", runtime_dpu_parser_imports.cpp.inc:546-552): the
// round stage keeps 15 fractional bits, the 32-bit result fx stands for fx * 2^-15, and that value is narrowed to
// fp16 with one round-to-nearest-even.  A float holds 24 bits: the 31-bit magnitude is first cut to 24 bits with
// the lost bits OR-ed into the last one (round to odd), which makes the hardware's second rounding to 11 bits exact.
__device__ __forceinline__ uint16_t f16_from_s1715(int fx, float lo, float hi) {
    unsigned a = fx < 0 ? 0u - (unsigned)fx : (unsigned)fx;
    const int lz = __builtin_clz(a | 1u);
    const int drop = lz < 8 ? 8 - lz : 0;
    const unsigned sticky = (a & ((1u << drop) - 1u)) != 0u ? 1u : 0u;
    a = (a >> drop) | sticky;
    float v = __builtin_ldexpf((float)a, drop - 15);  // exact
    v = fx < 0 ? -v : v;
    _Float16 h = (_Float16)v;
    const float r = (float)h;
    h = r < lo ? (_Float16)lo : h;
    h = r > hi ? (_Float16)hi : h;
    return __builtin_bit_cast(uint16_t, h);
}

// The same pipeline as ppe_requant up to the round stage, in 64-bit integers (general, slow form).
__device__ __forceinline__ uint16_t ppe_requant_f16(int acc, ChanParams c, Ppe p) {
    const int biased = (int)((unsigned)acc + (unsigned)c.bias);
    long long t = (long long)biased * (long long)c.mult;
    int s = c.shift - 15;
    if (t < 0) {
        t *= (long long)p.prelu_mult;
        s += p.prelu_shift;
    }
    long long r;
    if (s <= 0) {
        // |t| < 2^58 and s >= -15: saturate before the shift could overflow
        const long long lim = 0x7fffffffffffffffll >> (-s);
        r = t > lim ? 0x7fffffffffffffffll : (t < -lim ? -0x7fffffffffffffffll : t * (1ll << (-s)));
    } else if (s >= 64) {
        r = 0;
    } else {
        const long long q = t >> s;
        const unsigned long long rem = (unsigned long long)t & ((1ull << s) - 1ull);
        const unsigned long long half = 1ull << (s - 1);
        r = q + ((rem > half || (rem == half && (q & 1))) ? 1 : 0);
    }
    r = r > 2147483647ll ? 2147483647ll : (r < -2147483648ll ? -2147483648ll : r);
    return f16_from_s1715((int)r, p.f16_lo, p.f16_hi);
}

template <bool OUT_SIGNED>
__device__ __forceinline__ int saturate8i(int r) {
    if (OUT_SIGNED) return r < -128 ? -128 : (r > 127 ? 127 : r);
    return r < 0 ? 0 : (r > 255 ? 255 : r);
}
template <bool OUT_SIGNED>
__device__ __forceinline__ uint8_t saturate8(int r) {
    return (uint8_t)saturate8i<OUT_SIGNED>(r);
}

// Per-channel parameters prepared for the fast epilogue.  With f = mult * 2^-shift (exactly
// representable), one double-precision fused multiply-add b * f + 1.5 * 2^52 rounds the exact
// product to an integer, ties to even, in a single step: that IS the round-half-even shift of the
// integer pipeline, for every 32-bit b and every multiplier / shift the weight table can hold.
// The integer then sits in the low dword of the sum.  f_pos serves t >= 0 and
// f_neg = mult * prelu_mult * 2^-(shift + prelu_shift) serves t < 0.
struct ChanPrep {
    double f_pos;
    double f_neg;
    int bias;      // weight-table bias with the zero-point term folded in
    int sgn;       // -1 when mult < 0, else 0: t < 0  <=>  (b ^ sgn) < 0 for b != 0
    int bmax_pos;  // |b| beyond these makes |b * f| exceed 2^30: such b are clipped first, which
    int bmax_neg;  // cannot change a result that saturates anyway; INT_MAX when |f| <= 1/2
};
static_assert(sizeof(ChanPrep) == 32, "ChanPrep layout");

struct PpeFast {
    int zp_out, lo, hi;  // clamp bounds already intersected with the storage range
    // Weights with a zero point: rowterm[m] = (what is left of the weight zero point) x the sum of
    // (activation - zero point) under the window of output position m, added to every channel of that
    // position; null when the weights the kernel reads have none (see nce_pixel_sum_kernel).
    const int32_t* rowterm;
    float f16_lo, f16_hi;  // fp16 output: clamp bounds
};

// Any bound between the largest |b| whose result can still lie inside a clamp window and 2^30 / |f|
// serves; single precision is plenty.
__device__ __forceinline__ int ppe_bmax(double f) {
    const float a = __builtin_fabsf((float)f);
    return a <= 0.5f ? 0x7fffffff : (int)(1.0e9f * __builtin_amdgcn_rcpf(a));
}

__device__ __forceinline__ ChanPrep ppe_prepare(int mult, int shift, int bias, int prelu_mult, int prelu_shift) {
    ChanPrep c;
    c.bias = bias;
    c.sgn = mult < 0 ? -1 : 0;
    c.f_pos = __builtin_ldexp((double)mult, -shift);
    c.f_neg = __builtin_ldexp((double)((long long)mult * (long long)prelu_mult), -(shift + prelu_shift));
    c.bmax_pos = ppe_bmax(c.f_pos);
    c.bmax_neg = ppe_bmax(c.f_neg);
    return c;
}

// CLIP = false may be used when both bmax are INT_MAX (no clipping needed).
template <bool CLIP>
__device__ __forceinline__ int ppe_fast(int acc, const ChanPrep& c, const PpeFast& p) {
    int b = (int)((unsigned)acc + (unsigned)c.bias);
    const bool neg = (b ^ c.sgn) < 0;
    const double f = neg ? c.f_neg : c.f_pos;
    if (CLIP) {
        const int bm = neg ? c.bmax_neg : c.bmax_pos;
        b = b > bm ? bm : (b < -bm ? -bm : b);
    }
    // (double)b without a conversion instruction: the bit pattern of 2^52 + (b + 2^31), minus that offset
    const double bd = __builtin_bit_cast(double, 0x4330000000000000ull | (unsigned long long)((unsigned)b ^ 0x80000000u)) -
                      4503601774854144.0;
    constexpr double kMagic = 6755399441055744.0;  // 1.5 * 2^52
    const double y = __builtin_fma(bd, f, kMagic);
    const int q = (int)(unsigned)__builtin_bit_cast(unsigned long long, y) + p.zp_out;
    const int t = q > p.lo ? q : p.lo;
    return t < p.hi ? t : p.hi;
}

// The same narrowing from the fixed-point value held as a double (an integer v standing for v * 2^-15; any magnitude).
// v is first rounded to the eleven significant bits of an fp16 by adding and subtracting 2^(exponent of v + 42) with
// v's sign: the sum's last place is then 2^(exponent - 10), the addition rounds to nearest even there and the
// subtraction is exact.  What is left converts to single precision, scales by 2^-15 and converts to fp16 without
// further rounding (|v| < 2 is exact as it is: multiples of 2^-15 are fp16 subnormals' multiples of 2^-24), and values
// from 65520 on become infinite as in the direct conversion -- which is also what the 32-bit saturation of the
// fixed-point stage ends in (2^31 - 1 stands for 65535.99997), so that stage needs no step of its own here.
__device__ __forceinline__ uint16_t f16_from_scaled(double v, float lo, float hi) {
    const unsigned top = (unsigned)(__builtin_bit_cast(unsigned long long, v) >> 32);
    const unsigned mtop = ((top & 0x7ff00000u) + (42u << 20)) | (top & 0x80000000u);
    const double big = __builtin_bit_cast(double, (unsigned long long)mtop << 32);
    const double r = (v + big) - big;
    const float x = (float)r * 0x1p-15f;
    float y = x < lo ? lo : x;
    y = x > hi ? hi : y;
    return __builtin_bit_cast(uint16_t, (_Float16)y);
}

// fp16 output, fast form.  `c` comes from ppe_prepare with shift - 15, so b * f is the value in units of 2^-15;
// the fused multiply-add rounds the exact product once to an integer (ties to even) and the subtraction that
// follows is exact (products too large for that trick stay far above the fp16 range).
__device__ __forceinline__ uint16_t ppe_fast_f16(int acc, const ChanPrep& c, float lo, float hi) {
    const int b = (int)((unsigned)acc + (unsigned)c.bias);
    const bool neg = (b ^ c.sgn) < 0;
    const double f = neg ? c.f_neg : c.f_pos;
    constexpr double kMagic = 6755399441055744.0;  // 1.5 * 2^52
    const double v = __builtin_fma((double)b, f, kMagic) - kMagic;
    return f16_from_scaled(v, lo, hi);
}

// Four results of one output channel as four bytes.  Same arithmetic as ppe_fast with the tail
// shortened: the even part of the output zero point (plus 128 for signed storage) is folded into
// the rounding constant -- an odd offset there would flip which way ties round --, the clamp is
// one float median (all values involved are small integers, exact in fp32; anything larger lies
// outside the window on the correct side), and the byte is produced by the saturating
// convert-and-pack instruction.  Signed storage flips the top bits afterwards.
// GENERAL adds what few layers need: clipping of inputs whose product would leave the +-2^30
// range, and the odd unit of the zero point.
struct PpePack {
    double magic;  // 1.5 * 2^52 + the even part of (zp_out + 128 when the output is signed)
    int odd;       // the remaining 0 or 1
    int lo, hi;    // clamp window in the same shifted domain, inside [0, 255]
    unsigned flip; // 0x80808080 for signed storage, else 0
};

__device__ __forceinline__ PpePack make_ppe_pack(int zp_out, int lo, int hi, bool out_signed) {
    const int off = out_signed ? 128 : 0;
    const int z = zp_out + off;
    return PpePack{6755399441055744.0 + (double)(z & ~1), z & 1, lo + off, hi + off, out_signed ? 0x80808080u : 0u};
}

__device__ __forceinline__ int med3_i32(int v, int lo, int hi) {
    int r;
    asm("v_med3_i32 %0, %1, %2, %3" : "=v"(r) : "v"(v), "v"(lo), "v"(hi));
    return r;
}

// `c` must come from ppe_prepare_packed: its bias carries the +2^31 that turns the int -> double bit trick's sign
// flip into part of the bias addition, and for a negative multiplier its two factors (and bounds) are swapped, so
// that "the scaled value is negative" is simply "acc + bias is negative", whatever the multiplier's sign.
// (one value: the clamped integer in [0, 255] before the byte is placed and the sign bits flipped)
template <bool SAME_F, bool GENERAL>
__device__ __forceinline__ unsigned ppe_one(int a, const ChanPrep& c, const PpePack& p) {
    unsigned bu = (unsigned)a + (unsigned)c.bias;  // (acc + bias) ^ 0x80000000
    double f = c.f_pos;
    int bm = c.bmax_pos;
    if (!SAME_F) {
        const bool neg = (int)bu >= 0;  // flipped domain: top bit clear means acc + bias < 0
        f = neg ? c.f_neg : c.f_pos;
        if (GENERAL) bm = neg ? c.bmax_neg : c.bmax_pos;
    }
    if (GENERAL) {
        int b = (int)(bu ^ 0x80000000u);
        b = b > bm ? bm : (b < -bm ? -bm : b);
        bu = (unsigned)b ^ 0x80000000u;
    }
    const double bd = __builtin_bit_cast(double, 0x4330000000000000ull | (unsigned long long)bu) - 4503601774854144.0;
    const double y = __builtin_fma(bd, f, p.magic);
    int q = (int)(unsigned)__builtin_bit_cast(unsigned long long, y);
    if (GENERAL) q += p.odd;
    return (unsigned)med3_i32(q, p.lo, p.hi);
}

template <bool SAME_F, bool GENERAL>
__device__ __forceinline__ unsigned ppe_pack4(int a0, int a1, int a2, int a3, const ChanPrep& c, const PpePack& p) {
    const int a[4] = {a0, a1, a2, a3};
    unsigned w = 0;
#pragma unroll
    for (int r = 0; r < 4; r++) w |= ppe_one<SAME_F, GENERAL>(a[r], c, p) << (8 * r);
    return w ^ p.flip;
}

// ChanPrep for ppe_pack4: the bias carries the sign flip.
__device__ __forceinline__ ChanPrep ppe_prepare_packed(int mult, int shift, int bias, int prelu_mult, int prelu_shift) {
    ChanPrep c = ppe_prepare(mult, shift, bias, prelu_mult, prelu_shift);
    c.bias = (int)((unsigned)c.bias + 0x80000000u);
    if (c.sgn) {  // mult < 0: b < 0 scales to a non-negative value and takes f_pos, b > 0 takes f_neg (b = 0 gives 0 either way)
        const double f = c.f_pos;
        c.f_pos = c.f_neg;
        c.f_neg = f;
        const int bm = c.bmax_pos;
        c.bmax_pos = c.bmax_neg;
        c.bmax_neg = bm;
    }
    return c;
}

// The same four bytes from accumulators that already contain the bias (the MFMA chain started from it), for layers
// that need neither the clipping nor the odd zero-point unit of GENERAL: one conversion, one fused multiply-add,
// one median per value.  LEAKY: the negative branch scales by a slope in [0, 1] of the same sign (ReLU, LeakyReLU,
// PReLU up to 1): then b * f_neg >= b * f_pos exactly when b < 0, so the larger of the two rounded products is the
// result and no sign test is needed (rounding is monotone).  `c` comes from ppe_prepare (not _packed).
template <bool LEAKY>
__device__ __forceinline__ unsigned ppe_one_biased(int a, double f_pos, double f_neg, const PpePack& p) {
    const double bd = (double)a;
    int q = (int)(unsigned)__builtin_bit_cast(unsigned long long, __builtin_fma(bd, f_pos, p.magic));
    if (LEAKY) {
        const int qn = (int)(unsigned)__builtin_bit_cast(unsigned long long, __builtin_fma(bd, f_neg, p.magic));
        q = q > qn ? q : qn;
    }
    return (unsigned)med3_i32(q, p.lo, p.hi);
}

template <bool LEAKY>
__device__ __forceinline__ unsigned ppe_pack4_biased(int a0, int a1, int a2, int a3, double f_pos, double f_neg, const PpePack& p) {
    const int a[4] = {a0, a1, a2, a3};
    unsigned w = 0;
#pragma unroll
    for (int r = 0; r < 4; r++) w |= ppe_one_biased<LEAKY>(a[r], f_pos, f_neg, p) << (8 * r);
    return w ^ p.flip;
}

// ---------------------------------------------------------------- geometry of a task
struct ConvGeom {
    int64_t N, H, W, IC, OC, OH, OW;
    int KY, KX, SY, SX, PT, PL;
    // Where the operands' images, rows and pixels lie: the input in bytes, the output in elements (a dense NHWC tensor
    // has isw = IC, ish = W * isw, isn = H * ish and osw = OC, osh = OW * osw, osn = OH * osh; a view of a larger
    // tensor -- a channel slice, a window in H or W -- has the parent's).
    int64_t isn, ish, isw;
    int64_t osn, osh, osw;
    int out_flat;       // 2: output position m = (n, oy, ox) of N x OH x OW sits at m * osw; 1: that holds inside an image; 0: neither
    unsigned out_bits;  // the output's base address and its strides in bytes, or-ed: the alignment every row start shares
};

// Element offset of output position m, counted over the dense N x OH x OW positions.
__device__ __forceinline__ int64_t out_pos(const ConvGeom& g, int64_t m) {
    if (g.out_flat == 2) return m * g.osw;
    const int64_t ohow = g.OH * g.OW;
    const int64_t n = m / ohow, rem = m - n * ohow, oy = rem / g.OW, ox = rem - oy * g.OW;
    return n * g.osn + oy * g.osh + ox * g.osw;
}
// Byte offset of input pixel (n, iy, ix).
__device__ __forceinline__ int64_t in_pos(const ConvGeom& g, int64_t n, int64_t iy, int64_t ix) {
    return n * g.isn + iy * g.ish + ix * g.isw;
}
// Largest store (16, 8, 4 bytes, or 1) that every row start of the output is aligned to.
__device__ __forceinline__ int out_align(unsigned bits) {
    return (bits & 15) == 0 ? 16 : ((bits & 7) == 0 ? 8 : ((bits & 3) == 0 ? 4 : 1));
}

// ---------------------------------------------------------------- LDS tiles, DMA, byte transposes, ragged stores
// LDS tile of ROWS x BK bytes; the 16-byte chunk c of row r is kept at chunk slot c ^ swz(r) so
// that the lanes served together by a 128-bit LDS read hit different bank groups.
template <int BK>
__device__ __forceinline__ int lds_swz(int row) {
    constexpr int CPR = BK / 16;   // chunks per row
    constexpr int RPW = 16 / CPR;  // rows per 256-byte bank wrap
    return (row / RPW) % CPR;
}
template <int BK>
__device__ __forceinline__ int lds_offset(int row, int chunk) {
    return row * BK + ((chunk ^ lds_swz<BK>(row)) << 4);
}

// 16 bytes per lane from global memory straight into LDS: the wave's 64 lanes fill the 1 KiB that
// starts at the wave-uniform LDS byte address `lds_addr`, lane l at +16*l.  Issued as assembly so
// that the compiler keeps managing only the counter of the LDS reads; completion of these loads is
// awaited explicitly with dma_wait_all_and_barrier().
// The source is a wave-uniform base plus a 32-bit per-lane byte offset.
__device__ __forceinline__ void dma16(const void* gbase, unsigned goff, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(goff), "s"(gbase) : "memory");
}
__device__ __forceinline__ void dma_wait_all_and_barrier() {
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

template <typename T>
__device__ __forceinline__ unsigned lds_address(T* p) {
    return (unsigned)(size_t)(__attribute__((address_space(3))) char*)(p);
}

template <int CTRL>
__device__ __forceinline__ unsigned dpp_u32(unsigned v) {
    return (unsigned)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, 0xf, 0xf, true);
}

// Each lane of a quad holds one dword = 4 bytes of ONE column (rows R..R+3).  Afterwards lane t of
// the quad holds row R+t of the quad's FOUR columns, i.e. 4 bytes that are adjacent in memory.
// The two byte selectors depend on the lane only; QuadTranspose keeps them in registers so that a run of transposes
// does not rebuild them every time.
struct QuadTranspose {
    unsigned sel1, sel2;
    __device__ __forceinline__ explicit QuadTranspose(int lane) {
        // (v_perm_b32 selector bytes: 0-3 pick from the second source, 4-7 from the first)
        sel1 = (lane & 1) ? 0x03070105u : 0x06020400u;
        sel2 = (lane & 2) ? 0x03020706u : 0x05040100u;
        asm volatile("" : "+v"(sel1), "+v"(sel2));
    }
    __device__ __forceinline__ unsigned operator()(unsigned w) const {
        const unsigned p = dpp_u32<0xB1>(w);  // lane ^ 1
        // even lane: [w.b0, p.b0, w.b2, p.b2]   odd lane: [p.b1, w.b1, p.b3, w.b3]
        const unsigned a = __builtin_amdgcn_perm(p, w, sel1);
        const unsigned q = dpp_u32<0x4E>(a);  // lane ^ 2
        // lanes 0,1: [a.b0, a.b1, q.b0, q.b1]   lanes 2,3: [q.b2, q.b3, a.b2, a.b3]
        return __builtin_amdgcn_perm(q, a, sel2);
    }
};
__device__ __forceinline__ unsigned quad_transpose_bytes(unsigned w, int lane) {
    return QuadTranspose(lane)(w);
}

// The first `count` (at most 16) bytes of `v` to a destination that is not known to be 16-byte aligned or that ends
// early -- rows whose length is not a multiple of 16 bytes: whole 8- or 4-byte pieces where the row length and the
// tensor's base allow (`align`: 8, 4, or less), single bytes for what is left.  (72-, 88-, 120-, 200-channel layers
// are common in mobile networks; byte by byte their stores took three times the rest of the kernel.)
__device__ __forceinline__ void store_tail16(uint8_t* dst, const i32x4& v, int count, int align) {
    int e = 0;
    if (align >= 8) {
#pragma unroll
        for (int h = 0; h < 2; h++)
            if (count >= 8 * h + 8) {
                *reinterpret_cast<uint2*>(dst + 8 * h) = uint2{(unsigned)v[2 * h], (unsigned)v[2 * h + 1]};
                e = 8 * h + 8;
            }
    } else if (align >= 4) {
#pragma unroll
        for (int q = 0; q < 4; q++)
            if (count >= 4 * q + 4) {
                *reinterpret_cast<unsigned*>(dst + 4 * q) = (unsigned)v[q];
                e = 4 * q + 4;
            }
    }
    for (; e < count; e++) dst[e] = (uint8_t)(v[e >> 2] >> (8 * (e & 3)));
}
// alignment (8, 4 or 1) shared by every 16-byte-chunk start of rows `row_bytes` long in a tensor at `base`
__device__ __forceinline__ int row_align(const void* base, int64_t row_bytes) {
    const unsigned bits = (unsigned)reinterpret_cast<uintptr_t>(base) | (unsigned)row_bytes;
    return (bits & 7) == 0 ? 8 : ((bits & 3) == 0 ? 4 : 1);
}

constexpr int kOutStride = 288;  // bytes per row of the 256-column output staging tile in LDS
constexpr int kGemmLdsHead = 1024;  // bytes in front of the matmul kernel's panel buffers (column sums of B)

struct GemmPpe {
    int prelu_mult, prelu_shift;  // applied to negative scaled values (1,0 = none; 0,0 = ReLU)
    int corr;                     // zero-point term: acc_true = acc_raw + corr * sum_k B[n][k]
    int zp_out, lo, hi;           // clamp bounds already intersected with the storage range
    int out_signed;               // output storage is i8
    const int32_t* rowterm;       // as in PpeFast; padded past the last position, so edge tiles may read ahead
    float f16_lo, f16_hi;         // fp16 output: clamp bounds
    int out_f16;                  // the LDS-patch tile kernels: the output is fp16 (s17.15 narrowed), not bytes
};

// Where the rows of A sit: row m at byte m * K (a matrix, or a 1x1 stride-1 layer), or, for a 1x1 layer with a stride,
// output position m = (n, oy, ox) at pixel (n, oy * sy, ox * sx) of the input tensor -- the matmul kernel's loads
// take a byte offset per lane, so a strided 1x1 convolution is a matmul whose rows are picked from the input.
struct GemmRows {
    int strided;              // 0: row m at byte m * lda
    int64_t lda;
    int ow, ohow;             // output width, positions per image
    unsigned px, py, pimg;    // bytes from one output column / row / image to the next in the input (strides folded in)
};

// Where the rows of the result go: row m at element m * ldc (a matrix, a dense tensor, or a channel slice of one), or
// position m = (n, oy, ox) at n * sn + oy * sh + ox * sw (a window of a larger tensor).
struct GemmOut {
    int flat;                 // 1: row m at m * sw
    int64_t sn, sh, sw;
    int ow, ohow;
    unsigned bits;            // base address and strides in bytes, or-ed (see ConvGeom::out_bits)
    __device__ __forceinline__ int64_t row(int64_t m) const {
        if (flat) return m * sw;
        const unsigned mm = (unsigned)m, img = mm / (unsigned)ohow, rem = mm - img * (unsigned)ohow, oy = rem / (unsigned)ow, ox = rem - oy * (unsigned)ow;
        return (int64_t)img * sn + (int64_t)oy * sh + (int64_t)ox * sw;
    }
};

// A[M][K] x B[N][K]^T with the PPE fused; see the file header.  K must be a multiple of 64.
//
// Pipeline.  K is walked in panels of 64 bytes; a panel of A and B (32 KiB) goes from global memory
// straight into one of four LDS buffers.  In iteration kt the waves multiply panel kt, fetch panel
// kt+3 (8 DMA instructions per wave, spread between the MFMAs) and read the fragments one sub-step
// ahead; the only wait is for panel kt+1, which was requested two iterations earlier, and it sits
// with the workgroup barrier in the middle of the iteration, between the two sub-steps,
// so that the MFMAs of the second sub-step cover the first fragment reads of panel kt+1.  The column sums of B that the zero-point
// term needs come from nce_colsum_kernel (only when that term is not zero), and the per-column PPE

// ---------------------------------------------------------------- convolutions with the input patch in LDS
// A tile is `R` whole output rows of one image x 64 output channels.  The (R-1)*SY+KY input rows a
// tile needs are copied to LDS once, padding materialised with the zero-point byte and u8 re-biased
// to s8 on the way, so every tap of every output position is an LDS read.  The tile has
// MT = ceil(R*OW / 32) row blocks of 32 positions and one or two column blocks of 32 channels; wave
// w takes column block w % nt and the TMW row blocks w / nt + i * (waves / nt).  Row blocks past MT
// are computed on position 0 and dropped: the main loops have no branches.
//
// At the sizes these kernels serve a whole launch lasts a few microseconds, so index arithmetic
// counts: divisions by launch constants use multiply-high reciprocals prepared on the host.
struct FastDiv {
    uint32_t d, m;  // m = ceil(2^32 / d); exact for numerators below 2^32 / d
};
__device__ __forceinline__ int fdiv(int a, FastDiv f) {
    return f.d == 1 ? a : (int)__umulhi((unsigned)a, f.m);
}

struct PatchGeom {
    int R;        // output rows per tile
    int PH, PW;   // patch size in input pixels
    int MT;       // row blocks of 32 output positions per tile
    int nt;       // column blocks of 32 channels in use (1 or 2)
    int w_swz;    // weights rows are swizzled
    int ntiles;   // tiles per 64-channel block: N * tiles_y
    int patch_bytes;
    FastDiv tiles_y, cpr, cpp, upr, ow;  // tiles per image, chunks per weight row / pixel, units per patch row, OW
};

// Element offset of the tile's position p = r * OW + ox from the tile's first output position (rows osh apart).
__device__ __forceinline__ int64_t tile_out_pos(const ConvGeom& g, int p, FastDiv ow) {
    if (g.out_flat) return (int64_t)p * g.osw;
    const int r = fdiv(p, ow), ox = p - r * (int)ow.d;
    return (int64_t)r * g.osh + (int64_t)ox * g.osw;
}

constexpr int kPatchMaxMT = 14;
constexpr int kPatchOutStride = 80;  // bytes per output position in the staging tile
constexpr int kPatchOutStrideF16 = 144;  // the same for an fp16 output

// fp16 output of the tile kernels below (a wave holds row blocks mi0, mi0 + mstep, ... of 32 positions x the 32 channels
// of tile nj; accumulator register r of lane l is position 8*(r/4) + 4*(l/32) + r%4, channel l%32): values through the
// staging tile, 128 bytes a position, then whole runs of eight channels per store.  All threads of the workgroup call
// this after the barrier that frees the patch.
template <int TMW, int NT>
__device__ __forceinline__ void patch_epilogue_f16(i32x16 (&acc)[TMW], int mi0, int mstep, int nj, int MT, const ChanPrep& c,
                                                   const GemmPpe& ppe, const int32_t* rt, uint8_t* stage, uint16_t* out16,
                                                   int valid, int oc0, int OC, const ConvGeom& g, FastDiv ow) {
    const int tid = threadIdx.x, lane = tid & 63;
#pragma unroll
    for (int i = 0; i < TMW; i++) {
        const int mi = mi0 + i * mstep;
        if (mi >= MT) continue;
        uint8_t* const col = stage + (mi * 32 + 4 * (lane >> 5)) * kPatchOutStrideF16 + (nj * 32 + (lane & 31)) * 2;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int row = 8 * (r / 4) + (r % 4);
            const int extra = rt ? rt[mi * 32 + 4 * (lane >> 5) + row] : 0;
            *reinterpret_cast<uint16_t*>(col + row * kPatchOutStrideF16) = ppe_fast_f16(acc[i][r] + extra, c, ppe.f16_lo, ppe.f16_hi);
        }
    }
    __syncthreads();
    const bool vec_ok = (g.out_bits & 15) == 0;
    for (int cid = tid; cid < valid * 8; cid += NT) {
        const int row = cid >> 3, c8 = cid & 7;
        const int n = oc0 + c8 * 8;
        if (n >= OC) continue;
        const i32x4 v = *reinterpret_cast<const i32x4*>(stage + row * kPatchOutStrideF16 + c8 * 16);
        uint16_t* dst = out16 + (tile_out_pos(g, row, ow) + n);
        if (vec_ok && n + 8 <= OC) {
            __builtin_nontemporal_store(v, reinterpret_cast<i32x4*>(dst));
        } else {
            store_tail16(reinterpret_cast<uint8_t*>(dst), v, (OC - n < 8 ? OC - n : 8) * 2, out_align(g.out_bits));
        }
    }
}

// SAME_F (template parameter of the kernels below): the PPE treats both signs alike (no PReLU stage),
// which drops the per-value sign test.

// Weight slices of the streamed-weights convolution kernel.
struct StreamGeom {
    int ksl;       // channels per weight slice
    int spt;       // slices per tap = IC / ksl
};

// Tiles of the row-patch convolution kernel.
struct RowsGeom {
    int R, CW;       // output rows and columns per tile
    int PH;          // patch rows: (R - 1) * SY + KY
    int RB;          // bytes per patch row in LDS: m planes of `plane` chunks
    int row_chunks;  // 16-byte chunks per patch row
    int m, plane;    // chunks between neighbouring output positions; chunks per plane
    int S;           // MFMA steps: K / 16 chunks, two a step
    int WS;          // bytes per weight row in LDS: S * 32 + 16
    int ntiles;      // N * tiles per image
    FastDiv tiles_x, cw;  // column tiles per row of tiles, CW
    FastDiv tiles_y, ow, rc, cpp, kc, fm, rin;  // tiles per image, OW, row_chunks, chunks per pixel, 2 * S, m, chunks per kernel row
};

// TN: channel tiles of 32 per workgroup (1 for layers of up to 32 output channels; 4, with TM = 2, for short-K layers of
// many output channels, whose input rows are then staged by half as many workgroups).  MULTI: some workgroup takes more


// Kernels that may ask for more than 64 KiB of dynamic LDS are given the largest size any launch of them uses,
// once per (device, kernel): the attribute is then never changed again, so concurrent launches that want
// different sizes cannot undo each other's setting.
constexpr size_t kMaxDynLds = 160 * 1024 - 512;
int set_dyn_lds_attribute(const void* kernel);  // (nce.hip: once per device and kernel)
template <class KernelT>
int set_dyn_lds(KernelT kernel, size_t bytes) {
    if (bytes <= 64 * 1024) return VPX_RESULT_SUCCESS;
    VPX_REQUIRE(bytes <= kMaxDynLds, VPX_RESULT_ERROR_UNKNOWN, "a launch asks for %zu bytes of LDS", bytes);
    return set_dyn_lds_attribute(reinterpret_cast<const void*>(kernel));
}

// ---------------------------------------------------------------- what the dispatcher hands to a kernel family
// Dispatch overrides for tests and tuning.  The VPX_* environment variables of the same names are read once, at
// the first use; afterwards only vpx_set_tuning changes a value, so a launch never reads the environment.
enum { NCE_AUTO = 0, NCE_NAIVE, NCE_GATHER, NCE_CONV };
struct Tuning {
    std::atomic<int> nce_kernel{NCE_AUTO};  // VPX_NCE_KERNEL = naive | gather | conv: restrict the choice to slower, more general paths
    std::atomic<int> gemm_tile{0};          // VPX_GEMM_TILE = 128 | 256 (0: chosen from the shape)
    std::atomic<int> gemm_waves{0};         // VPX_GEMM_WAVES = 4 | 8
    std::atomic<int> gemm_regb{0};          // VPX_GEMM_REGB = on | wide | off: weights-in-registers matmul for K of 64, 128 or 256 (1, 2: with the most channel blocks per wave, -1; 0: chosen from the shape)
    std::atomic<int> gemm_pingpong{0};      // VPX_GEMM_PINGPONG = on | off: the waves of a SIMD take turns at the MFMAs
    std::atomic<int> conv_stream{0};        // VPX_CONV_KERNEL = regw | tile | stream: start the choice of LDS-patch kernel at this one (-1, 1, 2; 0: by size)
    std::atomic<int> conv_rows{0};          // VPX_CONV_ROWS = n: cap on the output rows per workgroup of the LDS-patch kernels
    std::atomic<int> conv_cols{0};          // VPX_CONV_COLS = n: output columns per tile of the row-patch kernel
    std::atomic<int> conv_waves{0};         // VPX_CONV_WAVES = 4 | 8
    std::atomic<int> stream_ksplit{1};      // VPX_STREAM_KSPLIT = off: the streamed-weights kernel never splits K over its waves
    std::atomic<int> mvn_fused{1};          // VPX_MVN_FUSED = off | nowait (see tuning_mvn_fused)
    std::atomic<int> calib_blocks{0};       // VPX_CALIB_BLOCKS = n: workgroups of the MFMA calibration loop (0: one per compute unit)
};
const Tuning& tuning();

// An operand of an NCE task as a view: the strides of its images, rows and pixels in elements (channels contiguous).
// All four task strides zero is the dense tensor.  Dimensions of size one take the stride that keeps the view as flat
// as the others allow (their own is never used).
struct View {
    int64_t sn, sh, sw;
    bool dense;   // the packed NHWC tensor
    int flat;     // 2: position m of N x H x W at m * sw; 1: that holds inside an image; 0: neither
    int64_t span; // elements from the first to one past the last
};
int operand_view(const int64_t st[4], int64_t N, int64_t H, int64_t W, int64_t C, const char* what, View* v);

// nce_gemm.hip.  `tile` 128 | 256, `waves` 4 | 8 (8 with the large tile only), `shortk`: K of at most three panels on
// the small tile; G groups on the grid's second dimension.
struct GemmLaunch {
    const int8_t* A;
    const int8_t* B;
    const int32_t* wt;
    uint8_t* out;
    int64_t M, N, K, G;
    int tile, waves;
    bool shortk, in_u8, pingpong;
    int out_kind;  // OutKind
    GemmPpe ppe;
    GemmRows rows;
    GemmOut dst;
};
int launch_gemm_mfma(const GemmLaunch& a, hipStream_t s);
// nce_gemm_regb.hip: K of 64, 128 or 256, rows of A and of the result at a fixed pitch, 16-byte aligned, N a multiple of
// 16, one group, byte output; `workgroups` x 4 waves, a multiple of
// (64-channel blocks / `cbw` / `gw`).
int launch_gemm_regb(const GemmLaunch& a, int cbw, int gw, int workgroups, hipStream_t s);
void gemm_regb_shape(int64_t M, int64_t N, int64_t K, int cus, bool widest, int* cbw, int* gw);  // 64-channel blocks per wave, groups of them per workgroup
int gemm_regb_workgroups_per_cu(bool same_f, int64_t K, int cbw);                   // resident workgroups the kernel's registers allow

// nce_conv_patch.hip: one workgroup per tile of `pg.R` output rows x 64 channels.
struct PatchLaunch {
    const int8_t* in;
    const int8_t* w;
    const int32_t* wt;
    const int32_t* colsum;  // streamed weights only: the sums of the weight rows, when the zero-point term needs them
    uint8_t* out;
    ConvGeom g;
    PatchGeom pg;
    StreamGeom sg;
    int pad_byte;
    GemmPpe ppe;
    bool in_u8, same_f;
    dim3 grid;
    size_t lds;
};
int launch_conv_regw(const PatchLaunch& a, hipStream_t s);
int launch_conv_tile(const PatchLaunch& a, int per_wave, int ics, int waves, hipStream_t s);
int launch_conv_stream(const PatchLaunch& a, int ksplit_waves, int per_wave, hipStream_t s);

// nce_conv_rows.hip: `bn` 32 | 64 | 128 channels per workgroup, `tm` 2 | 4 position blocks per wave block, `multi`: some
// workgroup takes more than one tile.
struct RowsLaunch {
    const int8_t* in;
    const int8_t* w;
    const int32_t* wt;
    uint8_t* out;
    ConvGeom g;
    RowsGeom rg;
    int pad_byte;
    GemmPpe ppe;
    bool in_u8, out_f16, multi;
    int bn, tm;
    dim3 grid;
    size_t lds;
};
int launch_conv_rows16(const RowsLaunch& a, hipStream_t s);

// nce_conv_gather.hip
int launch_fold(const int8_t* w, const int32_t* wt, ChanPrep* prep, int64_t OC, int64_t K, int corr, const Ppe& ppe, int shift_sub,
                hipStream_t s);
int launch_colsum(const int8_t* w, int32_t* colsum, int64_t OC, int64_t K, hipStream_t s);
int launch_conv_mfma(const int8_t* in, const int8_t* w, const ChanPrep* prep, uint8_t* out, const ConvGeom& g, int pad_byte,
                     const PpeFast& ppe, bool in_u8, int out_kind, hipStream_t s);
int launch_conv_mfma16(const int8_t* in, const int8_t* w, const ChanPrep* prep, uint8_t* out, const ConvGeom& g, int pad_byte,
                       const PpeFast& ppe, bool in_u8, int out_kind, hipStream_t s);
int launch_conv_naive(const uint8_t* in, const uint8_t* w, const int32_t* wt, uint8_t* out, const ConvGeom& g, int zp_in, int zp_w,
                      const Ppe& ppe, bool in_u8, bool w_u8, int out_kind, hipStream_t s);

// nce_eltwise.hip
int launch_nce_eltwise(const vpx_nce_task_t& t, const Ppe& ppe, hipStream_t s, const char** kernel_name);

}  // namespace nce
}  // namespace vpx
