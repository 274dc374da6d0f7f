// NCE cluster task on CDNA4: 8-bit convolution / matmul with int32 accumulation on the i8 MFMA
// units and the integer PPE fused into the epilogue.
//
// Device paths (chosen by vpx_nce_task):
//   nce_gemm_mfma   : 1x1 kernel, stride 1, no padding, more than 64 output channels (this is how
//                     NCE.MatMul arrives): a plain A[M][K] x B[N][K]^T GEMM.  256x256 output tile per
//                     workgroup, v_mfma_i32_32x32x32_i8, K panels from global memory straight into
//                     XOR-swizzled LDS (global_load_lds, no register staging), four buffers.
//   nce_conv_regw   : 3x3 taps of 64 input channels: the input rows of a tile sit in LDS, the weights of 64 output
//                     channels in the registers of every wave.
//   nce_conv_tile   : KYxKX / stride / padding with 64 or 128 input channels: the input rows of a tile
//                     and the weights of 64 output channels sit in LDS, every tap is an LDS read.
//   nce_conv_stream : the same with any multiple of 64 input channels: the weights pass through LDS a
//                     slice at a time.
//   nce_conv_mfma   : IC a multiple of 32, any size: activation fragments gathered from global
//                     memory, weights staged a K slice at a time.
//   nce_conv_mfma16 : IC a multiple of 16 only (stem layers), K up to 1008: two taps may share an MFMA step.
//   nce_eltwise_kernel : task type ELTWISE (quantized add / subtract).
//   nce_conv_naive  : any shape and any zero points, one output per lane.
//
// Zero points: the MFMA paths multiply raw bytes (u8 activations are re-biased to s8 by flipping
// the top bit) and add the missing term to the bias: acc_true = acc_raw + k * sum_k w[oc][k] with
// k = 128 - zp_in (u8) or -zp_in (i8); padded taps are filled with the byte that stands for the
// zero point so they contribute exactly 0, as the MPE does (runtime_dpu_parser_imports.cpp.inc:872-879).
// A weight zero point (mpe_wtbias, :940-945) adds one term per output position, prepared by two small
// kernels and added to the accumulators before the PPE (see nce_pixel_sum_kernel).
#include <atomic>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <set>
#include <type_traits>
#include <utility>

#include "vpx_common.h"

namespace vpx {

int launch_nce(const vpx_nce_task_t& t, hipStream_t s, const char** kernel_name);

namespace {

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

// ---------------------------------------------------------------- per-channel parameter fold
// One wavefront per output channel: sum of the channel's weights (for the zero-point term) and the
// prepared epilogue parameters.
__global__ __launch_bounds__(256) void nce_fold_kernel(const int8_t* __restrict__ w, const int32_t* __restrict__ wt,
                                                       ChanPrep* __restrict__ prep, int64_t OC, int64_t K, int corr,
                                                       Ppe ppe, int shift_sub) {
    const int lane = threadIdx.x & 63;
    const int64_t oc = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (oc >= OC) return;
    int sum = 0;
    if (corr != 0) {
        const int8_t* row = w + oc * K;
        if ((K & 15) == 0) {
            for (int64_t k = (int64_t)lane * 16; k < K; k += 64 * 16) {
                const i32x4 q = *reinterpret_cast<const i32x4*>(row + k);
#pragma unroll
                for (int j = 0; j < 4; j++) sum = __builtin_amdgcn_sdot4(q[j], 0x01010101, sum, false);
            }
        } else {
            for (int64_t k = lane; k < K; k += 64) sum += row[k];
        }
        for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
    }
    if (lane == 0) {
        const uint32_t w2 = (uint32_t)wt[oc * 4 + 2];
        // shift_sub = 15 for an fp16 output (the scaled value keeps 15 fractional bits), else 0
        const ChanPrep c = ppe_prepare((int)(int16_t)(w2 >> 16), (int)((w2 >> 8) & 0xffu) - shift_sub,
                                       (int)((unsigned)wt[oc * 4 + 3] + (unsigned)(corr * sum)), ppe.prelu_mult, ppe.prelu_shift);
        prep[oc] = c;
    }
}

// sum_k w[oc][k] alone (the GEMM path unpacks the weight table itself); one wavefront per channel,
// four 128-bit loads in flight per lane.
__global__ __launch_bounds__(256) void nce_colsum_kernel(const int8_t* __restrict__ w, int32_t* __restrict__ colsum,
                                                         int64_t OC, int64_t K) {
    const int lane = threadIdx.x & 63;
    const int64_t oc = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (oc >= OC) return;
    const int8_t* row = w + oc * K;
    int s0 = 0, s1 = 0, s2 = 0, s3 = 0;
    int64_t k = (int64_t)lane * 16;
    for (; k + 3 * 1024 < K; k += 4 * 1024) {
        const i32x4 q0 = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(row + k));
        const i32x4 q1 = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(row + k + 1024));
        const i32x4 q2 = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(row + k + 2048));
        const i32x4 q3 = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(row + k + 3072));
#pragma unroll
        for (int j = 0; j < 4; j++) {
            s0 = __builtin_amdgcn_sdot4(q0[j], 0x01010101, s0, false);
            s1 = __builtin_amdgcn_sdot4(q1[j], 0x01010101, s1, false);
            s2 = __builtin_amdgcn_sdot4(q2[j], 0x01010101, s2, false);
            s3 = __builtin_amdgcn_sdot4(q3[j], 0x01010101, s3, false);
        }
    }
    for (; k < K; k += 1024) {
        const i32x4 q = *reinterpret_cast<const i32x4*>(row + k);
#pragma unroll
        for (int j = 0; j < 4; j++) s0 = __builtin_amdgcn_sdot4(q[j], 0x01010101, s0, false);
    }
    int sum = (s0 + s1) + (s2 + s3);
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
    if (lane == 0) colsum[oc] = sum;
}

// ---------------------------------------------------------------- naive path
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

template <bool IN_SIGNED, bool W_SIGNED, int OUT>
__global__ __launch_bounds__(256) void nce_conv_naive(const uint8_t* __restrict__ in, const uint8_t* __restrict__ w,
                                                      const int32_t* __restrict__ wt, uint8_t* __restrict__ out,
                                                      ConvGeom g, int zp_in, int zp_w, Ppe ppe, int64_t total) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int64_t oc = idx % g.OC;
    const int64_t row = idx / g.OC;
    const int64_t ox = row % g.OW;
    const int64_t oy = (row / g.OW) % g.OH;
    const int64_t n = row / (g.OW * g.OH);
    int acc = 0;
    for (int ky = 0; ky < g.KY; ky++) {
        const int64_t iy = oy * g.SY + ky - g.PT;
        if (iy < 0 || iy >= g.H) continue;
        for (int kx = 0; kx < g.KX; kx++) {
            const int64_t ix = ox * g.SX + kx - g.PL;
            if (ix < 0 || ix >= g.W) continue;
            const uint8_t* pi = in + in_pos(g, n, iy, ix);
            const uint8_t* pw = w + ((oc * g.KY + ky) * g.KX + kx) * g.IC;
            for (int64_t ic = 0; ic < g.IC; ic++) {
                const int a = IN_SIGNED ? (int)(int8_t)pi[ic] : (int)pi[ic];
                const int b = W_SIGNED ? (int)(int8_t)pw[ic] : (int)pw[ic];
                acc += (a - zp_in) * (b - zp_w);
            }
        }
    }
    const uint32_t w2 = (uint32_t)wt[oc * 4 + 2];
    ChanParams c{wt[oc * 4 + 3], (int)(int16_t)(w2 >> 16), (int)((w2 >> 8) & 0xffu)};
    const int64_t o = n * g.osn + oy * g.osh + ox * g.osw + oc;
    if (OUT == OUT_F16) reinterpret_cast<uint16_t*>(out)[o] = ppe_requant_f16(acc, c, ppe);
    else out[o] = saturate8<OUT == OUT_I8>(ppe_requant(acc, c, ppe));
}

// ---------------------------------------------------------------- GEMM path
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
// parameters are unpacked from the weight table in the epilogue.
template <bool IN_U8, int OUT, int NW, int TILE = 256, bool SHORTK = false>
__global__ __launch_bounds__(64 * NW) void nce_gemm_mfma(const int8_t* __restrict__ A, const int8_t* __restrict__ B,
                                                     const int32_t* __restrict__ wt, const int32_t* __restrict__ colsum,
                                                     uint8_t* __restrict__ out,
                                                     int64_t M, int64_t N, int64_t K, int tiles_m, int tiles_n,
                                                     GemmPpe ppe, GemmRows rows, GemmOut dst) {
    // NW = 4: waves 2 x 2, 128 x 128 each, one per SIMD.  NW = 8: waves 2 x 4, 128 x 64 each, two per SIMD,
    // so that one wave's loads and address arithmetic issue while the other's MFMAs run.
    // TILE = 128 (four waves of 64 x 64, 64 KiB of LDS, two workgroups per CU) serves problems with too few 256 x 256 tiles.
    // SHORTK (K <= 192, three panels at most): all panels are fetched up front, nothing is pipelined and no panel buffer
    // is reused, so the workgroup asks only for the LDS it touches and more of them fit a CU (a matmul this short is
    // bound by its epilogue and stores, not by the MFMAs).
    constexpr int BM = TILE, BN = TILE, BK = 64, WM = BM / 2, WN = BN / (NW / 2), TM = WM / 32, TN = WN / 32;
    constexpr int MFMA_PER_DMA = TM * TN / (BM * BK / 1024 / NW);  // MFMAs between two DMA instructions of a sub-step
    static_assert(TM * TN >= TM + TN && MFMA_PER_DMA >= 1, "fragment reads and DMA instructions are interleaved with the MFMAs");
    constexpr int NT = 64 * NW;
    constexpr int NS = 4;                             // LDS panel buffers
    constexpr int CPR = BK / 16;                      // 16-byte chunks per tile row
    constexpr int RPI = 64 / CPR;                     // tile rows one 1 KiB DMA instruction covers
    constexpr int DMA_PER_WAVE = BM * BK / 1024 / NW;  // per operand, per panel
    constexpr int STAGE = (BM + BN) * BK;

    extern __shared__ __attribute__((aligned(16))) uint8_t smem_raw[];
    int* const colsums = reinterpret_cast<int*>(smem_raw);  // TILE column sums of B, handed from the upper waves to the lower
    uint8_t* const smem = smem_raw + kGemmLdsHead;          // the panel buffers, later the output staging tile

    // Grouped matmul: blockIdx.y is the group; every operand holds the groups one after the other.
    if (const int64_t grp = blockIdx.y) {
        A += grp * M * K;
        B += grp * N * K;
        wt += grp * N * 4;
        if (colsum) colsum += grp * N;
        out += grp * M * N * (OUT == OUT_F16 ? 2 : 1);
        if (ppe.rowterm) ppe.rowterm += grp * M;
    }

    // Workgroup ids are dealt round-robin to the 8 XCDs.  Give each XCD a contiguous run of tile
    // ids and walk tiles in groups of 4 tile-rows, so that workgroups resident on one XCD at the
    // same time share A and B panels in that XCD's L2.
    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) / 8;
    const int id = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (id >= total) return;
    constexpr int GM = 4;
    const int group = id / (GM * tiles_n);
    const int gm0 = group * GM;
    const int gsz = tiles_m - gm0 < GM ? tiles_m - gm0 : GM;
    const int in_group = id - group * GM * tiles_n;
    const int tm = gm0 + in_group % gsz;
    const int tn = in_group / gsz;
    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = NW == 4 ? (wave >> 1) * WM : (wave >> 2) * WM, wn0 = NW == 4 ? (wave & 1) * WN : (wave & 3) * WN;

    // Source addresses of this lane's DMA chunks.  Instruction q of a panel fills LDS bytes
    // [q*1024, q*1024+1024) of the operand's tile = rows q*RPI .. ; the lane sitting at chunk slot p
    // of row r fetches source chunk p ^ swz(r), which is what puts the swizzle in place.
    unsigned oa[DMA_PER_WAVE], ob[DMA_PER_WAVE];  // byte offsets from the tile's first row
#pragma unroll
    for (int i = 0; i < DMA_PER_WAVE; i++) {
        const int q = wave + NW * i;
        const int r = q * RPI + lane / CPR, p = lane % CPR;
        const int c = p ^ lds_swz<BK>(r);
        int64_t m = m0 + r, n = n0 + r;
        m = m < M ? m : M - 1;  // rows past the edge repeat the last one; their outputs are not stored
        n = n < N ? n : N - 1;
        oa[i] = (unsigned)((m - m0) * rows.lda + c * 16);
        if (rows.strided) {  // (offsets from the tensor's first byte; the host has checked that they fit 32 bits)
            const int mm = (int)m, img = mm / rows.ohow, rem = mm - img * rows.ohow, oy = rem / rows.ow, ox = rem - oy * rows.ow;
            oa[i] = (unsigned)img * rows.pimg + (unsigned)oy * rows.py + (unsigned)ox * rows.px + (unsigned)(c * 16);
        }
        ob[i] = (unsigned)((n - n0) * K + c * 16);
    }
    const int8_t* abase = rows.strided ? A : A + m0 * rows.lda;
    const int8_t* bbase = B + n0 * K;
    const unsigned lds0 = lds_address(smem);
    const int nk = (int)(K / BK);
    // d-th DMA instruction (first half A, second half B) of panel p.  Panels past the end keep the number of loads
    // in flight the same in every iteration: every lane re-fetches the tile's first 16 bytes (one cache line for
    // the whole instruction) into a buffer nobody reads.
    auto dma_one = [&](auto known_real, int p, int d) {
        const unsigned base = lds0 + (unsigned)((p & (NS - 1)) * STAGE);
        const bool real = decltype(known_real)::value || p < nk;  // (known: no select instructions in the loop body)
        const int64_t k0 = real ? (int64_t)p * BK : 0;
        if (d < DMA_PER_WAVE) dma16(abase + k0, real ? oa[d] : 0u, base + (unsigned)((wave + NW * d) * 1024));
        else dma16(bbase + k0, real ? ob[d - DMA_PER_WAVE] : 0u, base + (unsigned)(BM * BK + (wave + NW * (d - DMA_PER_WAVE)) * 1024));
    };

    i32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

    i32x4 fa[2][TM], fb[2][TN];
    auto load_frag = [&](const uint8_t* pa, int kk, int slot, int n) {
        const int chunk = kk * 2 + (lane >> 5);
        if (n == 0) fa[slot][0] = *reinterpret_cast<const i32x4*>(pa + lds_offset<BK>(wm0 + (lane & 31), chunk));
        else if (n <= TN) fb[slot][n - 1] = *reinterpret_cast<const i32x4*>(pa + BM * BK + lds_offset<BK>(wn0 + (n - 1) * 32 + (lane & 31), chunk));
        else fa[slot][n - TN] = *reinterpret_cast<const i32x4*>(pa + lds_offset<BK>(wm0 + (n - TN) * 32 + (lane & 31), chunk));
    };
    // The same reads for a panel buffer known at compile time: the lane's part of the address is one of eight registers
    // that do not change over the K loop (operand, sub-step, lower or upper pair of buffers) and everything else is the
    // instruction's immediate offset, so the unrolled loop below computes no LDS address.
    typedef const __attribute__((address_space(3))) uint8_t* lds_bytes_t;  // 32-bit LDS addresses: one register each
    typedef const __attribute__((address_space(3))) i32x4* lds_v4_t;
    lds_bytes_t frag_base[2][2][2];  // [buffer pair][operand: 0 = A, 1 = B][sub-step]
#pragma unroll
    for (int hi = 0; hi < 2; hi++)
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            const int chunk = kk * 2 + (lane >> 5);
            frag_base[hi][0][kk] = (lds_bytes_t)(smem + hi * 2 * STAGE + lds_offset<BK>(wm0 + (lane & 31), chunk));
            frag_base[hi][1][kk] = (lds_bytes_t)(smem + hi * 2 * STAGE + BM * BK + lds_offset<BK>(wn0 + (lane & 31), chunk));
            asm volatile("" : "+v"(frag_base[hi][0][kk]), "+v"(frag_base[hi][1][kk]));  // keep them: re-deriving costs vector ALU slots per read
        }
    auto load_frag_static = [&](auto stage_c, int kk, int slot, int n) {
        constexpr int stage = decltype(stage_c)::value;
        constexpr int imm = (stage & 1) * STAGE;
        // rows 32 apart are 32 * BK bytes apart and share their swizzle
        if (n == 0) fa[slot][0] = *(lds_v4_t)(frag_base[stage >> 1][0][kk] + imm);
        else if (n <= TN) fb[slot][n - 1] = *(lds_v4_t)(frag_base[stage >> 1][1][kk] + imm + (n - 1) * 32 * BK);
        else fa[slot][n - TN] = *(lds_v4_t)(frag_base[stage >> 1][0][kk] + imm + (n - TN) * 32 * BK);
    };
    // One sub-step: the TM x TN MFMAs on fragment slot `cur`; between them, the TM + TN fragment reads of the
    // next sub-step (panel at pnext, sub-step knext) into the other slot and this wave's DMA instructions
    // dma0.. of panel dma_p.
    // Column sums of B for the zero-point term, from the fragments as they pass: lane l sums the 16-byte chunks it
    // holds of column l % 32 (lanes l and l ^ 32 hold alternate chunks), four dot instructions per fragment.  Vector
    // ALU instructions between the MFMAs are not free (they take issue slots of the SIMD), so only the waves of the
    // tile's upper half (SUM) do this -- the lower half reads the same columns -- and hand the sums over through LDS.
    int cs[TN];
#pragma unroll
    for (int j = 0; j < TN; j++) cs[j] = 0;
    auto substep = [&](auto sum_c, auto next_stage_c, int cur, const uint8_t* pnext, int knext, int dma_p, int dma0) {
        constexpr bool SUM = decltype(sum_c)::value;
        constexpr int NEXT_STAGE = decltype(next_stage_c)::value;  // buffer the next sub-step's panel sits in, -1: see pnext
        auto load_next = [&](int n) {
            if constexpr (NEXT_STAGE >= 0) load_frag_static(next_stage_c, knext, cur ^ 1, n);
            else load_frag(pnext, knext, cur ^ 1, n);
        };
#pragma unroll
        for (int i = 0; i < TM; i++) {
            i32x4 a = fa[cur][i];
            if (IN_U8) a ^= (int32_t)0x80808080;  // u8 -> s8 (value - 128)
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const int idx = i * TN + j;
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, fb[cur][j], acc[i][j], 0, 0, 0);
                if (SUM && i == TM - 1) {  // behind the last MFMA that reads the fragment
#pragma unroll
                    for (int d = 0; d < 4; d++) cs[j] = __builtin_amdgcn_sdot4(fb[cur][j][d], 0x01010101, cs[j], false);
                }
                // all fragment reads of the next sub-step behind the first two MFMAs: the reads of the eight waves
                // queue at the LDS, and the last one issued must be back before this sub-step's MFMAs are through
                constexpr int FH = (TM + TN + 1) / 2;
                if (idx == 0) {
#pragma unroll
                    for (int n = 0; n < FH; n++) load_next(n);
                } else if (idx == 1) {
#pragma unroll
                    for (int n = FH; n < TM + TN; n++) load_next(n);
                }
                if (!SHORTK && idx % MFMA_PER_DMA == MFMA_PER_DMA - 1)
                    dma_one(std::integral_constant<bool, (NEXT_STAGE >= 0)>{}, dma_p, dma0 + idx / MFMA_PER_DMA);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    // per-column PPE words, fetched now so that the epilogue does not start with a memory round trip
    int w2r[TN], w3r[TN], csr[TN];
#pragma unroll
    for (int j = 0; j < TN; j++) {
        int64_t n = n0 + wn0 + j * 32 + (lane & 31);
        n = n < N ? n : N - 1;
        csr[j] = 0;
        w2r[j] = wt[n * 4 + 2];
        w3r[j] = wt[n * 4 + 3];
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // keeps the count of loads in flight below exact

    constexpr std::integral_constant<int, -1> kDynamicStage{};
    auto main_loop = [&](auto sum_c) {
        if (SHORTK) {
#pragma unroll
            for (int p = 0; p < NS - 1; p++)
                if (p < nk) {
#pragma unroll
                    for (int d = 0; d < 2 * DMA_PER_WAVE; d++) dma_one(std::false_type{}, p, d);
                }
            dma_wait_all_and_barrier();
#pragma unroll
            for (int n = 0; n < TM + TN; n++) load_frag(smem, 0, 0, n);
            for (int kt = 0; kt < nk; kt++) {
                const uint8_t* pcur = smem + kt * STAGE;
                const uint8_t* pnxt = kt + 1 < nk ? pcur + STAGE : pcur;  // the last step prefetches fragments nobody uses
                substep(sum_c, kDynamicStage, 0, pcur, 1, 0, 0);
                substep(sum_c, kDynamicStage, 1, pnxt, 0, 0, 0);
            }
        } else {
#pragma unroll
            for (int p = 0; p < NS - 1; p++)
#pragma unroll
                for (int d = 0; d < 2 * DMA_PER_WAVE; d++) dma_one(std::false_type{}, p, d);
            asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(4 * DMA_PER_WAVE) : "memory");  // panel 0 is in
#pragma unroll
            for (int n = 0; n < TM + TN; n++) load_frag(smem, 0, 0, n);
            int kt = 0;
            // Four panels per trip while all loads are real ones: the panel buffers are then known by number, the
            // fragment reads take immediate offsets and the loads need no selects.
            if ((nk & (NS - 1)) == 0) {
                auto one_panel = [&](auto u_c, int k) {
                    constexpr int u = decltype(u_c)::value;
                    substep(sum_c, std::integral_constant<int, u>{}, 0, nullptr, 1, k + NS - 1, 0);
                    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(3 * DMA_PER_WAVE) : "memory");
                    substep(sum_c, std::integral_constant<int, (u + 1) & (NS - 1)>{}, 1, nullptr, 0, k + NS - 1, DMA_PER_WAVE);
                };
                for (; kt + 2 * NS <= nk; kt += NS) {
                    one_panel(std::integral_constant<int, 0>{}, kt);
                    one_panel(std::integral_constant<int, 1>{}, kt + 1);
                    one_panel(std::integral_constant<int, 2>{}, kt + 2);
                    one_panel(std::integral_constant<int, 3>{}, kt + 3);
                }
            }
            for (; kt < nk; kt++) {
                const uint8_t* pcur = smem + (kt & (NS - 1)) * STAGE;
                const uint8_t* pnxt = smem + ((kt + 1) & (NS - 1)) * STAGE;
                substep(sum_c, kDynamicStage, 0, pcur, 1, kt + NS - 1, 0);
                // Loads in flight here, oldest first: panel kt+1, panel kt+2 (2 * DMA_PER_WAVE each), half of panel kt+3.
                // Behind the barrier panel kt+1 is complete for every wave and nobody reads panel kt-1 any
                // more, whose buffer panel kt+3 is being written to.
                asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(3 * DMA_PER_WAVE) : "memory");
                substep(sum_c, kDynamicStage, 1, pnxt, 0, kt + NS - 1, DMA_PER_WAVE);
            }
        }
    };
    // (a matmul of at most three panels is all epilogue: there every wave sums its own columns and nothing is handed over)
    if (SHORTK || wm0 == 0) main_loop(std::true_type{});
    else main_loop(std::false_type{});
#pragma unroll
    for (int j = 0; j < TN; j++) {
        csr[j] = cs[j] + __shfl_xor(cs[j], 32, 64);  // every lane takes part
        if (!SHORTK && wm0 == 0 && lane < 32) colsums[wn0 + j * 32 + lane] = csr[j];
    }
    dma_wait_all_and_barrier();  // every wave is done with the panels: LDS becomes the output staging tile
    if (!SHORTK) {
#pragma unroll
        for (int j = 0; j < TN; j++) csr[j] = colsums[wn0 + j * 32 + (lane & 31)];  // sum_k B[n][k] of column n of block j
    }

    // Epilogue.  Accumulator register r of lane l is C[8*(r/4) + 4*(l/32) + r%4][l%32] of its 32x32 tile.
    if constexpr (OUT == OUT_F16) {
        // fp16 output: through the staging tile like the bytes below, half of a 256-row tile at a time (128 rows x 544
        // bytes), so that the tile leaves in whole rows of 16-byte stores (two-byte stores straight from the registers,
        // 64 bytes of a row per half-wavefront, cost the [4096 x 4096] . [4096 x 11008] matmul 60 us).
        constexpr int PASSES = TILE == 256 ? 2 : 1, ROWS = BM / PASSES, STR = BN * 2 + 32;
        static_assert(ROWS * STR <= NS * STAGE, "the fp16 staging tile fits the panel buffers");
        uint16_t* out16 = reinterpret_cast<uint16_t*>(out);
        if (ppe.rowterm) {  // (padded past the last row: edge tiles may read ahead)
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const i32x4 v = *reinterpret_cast<const i32x4*>(ppe.rowterm + m0 + wm0 + i * 32 + 8 * g + 4 * (lane >> 5));
#pragma unroll
                    for (int j = 0; j < TN; j++)
#pragma unroll
                        for (int q = 0; q < 4; q++) acc[i][j][g * 4 + q] += v[q];
                }
        }
        const bool vec_ok = (dst.bits & 15) == 0;
#pragma unroll
        for (int pass = 0; pass < PASSES; pass++) {
            if (wm0 / ROWS == pass) {
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const uint32_t w2 = (uint32_t)w2r[j];
                    const ChanPrep c = ppe_prepare((int)(int16_t)(w2 >> 16), (int)((w2 >> 8) & 0xffu) - 15,
                                                   (int)((unsigned)w3r[j] + (unsigned)(ppe.corr * csr[j])), ppe.prelu_mult, ppe.prelu_shift);
                    uint8_t* const col = smem + (wm0 - pass * ROWS + 4 * (lane >> 5)) * STR + (wn0 + j * 32 + (lane & 31)) * 2;
#pragma unroll
                    for (int i = 0; i < TM; i++)
#pragma unroll
                        for (int r = 0; r < 16; r++)
                            *reinterpret_cast<uint16_t*>(col + (i * 32 + 8 * (r / 4) + (r % 4)) * STR) = ppe_fast_f16(acc[i][j][r], c, ppe.f16_lo, ppe.f16_hi);
                }
            }
            __syncthreads();
            for (int it = 0; it < ROWS * (BN / 8) / NT; it++) {
                const int cid = tid + NT * it;
                const int row = cid / (BN / 8), c8 = cid % (BN / 8);
                const int64_t m = m0 + pass * ROWS + row, n = n0 + c8 * 8;
                if (m >= M || n >= N) continue;
                const i32x4 v = *reinterpret_cast<const i32x4*>(smem + row * STR + c8 * 16);
                uint16_t* const to = out16 + dst.row(m) + n;
                if (vec_ok && n + 8 <= N) {
                    __builtin_nontemporal_store(v, reinterpret_cast<i32x4*>(to));
                } else {
                    store_tail16(reinterpret_cast<uint8_t*>(to), v, (int)(N - n < 8 ? N - n : 8) * 2, out_align(dst.bits));
                }
            }
            if (pass + 1 < PASSES) __syncthreads();  // the other half overwrites the staging tile
        }
        return;
    }
    constexpr bool OUT_SIGNED = OUT == OUT_I8;
    ChanPrep cp[TN];
    bool clip = false;
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const uint32_t w2 = (uint32_t)w2r[j];
        cp[j] = ppe_prepare_packed((int)(int16_t)(w2 >> 16), (int)((w2 >> 8) & 0xffu),
                                   (int)((unsigned)w3r[j] + (unsigned)(ppe.corr * csr[j])), ppe.prelu_mult, ppe.prelu_shift);
        clip = clip || cp[j].bmax_pos != 0x7fffffff || cp[j].bmax_neg != 0x7fffffff;
        // keep the prepared factors in registers: without this the compiler re-derives them per element
        asm volatile("" : "+v"(cp[j].f_pos), "+v"(cp[j].f_neg));
    }
    const PpePack pk = make_ppe_pack(ppe.zp_out, ppe.lo, ppe.hi, OUT_SIGNED);
    if (ppe.rowterm) {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const i32x4 v = *reinterpret_cast<const i32x4*>(ppe.rowterm + m0 + wm0 + i * 32 + 8 * g + 4 * (lane >> 5));
#pragma unroll
                for (int j = 0; j < TN; j++)
#pragma unroll
                    for (int q = 0; q < 4; q++) acc[i][j][g * 4 + q] += v[q];
            }
    }
    // kind 0: every PPE setting; 1: no clipping, even zero-point offset, slope in [0, 1] (ReLU, LeakyReLU): no sign
    // test, see ppe_pack4_biased; 2: the same with slope 1 (no PReLU stage)
    auto requant_tile = [&](auto kind_c) {
        constexpr int KIND = decltype(kind_c)::value;
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int col4 = wn0 + j * 32 + ((lane & 31) & ~3);
            const int pb = (int)((unsigned)cp[j].bias - 0x80000000u);  // the bias without the sign flip of the packed form
#pragma unroll
            for (int i = 0; i < TM; i++) {
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    unsigned w;
                    if constexpr (KIND == 0)
                        w = ppe_pack4<false, true>(acc[i][j][g * 4], acc[i][j][g * 4 + 1], acc[i][j][g * 4 + 2], acc[i][j][g * 4 + 3], cp[j], pk);
                    else  // (the larger of the two products is the same whichever way a negative multiplier swapped the factors)
                        w = ppe_pack4_biased<KIND == 1>(acc[i][j][g * 4] + pb, acc[i][j][g * 4 + 1] + pb, acc[i][j][g * 4 + 2] + pb,
                                                        acc[i][j][g * 4 + 3] + pb, cp[j].f_pos, cp[j].f_neg, pk);
                    w = quad_transpose_bytes(w, lane);
                    const int row = wm0 + i * 32 + 8 * g + 4 * (lane >> 5) + (lane & 3);
                    *reinterpret_cast<unsigned*>(smem + row * kOutStride + col4) = w;
                }
            }
        }
    };
    // scale factors above 1/2 are rare (shift < 15), as are odd zero-point offsets and slopes outside [0, 1]
    const bool slope_ok = ppe.prelu_mult >= 0 && (ppe.prelu_shift >= 31 || ppe.prelu_mult <= (1 << ppe.prelu_shift));
    if (__builtin_amdgcn_ballot_w64(clip) != 0 || pk.odd != 0 || !slope_ok) requant_tile(std::integral_constant<int, 0>{});
    else if (ppe.prelu_mult == 1 && ppe.prelu_shift == 0) requant_tile(std::integral_constant<int, 2>{});
    else requant_tile(std::integral_constant<int, 1>{});
    __syncthreads();
    const bool vec_ok = (dst.bits & 15) == 0;
    for (int it = 0; it < BM * (BN / 16) / NT; it++) {
        const int cid = tid + NT * it;
        const int row = cid / (BN / 16), c16 = cid % (BN / 16);
        const int64_t m = m0 + row, n = n0 + c16 * 16;
        if (m >= M || n >= N) continue;
        const i32x4 v = *reinterpret_cast<const i32x4*>(smem + row * kOutStride + c16 * 16);
        uint8_t* const to = out + dst.row(m) + n;
        if (vec_ok && n + 16 <= N) {
            __builtin_nontemporal_store(v, reinterpret_cast<i32x4*>(to));
        } else {
            store_tail16(to, v, (int)(N - n < 16 ? N - n : 16), out_align(dst.bits));
        }
    }
}

// ---------------------------------------------------------------- implicit-GEMM convolution path
// Workgroup: BM output positions (flattened n, oy, ox) x BN output channels, 4 waves split BM.
// The weights of the BN channels, all taps, sit in LDS as [BN][KY*KX*IC] rows (swizzle as above
// on 64-byte granules, applied when a row is a whole number of them); activation fragments come
// straight from global memory, 16 bytes per lane.
template <int BM, int BN, bool IN_U8, int OUT>
__global__ __launch_bounds__(256) void nce_conv_mfma(const int8_t* __restrict__ in, const int8_t* __restrict__ w,
                                                     const ChanPrep* __restrict__ prep, uint8_t* __restrict__ out,
                                                     ConvGeom g, int pad_byte, int swz, int tc, int icc, PpeFast ppe) {
    constexpr int WM = BM / 4;
    constexpr int TM = WM / 32, TN = BN / 32;
    // Weights are staged a slice of K at a time: `tc` taps x `icc` channels of each of the BN rows
    // (the whole of K when it fits).  Slice row stride KC = tc * icc bytes.
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];  // [BN][KC]
    const int64_t Ktot = (int64_t)g.KY * g.KX * g.IC;
    const int64_t Mtot = g.N * g.OH * g.OW;
    const int64_t m0 = (int64_t)blockIdx.x * BM;
    const int64_t oc0 = (int64_t)blockIdx.y * BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int taps = g.KY * g.KX;
    const int KC = tc * icc;

    // positions of this lane's rows
    int64_t base_n[TM];
    int oy[TM], ox[TM];
#pragma unroll
    for (int i = 0; i < TM; i++) {
        int64_t m = m0 + wave * WM + i * 32 + (lane & 31);
        m = m < Mtot ? m : Mtot - 1;
        ox[i] = (int)(m % g.OW);
        oy[i] = (int)((m / g.OW) % g.OH);
        base_n[i] = (m / (g.OW * g.OH)) * g.isn;
    }
    const int pad32 = (pad_byte & 0xff) * 0x01010101;

    i32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

    const int kgroup = lane >> 5;  // which 16-byte half of a 32-wide K step this lane feeds
    for (int tap0 = 0; tap0 < taps; tap0 += tc) {
        const int ntap = taps - tap0 < tc ? taps - tap0 : tc;
        for (int ic0 = 0; ic0 < (int)g.IC; ic0 += icc) {
            const int icn = (int)g.IC - ic0 < icc ? (int)g.IC - ic0 : icc;
            // stage the slice: 16-byte chunks, chunk index xor-ed with (row>>2)&3 inside 64-byte granules
            const int cpt = icn / 16;  // chunks per tap of this slice
            const int chunks_per_row = ntap * cpt;
            __syncthreads();           // everybody is done with the previous slice
            for (int cid = tid; cid < BN * chunks_per_row; cid += 256) {
                const int row = cid / chunks_per_row;
                const int c = cid - row * chunks_per_row;
                const int tl = c / cpt, cc = c - tl * cpt;
                int64_t oc = oc0 + row;
                oc = oc < g.OC ? oc : g.OC - 1;
                const i32x4 q = *reinterpret_cast<const i32x4*>(w + oc * Ktot + (int64_t)(tap0 + tl) * g.IC + ic0 + cc * 16);
                const int lc = tl * (icc / 16) + cc;  // chunk position in the slice row
                const int cs = swz ? ((lc & ~3) | ((lc ^ (row >> 2)) & 3)) : lc;
                *reinterpret_cast<i32x4*>(smem + row * KC + cs * 16) = q;
            }
            __syncthreads();
            for (int tl = 0; tl < ntap; tl++) {
                const int tap = tap0 + tl;
                const int ky = tap / g.KX, kx = tap - ky * g.KX;
                const int8_t* pin[TM];
                bool inside[TM];
#pragma unroll
                for (int i = 0; i < TM; i++) {
                    const int iy = oy[i] * g.SY + ky - g.PT;
                    const int ix = ox[i] * g.SX + kx - g.PL;
                    inside[i] = iy >= 0 && iy < g.H && ix >= 0 && ix < g.W;
                    pin[i] = in + base_n[i] + (int64_t)(inside[i] ? iy : 0) * g.ish + (int64_t)(inside[i] ? ix : 0) * g.isw + ic0 + kgroup * 16;
                }
                for (int ic = 0; ic < icn; ic += 32) {
                    i32x4 fa[TM], fb[TN];
#pragma unroll
                    for (int i = 0; i < TM; i++) {
                        i32x4 q = *reinterpret_cast<const i32x4*>(pin[i] + ic);
                        if (!inside[i]) q = i32x4{pad32, pad32, pad32, pad32};
                        if (IN_U8) q ^= (int32_t)0x80808080;
                        fa[i] = q;
                    }
                    const int c = tl * (icc / 16) + ic / 16 + kgroup;
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        const int row = j * 32 + (lane & 31);
                        const int cs = swz ? ((c & ~3) | ((c ^ (row >> 2)) & 3)) : c;
                        fb[j] = *reinterpret_cast<const i32x4*>(smem + row * KC + cs * 16);
                    }
#pragma unroll
                    for (int i = 0; i < TM; i++)
#pragma unroll
                        for (int j = 0; j < TN; j++)
                            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
                }
            }
        }
    }

#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int64_t oc = oc0 + j * 32 + (lane & 31);
        if (oc >= g.OC) continue;
        const ChanPrep cp = prep[oc];
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int64_t m = m0 + wave * WM + i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
                if (m >= Mtot) continue;
                const int a = acc[i][j][r] + (ppe.rowterm ? ppe.rowterm[m] : 0);
                const int64_t o = out_pos(g, m) + oc;
                if (OUT == OUT_F16) reinterpret_cast<uint16_t*>(out)[o] = ppe_fast_f16(a, cp, ppe.f16_lo, ppe.f16_hi);
                else out[o] = (uint8_t)ppe_fast<true>(a, cp, ppe);
            }
        }
    }
}

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

// ---------------------------------------------------------------- patch convolution, one tile per workgroup
// Everything here is shaped for few instructions, which is what
// bounds a convolution of a few microseconds: LDS rows are padded by 16 bytes instead of
// xor-swizzled (pixel stride IC + 16, weight-row stride Ktot + 16: with IC a multiple of 64 the 16
// lanes an LDS pass serves fall on 16 different 4-bank groups), so a fragment address is one add of
// a per-tap scalar to a per-lane constant and the K steps inside a tap are immediate offsets;
// one workgroup computes one tile; fragments of tap t+1 are read while the MFMAs of tap t run.
// ICS = IC / 64.
template <bool IN_U8, int TMW, bool SAME_F, int ICS, int NW>
__global__ __launch_bounds__(64 * NW, NW == 8 ? 1 : (TMW <= 4 ? 2 : 1)) void nce_conv_tile(const int8_t* __restrict__ in,
                                                                      const int8_t* __restrict__ w,
                                                                      const int32_t* __restrict__ wt,
                                                                      uint8_t* __restrict__ out, ConvGeom g, PatchGeom pg,
                                                                      int pad_byte, GemmPpe ppe) {
    constexpr int BN = 64, IC = ICS * 64, KS = ICS * 2, PS = IC + 16, NT = 64 * NW;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int Ktot = g.KY * g.KX * IC, WS = Ktot + 16;
    uint8_t* const wlds = smem;             // [64][Ktot + 16]
    uint8_t* const patch = smem + BN * WS;  // [PH*PW][IC + 16], later the output staging tile
    __shared__ int csum[BN];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int img = fdiv(blockIdx.x, pg.tiles_y);
    const int oy0 = (blockIdx.x - img * (int)pg.tiles_y.d) * pg.R;
    const int oc0 = blockIdx.y * BN;

    // ---- weights and patch -> LDS; every load is issued before the first LDS store
    {
        constexpr int UW = NW == 8 ? 5 : 9, UP = NW == 8 ? 3 : 6;
        const int cpr = (int)pg.cpr.d;                 // 16-byte chunks per weight row
        const int wchunks = BN * cpr;
        constexpr int cpp = IC / 16;
        const int row_chunks = pg.PW * cpp;
        const int upr = (int)pg.upr.d, units = pg.PH * upr;
        const int pad32 = (pad_byte & 0xff) * 0x01010101;
        const int8_t* img_base = in + (int64_t)img * g.isn;
        const int iy0 = oy0 * g.SY - g.PT;
        const bool full_rows = oc0 + BN <= g.OC;       // the 64 weight rows are one contiguous run
        for (int q0 = 0, u0 = 0; q0 < wchunks || u0 < units; q0 += NT * UW, u0 += NW * UP) {
            i32x4 qw[UW], qp[UP];
            int dw[UW], dp[UP];
#pragma unroll
            for (int u = 0; u < UW; u++) {
                const int q = q0 + u * NT + tid;
                const bool ok = q < wchunks;
                const int qq = ok ? q : 0;
                const int row = fdiv(qq, pg.cpr);
                int64_t src = (int64_t)qq * 16;
                if (!full_rows) {
                    const int64_t oc = oc0 + row < g.OC ? row : g.OC - 1 - oc0;
                    src = oc * Ktot + (int64_t)(qq - row * cpr) * 16;
                }
                qw[u] = *reinterpret_cast<const i32x4*>(w + (int64_t)oc0 * Ktot + src);
                dw[u] = ok ? (qq + row) * 16 : -1;
            }
#pragma unroll
            for (int u = 0; u < UP; u++) {
                const int unit = u0 + wave + NW * u;
                const int py = fdiv(unit, pg.upr);  // wave-uniform
                const int qi = (unit - py * upr) * 64 + lane;
                const bool ok = unit < units && qi < row_chunks;
                const int px = qi / cpp, cc = qi % cpp;
                const int iy = iy0 + py, ix = px - g.PL;
                const bool inside = ok && iy >= 0 && iy < g.H && ix >= 0 && ix < g.W;
                const int64_t off = inside ? (int64_t)iy * g.ish + (int64_t)ix * g.isw + cc * 16 : 0;
                const i32x4 v = *reinterpret_cast<const i32x4*>(img_base + off);
                qp[u] = inside ? v : i32x4{pad32, pad32, pad32, pad32};
                dp[u] = ok ? (py * pg.PW + px) * PS + cc * 16 : -1;
            }
#pragma unroll
            for (int u = 0; u < UW; u++)
                if (dw[u] >= 0) *reinterpret_cast<i32x4*>(wlds + dw[u]) = qw[u];
#pragma unroll
            for (int u = 0; u < UP; u++)
                if (dp[u] >= 0) {
                    if (IN_U8) qp[u] ^= (int32_t)0x80808080;
                    *reinterpret_cast<i32x4*>(patch + dp[u]) = qp[u];
                }
        }
    }
    __syncthreads();

    // ---- per-channel weight sums from the LDS copy
    if (ppe.corr != 0 && tid < 256) {
        const int row = tid >> 2, part = tid & 3;
        int sum = 0;
        for (int c = part; c < (int)pg.cpr.d; c += 4) {
            const i32x4 q = *reinterpret_cast<const i32x4*>(wlds + row * WS + c * 16);
#pragma unroll
            for (int j = 0; j < 4; j++) sum = __builtin_amdgcn_sdot4(q[j], 0x01010101, sum, false);
        }
        sum += (int)dpp_u32<0xB1>((unsigned)sum);
        sum += (int)dpp_u32<0x4E>((unsigned)sum);
        if (part == 0) csum[row] = sum;
    }

    // ---- main loop
    const int nj = pg.nt == 2 ? wave & 1 : 0;
    const int mi0 = pg.nt == 2 ? wave >> 1 : wave, mstep = pg.nt == 2 ? NW / 2 : NW;
    const int npos = pg.R * (int)g.OW;
    const int kgroup = lane >> 5;
    int abase[TMW];
#pragma unroll
    for (int i = 0; i < TMW; i++) {
        int p = (mi0 + i * mstep) * 32 + (lane & 31);
        p = p < npos ? p : 0;
        const int r = fdiv(p, pg.ow), ox = p - r * (int)g.OW;
        abase[i] = (r * g.SY * pg.PW + ox * g.SX) * PS + kgroup * 16;
    }
    const int brow = nj * 32 + (lane & 31);
    const int bbase = brow * WS + kgroup * 16;

    i32x4 fa[2][KS][TMW], fb[2][KS];
    auto read_tap = [&](auto buf_c, int soff_a, int soff_b) {
        constexpr int buf = decltype(buf_c)::value;
        const uint8_t* pb = wlds + bbase + soff_b;
#pragma unroll
        for (int k = 0; k < KS; k++) fb[buf][k] = *reinterpret_cast<const i32x4*>(pb + k * 32);
#pragma unroll
        for (int i = 0; i < TMW; i++) {
            const uint8_t* pa = patch + abase[i] + soff_a;
#pragma unroll
            for (int k = 0; k < KS; k++) fa[buf][k][i] = *reinterpret_cast<const i32x4*>(pa + k * 32);
        }
    };
    i32x16 acc[TMW];
#pragma unroll
    for (int i = 0; i < TMW; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0;
    auto mfma_tap = [&](auto buf_c) {
        constexpr int buf = decltype(buf_c)::value;
#pragma unroll
        for (int k = 0; k < KS; k++)
#pragma unroll
            for (int i = 0; i < TMW; i++) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[buf][k][i], fb[buf][k], acc[i], 0, 0, 0);
    };
    const int taps = g.KY * g.KX;
    int ky = 0, kx = 0, tap = 0;
    auto next_tap = [&]() {  // advances (ky, kx, tap); returns false past the last one
        tap++;
        kx++;
        if (kx == g.KX) {
            kx = 0;
            ky++;
        }
        return tap < taps;
    };
    read_tap(std::integral_constant<int, 0>{}, 0, 0);
    for (;;) {
        const bool more1 = next_tap();
        if (more1) read_tap(std::integral_constant<int, 1>{}, (ky * pg.PW + kx) * PS, tap * IC);
        mfma_tap(std::integral_constant<int, 0>{});
        if (!more1) break;
        const bool more0 = next_tap();
        if (more0) read_tap(std::integral_constant<int, 0>{}, (ky * pg.PW + kx) * PS, tap * IC);
        mfma_tap(std::integral_constant<int, 1>{});
        if (!more0) break;
    }
    __syncthreads();  // all waves are done with the patch: its LDS becomes the output staging tile

    // ---- epilogue
    if (ppe.out_f16) {
        int64_t n = oc0 + brow;
        n = n < g.OC ? n : g.OC - 1;
        const uint32_t w2 = (uint32_t)wt[n * 4 + 2];
        const ChanPrep c = ppe_prepare((int)(int16_t)(w2 >> 16), (int)((w2 >> 8) & 0xffu) - 15,
                                       (int)((unsigned)wt[n * 4 + 3] + (unsigned)(ppe.corr * (ppe.corr != 0 ? csum[brow] : 0))),
                                       ppe.prelu_mult, ppe.prelu_shift);
        const int rows_here = g.OH - oy0 < pg.R ? (int)(g.OH - oy0) : pg.R;
        const int64_t pos0 = ((int64_t)img * g.OH + oy0) * g.OW;
        patch_epilogue_f16<TMW, NT>(acc, mi0, mstep, nj, pg.MT, c, ppe, ppe.rowterm ? ppe.rowterm + pos0 : nullptr, patch,
                                    reinterpret_cast<uint16_t*>(out) + ((int64_t)img * g.osn + (int64_t)oy0 * g.osh),
                                    rows_here * (int)g.OW, oc0, (int)g.OC, g, pg.ow);
        return;
    }
    {
        int64_t n = oc0 + brow;
        n = n < g.OC ? n : g.OC - 1;
        const int cs = ppe.corr != 0 ? csum[brow] : 0;
        const uint32_t w2 = (uint32_t)wt[n * 4 + 2];
        ChanPrep cp = ppe_prepare_packed((int)(int16_t)(w2 >> 16), (int)((w2 >> 8) & 0xffu),
                                         (int)((unsigned)wt[n * 4 + 3] + (unsigned)(ppe.corr * cs)), ppe.prelu_mult, ppe.prelu_shift);
        asm volatile("" : "+v"(cp.f_pos), "+v"(cp.f_neg));
        const PpePack pk = make_ppe_pack(ppe.zp_out, ppe.lo, ppe.hi, ppe.out_signed != 0);
        // (the short PPE serves slopes in [0, 1], an even zero-point offset and scales up to 1/2: see ppe_pack4_biased)
        const bool slope_ok = SAME_F || (ppe.prelu_mult >= 0 && (ppe.prelu_shift >= 31 || ppe.prelu_mult <= (1 << ppe.prelu_shift)));
        const bool general = __builtin_amdgcn_ballot_w64(cp.bmax_pos != 0x7fffffff || cp.bmax_neg != 0x7fffffff) != 0 || pk.odd != 0 || !slope_ok;
        const int pb = (int)((unsigned)cp.bias - 0x80000000u);  // the bias without the sign flip of the packed form
        const int col4 = nj * 32 + ((lane & 31) & ~3);
        if (ppe.rowterm) {
            const int32_t* rt = ppe.rowterm + ((int64_t)img * g.OH + oy0) * g.OW;
#pragma unroll
            for (int i = 0; i < TMW; i++) {
                if (mi0 + i * mstep >= pg.MT) continue;
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][r] += rt[(mi0 + i * mstep) * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4)];
            }
        }
        auto requant = [&](auto general_c) {
#pragma unroll
            for (int i = 0; i < TMW; i++) {
                if (mi0 + i * mstep >= pg.MT) continue;
#pragma unroll
                for (int gq = 0; gq < 4; gq++) {
                    unsigned v;
                    if constexpr (decltype(general_c)::value)
                        v = ppe_pack4<SAME_F, true>(acc[i][gq * 4], acc[i][gq * 4 + 1], acc[i][gq * 4 + 2], acc[i][gq * 4 + 3], cp, pk);
                    else
                        v = ppe_pack4_biased<!SAME_F>(acc[i][gq * 4] + pb, acc[i][gq * 4 + 1] + pb, acc[i][gq * 4 + 2] + pb,
                                                      acc[i][gq * 4 + 3] + pb, cp.f_pos, cp.f_neg, pk);
                    v = quad_transpose_bytes(v, lane);
                    const int row = (mi0 + i * mstep) * 32 + 8 * gq + 4 * (lane >> 5) + (lane & 3);
                    *reinterpret_cast<unsigned*>(patch + row * kPatchOutStride + col4) = v;
                }
            }
        };
        if (general) requant(std::true_type{});
        else requant(std::false_type{});
    }
    __syncthreads();
    const int rows_here = g.OH - oy0 < pg.R ? (int)(g.OH - oy0) : pg.R;
    const int valid = rows_here * (int)g.OW;
    uint8_t* const out0 = out + ((int64_t)img * g.osn + (int64_t)oy0 * g.osh);  // the tile's first output position
    const bool vec_ok = (g.out_bits & 15) == 0;
    for (int cid = tid; cid < valid * 4; cid += NT) {
        const int row = cid >> 2, c16 = cid & 3;
        const int64_t n = oc0 + c16 * 16;
        if (n >= g.OC) continue;
        const i32x4 v = *reinterpret_cast<const i32x4*>(patch + row * kPatchOutStride + c16 * 16);
        uint8_t* dst = out0 + tile_out_pos(g, row, pg.ow) + n;
        if (vec_ok && n + 16 <= g.OC) {
            __builtin_nontemporal_store(v, reinterpret_cast<i32x4*>(dst));
        } else {
            store_tail16(dst, v, (int)(g.OC - n < 16 ? g.OC - n : 16), out_align(g.out_bits));
        }
    }
}

// ---------------------------------------------------------------- patch convolution, weights in registers
// KY x KX taps of 64 input channels: the weights of a 64-channel block are 16 x KY x KX vector registers per lane in
// the B layout of `v_mfma_i32_16x16x64_i8`, so every wave keeps all of them and the main loop reads only activations
// from LDS (one 16-byte fragment per four MFMAs, where nce_conv_tile reads six per four).  A wave walks blocks of 16
// output positions x 64 channels: KY*KX fragment reads and 4*KY*KX MFMAs, then the PPE of the block's 16 values per
// lane and one 16-byte store per lane -- no workgroup barrier after the staging, no output staging in LDS.
// (On this part the vector ALU work of one wave does not run under the MFMAs of the other wave of its SIMD, and
// interleaving the PPE of block b-1 with the MFMAs of block b inside a wave needs a second set of accumulators,
// which at two waves per SIMD spills: measured, a pipelined four-wave form with 32x32x32 MFMAs took 10.7 us where
// this one takes 9.6 us at [32,56,56,64] -> 64.)
//
// Channel order inside a block: column n of MFMA tile j is output channel 16*(n/4) + 4*j + n%4.  After the 4x4 byte
// transpose a lane then holds channels 16*q .. 16*q+15 of one position in its four result dwords (tile j -> dword j),
// which is the 16 bytes it stores.  The weight rows sit in LDS in tile order (row 16*j + n), which the fragment reads
// of sixteen lanes walk conflict-free.
template <bool IN_U8, bool SAME_F, int KY, int KX>
__global__ __launch_bounds__(512) void nce_conv_regw(const int8_t* __restrict__ in, const int8_t* __restrict__ w,
                                                     const int32_t* __restrict__ wt, uint8_t* __restrict__ out, ConvGeom g,
                                                     PatchGeom pg, int pad_byte, GemmPpe ppe) {
    constexpr int BN = 64, IC = 64, PS = IC + 16, NW = 8, NT = 64 * NW, TAPS = KY * KX, Ktot = TAPS * IC, WS = Ktot + 16;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* const wlds = smem;             // [64][Ktot + 16], rows in tile order
    uint8_t* const patch = smem + BN * WS;  // [PH*PW][IC + 16]
    __shared__ int csum[BN];                // weight sums, by LDS row

    // A launch of a few microseconds is bound by instructions as much as by anything else: all index arithmetic below
    // is 32-bit, on offsets from a few 64-bit bases that are the same for the whole wave.
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int H = (int)g.H, W = (int)g.W, OC = (int)g.OC, OW = (int)g.OW, OH = (int)g.OH;
    const int img = fdiv(blockIdx.x, pg.tiles_y);
    const int oy0 = (blockIdx.x - img * (int)pg.tiles_y.d) * pg.R;
    const int oc0 = blockIdx.y * BN;

    // ---- weights and patch -> LDS.  All loads are issued up front, weights first: they come from L2 and are back
    // before the patch rows are, so the waves copy their weight fragments to registers while the patch is on its way.
    const int n16 = lane & 15, c4 = lane >> 4;
    i32x4 wb[TAPS][4];
    {
        constexpr int cpr = Ktot / 16;                 // 16-byte chunks per weight row
        constexpr int wchunks = BN * cpr;
        constexpr int UW = (wchunks + NT - 1) / NT, UP = 5;
        constexpr int cpp = IC / 16;
        const int row_chunks = pg.PW * cpp;
        const int upr = (int)pg.upr.d, units = pg.PH * upr;
        const int pad32 = (pad_byte & 0xff) * 0x01010101;
        const int iy0 = oy0 * g.SY - g.PT;
        // patch pixel (py, px) is input pixel (iy0 + py, px - PL): byte offset py * W*IC + px * IC from `corner`, which
        // may lie outside the tensor; lanes whose pixel is padding read the first pixel of the tile's first real row
        const int isw = (int)g.isw, ish = (int)g.ish;  // (the host sends layers here whose patch offsets fit 32 bits)
        const int8_t* corner = in + ((int64_t)img * g.isn + (int64_t)iy0 * g.ish - (int64_t)g.PL * g.isw);
        const int safe_off = (iy0 < 0 ? -iy0 : 0) * ish + g.PL * isw;
        const int8_t* wsrc = w + (int64_t)oc0 * Ktot;
        const bool full_rows = oc0 + BN <= OC;         // the 64 weight rows are one contiguous run
        i32x4 qw[UW], qp[UP];
        int dw[UW], dp[UP];
        bool pin[UP];
        // (nothing here may use a loaded value: the first use is where the wave waits for the load)
        auto load_patch = [&](int u0) {
#pragma unroll
            for (int u = 0; u < UP; u++) {
                const int unit = u0 + wave + NW * u;   // wave-uniform, as are py and sub
                const int py = fdiv(unit, pg.upr), sub = unit - py * upr;
                const int qi = sub * 64 + lane;
                const bool ok = unit < units && qi < row_chunks;
                const int px = qi / cpp;
                const int iy = iy0 + py;
                const bool inside = ok && (unsigned)iy < (unsigned)H && (unsigned)(px - g.PL) < (unsigned)W;
                const int off = inside ? py * ish + px * isw + (qi % cpp) * 16 : safe_off;
                qp[u] = *reinterpret_cast<const i32x4*>(corner + off);
                pin[u] = inside;
                dp[u] = ok ? py * (pg.PW * PS) + px * PS + (qi % cpp) * 16 : -1;
            }
        };
        auto store_patch = [&]() {
#pragma unroll
            for (int u = 0; u < UP; u++)
                if (dp[u] >= 0) {
                    i32x4 v = pin[u] ? qp[u] : i32x4{pad32, pad32, pad32, pad32};
                    if (IN_U8) v ^= (int32_t)0x80808080;
                    *reinterpret_cast<i32x4*>(patch + dp[u]) = v;
                }
        };
#pragma unroll
        for (int u = 0; u < UW; u++) {
            const int q = u * NT + tid;
            const bool ok = q < wchunks;
            const int qq = ok ? q : 0;
            const int row = qq / cpr, c = qq - row * cpr;
            int src = qq * 16;
            if (!full_rows) src = (oc0 + row < OC ? row : OC - 1 - oc0) * Ktot + c * 16;  // channels past the end repeat the last one
            qw[u] = *reinterpret_cast<const i32x4*>(wsrc + src);
            const int lrow = ((row >> 2) & 3) * 16 + (row >> 4) * 4 + (row & 3);
            dw[u] = ok ? lrow * WS + c * 16 : -1;
        }
        load_patch(0);
#pragma unroll
        for (int u = 0; u < UW; u++)
            if (dw[u] >= 0) *reinterpret_cast<i32x4*>(wlds + dw[u]) = qw[u];
        __syncthreads();
        // this wave's copy of the weights
#pragma unroll
        for (int t = 0; t < TAPS; t++)
#pragma unroll
            for (int j = 0; j < 4; j++) wb[t][j] = *reinterpret_cast<const i32x4*>(wlds + (j * 16 + n16) * WS + t * IC + c4 * 16);
        // the sums of the weight rows where the zero-point term needs them
        if (ppe.corr != 0 && tid < 256) {
            const int row = tid >> 2, part = tid & 3;
            int sum = 0;
            for (int c = part; c < Ktot / 16; c += 4) {
                const i32x4 q = *reinterpret_cast<const i32x4*>(wlds + row * WS + c * 16);
#pragma unroll
                for (int j = 0; j < 4; j++) sum = __builtin_amdgcn_sdot4(q[j], 0x01010101, sum, false);
            }
            sum += (int)dpp_u32<0xB1>((unsigned)sum);
            sum += (int)dpp_u32<0x4E>((unsigned)sum);
            if (part == 0) csum[row] = sum;
        }
        store_patch();
        for (int u0 = NW * UP; u0 < units; u0 += NW * UP) {  // tall patches: the rest, a round trip each
            load_patch(u0);
            store_patch();
        }
    }
    __syncthreads();

    // ---- per-channel PPE parameters of the lane's four channels
    ChanPrep cp[4];
    bool clip = false;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        int n = oc0 + (n16 >> 2) * 16 + j * 4 + (n16 & 3);
        n = n < OC ? n : OC - 1;
        const int cs = ppe.corr != 0 ? csum[j * 16 + n16] : 0;
        const uint32_t w2 = (uint32_t)wt[n * 4 + 2];
        cp[j] = ppe_prepare((int)(int16_t)(w2 >> 16), (int)((w2 >> 8) & 0xffu),
                            (int)((unsigned)wt[n * 4 + 3] + (unsigned)(ppe.corr * cs)), ppe.prelu_mult, ppe.prelu_shift);
        clip = clip || cp[j].bmax_pos != 0x7fffffff || cp[j].bmax_neg != 0x7fffffff;
        asm volatile("" : "+v"(cp[j].f_pos), "+v"(cp[j].f_neg));
    }
    const PpePack pk = make_ppe_pack(ppe.zp_out, ppe.lo, ppe.hi, ppe.out_signed != 0);
    // the short PPE serves slopes in [0, 1] (ReLU, LeakyReLU), an even zero-point offset and scales up to 1/2
    const bool slope_ok = SAME_F || (ppe.prelu_mult >= 0 && (ppe.prelu_shift >= 31 || ppe.prelu_mult <= (1 << ppe.prelu_shift)));
    const bool general = __builtin_amdgcn_ballot_w64(clip) != 0 || pk.odd != 0 || !slope_ok;
    const QuadTranspose transpose(lane);

    const int rows_here = OH - oy0 < pg.R ? OH - oy0 : pg.R;
    const int valid = rows_here * OW;
    const int nblk = (valid + 15) >> 4;
    const int64_t pos0 = ((int64_t)img * OH + oy0) * OW;
    const int32_t* rt = ppe.rowterm ? ppe.rowterm + pos0 : nullptr;
    uint8_t* const out0 = out + ((int64_t)img * g.osn + (int64_t)oy0 * g.osh);  // the tile's first output position
    const bool vec_ok = (g.out_bits & 15) == 0;
    const int q16 = oc0 + (n16 >> 2) * 16;  // first of the 16 channels this lane stores
    int soff[TAPS];
#pragma unroll
    for (int t = 0; t < TAPS; t++) soff[t] = ((t / KX) * pg.PW + (t % KX)) * PS;

    auto one_block = [&](int b, auto general_c) {
        int p = b * 16 + n16;
        p = p < valid ? p : 0;
        const int r = fdiv(p, pg.ow), ox = p - r * OW;
        const uint8_t* pa = patch + (r * g.SY * pg.PW + ox * g.SX) * PS + c4 * 16;
        constexpr bool GENERAL = decltype(general_c)::value;
        i32x4 acc[4];  // the short PPE's accumulators start from the bias
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int b0 = GENERAL ? 0 : cp[j].bias;
            acc[j] = i32x4{b0, b0, b0, b0};
        }
        i32x4 fa[TAPS];  // all of the block's fragments are asked for before the first MFMA waits for one
#pragma unroll
        for (int t = 0; t < TAPS; t++) fa[t] = *reinterpret_cast<const i32x4*>(pa + soff[t]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < TAPS; t++)
#pragma unroll
            for (int j = 0; j < 4; j++) acc[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[t], wb[t][j], acc[j], 0, 0, 0);
        if (rt) {  // (padded past the last position: an edge block may read ahead)
            i32x4 v;
#pragma unroll
            for (int r4 = 0; r4 < 4; r4++) v[r4] = rt[b * 16 + 4 * c4 + r4];
#pragma unroll
            for (int j = 0; j < 4; j++) acc[j] += v;
        }
        i32x4 o;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            unsigned v;
            if constexpr (GENERAL) {
                ChanPrep c = cp[j];  // the form ppe_pack4 takes: sign flip in the bias, factors swapped for a negative multiplier
                c.bias = (int)((unsigned)c.bias + 0x80000000u);
                if (c.sgn) {
                    c.f_pos = cp[j].f_neg;
                    c.f_neg = cp[j].f_pos;
                    c.bmax_pos = cp[j].bmax_neg;
                    c.bmax_neg = cp[j].bmax_pos;
                }
                v = ppe_pack4<SAME_F, true>(acc[j][0], acc[j][1], acc[j][2], acc[j][3], c, pk);
            } else {
                v = ppe_pack4_biased<!SAME_F>(acc[j][0], acc[j][1], acc[j][2], acc[j][3], cp[j].f_pos, cp[j].f_neg, pk);
            }
            o[j] = (int)transpose(v);
        }
        const int pi = b * 16 + 4 * c4 + (lane & 3);
        if (pi < valid && q16 < OC) {
            uint8_t* dst = out0 + (tile_out_pos(g, pi, pg.ow) + q16);
            if (vec_ok && q16 + 16 <= OC) {
                __builtin_nontemporal_store(o, reinterpret_cast<i32x4*>(dst));
            } else {
                store_tail16(dst, o, OC - q16 < 16 ? OC - q16 : 16, out_align(g.out_bits));
            }
        }
    };
    if (general) {
        for (int b = wave; b < nblk; b += NW) one_block(b, std::true_type{});
    } else {
        for (int b = wave; b < nblk; b += NW) one_block(b, std::false_type{});
    }
}

// ---------------------------------------------------------------- patch convolution with streamed weights
// For layers whose weights do not fit LDS next to the input patch (many input channels): the patch
// stays resident, the weights pass through two small LDS buffers a slice at a time -- one tap x KSL
// channels of the 64 output channels (KSL = 64, 128 or 256, a divisor of IC).  The global loads of
// slice s+1 are issued before the MFMAs of slice s and written to the other buffer after them;
// one barrier per slice.  Same padded LDS rows and addressing as nce_conv_tile; IC is a run-time
// multiple of 64.
struct StreamGeom {
    int ksl;       // channels per weight slice
    int spt;       // slices per tap = IC / ksl
};

//
// KSPLIT (tiles of up to 64 positions per four waves -- 7 x 7 planes, halves of 14 x 14 ones): with a 32 x 32 tile per wave
// every MFMA reads two fragments from LDS, four times what LDS delivers while the four SIMDs multiply.  Here the four
// waves of a group each take a quarter of a slice's K steps over the whole 64 x 64 tile (four MFMAs per four fragments),
// and their partial sums meet in LDS after the last slice; each wave then finishes one 32 x 32 tile as before.
template <bool IN_U8, int TMW, bool SAME_F, int NW, int KSPLIT = 0>
__global__ __launch_bounds__(64 * NW, NW == 8 ? 1 : 2) void nce_conv_stream(const int8_t* __restrict__ in,
                                                                           const int8_t* __restrict__ w,
                                                                           const int32_t* __restrict__ wt,
                                                                           const int32_t* __restrict__ colsum,
                                                                           uint8_t* __restrict__ out, ConvGeom g,
                                                                           PatchGeom pg, StreamGeom sg, int pad_byte,
                                                                           GemmPpe ppe) {
    constexpr int BN = 64, NT = 64 * NW, UWS = 256 * BN / 16 / NT;  // chunks of a 256-channel slice per thread
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int IC = (int)g.IC, PS = IC + 16;
    const int Ktot = g.KY * g.KX * IC;
    const int KSL = sg.ksl, WS = KSL + 16;
    uint8_t* const wbuf = smem;                 // [2][64][KSL + 16]
    uint8_t* const patch = smem + 2 * BN * WS;  // [PH*PW][IC + 16], later the output staging tile

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int img = fdiv(blockIdx.x, pg.tiles_y);
    const int oy0 = (blockIdx.x - img * (int)pg.tiles_y.d) * pg.R;
    const int oc0 = blockIdx.y * BN;

    // weight slice transfer: chunk q of a slice = (row q / cps, chunk q % cps), cps = KSL / 16 (4, 8 or 16)
    const int cps_shift = KSL == 64 ? 2 : (KSL == 128 ? 3 : 4);
    const int slice_chunks = BN << cps_shift;
    // (a thread's chunks sit at the same place of every slice: their addresses are worked out once, and a slice adds
    // its offset tap * IC + ic0 = sl * KSL, since the slices of a weight row follow each other in K order)
    const int8_t* wsrc[UWS];
#pragma unroll
    for (int u = 0; u < UWS; u++) {
        const int qi = u * NT + tid;
        const int qq = qi < slice_chunks ? qi : 0;
        const int row = qq >> cps_shift, c = qq & ((1 << cps_shift) - 1);
        int64_t oc = oc0 + row;
        oc = oc < g.OC ? oc : g.OC - 1;
        wsrc[u] = w + oc * Ktot + c * 16;
    }
    auto slice_issue = [&](int sl, i32x4(&q)[UWS]) {
        const int off = sl * KSL;
#pragma unroll
        for (int u = 0; u < UWS; u++) q[u] = *reinterpret_cast<const i32x4*>(wsrc[u] + off);
    };
    auto slice_commit = [&](int buf, const i32x4(&q)[UWS]) {
#pragma unroll
        for (int u = 0; u < UWS; u++) {
            const int qi = u * NT + tid;
            if (qi < slice_chunks) {
                const int row = qi >> cps_shift, c = qi & ((1 << cps_shift) - 1);
                *reinterpret_cast<i32x4*>(wbuf + buf * BN * WS + row * WS + c * 16) = q[u];
            }
        }
    };

    // ---- patch and the first weight slice -> LDS.  Weight slices are asked for DEPTH slices ahead and wait in
    // registers: the MFMAs of a slice (a few hundred clocks) are much shorter than a trip to L2, and with two slices in
    // flight a workgroup moved 32 KiB per memory latency ([32,7,7,512] -> 512 3x3: 18 slices, 17.9 us).
    constexpr int DEPTH = 6;
    const int slices = g.KY * g.KX * sg.spt;
    i32x4 wq[DEPTH][UWS];
#pragma unroll
    for (int d = 0; d < DEPTH; d++)
        if (d < slices) slice_issue(d, wq[d]);
    {
        constexpr int UP = NW == 8 ? 4 : 6;
        const int cpp = IC / 16;
        const int row_chunks = pg.PW * cpp;
        const int upr = (int)pg.upr.d, units = pg.PH * upr;
        const int pad32 = (pad_byte & 0xff) * 0x01010101;
        const int8_t* img_base = in + (int64_t)img * g.isn;
        const int iy0 = oy0 * g.SY - g.PT;
        for (int u0 = 0; u0 < units; u0 += NW * UP) {
            i32x4 qp[UP];
            int dp[UP];
#pragma unroll
            for (int u = 0; u < UP; u++) {
                const int unit = u0 + wave + NW * u;
                const int py = fdiv(unit, pg.upr);  // wave-uniform
                const int qi = (unit - py * upr) * 64 + lane;
                const bool ok = unit < units && qi < row_chunks;
                const int px = fdiv(qi, pg.cpp), cc = qi - px * cpp;
                const int iy = iy0 + py, ix = px - g.PL;
                const bool inside = ok && iy >= 0 && iy < g.H && ix >= 0 && ix < g.W;
                const int64_t off = inside ? (int64_t)iy * g.ish + (int64_t)ix * g.isw + cc * 16 : 0;
                const i32x4 v = *reinterpret_cast<const i32x4*>(img_base + off);
                qp[u] = inside ? v : i32x4{pad32, pad32, pad32, pad32};
                dp[u] = ok ? (py * pg.PW + px) * PS + cc * 16 : -1;
            }
#pragma unroll
            for (int u = 0; u < UP; u++)
                if (dp[u] >= 0) {
                    if (IN_U8) qp[u] ^= (int32_t)0x80808080;
                    *reinterpret_cast<i32x4*>(patch + dp[u]) = qp[u];
                }
        }
    }
    slice_commit(0, wq[0]);
    __syncthreads();

    // ---- main loop
    static_assert(!KSPLIT || (TMW == 1 && (KSPLIT == 4 || KSPLIT == 8) && NW % KSPLIT == 0), "a K-split wave finishes one row block");
    constexpr int KS = KSPLIT ? KSPLIT : 4;
    const int grp = wave / KS, ks = wave % KS;  // KSPLIT: group of KS waves, this wave's share of K
    const int nj = KSPLIT ? ks & 1 : (pg.nt == 2 ? wave & 1 : 0);
    // (of eight waves that split K the first four finish a tile each; the others only contribute: a row block past the end)
    const int mi0 = KSPLIT ? (ks < 4 ? 2 * grp + (ks >> 1) : kPatchMaxMT) : (pg.nt == 2 ? wave >> 1 : wave);
    const int mstep = pg.nt == 2 ? NW / 2 : NW;
    const int npos = pg.R * (int)g.OW;
    const int kgroup = lane >> 5;
    int abase[TMW];
#pragma unroll
    for (int i = 0; i < TMW; i++) {
        int p = (mi0 + i * mstep) * 32 + (lane & 31);
        p = p < npos ? p : 0;
        const int r = fdiv(p, pg.ow), ox = p - r * (int)g.OW;
        abase[i] = (r * g.SY * pg.PW + ox * g.SX) * PS + kgroup * 16;
    }
    const int brow = nj * 32 + (lane & 31);
    const int bbase = brow * WS + kgroup * 16;
    int abase4[2], bbase4[2];  // KSPLIT: both row blocks of the group, both channel tiles
#pragma unroll
    for (int i = 0; i < 2; i++) {
        int p = (2 * grp + i) * 32 + (lane & 31);
        p = p < npos ? p : 0;
        const int r = fdiv(p, pg.ow), ox = p - r * (int)g.OW;
        abase4[i] = (r * g.SY * pg.PW + ox * g.SX) * PS + kgroup * 16;
        bbase4[i] = (i * 32 + (lane & 31)) * WS + kgroup * 16;
    }
    i32x16 acc4[2][2];
    if (KSPLIT != 0) {
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc4[i][j][r] = 0;
    }

    i32x16 acc[TMW];
#pragma unroll
    for (int i = 0; i < TMW; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0;

    const int ksteps = KSL / 32;
    int ky = 0, kx = 0, sub = 0;  // position of the current slice
    // slice sl: its registers (set sl % DEPTH) were stored to LDS an iteration ago and take slice sl + DEPTH now
    auto one_slice = [&](int sl, auto set_c) {
        constexpr int set = decltype(set_c)::value;
        const int buf = set & 1;  // (DEPTH is even)
        const bool more = sl + 1 < slices;
        if (sl + DEPTH < slices) slice_issue(sl + DEPTH, wq[set]);
        const uint8_t* pa0 = patch + (ky * pg.PW + kx) * PS + sub * KSL;
        if constexpr (KSPLIT != 0) {
            // this wave's K steps of the slice: ks and, where a slice has twice as many steps as the group has waves, ks + KS
            // (the host asks for slices of KS or 2 KS steps)
            const uint8_t* pw = wbuf + buf * BN * WS;
            i32x4 fa[2][2], fb[2][2];
            const bool two = ksteps > KS;
#pragma unroll
            for (int h = 0; h < 2; h++) {
                if (h == 1 && !two) break;
                const int k = ks + KS * h;
#pragma unroll
                for (int i = 0; i < 2; i++) {
                    fa[h][i] = *reinterpret_cast<const i32x4*>(pa0 + abase4[i] + k * 32);
                    fb[h][i] = *reinterpret_cast<const i32x4*>(pw + bbase4[i] + k * 32);
                }
            }
#pragma unroll
            for (int h = 0; h < 2; h++) {
                if (h == 1 && !two) break;
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int j = 0; j < 2; j++)
                        acc4[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[h][i], fb[h][j], acc4[i][j], 0, 0, 0);
            }
        } else {
        const uint8_t* pb = wbuf + buf * BN * WS + bbase;
        i32x4 fa[2][TMW], fb[2];
        auto read_frags = [&](int slot, int k) {
            fb[slot] = *reinterpret_cast<const i32x4*>(pb + k * 32);
#pragma unroll
            for (int i = 0; i < TMW; i++) fa[slot][i] = *reinterpret_cast<const i32x4*>(pa0 + abase[i] + k * 32);
        };
        read_frags(0, 0);
        for (int k = 0; k < ksteps; k += 2) {  // ksteps is even
            read_frags(1, k + 1);
#pragma unroll
            for (int i = 0; i < TMW; i++) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[0][i], fb[0], acc[i], 0, 0, 0);
            if (k + 2 < ksteps) read_frags(0, k + 2);
#pragma unroll
            for (int i = 0; i < TMW; i++) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[1][i], fb[1], acc[i], 0, 0, 0);
        }
        }
        if (more) slice_commit(buf ^ 1, wq[(set + 1) % DEPTH]);
        __syncthreads();  // slice sl+1 is visible; nobody reads buffer `buf` any more
        sub++;
        if (sub == sg.spt) {
            sub = 0;
            kx++;
            if (kx == g.KX) {
                kx = 0;
                ky++;
            }
        }
    };
    static_assert(DEPTH == 6, "the loop below names the register sets one by one");
    for (int sl = 0; sl < slices; sl += DEPTH) {
        one_slice(sl, std::integral_constant<int, 0>{});
        if (sl + 1 < slices) one_slice(sl + 1, std::integral_constant<int, 1>{});
        if (sl + 2 < slices) one_slice(sl + 2, std::integral_constant<int, 2>{});
        if (sl + 3 < slices) one_slice(sl + 3, std::integral_constant<int, 3>{});
        if (sl + 4 < slices) one_slice(sl + 4, std::integral_constant<int, 4>{});
        if (sl + 5 < slices) one_slice(sl + 5, std::integral_constant<int, 5>{});
    }

    // ---- KSPLIT: the partial sums of a group's waves meet in LDS (the last barrier of the loop has freed all of it);
    // wave ks < 4 keeps tile (ks / 2, ks % 2) and adds what the others hold of it
    if constexpr (KSPLIT != 0) {
        uint8_t* const red = smem;  // [wave][tile][quad][lane] x 16 bytes
#pragma unroll
        for (int t = 0; t < 4; t++) {
            if (t == ks) continue;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const i32x16& a = acc4[t >> 1][t & 1];
                *reinterpret_cast<i32x4*>(red + ((((wave * 4 + t) * 4 + q) * 64 + lane) << 4)) = i32x4{a[4 * q], a[4 * q + 1], a[4 * q + 2], a[4 * q + 3]};
            }
        }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < 4; t++)
            if (t == ks) acc[0] = acc4[t >> 1][t & 1];
#pragma unroll
        for (int o = 1; o < KS; o++) {
            const int v = grp * KS + ((ks + o) % KS);
            if (ks >= 4) break;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const i32x4 part = *reinterpret_cast<const i32x4*>(red + ((((v * 4 + ks) * 4 + q) * 64 + lane) << 4));
#pragma unroll
                for (int r = 0; r < 4; r++) acc[0][4 * q + r] += part[r];
            }
        }
        __syncthreads();  // the output staging below overwrites the partial sums
    }

    // ---- epilogue (the last barrier of the loop has freed the patch)
    if (ppe.out_f16) {
        int64_t n = oc0 + brow;
        n = n < g.OC ? n : g.OC - 1;
        const uint32_t w2 = (uint32_t)wt[n * 4 + 2];
        const ChanPrep c = ppe_prepare((int)(int16_t)(w2 >> 16), (int)((w2 >> 8) & 0xffu) - 15,
                                       (int)((unsigned)wt[n * 4 + 3] + (unsigned)(ppe.corr * (colsum ? colsum[n] : 0))), ppe.prelu_mult,
                                       ppe.prelu_shift);
        const int rows_here = g.OH - oy0 < pg.R ? (int)(g.OH - oy0) : pg.R;
        const int64_t pos0 = ((int64_t)img * g.OH + oy0) * g.OW;
        patch_epilogue_f16<TMW, NT>(acc, mi0, mstep, nj, pg.MT, c, ppe, ppe.rowterm ? ppe.rowterm + pos0 : nullptr, patch,
                                    reinterpret_cast<uint16_t*>(out) + ((int64_t)img * g.osn + (int64_t)oy0 * g.osh),
                                    rows_here * (int)g.OW, oc0, (int)g.OC, g, pg.ow);
        return;
    }
    {
        int64_t n = oc0 + brow;
        n = n < g.OC ? n : g.OC - 1;
        const int cs = colsum ? colsum[n] : 0;
        const uint32_t w2 = (uint32_t)wt[n * 4 + 2];
        ChanPrep cp = ppe_prepare_packed((int)(int16_t)(w2 >> 16), (int)((w2 >> 8) & 0xffu),
                                         (int)((unsigned)wt[n * 4 + 3] + (unsigned)(ppe.corr * cs)), ppe.prelu_mult, ppe.prelu_shift);
        asm volatile("" : "+v"(cp.f_pos), "+v"(cp.f_neg));
        const PpePack pk = make_ppe_pack(ppe.zp_out, ppe.lo, ppe.hi, ppe.out_signed != 0);
        // (the short PPE serves slopes in [0, 1], an even zero-point offset and scales up to 1/2: see ppe_pack4_biased)
        const bool slope_ok = SAME_F || (ppe.prelu_mult >= 0 && (ppe.prelu_shift >= 31 || ppe.prelu_mult <= (1 << ppe.prelu_shift)));
        const bool general = __builtin_amdgcn_ballot_w64(cp.bmax_pos != 0x7fffffff || cp.bmax_neg != 0x7fffffff) != 0 || pk.odd != 0 || !slope_ok;
        const int pb = (int)((unsigned)cp.bias - 0x80000000u);  // the bias without the sign flip of the packed form
        const int col4 = nj * 32 + ((lane & 31) & ~3);
        if (ppe.rowterm) {
            const int32_t* rt = ppe.rowterm + ((int64_t)img * g.OH + oy0) * g.OW;
#pragma unroll
            for (int i = 0; i < TMW; i++) {
                if (mi0 + i * mstep >= pg.MT) continue;
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][r] += rt[(mi0 + i * mstep) * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4)];
            }
        }
        auto requant = [&](auto general_c) {
#pragma unroll
            for (int i = 0; i < TMW; i++) {
                if (mi0 + i * mstep >= pg.MT) continue;
#pragma unroll
                for (int gq = 0; gq < 4; gq++) {
                    unsigned v;
                    if constexpr (decltype(general_c)::value)
                        v = ppe_pack4<SAME_F, true>(acc[i][gq * 4], acc[i][gq * 4 + 1], acc[i][gq * 4 + 2], acc[i][gq * 4 + 3], cp, pk);
                    else
                        v = ppe_pack4_biased<!SAME_F>(acc[i][gq * 4] + pb, acc[i][gq * 4 + 1] + pb, acc[i][gq * 4 + 2] + pb,
                                                      acc[i][gq * 4 + 3] + pb, cp.f_pos, cp.f_neg, pk);
                    v = quad_transpose_bytes(v, lane);
                    const int row = (mi0 + i * mstep) * 32 + 8 * gq + 4 * (lane >> 5) + (lane & 3);
                    *reinterpret_cast<unsigned*>(patch + row * kPatchOutStride + col4) = v;
                }
            }
        };
        if (general) requant(std::true_type{});
        else requant(std::false_type{});
    }
    __syncthreads();
    const int rows_here = g.OH - oy0 < pg.R ? (int)(g.OH - oy0) : pg.R;
    const int valid = rows_here * (int)g.OW;
    uint8_t* const out0 = out + ((int64_t)img * g.osn + (int64_t)oy0 * g.osh);  // the tile's first output position
    const bool vec_ok = (g.out_bits & 15) == 0;
    for (int cid = tid; cid < valid * 4; cid += NT) {
        const int row = cid >> 2, c16 = cid & 3;
        const int64_t n = oc0 + c16 * 16;
        if (n >= g.OC) continue;
        const i32x4 v = *reinterpret_cast<const i32x4*>(patch + row * kPatchOutStride + c16 * 16);
        uint8_t* dst = out0 + tile_out_pos(g, row, pg.ow) + n;
        if (vec_ok && n + 16 <= g.OC) {
            __builtin_nontemporal_store(v, reinterpret_cast<i32x4*>(dst));
        } else {
            store_tail16(dst, v, (int)(g.OC - n < 16 ? g.OC - n : 16), out_align(g.out_bits));
        }
    }
}

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

// ---------------------------------------------------------------- gather convolution, IC a multiple of 16
// Stem layers (3 or 4 image channels padded to 16) and other channel counts that are a multiple of
// 16 but not of 32.  K = KY*KX*IC is walked as a flat run of 16-byte chunks, two per MFMA step:
// lanes 0-31 feed chunk 2j, lanes 32-63 chunk 2j+1, which may belong to different taps.  All
// weights of the 64 output channels (K rounded up to 32, zero-filled) sit in LDS.
template <bool IN_U8, int OUT>
__global__ __launch_bounds__(256) void nce_conv_mfma16(const int8_t* __restrict__ in, const int8_t* __restrict__ w,
                                                       const ChanPrep* __restrict__ prep, uint8_t* __restrict__ out,
                                                       ConvGeom g, int pad_byte, PpeFast ppe) {
    constexpr int BM = 256, BN = 64, WM = BM / 4, TM = WM / 32, TN = BN / 32;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];  // [BN][K32 + 16]
    const int Ktot = g.KY * g.KX * (int)g.IC;
    const int K32 = (Ktot + 31) & ~31, WS = K32 + 16;
    const int64_t Mtot = g.N * g.OH * g.OW;
    const int64_t m0 = (int64_t)blockIdx.x * BM;
    const int64_t oc0 = (int64_t)blockIdx.y * BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int cpr = K32 / 16, cpt = (int)g.IC / 16;

    for (int cid = tid; cid < BN * cpr; cid += 256) {
        const int row = cid / cpr, c = cid - row * cpr;
        int64_t oc = oc0 + row;
        oc = oc < g.OC ? oc : g.OC - 1;
        i32x4 q = i32x4{0, 0, 0, 0};
        if (c * 16 < Ktot) q = *reinterpret_cast<const i32x4*>(w + oc * Ktot + c * 16);
        *reinterpret_cast<i32x4*>(smem + row * WS + c * 16) = q;
    }
    __syncthreads();

    int64_t base_n[TM];
    int oy[TM], ox[TM];
#pragma unroll
    for (int i = 0; i < TM; i++) {
        int64_t m = m0 + wave * WM + i * 32 + (lane & 31);
        m = m < Mtot ? m : Mtot - 1;
        ox[i] = (int)(m % g.OW) * g.SX - g.PL;
        oy[i] = (int)((m / g.OW) % g.OH) * g.SY - g.PT;
        base_n[i] = (m / (g.OW * g.OH)) * g.isn;
    }
    const int pad32 = (pad_byte & 0xff) * 0x01010101;
    i32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

    const int kgroup = lane >> 5;
    const int last_tap = g.KY * g.KX - 1;
    for (int c = kgroup; c < cpr; c += 2) {  // this lane's chunk of every step
        int tap = c / cpt;
        const int cc = c - tap * cpt;
        const bool real = tap <= last_tap;   // the zero-filled tail of K: any finite activation will do
        tap = real ? tap : last_tap;
        const int ky = tap / g.KX, kx = tap - ky * g.KX;
        i32x4 fa[TM], fb[TN];
#pragma unroll
        for (int i = 0; i < TM; i++) {
            const int iy = oy[i] + ky, ix = ox[i] + kx;
            const bool inside = iy >= 0 && iy < g.H && ix >= 0 && ix < g.W;
            const int64_t off = inside ? (int64_t)iy * g.ish + (int64_t)ix * g.isw + cc * 16 : 0;
            i32x4 q = *reinterpret_cast<const i32x4*>(in + base_n[i] + off);
            if (!inside) q = i32x4{pad32, pad32, pad32, pad32};
            if (IN_U8) q ^= (int32_t)0x80808080;
            fa[i] = q;
        }
#pragma unroll
        for (int j = 0; j < TN; j++) fb[j] = *reinterpret_cast<const i32x4*>(smem + (j * 32 + (lane & 31)) * WS + c * 16);
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }

#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int64_t oc = oc0 + j * 32 + (lane & 31);
        if (oc >= g.OC) continue;
        const ChanPrep cp = prep[oc];
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int64_t m = m0 + wave * WM + i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
                if (m >= Mtot) continue;
                const int a = acc[i][j][r] + (ppe.rowterm ? ppe.rowterm[m] : 0);
                const int64_t o = out_pos(g, m) + oc;
                if (OUT == OUT_F16) reinterpret_cast<uint16_t*>(out)[o] = ppe_fast_f16(a, cp, ppe.f16_lo, ppe.f16_hi);
                else out[o] = (uint8_t)ppe_fast<true>(a, cp, ppe);
            }
        }
    }
}

// ---------------------------------------------------------------- row-patch convolution, IC a multiple of 16
// Stem layers again (few input channels, many taps), with the input rows under a band of output rows resident in
// LDS.  A pixel's channels are contiguous and so are the pixels of a row, hence the KX * IC bytes under one kernel
// row of one output position are one contiguous run of the patch row: the convolution is KY matmuls over runs that
// start SX * IC bytes apart.  K is walked in its natural order in 16-byte chunks, two per MFMA step (lanes 0-31 the
// even chunk, lanes 32-63 the odd one, which may lie in the next kernel row; an odd chunk count ends on a chunk of
// zero weights).  A fragment address is a per-lane base plus one of two wave-uniform offsets, by lane half, which a
// small table in LDS holds per step: no bounds test, padding value or sign flip inside the loop (the staging applies
// them once per input byte).
//
// Patch rows are stored de-interleaved.  Neighbouring output positions start m = SX * IC / 16 chunks apart, so chunk u
// of a row sits at (u % m) * plane + u / m: the 32 lanes of a fragment read then fall on 32 consecutive chunks
// whatever the stride (with the plain layout a stride of two puts them on every other chunk, and two lanes of each
// LDS pass on the same banks: measured 23 against 19.5 us in the loop of a 7x7 stem).
//
// The weights are the A operand and the activations the B operand, so a lane ends up with one position and
// sixteen channels: LDS row 8q + 4h + r of a 32-row tile holds channel 16h + 4q + r, and the sixteen accumulator
// registers of lane half h are channels 16h .. 16h + 15 of its position, stored as one 16-byte word.
// Workgroups are persistent: the weights of their 64 channels are staged once, then tiles of R output rows x CW output
// columns follow (the whole width where the rows under it fit LDS, else column tiles: wide images).
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
// than one tile.  F16: the output is fp16 (the s17.15 PPE; sixteen channels of a position are two 16-byte stores).
template <bool IN_U8, int TM, int TN, bool MULTI, bool F16 = false>
__global__ __launch_bounds__(512) void nce_conv_rows16(const int8_t* __restrict__ in, const int8_t* __restrict__ w,
                                                       const int32_t* __restrict__ wt, uint8_t* __restrict__ out, ConvGeom g,
                                                       RowsGeom rg, int pad_byte, GemmPpe ppe) {
    constexpr int BN = 32 * TN, NW = 8, NT = 64 * NW, BP = 32 * TM;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* const wlds = smem;                                          // [64][WS], rows in tile order
    ChanPrep* const sprep = reinterpret_cast<ChanPrep*>(smem + BN * rg.WS);  // [64], by channel
    int* const sbias = reinterpret_cast<int*>(sprep + BN);               // [64] biases, [64] row sums, one flag
    int* const csum = sbias + BN;
    int* const sflag = csum + BN;
    int* const stab = sflag + 4;                                         // [S][2] fragment offsets, by step and lane half
    uint8_t* const patch = reinterpret_cast<uint8_t*>(stab + (2 * rg.S + 3) / 4 * 4);  // [PH][RB]

    const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int H = (int)g.H, W = (int)g.W, IC = (int)g.IC, OC = (int)g.OC, OW = (int)g.OW, OH = (int)g.OH;
    const int oc0 = blockIdx.y * BN;
    const int Ktot = g.KY * g.KX * IC, row_in = g.KX * (IC / 16), nchunks = g.KY * row_in;
    const int S = rg.S, kc = 2 * S;

    // ---- input rows -> LDS: patch row py is input row iy0 + py from pixel -PL on; padding and the sign flip applied here.
    // The first UPF chunks of every thread stay in registers from the load (issued a tile ahead) to the store.
    constexpr int UPF = TM * TN >= 8 ? 6 : 9;  // (what the registers beside the accumulators allow)
    const int pad32 = (pad_byte & 0xff) * 0x01010101;
    const int total_chunks = rg.PH * rg.row_chunks;
    i32x4 qv[UPF];
    struct Chunk {
        bool ok, inside;
        int src, dst;
    };
    struct Origin {
        const int8_t* corner;   // of the patch in the input; may lie outside the tensor
        int iy0, ix0, safe_off;  // first input row and column; offset from the corner to a pixel that exists
    };
    struct TilePos {
        int img, oy0, ox0;
    };
    auto tile_pos = [&](int tile_) {  // tiles in the order (image, row of tiles, column tile)
        const int tr = fdiv(tile_, rg.tiles_x), tx = tile_ - tr * (int)rg.tiles_x.d;
        const int img = fdiv(tr, rg.tiles_y);
        return TilePos{img, (tr - img * (int)rg.tiles_y.d) * rg.R, tx * rg.CW};
    };
    auto origin = [&](int tile_) {
        const TilePos tp = tile_pos(tile_);
        const int iy0 = tp.oy0 * g.SY - g.PT, ix0 = tp.ox0 * g.SX - g.PL;
        const int safe_row = iy0 < 0 ? 0 : (iy0 < H ? iy0 : H - 1);
        return Origin{in + ((int64_t)tp.img * g.isn + (int64_t)iy0 * g.ish + (int64_t)ix0 * g.isw), iy0, ix0,
                      (safe_row - iy0) * (int)g.ish - ix0 * (int)g.isw};
    };
    auto chunk = [&](const Origin& o, int q) {
        Chunk c;
        c.ok = q < total_chunks;
        const int qq = c.ok ? q : 0;
        const int py = fdiv(qq, rg.rc), qi = qq - py * rg.row_chunks;
        const int px = fdiv(qi, rg.cpp);
        c.inside = c.ok && (unsigned)(o.iy0 + py) < (unsigned)H && (unsigned)(o.ix0 + px) < (unsigned)W;
        c.src = c.inside ? py * (int)g.ish + px * (int)g.isw + (qi - px * (int)rg.cpp.d) * 16 : o.safe_off;
        const int qd = fdiv(qi, rg.fm);
        c.dst = py * rg.RB + ((qi - qd * rg.m) * rg.plane + qd) * 16;
        return c;
    };
    auto put = [&](const Chunk& c, i32x4 v) {
        if (!c.ok) return;
        if (!c.inside) v = i32x4{pad32, pad32, pad32, pad32};
        if (IN_U8) v ^= (int32_t)0x80808080;
        *reinterpret_cast<i32x4*>(patch + c.dst) = v;
    };
    // (the chunks' places do not depend on the tile, but worked out once they would sit in registers for the whole
    // kernel: the thread index goes through an opaque move so that they are worked out where they are used)
    auto load_patch = [&](int tile_) {
        const Origin o = origin(tile_);
        int t0 = tid;
        asm volatile("" : "+v"(t0));
#pragma unroll
        for (int u = 0; u < UPF; u++) qv[u] = *reinterpret_cast<const i32x4*>(o.corner + chunk(o, u * NT + t0).src);
    };
    auto store_patch = [&](int tile_) {
        const Origin o = origin(tile_);
        int t0 = tid;
        asm volatile("" : "+v"(t0));
#pragma unroll
        for (int u = 0; u < UPF; u++) put(chunk(o, u * NT + t0), qv[u]);
        for (int q0 = UPF * NT; q0 < total_chunks; q0 += 4 * NT) {  // tall patches: the rest, a round trip each
            i32x4 rest[4];
#pragma unroll
            for (int u = 0; u < 4; u++) rest[u] = *reinterpret_cast<const i32x4*>(o.corner + chunk(o, q0 + u * NT + tid).src);
#pragma unroll
            for (int u = 0; u < 4; u++) put(chunk(o, q0 + u * NT + tid), rest[u]);
        }
    };
    int wt2 = 0, wt3 = 0;  // this thread's channel of the weight table, asked for before anything else
    if (tid < BN) {
        const int n = oc0 + tid < OC ? oc0 + tid : OC - 1;
        wt2 = wt[n * 4 + 2];
        wt3 = wt[n * 4 + 3];
    }
    load_patch(blockIdx.x);  // (under the staging of the weights)

    // ---- weights -> LDS, once; the table of fragment offsets
    for (int c = tid; c < 2 * rg.S; c += NT) {
        const int ky = fdiv(c, rg.rin), e = c - ky * row_in;
        const int ed = fdiv(e, rg.fm);
        stab[c] = c < nchunks ? ky * rg.RB + ((e - ed * rg.m) * rg.plane + ed) * 16 : 0;  // (the chunk past the end: zero weights, any bytes)
    }
    for (int q = tid; q < BN * kc; q += NT) {
        const int n = fdiv(q, rg.kc), c = q - n * kc;
        const int oc = oc0 + n < OC ? oc0 + n : OC - 1;  // channels past the end repeat the last one
        i32x4 v = i32x4{0, 0, 0, 0};
        if (c < nchunks) v = *reinterpret_cast<const i32x4*>(w + (int64_t)oc * Ktot + c * 16);
        const int lrow = (n & ~31) + 8 * ((n >> 2) & 3) + 4 * ((n >> 4) & 1) + (n & 3);
        *reinterpret_cast<i32x4*>(wlds + lrow * rg.WS + c * 16) = v;
    }
    __syncthreads();
    if (tid < 4 * BN) {  // the sums of the weight rows, for the zero-point term
        const int n = tid >> 2, part = tid & 3;
        const int lrow = (n & ~31) + 8 * ((n >> 2) & 3) + 4 * ((n >> 4) & 1) + (n & 3);
        int sum = 0;
        if (ppe.corr != 0)
            for (int c = part; c < kc; c += 4) {
                const i32x4 q = *reinterpret_cast<const i32x4*>(wlds + lrow * rg.WS + c * 16);
#pragma unroll
                for (int j = 0; j < 4; j++) sum = __builtin_amdgcn_sdot4(q[j], 0x01010101, sum, false);
            }
        sum += (int)dpp_u32<0xB1>((unsigned)sum);
        sum += (int)dpp_u32<0x4E>((unsigned)sum);
        if (part == 0) csum[n] = sum;
    }
    __syncthreads();
    const PpePack pk = make_ppe_pack(ppe.zp_out, ppe.lo, ppe.hi, ppe.out_signed != 0);
    if (tid < BN) {
        const uint32_t w2 = (uint32_t)wt2;
        // (an fp16 output keeps 15 fractional bits of the scaled value)
        const ChanPrep c = ppe_prepare((int)(int16_t)(w2 >> 16), (int)((w2 >> 8) & 0xffu) - (F16 ? 15 : 0),
                                       (int)((unsigned)wt3 + (unsigned)(ppe.corr * csum[tid])), ppe.prelu_mult, ppe.prelu_shift);
        sprep[tid] = c;
        sbias[tid] = c.bias;
        // the short PPE serves slopes in [0, 1] (ReLU, LeakyReLU), an even zero-point offset and scales up to 1/2
        const bool slope_ok = (ppe.prelu_mult >= 0 && (ppe.prelu_shift >= 31 || ppe.prelu_mult <= (1 << ppe.prelu_shift)));
        const bool clip = c.bmax_pos != 0x7fffffff || c.bmax_neg != 0x7fffffff;
        const bool general = __builtin_amdgcn_ballot_w64(clip) != 0 || pk.odd != 0 || !slope_ok;
        if (tid == 0) sflag[0] = general ? 1 : 0;
    }
    // (the barrier after the first patch makes these visible)

    const bool same_f = ppe.prelu_mult == 1 && ppe.prelu_shift == 0;  // no PReLU stage (or a slope of zero, which the host turns into a clamp)
    const bool vec_ok = (g.out_bits & 15) == 0;
    const bool half_ok = (g.out_bits & 7) == 0;
    const uint8_t* const wl = wlds + (lane & 31) * rg.WS + half * 16;
    const int q16 = oc0 + half * 16;  // first of the 16 channels this lane stores in channel tile 0

    for (int tile = blockIdx.x; tile < rg.ntiles; tile += gridDim.x) {
        const TilePos tp = tile_pos(tile);
        const int img = tp.img, oy0 = tp.oy0, ox0 = tp.ox0;
        store_patch(tile);
        __syncthreads();
        // the next tile's rows travel while this one is computed (after the last tile: the same rows once more, so that
        // no branch stands between these loads and their use; a launch of one tile per workgroup has none of this)
        if (MULTI) load_patch(tile + (int)gridDim.x < rg.ntiles ? tile + (int)gridDim.x : tile);
        const bool general = sflag[0] != 0;

        // positions of a tile are counted over R x CW; those past the last row or column of the tensor are skipped
        const int rows_here = OH - oy0 < rg.R ? OH - oy0 : rg.R;
        const int cols_here = OW - ox0 < rg.CW ? OW - ox0 : rg.CW;
        const int nblk = (rows_here * rg.CW + BP - 1) / BP;
        const int64_t pos0 = ((int64_t)img * OH + oy0) * OW + ox0;
        const int32_t* rt = ppe.rowterm ? ppe.rowterm + pos0 : nullptr;
        const int64_t opos0 = (int64_t)img * g.osn + (int64_t)oy0 * g.osh + (int64_t)ox0 * g.osw;  // the tile's first output position
        uint8_t* const out0 = out + opos0;
        // element offset of the position r * OW + c from there
        auto out_off = [&](int pcv) {
            if (g.out_flat) return (int64_t)pcv * g.osw;
            const int r = fdiv(pcv, rg.ow), c = pcv - r * OW;
            return (int64_t)r * g.osh + (int64_t)c * g.osw;
        };

        auto one_block = [&](int b, auto kind_c) {
            // PPE kinds.  0: the general form; 1: two factors, the short form (see ppe_pack4_biased); 2: one factor;
            // 3: fp16 output (like the general form the accumulators start from zero and the PPE adds the bias)
            constexpr int KIND = decltype(kind_c)::value;
            constexpr bool GENERAL = KIND == 0 || KIND == 3;
            const uint8_t* pl[TM];
            int pc[TM];  // the position's offset from the tile's first one in the output, -1 for none
#pragma unroll
            for (int i = 0; i < TM; i++) {
                const int p = b * BP + i * 32 + (lane & 31);
                int r = fdiv(p, rg.cw), c = p - r * rg.CW;
                const bool ok = r < rows_here && c < cols_here;
                r = ok ? r : 0;
                c = ok ? c : 0;
                pc[i] = ok ? r * OW + c : -1;
                pl[i] = patch + r * g.SY * rg.RB + c * 16;
            }
            // The short PPE's accumulators start from the bias: the lane's sixteen channels of a channel tile are the C
            // operand of the first step's MFMAs (no copies into every position block's accumulators).
            i32x16 acc[TM][TN], start[TN];
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    i32x4 b4 = i32x4{0, 0, 0, 0};
                    if (!GENERAL) b4 = *reinterpret_cast<const i32x4*>(sbias + 32 * j + 16 * half + 4 * q);
#pragma unroll
                    for (int r = 0; r < 4; r++) start[j][4 * q + r] = b4[r];
                }

            // fragments of step s + 1 are read before the MFMAs of step s, their offset in the patch a step before that
            int ls = 0;  // the next step to read
            const int* const tab = stab + half;
            int poff = tab[0];
            i32x4 fa[2][TN], fb[2][TM];
            auto read = [&](auto buf_c) {
                constexpr int buf = decltype(buf_c)::value;
                const int woff = ls * 32;
#pragma unroll
                for (int j = 0; j < TN; j++) fa[buf][j] = *reinterpret_cast<const i32x4*>(wl + j * 32 * rg.WS + woff);
#pragma unroll
                for (int i = 0; i < TM; i++) fb[buf][i] = *reinterpret_cast<const i32x4*>(pl[i] + poff);
                if (ls + 1 < S) ls++;  // (past the end the last step is read again)
                poff = tab[2 * ls];
            };
            auto multiply = [&](auto buf_c) {
                constexpr int buf = decltype(buf_c)::value;
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[buf][j], fb[buf][i], acc[i][j], 0, 0, 0);
            };
            read(std::integral_constant<int, 0>{});
            read(std::integral_constant<int, 1>{});
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[0][j], fb[0][i], start[j], 0, 0, 0);
            for (int s = 1; s < S; s += 2) {
                read(std::integral_constant<int, 0>{});
                multiply(std::integral_constant<int, 1>{});
                if (s + 1 < S) {
                    read(std::integral_constant<int, 1>{});
                    multiply(std::integral_constant<int, 0>{});
                }
            }

            if (rt) {
#pragma unroll
                for (int i = 0; i < TM; i++) {
                    const int v = rt[pc[i] < 0 ? 0 : pc[i]];
#pragma unroll
                    for (int j = 0; j < TN; j++)
#pragma unroll
                        for (int r = 0; r < 16; r++) acc[i][j][r] += v;
                }
            }
            if constexpr (KIND == 3) {
                uint16_t* const out16 = reinterpret_cast<uint16_t*>(out) + opos0;
                const bool vec16_ok = vec_ok;
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const int qc = q16 + 32 * j;
#pragma unroll
                    for (int half8 = 0; half8 < 2; half8++) {  // channels 0-7, then 8-15 of the lane's sixteen
                        i32x4 o8[TM];
#pragma unroll
                        for (int i = 0; i < TM; i++) o8[i] = i32x4{0, 0, 0, 0};
#pragma unroll
                        for (int r8 = 0; r8 < 8; r8++) {
                            const int r = half8 * 8 + r8;
                            const ChanPrep c = sprep[32 * j + 16 * half + r];
#pragma unroll
                            for (int i = 0; i < TM; i++)
                                o8[i][r8 >> 1] |= (int)ppe_fast_f16(acc[i][j][r], c, ppe.f16_lo, ppe.f16_hi) << (16 * (r8 & 1));
                            __builtin_amdgcn_sched_barrier(0);  // (a channel at a time: hoisted, the parameters of all sixteen fill the register file)
                        }
#pragma unroll
                        for (int i = 0; i < TM; i++) {
                            if (pc[i] < 0 || qc + 8 * half8 >= OC) continue;
                            uint16_t* dst = out16 + (out_off(pc[i]) + qc + 8 * half8);
                            if (vec16_ok && qc + 8 * half8 + 8 <= OC) {
                                __builtin_nontemporal_store(o8[i], reinterpret_cast<i32x4*>(dst));
                            } else {
                                for (int e = 0; e < 8 && qc + 8 * half8 + e < OC; e++) dst[e] = (uint16_t)(o8[i][e >> 1] >> (16 * (e & 1)));
                            }
                        }
                    }
                }
                return;
            }
#pragma unroll
            for (int j = 0; j < TN; j++) {
                i32x4 o[TM];
#pragma unroll
                for (int i = 0; i < TM; i++) o[i] = i32x4{0, 0, 0, 0};
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const ChanPrep* cpp = sprep + 32 * j + 16 * half + r;
                    if constexpr (KIND == 0) {
                        ChanPrep c = *cpp;  // the form ppe_one takes: sign flip in the bias, factors swapped for a negative multiplier
                        c.bias = (int)((unsigned)c.bias + 0x80000000u);
                        if (c.sgn) {
                            const double f = c.f_pos;
                            c.f_pos = c.f_neg;
                            c.f_neg = f;
                            const int bm = c.bmax_pos;
                            c.bmax_pos = c.bmax_neg;
                            c.bmax_neg = bm;
                        }
#pragma unroll
                        for (int i = 0; i < TM; i++) o[i][r >> 2] |= (int)(ppe_one<false, true>(acc[i][j][r], c, pk) << (8 * (r & 3)));
                    } else {
                        const double f_pos = cpp->f_pos, f_neg = KIND == 2 ? 0.0 : cpp->f_neg;
#pragma unroll
                        for (int i = 0; i < TM; i++)
                            o[i][r >> 2] |= (int)(ppe_one_biased<KIND == 1>(acc[i][j][r], f_pos, f_neg, pk) << (8 * (r & 3)));
                    }
                }
                const int qc = q16 + 32 * j;
#pragma unroll
                for (int i = 0; i < TM; i++) {
                    if (pc[i] < 0 || qc >= OC) continue;
                    o[i] ^= (int)pk.flip;
                    uint8_t* dst = out0 + (out_off(pc[i]) + qc);
                    if (vec_ok && qc + 16 <= OC) {
                        __builtin_nontemporal_store(o[i], reinterpret_cast<i32x4*>(dst));
                    } else if (half_ok && qc + 16 <= OC) {  // (rows a multiple of 8 bytes long: 72, 88, 120 channels)
                        *reinterpret_cast<uint2*>(dst) = uint2{(unsigned)o[i][0], (unsigned)o[i][1]};
                        *reinterpret_cast<uint2*>(dst + 8) = uint2{(unsigned)o[i][2], (unsigned)o[i][3]};
                    } else {
                        for (int e = 0; e < 16 && qc + e < OC; e++) dst[e] = (uint8_t)(o[i][e >> 2] >> (8 * (e & 3)));
                    }
                }
            }
        };
        if constexpr (F16) {
            for (int b = wave; b < nblk; b += NW) one_block(b, std::integral_constant<int, 3>{});
        } else if (general) {
            for (int b = wave; b < nblk; b += NW) one_block(b, std::integral_constant<int, 0>{});
        } else if (same_f) {
            for (int b = wave; b < nblk; b += NW) one_block(b, std::integral_constant<int, 2>{});
        } else {
            for (int b = wave; b < nblk; b += NW) one_block(b, std::integral_constant<int, 1>{});
        }
        __syncthreads();  // the next tile's rows replace this patch
    }
}

// Kernels that may ask for more than 64 KiB of dynamic LDS are given the largest size any launch of them uses,
// once per (device, kernel): the attribute is then never changed again, so concurrent launches that want
// different sizes cannot undo each other's setting.
constexpr size_t kMaxDynLds = 160 * 1024 - 512;
std::mutex g_lds_mutex;
std::set<std::pair<int, const void*>> g_lds_done;

template <class KernelT>
int set_dyn_lds(KernelT kernel, size_t bytes) {
    if (bytes <= 64 * 1024) return VPX_RESULT_SUCCESS;
    VPX_REQUIRE(bytes <= kMaxDynLds, VPX_RESULT_ERROR_UNKNOWN, "a launch asks for %zu bytes of LDS", bytes);
    int dev = 0;
    VPX_HIP_CHECK(hipGetDevice(&dev));
    const void* fn = reinterpret_cast<const void*>(kernel);
    std::lock_guard<std::mutex> lock(g_lds_mutex);
    if (g_lds_done.count({dev, fn})) return VPX_RESULT_SUCCESS;
    VPX_HIP_CHECK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxDynLds));
    g_lds_done.insert({dev, fn});
    return VPX_RESULT_SUCCESS;
}

// An operand of an NCE task as a view: the strides of its images, rows and pixels in elements (channels contiguous).
// All four task strides zero is the dense tensor.  Dimensions of size one take the stride that keeps the view as flat
// as the others allow (their own is never used).
struct View {
    int64_t sn, sh, sw;
    bool dense;   // the packed NHWC tensor
    int flat;     // 2: position m of N x H x W at m * sw; 1: that holds inside an image; 0: neither
    int64_t span; // elements from the first to one past the last
};
int operand_view(const int64_t st[4], int64_t N, int64_t H, int64_t W, int64_t C, const char* what, View* v) {
    if ((st[0] | st[1] | st[2] | st[3]) == 0) {
        *v = View{H * W * C, W * C, C, true, 2, N * H * W * C};
        return VPX_RESULT_SUCCESS;
    }
    VPX_REQUIRE(st[3] == 1, VPX_RESULT_ERROR_INVALID_ARGUMENT, "NCE task: the %s's channel stride is %lld; channels must be contiguous (1)", what,
                (long long)st[3]);
    VPX_REQUIRE(st[0] >= 0 && st[1] >= 0 && st[2] >= 0, VPX_RESULT_ERROR_INVALID_ARGUMENT, "NCE task: the %s has a negative stride", what);
    const int64_t ext_w = (W - 1) * st[2] + C;
    VPX_REQUIRE(W <= 1 || st[2] >= C, VPX_RESULT_ERROR_INVALID_ARGUMENT, "NCE task: the %s's W stride %lld is below its %lld channels", what,
                (long long)st[2], (long long)C);
    VPX_REQUIRE(H <= 1 || st[1] >= ext_w, VPX_RESULT_ERROR_INVALID_ARGUMENT, "NCE task: the %s's H stride %lld is below the %lld elements a row spans",
                what, (long long)st[1], (long long)ext_w);
    const int64_t ext_h = (H - 1) * st[1] + ext_w;
    VPX_REQUIRE(N <= 1 || st[0] >= ext_h, VPX_RESULT_ERROR_INVALID_ARGUMENT, "NCE task: the %s's N stride %lld is below the %lld elements an image spans",
                what, (long long)st[0], (long long)ext_h);
    int64_t sn = st[0], sh = st[1], sw = st[2];
    if (W <= 1) sw = H > 1 ? sh : (N > 1 ? sn : C);
    if (H <= 1) sh = N > 1 && W <= 1 ? sn : W * sw;
    if (N <= 1) sn = H * sh;
    v->sn = sn;
    v->sh = sh;
    v->sw = sw;
    v->flat = sh == W * sw ? (sn == H * sh ? 2 : 1) : 0;
    v->dense = v->flat == 2 && sw == C;
    v->span = (N > 0 && H > 0 && W > 0) ? (N - 1) * sn + (H - 1) * sh + (W - 1) * sw + C : 0;
    return VPX_RESULT_SUCCESS;
}

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

// Weights with a zero point zw.  The MFMA kernels multiply signed bytes W = w - cw (cw = 128 for unsigned storage,
// re-biased into a scratch copy, else 0), so sum (a - za)(w - zw) lacks (cw - zw) * sum (a - za) over the taps
// inside the image: one value per output position, the same for all its channels.  Two small kernels prepare
// it: the channel sum of every input pixel, then the sum of those under each window times (cw - zw); the
// convolution kernels add the result to their accumulators before the PPE.  A 1x1, stride-1, unpadded layer
// (a matmul) needs only the first, which then applies the factor itself.
__global__ __launch_bounds__(256) void nce_pixel_sum_kernel(const uint8_t* __restrict__ in, int32_t* __restrict__ cs, int64_t pixels,
                                                            int IC, int lpp, int flip, int offset, int factor, ConvGeom g, int in_flat) {
    // lpp lanes (a power of two, at most 64) share a pixel; each sums 16-byte chunks
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t pixel = t / lpp;
    const int sub = (int)(t % lpp);
    unsigned sum = 0;
    if (pixel < pixels) {
        // (pixels are counted over the dense N x H x W grid; a view of a larger tensor has them isw / ish / isn apart)
        int64_t at = pixel * g.isw;
        if (!in_flat) {
            const int64_t hw = g.H * g.W, n = pixel / hw, rem = pixel - n * hw, y = rem / g.W;
            at = in_pos(g, n, y, rem - y * g.W);
        }
        const i32x4* row = reinterpret_cast<const i32x4*>(in + at);
        for (int c = sub; c < IC / 16; c += lpp) {
            const i32x4 q = row[c];
#pragma unroll
            for (int k = 0; k < 4; k++) sum = __builtin_amdgcn_sad_u8((unsigned)(q[k] ^ flip), 0u, sum);  // four bytes at once
        }
    }
    for (int o = lpp >> 1; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
    if (pixel < pixels && sub == 0) cs[pixel] = ((int)sum - offset) * factor;
}

__global__ __launch_bounds__(256) void nce_window_sum_kernel(const int32_t* __restrict__ cs, int32_t* __restrict__ rowterm, ConvGeom g,
                                                             int factor, int64_t total) {
    const int64_t m = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (m >= total) return;
    const int64_t ox = m % g.OW, oy = (m / g.OW) % g.OH, n = m / (g.OW * g.OH);
    int sum = 0;
    for (int ky = 0; ky < g.KY; ky++) {
        const int64_t iy = oy * g.SY + ky - g.PT;
        if (iy < 0 || iy >= g.H) continue;
        for (int kx = 0; kx < g.KX; kx++) {
            const int64_t ix = ox * g.SX + kx - g.PL;
            if (ix >= 0 && ix < g.W) sum += cs[(n * g.H + iy) * g.W + ix];
        }
    }
    rowterm[m] = sum * factor;
}

// u8 weights whose zero point is 128 (symmetric weights kept in unsigned storage) are the signed weights
// w - 128: one pass flips the top bit of every byte into a scratch copy and the signed kernels run on that.
__global__ __launch_bounds__(256) void nce_weights_to_s8_kernel(const i32x4* __restrict__ in, i32x4* __restrict__ out, int64_t n_vec) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n_vec; i += (int64_t)gridDim.x * 256) out[i] = in[i] ^ (int32_t)0x80808080;
}


// Dispatch overrides for tests and tuning.  The VPX_* environment variables of the same names are read once, at
// the first use; afterwards only vpx_set_tuning changes a value, so a launch never reads the environment.
enum { NCE_AUTO = 0, NCE_NAIVE, NCE_GATHER, NCE_CONV };
struct Tuning {
    std::atomic<int> nce_kernel{NCE_AUTO};  // VPX_NCE_KERNEL = naive | gather | conv: restrict the choice to slower, more general paths
    std::atomic<int> gemm_tile{0};          // VPX_GEMM_TILE = 128 | 256 (0: chosen from the shape)
    std::atomic<int> gemm_waves{0};         // VPX_GEMM_WAVES = 4 | 8
    std::atomic<int> conv_stream{0};        // VPX_CONV_KERNEL = regw | tile | stream: start the choice of LDS-patch kernel at this one (-1, 1, 2; 0: by size)
    std::atomic<int> conv_rows{0};          // VPX_CONV_ROWS = n: cap on the output rows per workgroup of the LDS-patch kernels
    std::atomic<int> conv_cols{0};          // VPX_CONV_COLS = n: output columns per tile of the row-patch kernel
    std::atomic<int> conv_waves{0};         // VPX_CONV_WAVES = 4 | 8
    std::atomic<int> stream_ksplit{1};      // VPX_STREAM_KSPLIT = off: the streamed-weights kernel never splits K over its waves
    std::atomic<int> mvn_fused{1};          // VPX_MVN_FUSED = off | nowait (see tuning_mvn_fused)
};
Tuning g_tuning;
std::once_flag g_tuning_once;

bool set_knob(const char* knob, const char* value) {
    const char* v = value ? value : "";
    if (!std::strcmp(knob, "VPX_NCE_KERNEL")) {
        g_tuning.nce_kernel = !std::strcmp(v, "naive") ? NCE_NAIVE : (!std::strcmp(v, "gather") ? NCE_GATHER : (!std::strcmp(v, "conv") ? NCE_CONV : NCE_AUTO));
    } else if (!std::strcmp(knob, "VPX_GEMM_TILE")) {
        g_tuning.gemm_tile = *v ? (std::atoi(v) == 128 ? 128 : 256) : 0;
    } else if (!std::strcmp(knob, "VPX_GEMM_WAVES")) {
        g_tuning.gemm_waves = *v ? (std::atoi(v) == 4 ? 4 : 8) : 0;
    } else if (!std::strcmp(knob, "VPX_CONV_KERNEL")) {
        g_tuning.conv_stream = !std::strcmp(v, "stream") ? 2 : (!std::strcmp(v, "tile") ? 1 : (!std::strcmp(v, "regw") ? -1 : 0));
    } else if (!std::strcmp(knob, "VPX_CONV_ROWS")) {
        g_tuning.conv_rows = std::atoi(v) > 0 ? std::atoi(v) : 0;
    } else if (!std::strcmp(knob, "VPX_CONV_COLS")) {
        g_tuning.conv_cols = std::atoi(v) > 0 ? std::atoi(v) : 0;
    } else if (!std::strcmp(knob, "VPX_CONV_WAVES")) {
        g_tuning.conv_waves = std::atoi(v) == 4 ? 4 : 0;
    } else if (!std::strcmp(knob, "VPX_STREAM_KSPLIT")) {
        g_tuning.stream_ksplit = (!std::strcmp(v, "off") || !std::strcmp(v, "0")) ? 0 : 1;
    } else if (!std::strcmp(knob, "VPX_MVN_FUSED")) {
        g_tuning.mvn_fused = !std::strcmp(v, "off") ? 0 : (!std::strcmp(v, "nowait") ? 2 : 1);
    } else {
        return false;
    }
    return true;
}

const Tuning& tuning() {
    std::call_once(g_tuning_once, [] {
        for (const char* k : {"VPX_NCE_KERNEL", "VPX_GEMM_TILE", "VPX_GEMM_WAVES", "VPX_CONV_KERNEL", "VPX_CONV_ROWS", "VPX_CONV_COLS", "VPX_CONV_WAVES", "VPX_STREAM_KSPLIT", "VPX_MVN_FUSED"})
            if (const char* v = std::getenv(k)) set_knob(k, v);
    });
    return g_tuning;
}

}  // namespace

int tuning_mvn_fused() {
    return tuning().mvn_fused.load();
}

int set_tuning(const char* knob, const char* value) {
    (void)tuning();  // the environment is consulted before the first explicit setting, never after it
    VPX_REQUIRE(knob != nullptr, VPX_RESULT_ERROR_INVALID_NULL_HANDLE, "tuning knob name is null");
    VPX_REQUIRE(set_knob(knob, value), VPX_RESULT_ERROR_INVALID_ARGUMENT, "unknown tuning knob '%s'", knob);
    return VPX_RESULT_SUCCESS;
}

int launch_nce(const vpx_nce_task_t& t, hipStream_t s, const char** kernel_name) {
    const bool in_u8 = t.input_type == VPX_NN_U8, w_u8 = t.weights_type == VPX_NN_U8,
               out_signed = t.output_type == VPX_NN_I8, out_f16 = t.output_type == VPX_NN_FP16;
    ConvGeom g{};
    g.N = t.N; g.H = t.H; g.W = t.W; g.IC = t.IC; g.OC = t.OC;
    g.KY = t.kernel_size[0]; g.KX = t.kernel_size[1];
    g.SY = t.kernel_strides[0]; g.SX = t.kernel_strides[1];
    g.PL = t.kernel_padding[0]; g.PT = t.kernel_padding[2];
    g.OH = (t.H + t.kernel_padding[2] + t.kernel_padding[3] - g.KY) / g.SY + 1;
    g.OW = (t.W + t.kernel_padding[0] + t.kernel_padding[1] - g.KX) / g.SX + 1;
    VPX_REQUIRE(g.OH > 0 && g.OW > 0, VPX_RESULT_ERROR_INVALID_ARGUMENT, "NCE task: kernel %dx%d does not fit the padded input",
                g.KY, g.KX);

    Ppe ppe;
    ppe.zp_out = t.zp_out;
    ppe.clamp_lo = t.ppe.clamp_low;
    ppe.clamp_hi = t.ppe.clamp_high;
    ppe.f16_lo = -INFINITY;
    ppe.f16_hi = INFINITY;
    if (out_f16 && t.ppe.clamp_high != INT32_MAX) {
        // two fp16 bounds in one word, 0xllllhhhh (dialect/VPU/utils/ppe_utils.hpp:36-87); clamp_low is not used
        const auto half = [](uint32_t h) {
            const uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
            const float mag = e == 0 ? std::ldexp((float)m, -24) : (e == 31 ? (m ? NAN : INFINITY) : std::ldexp((float)(m | 0x400u), (int)e - 25));
            return (h & 0x8000u) ? -mag : mag;
        };
        const float lo = half(((uint32_t)t.ppe.clamp_high >> 16) & 0xffffu), hi = half((uint32_t)t.ppe.clamp_high & 0xffffu);
        if (!std::isnan(lo)) ppe.f16_lo = lo;
        if (!std::isnan(hi)) ppe.f16_hi = hi;
    }
    switch (t.ppe.mode) {
    case VPX_PPE_NOOP: ppe.prelu_mult = 1; ppe.prelu_shift = 0; break;
    case VPX_PPE_LRELU:
    case VPX_PPE_LRELUX: ppe.prelu_mult = 0; ppe.prelu_shift = 0; break;
    case VPX_PPE_LPRELU: ppe.prelu_mult = t.ppe.lrelu_mult; ppe.prelu_shift = t.ppe.lrelu_shift; break;
    default: return fail(VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "NCE task: PPE mode %d is not an integer-pipeline mode", t.ppe.mode);
    }

    if (t.task_type == VPX_NCE_ELTWISE) return launch_nce_eltwise(t, ppe, s, kernel_name);

    // A slope of zero (ReLU) is a clamp: the negative branch ends at the zero point whatever the accumulator, and rounding
    // is monotone, so the result is that of a layer without a PReLU stage held at or above the zero point before the
    // clamp (max, then min) -- the same layer with the lower bound raised to the zero point.  Every kernel's epilogue then
    // runs its one-factor form: no sign test, no second product.  (Integer outputs only: an fp16 zero keeps its sign.)
    if (!out_f16 && ppe.prelu_mult == 0) {
        ppe.prelu_mult = 1;
        ppe.prelu_shift = 0;
        if (ppe.clamp_lo < t.zp_out) ppe.clamp_lo = t.zp_out;
    }

    const int64_t Mtot = g.N * g.OH * g.OW;
    const int64_t Ktot = (int64_t)g.KY * g.KX * g.IC;
    if (Mtot == 0 || g.OC == 0) return VPX_RESULT_SUCCESS;

    // Input and output as views (dense unless the task gives strides); the weights are always dense.
    View vin, vout;
    {
        int rc = operand_view(t.input_strides, g.N, g.H, g.W, g.IC, "input", &vin);
        if (!rc) rc = operand_view(t.output_strides, g.N, g.OH, g.OW, g.OC, "output", &vout);
        if (rc) return rc;
        VPX_REQUIRE(t.groups <= 1 || (vin.dense && vout.dense), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                    "NCE task: a grouped task takes dense operands (strides were given with groups = %d)", t.groups);
    }
    g.isn = vin.sn; g.ish = vin.sh; g.isw = vin.sw;
    g.osn = vout.sn; g.osh = vout.sh; g.osw = vout.sw;
    g.out_flat = vout.flat;
    g.out_bits = (unsigned)(reinterpret_cast<uintptr_t>(t.output) | (uintptr_t)((vout.sn | vout.sh | vout.sw) * (out_f16 ? 2 : 1)));
    const bool in_flat = vin.flat == 2;

    const bool zp_in_ok = in_u8 ? (t.zp_in >= 0 && t.zp_in <= 255) : (t.zp_in >= -128 && t.zp_in <= 127);
    // the fast epilogue adds the output zero point after limiting the scaled value to +-2^30
    const bool zp_out_ok = t.zp_out >= -(1 << 20) && t.zp_out <= (1 << 20);
    // Unsigned weights are re-biased by 128 into a signed scratch copy; what is left of the weight zero point
    // (wz_rest = 128 - zp_w, or -zp_w for signed storage) enters through one term per output position.
    const bool w_rebias = w_u8 && Ktot % 16 == 0;
    const bool zp_w_ok = w_u8 ? (t.zp_w >= 0 && t.zp_w <= 255) : (t.zp_w >= -128 && t.zp_w <= 127);
    const int wz_rest = (w_u8 ? 128 : 0) - t.zp_w;
    const bool mfma_ok = (!w_u8 || w_rebias) && zp_w_ok && zp_in_ok && zp_out_ok && Mtot < (1ll << 31) && g.OC < (1ll << 31) &&
                         (wz_rest == 0 || (g.IC % 16 == 0 && g.N * g.H * g.W < (1ll << 31) && g.IC < (1 << 23)));
    const bool is_1x1 = g.KY == 1 && g.KX == 1 && t.kernel_padding[0] == 0 && t.kernel_padding[1] == 0 &&
                        t.kernel_padding[2] == 0 && t.kernel_padding[3] == 0;
    const bool is_gemm = is_1x1 && g.SY == 1 && g.SX == 1;
    // a 1x1 layer with a stride, or whose input pixels are not evenly spaced (a window of a larger tensor), is a matmul
    // over rows picked from the input (one group, the view spanning less than 4 GiB)
    const bool picks_rows = !(is_gemm && in_flat);
    const bool is_strided_gemm = is_1x1 && picks_rows && t.groups <= 1 && vin.span < (1ll << 32);
    const bool is_flat_gemm = is_gemm && in_flat && vin.sw < (1ll << 23);
    // (the MFMA kernels read 16 bytes at a time from wherever a pixel starts)
    const bool aligned = ((reinterpret_cast<uintptr_t>(t.input) | reinterpret_cast<uintptr_t>(t.weights) |
                           (uintptr_t)(vin.sn | vin.sh | vin.sw)) & 15) == 0;
    // VPX_NCE_KERNEL=naive|gather|conv restricts the choice to the slower, more general paths (used by tests
    // to check the device paths against each other).
    const Tuning& knobs = tuning();
    const int force = knobs.nce_kernel.load();
    const bool allow_gemm = force == NCE_AUTO;
    const bool allow_lds = allow_gemm || force == NCE_CONV;
    const bool allow_mfma = allow_lds || force == NCE_GATHER;

    // A matmul tile wastes half (128 columns) or three quarters of its MFMAs on 64 output channels: such 1x1 layers go
    // to the convolution kernels, whose tiles are 64 channels wide (7.5 us against 9.5 us at [100352 x 64 x 64]), unless K
    // is long enough for the matmul kernel's deeper pipeline to make up for it (from 192 channels on: [100352 x 192 x 64]
    // 13.8 -> 11.1 us, [25088 x 512 x 64] 8.6 -> 7.5 us, [6272 x 1024 x 64] 11.1 -> 9.0 us; 128 channels: even).
    const int64_t gemm_tiles = ((Mtot + 255) / 256) * ((g.OC + 255) / 256);
    const bool use_gemm = allow_gemm && (is_flat_gemm || is_strided_gemm) && g.IC % 64 == 0 && g.IC < (1 << 24) && (g.OC > 64 || (g.OC > 48 && g.IC >= 192) || Mtot < 1024);
    // VPU.NCE.MatMul's groups: one launch of the matmul kernel when it serves the shape (the preparation passes then
    // walk all groups' weights / activations as one tensor), else one task after the other on the stream.
    const int64_t G = t.groups > 1 ? t.groups : 1;
    const bool one_launch = G > 1 && allow_mfma && mfma_ok && aligned && use_gemm && (wz_rest == 0 || Mtot % 4 == 0) && G <= 65535 &&
                            G * g.OC < (1ll << 31) && G * Mtot < (1ll << 31);
    if (G > 1 && !one_launch) {
        const int64_t out_bytes = out_f16 ? 2 : 1;
        for (int64_t grp = 0; grp < G; grp++) {
            vpx_nce_task_t sub = t;
            sub.groups = 1;
            sub.input = (const char*)t.input + grp * g.N * g.H * g.W * g.IC;
            sub.weights = (const char*)t.weights + grp * g.OC * Ktot;
            sub.weight_table = t.weight_table + grp * g.OC * 4;
            sub.output = (char*)t.output + grp * Mtot * g.OC * out_bytes;
            const int rc = launch_nce(sub, s, kernel_name);
            if (rc) return rc;
        }
        return VPX_RESULT_SUCCESS;
    }
    const void* wptr = t.weights;  // the signed weights the MFMA kernels read
    size_t wofs = 0;               // scratch bytes taken by their re-biased copy
    const auto scratch = [&](size_t bytes, void** out) {
        void* base = nullptr;
        const int r = get_workspace(s, wofs + bytes, &base);
        *out = (char*)base + wofs;
        return r;
    };
    const int32_t* rowterm = nullptr;  // the per-position term of the weight zero point, when there is one
    const auto rebias_weights = [&]() -> int {
        // (G > 1 here only on the matmul path: all groups' weights and pixels are walked as one tensor)
        const size_t wbytes = w_rebias ? ((size_t)(G * g.OC) * (size_t)Ktot + 255) / 256 * 256 : 0;
        const int64_t pixels = G * g.N * g.H * g.W;
        const bool direct = is_gemm;  // every output position is one input pixel
        constexpr int64_t kRowPad = 32 * kPatchMaxMT + 256;  // edge tiles read past the last position
        const size_t rbytes = wz_rest != 0 ? (size_t)(G * Mtot + kRowPad + (direct ? 0 : pixels)) * sizeof(int32_t) : 0;
        if (wbytes + rbytes == 0) return VPX_RESULT_SUCCESS;
        void* base = nullptr;
        const int r = get_workspace(s, wbytes + (rbytes + 255) / 256 * 256, &base);
        if (r) return r;
        if (w_rebias) {
            const int64_t n_vec = G * g.OC * Ktot / 16;
            const int64_t blocks = (n_vec + 255) / 256;
            hipLaunchKernelGGL(nce_weights_to_s8_kernel, dim3((unsigned)(blocks < 4096 ? blocks : 4096)), dim3(256), 0, s,
                               (const i32x4*)t.weights, (i32x4*)base, n_vec);
            VPX_HIP_CHECK(hipGetLastError());
            wptr = base;
        }
        if (wz_rest != 0) {
            int32_t* rt = (int32_t*)((char*)base + wbytes);
            int32_t* cs = direct ? rt : rt + G * Mtot + kRowPad;
            int lpp = 1;
            while (lpp < g.IC / 16 && lpp < 64) lpp *= 2;
            const int64_t blocks = (pixels * lpp + 255) / 256;
            VPX_REQUIRE(blocks < (1ll << 31), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "NCE task: input of %lld pixels exceeds the launch limit",
                        (long long)pixels);
            hipLaunchKernelGGL(nce_pixel_sum_kernel, dim3((unsigned)blocks), dim3(256), 0, s, (const uint8_t*)t.input, cs, pixels,
                               (int)g.IC, lpp, in_u8 ? 0 : (int)0x80808080, (int)((in_u8 ? 0 : 128) * g.IC + t.zp_in * g.IC),
                               direct ? wz_rest : 1, g, in_flat ? 1 : 0);
            VPX_HIP_CHECK(hipGetLastError());
            if (!direct) {
                hipLaunchKernelGGL(nce_window_sum_kernel, dim3((unsigned)((Mtot + 255) / 256)), dim3(256), 0, s, cs, rt, g, wz_rest, Mtot);
                VPX_HIP_CHECK(hipGetLastError());
            }
            rowterm = rt;
        }
        wofs = wbytes + (rbytes + 255) / 256 * 256;
        return VPX_RESULT_SUCCESS;
    };
    // Channel counts that are a multiple of 16 but not of 64 (stem layers; 32, 96, 160 ... channels): the row-patch kernel
    // where a band of input rows and the weights fit LDS together, else the gather kernels below.  (Multiples of 32 have a
    // gather kernel that takes any K: they come here while the weights leave most of LDS to the rows -- [32,112,112,32] ->
    // 64 3x3: 27 us against 64 us, [32,14,14,160] -> 320 1x1: 9 against 19.5; 5x5 x 96 channels, 154 KiB of weights: 183 against 47.)
    if (allow_lds && !use_gemm && mfma_ok && aligned && g.IC % 16 == 0 &&
        (g.IC % 32 != 0 || (g.IC % 64 != 0 && (g.OC <= 32 ? 32 : 64) * ((g.KY * g.KX * (g.IC / 16) + 1) / 2 * 32 + 16) <= 100 * 1024)) &&
        g.H * g.ish < (1ll << 31) &&
        g.N * g.OH < (1ll << 30) && g.OC < (1 << 24) && g.KY * g.KX * g.IC < (1 << 16)) {
        RowsGeom rg{};
        const int cpt = (int)g.IC / 16;
        rg.S = (g.KY * g.KX * cpt + 1) / 2;
        rg.WS = rg.S * 32 + 16;
        rg.m = g.SX * cpt;
        // bytes per patch row under CW output columns: m planes of chunks
        auto row_bytes = [&](int64_t CW) { return (((CW - 1) * g.SX + g.KX) * cpt + rg.m - 1) / rg.m * rg.m * 16; };
        // channels per workgroup: 128 where more than 64 are wanted, their weights are short (a quarter of LDS at most) and
        // blocks of 128 leave at most an eighth of the last one empty ([32,28,28,96] -> 576 1x1: 21.6 -> 16.4 us; 192 channels,
        // a third of two blocks empty: 21.7 -> 23.9 us, so those stay with blocks of 64)
        const bool wide = g.OC > 64 && 128 * (size_t)rg.WS <= 40 * 1024 && ((g.OC + 127) / 128 * 128 - g.OC) * 8 <= g.OC;
        const int bn = g.OC <= 32 ? 32 : (wide ? 128 : 64);
        const size_t fixed = bn * (size_t)rg.WS + bn * sizeof(ChanPrep) + 2 * bn * sizeof(int) + 16 + (size_t)(2 * rg.S + 3) / 4 * 16;
        auto need = [&](int64_t R, int64_t CW) { return fixed + (size_t)((R - 1) * g.SY + g.KY) * (size_t)row_bytes(CW); };
        int cus = 0;
        int rc = device_compute_units(&cus);
        if (rc) return rc;
        const int64_t ocb = (g.OC + bn - 1) / bn;
        const int64_t slots = cus / ocb > 0 ? cus / ocb : 1;  // workgroups per block of channels
        // Tile height and positions per wave block: the cheapest of all that fit, counted in MFMA time (32 clocks
        // each) plus the staging of the rows at about 64 bytes per clock; a workgroup's eight waves take a block each.
        const int S = rg.S;
        int best_r = 0, best_tm = 0;
        int64_t best_cw = 0;
        double best = 0;
        // (the whole width, or the width in 2 .. 32 column tiles: the rows under a band of a wide image do not fit LDS)
        for (int tx = 1; tx <= 32 && (tx == 1 || best_tm == 0 || g.OW / tx >= 64); tx++) {
            const int64_t CW = (g.OW + tx - 1) / tx, RB = row_bytes(CW);
            if (tx > 1 && (g.OW + CW - 1) / CW != tx) continue;
            for (int64_t R = 1; R <= g.OH && need(R, CW) <= kMaxDynLds; R++) {
                const int64_t ntiles = g.N * ((g.OH + R - 1) / R) * tx;
                const int64_t per_wg = (ntiles + slots - 1) / slots;
                for (int tm = 2; tm <= (bn == 128 ? 2 : 4); tm += 2) {
                    const int64_t blocks = (R * CW + 32 * tm - 1) / (32 * tm);
                    const double cost = (double)per_wg * ((double)((blocks + 7) / 8) * tm * (bn / 32) * (S * 32.0 + 400) * 2 +
                                                          (double)((R - 1) * g.SY + g.KY) * (double)RB / 64 + 1500);
                    if (best_tm == 0 || cost < best || (cost == best && (int)R == best_r && CW == best_cw)) {  // (a tie between the block sizes of one tile: the larger)
                        best = cost;
                        best_r = (int)R;
                        best_cw = CW;
                        best_tm = tm;
                    }
                }
            }
        }
        if (const int v = knobs.conv_rows.load()) {
            if (best_tm != 0 && v >= 1 && v <= g.OH && need(v, best_cw) <= kMaxDynLds) best_r = v;
        }
        if (const int v = knobs.conv_cols.load()) {
            if (best_tm != 0 && v >= 1 && v <= g.OW && need(best_r, v) <= kMaxDynLds) best_cw = v;
        }
        const int64_t RB = best_tm ? row_bytes(best_cw) : 0;
        if (best_tm != 0 && RB < (1 << 20) && g.N * ((g.OH + best_r - 1) / best_r) * ((g.OW + best_cw - 1) / best_cw) < (1ll << 30)) {
            const int corr = in_u8 ? 128 - t.zp_in : -t.zp_in;
            rc = rebias_weights();
            if (rc) return rc;
            const int tmin = out_signed ? -128 : 0, tmax = out_signed ? 127 : 255;
            int lo = ppe.clamp_lo > tmin ? ppe.clamp_lo : tmin, hi = ppe.clamp_hi < tmax ? ppe.clamp_hi : tmax;
            if (lo > tmax) lo = tmax;
            if (hi < tmin) hi = tmin;
            if (lo > hi) lo = hi;
            auto fd = [](int64_t d) { return FastDiv{(uint32_t)d, (uint32_t)(((1ull << 32) + (uint64_t)d - 1) / (uint64_t)d)}; };
            const int tiles_y = (int)((g.OH + best_r - 1) / best_r), tiles_x = (int)((g.OW + best_cw - 1) / best_cw);
            rg.R = best_r;
            rg.CW = (int)best_cw;
            rg.PH = (best_r - 1) * g.SY + g.KY;
            rg.RB = (int)RB;
            rg.plane = (int)(RB / 16 / rg.m);
            rg.row_chunks = (int)(((best_cw - 1) * g.SX + g.KX) * cpt);
            rg.ntiles = (int)(g.N * tiles_y * tiles_x);
            rg.tiles_y = fd(tiles_y);
            rg.tiles_x = fd(tiles_x);
            rg.cw = fd(best_cw);
            rg.ow = fd(g.OW);
            rg.rc = fd(rg.row_chunks);
            rg.cpp = fd(cpt);
            rg.kc = fd(2 * rg.S);
            rg.fm = fd(rg.m);
            rg.rin = fd(g.KX * cpt);
            const size_t lds = need(best_r, best_cw);
            const int64_t per_wg = (rg.ntiles + slots - 1) / slots;
            const dim3 grid((unsigned)((rg.ntiles + per_wg - 1) / per_wg), (unsigned)ocb);
            GemmPpe gp{ppe.prelu_mult, ppe.prelu_shift, corr, t.zp_out, lo, hi, out_signed ? 1 : 0, rowterm, ppe.f16_lo, ppe.f16_hi, out_f16 ? 1 : 0};
            const int pad_byte = t.zp_in & 0xff;
#define VPX_ROWS_T(U8, TNV, TMV, MULTIV)                                                                              \
    do {                                                                                                              \
        if (out_f16) {                                                                                                \
            auto kern = nce_conv_rows16<U8, TMV, TNV, MULTIV, true>;                                                  \
            rc = set_dyn_lds(kern, lds);                                                                              \
            if (rc) return rc;                                                                                        \
            hipLaunchKernelGGL(kern, grid, dim3(512), lds, s, (const int8_t*)t.input, (const int8_t*)wptr,       \
                               t.weight_table, (uint8_t*)t.output, g, rg, pad_byte, gp);                              \
        } else {                                                                                                      \
            auto kern = nce_conv_rows16<U8, TMV, TNV, MULTIV, false>;                                                 \
            rc = set_dyn_lds(kern, lds);                                                                              \
            if (rc) return rc;                                                                                        \
            hipLaunchKernelGGL(kern, grid, dim3(512), lds, s, (const int8_t*)t.input, (const int8_t*)wptr,       \
                               t.weight_table, (uint8_t*)t.output, g, rg, pad_byte, gp);                              \
        }                                                                                                             \
    } while (0)
#define VPX_ROWS(U8, TNV)                                                                                             \
    do {                                                                                                              \
        if (best_tm == 4 && per_wg > 1) VPX_ROWS_T(U8, TNV, 4, true);                                                \
        else if (best_tm == 4) VPX_ROWS_T(U8, TNV, 4, false);                                                        \
        else if (per_wg > 1) VPX_ROWS_T(U8, TNV, 2, true);                                                           \
        else VPX_ROWS_T(U8, TNV, 2, false);                                                                          \
    } while (0)
            if (bn == 128) {  // (TM = 2 only: eight accumulator tiles a wave)
                if (in_u8 && per_wg > 1) VPX_ROWS_T(true, 4, 2, true);
                else if (in_u8) VPX_ROWS_T(true, 4, 2, false);
                else if (per_wg > 1) VPX_ROWS_T(false, 4, 2, true);
                else VPX_ROWS_T(false, 4, 2, false);
            } else if (in_u8 && bn == 32) VPX_ROWS(true, 1);
            else if (in_u8) VPX_ROWS(true, 2);
            else if (bn == 32) VPX_ROWS(false, 1);
            else VPX_ROWS(false, 2);
#undef VPX_ROWS
#undef VPX_ROWS_T
            VPX_HIP_CHECK(hipGetLastError());
            *kernel_name = "nce_conv_rows16";
            return VPX_RESULT_SUCCESS;
        }
    }

    if (allow_mfma && mfma_ok && aligned && (use_gemm || g.IC % 32 == 0)) {
        int rc = VPX_RESULT_SUCCESS;
        rc = rebias_weights();
        if (rc) return rc;
        const int corr = in_u8 ? 128 - t.zp_in : -t.zp_in;
        PpeFast pf{};
        pf.zp_out = t.zp_out;
        pf.rowterm = rowterm;
        pf.f16_lo = ppe.f16_lo;
        pf.f16_hi = ppe.f16_hi;
        const int tmin = out_signed ? -128 : 0, tmax = out_signed ? 127 : 255;
        pf.lo = ppe.clamp_lo > tmin ? ppe.clamp_lo : tmin;
        pf.hi = ppe.clamp_hi < tmax ? ppe.clamp_hi : tmax;
        if (pf.lo > tmax) pf.lo = tmax;  // clamp window entirely above / below the storage range
        if (pf.hi < tmin) pf.hi = tmin;
        if (pf.lo > pf.hi) pf.lo = pf.hi;  // inverted window: max-then-min always ends at the upper bound

        if (use_gemm) {
            // 256 x 256 tiles (one workgroup per CU) or 128 x 128 (four times as many, two workgroups per CU): whichever
            // leaves less of the chip idle, counting the padding of edge tiles and the empty part of the last round of
            // workgroups; at equal use the large tile is about an eighth faster from K = 256 on (half the operand traffic per
            // MFMA), about equal at K = 128 and slower at K = 64 (all epilogue).  [25088 x 512 x 128] 14.1 -> 7.8 us,
            // [100352 x 256 x 128] 23.8 -> 14.4 us, [512 x 4096 x 4096] 43 -> 24 us with the small tile; [25088 x 256 x 512]
            // 14.3 -> 11.4 us, [12544 x 1024 x 1024] 26.5 -> 21.1 us with the large one.  VPX_GEMM_TILE=128|256 overrides.
            int cus_gemm = 0;
            rc = device_compute_units(&cus_gemm);
            if (rc) return rc;
            const int64_t t256 = gemm_tiles * G, t128 = ((Mtot + 127) / 128) * ((g.OC + 127) / 128) * G;
            const double work = (double)Mtot * (double)g.OC * (double)G;
            const double use256 = work / ((double)((t256 + cus_gemm - 1) / cus_gemm) * cus_gemm * 65536.0);
            const double use128 = work / ((double)((t128 + 2 * cus_gemm - 1) / (2 * cus_gemm)) * 2 * cus_gemm * 16384.0);
            // (fp16 outputs: the large tile's epilogue leaves in two passes and costs more than its main loop saves up to
            // K = 1024 -- [32768 x 512 x 512] 26.6 us small, 30.4 us large; [32768 x 2048 x 512] 58.4 and 54.8)
            const bool large = out_f16 ? (g.IC >= 2048 && use256 * 1.06 > use128)
                               : g.IC >= 256 ? use256 * 1.12 > use128
                                             : (g.IC >= 128 && t256 * 10 >= cus_gemm * 7 && t256 <= cus_gemm && use256 * 1.03 > use128);
            const int tile_knob = knobs.gemm_tile.load();
            const int tile = tile_knob ? tile_knob : (large ? 256 : 128);
            const int tiles_m = (int)((Mtot + tile - 1) / tile), tiles_n = (int)((g.OC + tile - 1) / tile);
            const int per_xcd = (tiles_m * tiles_n + 7) / 8;
            // Eight waves (two per SIMD: one wave's reads and loads issue under the other's MFMAs) win at every K
            // (8192^3: 466 us against 483 us with four waves of 128 x 128).  VPX_GEMM_WAVES=4|8 overrides.
            const int waves_knob = knobs.gemm_waves.load();
            // (an fp16 output exists in the eight-wave form of the large tile only: the knob does not apply to it)
            const int nw = tile == 128 ? 4 : (out_f16 ? 8 : (waves_knob ? waves_knob : 8));
            const dim3 grid((unsigned)(per_xcd * 8), (unsigned)G), block(64 * nw);
            const int64_t nk = g.IC / 64;
            const bool shortk = tile == 128 && nk <= 3 && !out_f16;
            size_t lds = 4 * (size_t)(tile + tile) * 64;  // four K panels; the output staging tile reuses them
            if (shortk) {
                lds = (size_t)nk * (tile + tile) * 64;  // only the panels there are ...
                if (lds < (size_t)tile * kOutStride) lds = (size_t)tile * kOutStride;  // ... or the staging tile
            }
            lds += kGemmLdsHead;
            GemmPpe gp{ppe.prelu_mult, ppe.prelu_shift, corr, pf.zp_out, pf.lo, pf.hi, out_signed ? 1 : 0, rowterm, ppe.f16_lo, ppe.f16_hi};
            const int32_t* colsum = nullptr;  // the kernel sums the columns of B itself, from the fragments it reads
            const GemmRows rows{picks_rows ? 1 : 0, vin.sw, (int)g.OW, (int)(g.OH * g.OW), (unsigned)(g.SX * vin.sw), (unsigned)(g.SY * vin.sh),
                                (unsigned)vin.sn};
            const GemmOut dst{vout.flat == 2 ? 1 : 0, vout.sn, vout.sh, vout.sw, (int)g.OW, (int)(g.OH * g.OW), g.out_bits};
#define VPX_GEMM_W(U8, SGN, NW, TILE, SHORTK)                                                                        \
    do {                                                                                                             \
        auto kern = nce_gemm_mfma<U8, SGN, NW, TILE, SHORTK>;                                                        \
        rc = set_dyn_lds(kern, lds);                                                                                 \
        if (rc) return rc;                                                                                           \
        hipLaunchKernelGGL(kern, grid, block, lds, s, (const int8_t*)t.input, (const int8_t*)wptr,              \
                           t.weight_table, colsum, (uint8_t*)t.output, Mtot, g.OC, g.IC, tiles_m, tiles_n, gp, rows, dst); \
    } while (0)
#define VPX_GEMM(U8, SGN)                                                                                            \
    do {                                                                                                             \
        if (shortk) VPX_GEMM_W(U8, SGN, 4, 128, true);                                                               \
        else if (tile == 128) VPX_GEMM_W(U8, SGN, 4, 128, false);                                                    \
        else if (nw == 4) VPX_GEMM_W(U8, SGN, 4, 256, false);                                                        \
        else VPX_GEMM_W(U8, SGN, 8, 256, false);                                                                     \
    } while (0)
            if (out_f16) {
                // fp16 output: the eight-wave 256-tile and the four-wave 128-tile forms only
                if (in_u8) { if (tile == 128) VPX_GEMM_W(true, OUT_F16, 4, 128, false); else VPX_GEMM_W(true, OUT_F16, 8, 256, false); }
                else { if (tile == 128) VPX_GEMM_W(false, OUT_F16, 4, 128, false); else VPX_GEMM_W(false, OUT_F16, 8, 256, false); }
            }
            else if (in_u8 && out_signed) VPX_GEMM(true, OUT_I8);
            else if (in_u8) VPX_GEMM(true, OUT_U8);
            else if (out_signed) VPX_GEMM(false, OUT_I8);
            else VPX_GEMM(false, OUT_U8);
#undef VPX_GEMM
#undef VPX_GEMM_W
            VPX_HIP_CHECK(hipGetLastError());
            *kernel_name = "nce_gemm_mfma";
            return VPX_RESULT_SUCCESS;
        }

        // Preferred: input patch in LDS, one launch.  R = output rows per workgroup.
        // (an fp16 output takes the gather kernel below: the tile kernels' epilogues stage bytes)
        if (allow_lds && g.IC % 64 == 0 && g.OW <= 32 * kPatchMaxMT && g.N * g.OH < (1ll << 30) && Ktot < (1 << 20) &&
            g.IC < (1 << 14) && g.W * g.SX < (1 << 14) && g.N * g.OH * g.OW < (1ll << 31)) {
            // IC of 64 or 128: the one-tile-per-workgroup kernel with padded LDS rows (a tap's fragments of more
            // channels do not fit the registers twice)
            // VPX_CONV_KERNEL=stream starts the choice below the tile kernel (tests compare them)
            const int first = knobs.conv_stream.load();
            int cus_here = 0;
            rc = device_compute_units(&cus_here);
            if (rc) return rc;
            // (with 128 channels and a stride the haloed patch crowds the resident weights out of LDS: the
            // streamed-weights kernel below measures 15.7 us against 20.2 at [32,56,56,128] -> 128, 3x3, stride 2)
            // 3x3 taps of 64 channels: the weights fit the registers of every wave.  Copying them there costs about a
            // microsecond per workgroup, which pays from about 50 000 output positions on ([32,56,56,64] -> 64: 9.1 us
            // against 9.5 us; [4,224,224,64] -> 64: 13.9 against 29.2; [32,28,28,64] -> 64: 7.0 against 6.0; the same input
            // at stride 2: 7.5 against 7.1).
            const size_t out_stride = out_f16 ? kPatchOutStrideF16 : kPatchOutStride;  // staging bytes per position
            // (the weights-in-registers kernel stores bytes straight from its registers: integer outputs only)
            if (!out_f16 && g.IC == 64 && g.KY == 3 && g.KX == 3 && g.H * g.ish < (1ll << 31) &&
                (first < 0 || (first == 0 && g.N * g.OH * g.OW >= 50000))) {
                PatchGeom pg{};
                const int64_t PS = g.IC + 16, WS = Ktot + 16;
                auto need = [&](int R) {
                    return 64 * (size_t)WS + (size_t)((R - 1) * g.SY + g.KY) * (size_t)((g.OW - 1) * g.SX + g.KX) * (size_t)PS;
                };
                int cus = 0;
                rc = device_compute_units(&cus);
                if (rc) return rc;
                const int64_t ocb = (g.OC + 63) / 64;
                // one workgroup per compute unit where the layer allows: rows per tile from the rows there are
                int R = (int)((g.N * g.OH * ocb + cus - 1) / cus);
                const int rmin = (int)((128 + g.OW - 1) / g.OW);  // eight waves want eight blocks of 16 positions
                if (R < rmin) R = rmin;
                if (R > g.OH) R = (int)g.OH;
                while (R > 1 && need(R) > kMaxDynLds) R--;
                if (const int v = knobs.conv_rows.load()) {
                    if (v >= 1 && v <= R) R = v;
                }
                if (need(R) <= kMaxDynLds) {
                    const int tiles_y = (int)((g.OH + R - 1) / R);
                    auto fd = [](int64_t d) { return FastDiv{(uint32_t)d, (uint32_t)(((1ull << 32) + (uint64_t)d - 1) / (uint64_t)d)}; };
                    pg.R = (int)((g.OH + tiles_y - 1) / tiles_y);
                    pg.PH = (pg.R - 1) * g.SY + g.KY;
                    pg.PW = (int)(g.OW - 1) * g.SX + g.KX;
                    pg.MT = (int)((pg.R * g.OW + 31) / 32);
                    pg.nt = 2;
                    pg.ntiles = (int)(g.N * tiles_y);
                    pg.tiles_y = fd(tiles_y);
                    pg.cpr = fd(Ktot / 16);
                    pg.cpp = fd(g.IC / 16);
                    pg.upr = fd((pg.PW * (g.IC / 16) + 63) / 64);
                    pg.ow = fd(g.OW);
                    const size_t lds = need(pg.R);
                    const dim3 grid((unsigned)(g.N * tiles_y), (unsigned)ocb);
                    GemmPpe gp{ppe.prelu_mult, ppe.prelu_shift, corr, pf.zp_out, pf.lo, pf.hi, out_signed ? 1 : 0, rowterm, ppe.f16_lo, ppe.f16_hi, out_f16 ? 1 : 0};
                    const int pad_byte = t.zp_in & 0xff;
                    const bool same_f = ppe.prelu_mult == 1 && ppe.prelu_shift == 0;
#define VPX_REGW(U8, SAME)                                                                                            \
    do {                                                                                                              \
        auto kern = nce_conv_regw<U8, SAME, 3, 3>;                                                                    \
        rc = set_dyn_lds(kern, lds);                                                                                  \
        if (rc) return rc;                                                                                            \
        hipLaunchKernelGGL(kern, grid, dim3(512), lds, s, (const int8_t*)t.input, (const int8_t*)wptr, t.weight_table, \
                           (uint8_t*)t.output, g, pg, pad_byte, gp);                                                  \
    } while (0)
                    if (in_u8 && same_f) VPX_REGW(true, true);
                    else if (in_u8) VPX_REGW(true, false);
                    else if (same_f) VPX_REGW(false, true);
                    else VPX_REGW(false, false);
#undef VPX_REGW
                    VPX_HIP_CHECK(hipGetLastError());
                    *kernel_name = "nce_conv_regw";
                    return VPX_RESULT_SUCCESS;
                }
            }
            if ((g.IC == 64 || (g.IC == 128 && g.SY * g.SX == 1)) && first <= 1) {
                PatchGeom pg{};
                const int64_t PS = g.IC + 16, WS = Ktot + 16;
                auto need = [&](int R) {
                    const size_t patch = (size_t)((R - 1) * g.SY + g.KY) * (size_t)((g.OW - 1) * g.SX + g.KX) * (size_t)PS;
                    const size_t stage = (size_t)((R * g.OW + 31) / 32) * 32 * out_stride;
                    return 64 * (size_t)WS + (patch > stage ? patch : stage);
                };
                int R = (int)(32 * kPatchMaxMT / g.OW);
                if (R > g.OH) R = (int)g.OH;
                while (R > 1 && need(R) > 160 * 1024 - 512) R--;
                if (need(R) <= 160 * 1024 - 512) {
                    const int64_t ocb = (g.OC + 63) / 64;
                    // shorter tiles while they are few: down to 128 positions, or to 64 while there are fewer tiles
                    // than compute units ([32,14,14,256] -> 256, 3x3: 12.1 us with 256 tiles of 7 rows, 15.4 us with 128 of 14)
                    while (R > 1) {
                        const int64_t tiles = g.N * ((g.OH + R - 1) / R) * ocb;
                        if (tiles >= 512 || ((R + 1) / 2) * g.OW < (tiles < cus_here ? 64 : 128)) break;
                        R = (R + 1) / 2;
                    }
                    if (const int v = knobs.conv_rows.load()) {
                        if (v >= 1 && v <= R) R = v;
                    }
                    const int tiles_y = (int)((g.OH + R - 1) / R);
                    auto fd = [](int64_t d) { return FastDiv{(uint32_t)d, (uint32_t)(((1ull << 32) + (uint64_t)d - 1) / (uint64_t)d)}; };
                    pg.R = (int)((g.OH + tiles_y - 1) / tiles_y);
                    pg.PH = (pg.R - 1) * g.SY + g.KY;
                    pg.PW = (int)(g.OW - 1) * g.SX + g.KX;
                    pg.MT = (int)((pg.R * g.OW + 31) / 32);
                    pg.nt = g.OC <= 32 ? 1 : 2;
                    pg.ntiles = (int)(g.N * tiles_y);
                    pg.tiles_y = fd(tiles_y);
                    pg.cpr = fd(Ktot / 16);
                    pg.cpp = fd(g.IC / 16);
                    pg.upr = fd((pg.PW * (g.IC / 16) + 63) / 64);
                    pg.ow = fd(g.OW);
                    const size_t lds = need(pg.R);
                    const dim3 grid((unsigned)(g.N * tiles_y), (unsigned)ocb);
                    GemmPpe gp{ppe.prelu_mult, ppe.prelu_shift, corr, pf.zp_out, pf.lo, pf.hi, out_signed ? 1 : 0, rowterm, ppe.f16_lo, ppe.f16_hi, out_f16 ? 1 : 0};
                    const int pad_byte = t.zp_in & 0xff;
                    const bool same_f = ppe.prelu_mult == 1 && ppe.prelu_shift == 0;
                    const int nw = knobs.conv_waves.load() == 4 ? 4 : 8;
                    const int per_wave = (pg.MT + nw / pg.nt - 1) / (nw / pg.nt);
                    const int ics = (int)(g.IC / 64);
#define VPX_TILE_W(U8, TMW, SAME, ICS, NW)                                                                            \
    do {                                                                                                              \
        auto kern = nce_conv_tile<U8, TMW, SAME, ICS, NW>;                                                            \
        rc = set_dyn_lds(kern, lds);                                                                                  \
        if (rc) return rc;                                                                                            \
        hipLaunchKernelGGL(kern, grid, dim3(64 * NW), lds, s, (const int8_t*)t.input, (const int8_t*)wptr,       \
                           t.weight_table, (uint8_t*)t.output, g, pg, pad_byte, gp);                                  \
    } while (0)
#define VPX_TILE(U8, TMW, SAME, ICS)                                                                                  \
    do {                                                                                                              \
        if (nw == 8 && TMW <= 4) VPX_TILE_W(U8, (TMW <= 4 ? TMW : 4), SAME, ICS, 8);                                  \
        else VPX_TILE_W(U8, TMW, SAME, ICS, 4);                                                                       \
    } while (0)
#define VPX_TILE_I(U8, TMW, SAME)                                                                                     \
    do {                                                                                                              \
        if (ics == 1) VPX_TILE(U8, TMW, SAME, 1);                                                                     \
        else VPX_TILE(U8, TMW, SAME, 2);                                                                              \
    } while (0)
#define VPX_TILE_T(TMW)                                                                                               \
    do {                                                                                                              \
        if (in_u8 && same_f) VPX_TILE_I(true, TMW, true);                                                             \
        else if (in_u8) VPX_TILE_I(true, TMW, false);                                                                 \
        else if (same_f) VPX_TILE_I(false, TMW, true);                                                                \
        else VPX_TILE_I(false, TMW, false);                                                                           \
    } while (0)
                    if (per_wave <= 2) VPX_TILE_T(2);
                    else if (per_wave <= 4) VPX_TILE_T(4);
                    else VPX_TILE_T(7);
#undef VPX_TILE_T
#undef VPX_TILE_I
#undef VPX_TILE
#undef VPX_TILE_W
                    VPX_HIP_CHECK(hipGetLastError());
                    *kernel_name = "nce_conv_tile";
                    return VPX_RESULT_SUCCESS;
                }
            }
            // any IC that is a multiple of 64: resident patch, weights streamed a slice at a time
            if (first <= 2) {
                PatchGeom pg{};
                StreamGeom sg{};
                sg.ksl = g.IC % 256 == 0 ? 256 : (g.IC % 128 == 0 ? 128 : 64);
                sg.spt = (int)(g.IC / sg.ksl);
                const int64_t PS = g.IC + 16;
                auto need = [&](int R) {
                    const size_t patch = (size_t)((R - 1) * g.SY + g.KY) * (size_t)((g.OW - 1) * g.SX + g.KX) * (size_t)PS;
                    const size_t stage = (size_t)((R * g.OW + 31) / 32) * 32 * out_stride;
                    return 2 * 64 * (size_t)(sg.ksl + 16) + (patch > stage ? patch : stage);
                };
                int R = (int)(32 * kPatchMaxMT / g.OW);
                if (R > g.OH) R = (int)g.OH;
                while (R > 1 && need(R) > 160 * 1024 - 512) R--;
                if (need(R) <= 160 * 1024 - 512) {
                    const int64_t ocb = (g.OC + 63) / 64;
                    // shorter tiles while they are few: down to 128 positions, or to 64 while there are fewer tiles
                    // than compute units ([32,14,14,256] -> 256, 3x3: 12.1 us with 256 tiles of 7 rows, 15.4 us with 128 of 14)
                    while (R > 1) {
                        const int64_t tiles = g.N * ((g.OH + R - 1) / R) * ocb;
                        if (tiles >= 512 || ((R + 1) / 2) * g.OW < (tiles < cus_here ? 64 : 128)) break;
                        R = (R + 1) / 2;
                    }
                    if (const int v = knobs.conv_rows.load()) {
                        if (v >= 1 && v <= R) R = v;
                    }
                    const int tiles_y = (int)((g.OH + R - 1) / R);
                    auto fd = [](int64_t d) { return FastDiv{(uint32_t)d, (uint32_t)(((1ull << 32) + (uint64_t)d - 1) / (uint64_t)d)}; };
                    pg.R = (int)((g.OH + tiles_y - 1) / tiles_y);
                    pg.PH = (pg.R - 1) * g.SY + g.KY;
                    pg.PW = (int)(g.OW - 1) * g.SX + g.KX;
                    pg.MT = (int)((pg.R * g.OW + 31) / 32);
                    pg.nt = g.OC <= 32 ? 1 : 2;
                    pg.ntiles = (int)(g.N * tiles_y);
                    pg.tiles_y = fd(tiles_y);
                    pg.cpr = fd(Ktot / 16);
                    pg.cpp = fd(g.IC / 16);
                    pg.upr = fd((pg.PW * (g.IC / 16) + 63) / 64);
                    pg.ow = fd(g.OW);
                    // tiles of at most 64 positions per four waves: K split over the waves of a group (slices of four or
                    // eight K steps, both channel tiles in use)
                    // (one tile of 64 positions: eight waves, eight shares of K, where a slice has eight K steps)
                    const int ksplit_waves = knobs.stream_ksplit.load() && pg.nt == 2 && sg.ksl >= 128 ? (pg.MT <= 2 ? (sg.ksl == 256 ? 88 : 4) : (pg.MT <= 4 ? 8 : 0)) : 0;
                    size_t lds = need(pg.R);
                    if (lds < (size_t)(ksplit_waves % 80) * 16384) lds = (size_t)(ksplit_waves % 80) * 16384;  // the partial sums
                    const dim3 grid((unsigned)(g.N * tiles_y), (unsigned)ocb);
                    GemmPpe gp{ppe.prelu_mult, ppe.prelu_shift, corr, pf.zp_out, pf.lo, pf.hi, out_signed ? 1 : 0, rowterm, ppe.f16_lo, ppe.f16_hi, out_f16 ? 1 : 0};
                    const int pad_byte = t.zp_in & 0xff;
                    const bool same_f = ppe.prelu_mult == 1 && ppe.prelu_shift == 0;
                    int32_t* colsum = nullptr;
                    if (corr != 0) {
                        void* ws = nullptr;
                        rc = scratch(sizeof(int32_t) * (size_t)g.OC, &ws);
                        if (rc) return rc;
                        colsum = (int32_t*)ws;
                        hipLaunchKernelGGL(nce_colsum_kernel, dim3((unsigned)((g.OC + 3) / 4)), dim3(256), 0, s,
                                           (const int8_t*)wptr, colsum, g.OC, Ktot);
                        VPX_HIP_CHECK(hipGetLastError());
                    }
                    const int per_wave = (pg.MT + 8 / pg.nt - 1) / (8 / pg.nt);  // eight waves: at most 4 row blocks each
#define VPX_STREAM_W(U8, TMW, SAME, NW, KS)                                                                           \
    do {                                                                                                              \
        auto kern = nce_conv_stream<U8, TMW, SAME, NW, KS>;                                                           \
        rc = set_dyn_lds(kern, lds);                                                                                  \
        if (rc) return rc;                                                                                            \
        hipLaunchKernelGGL(kern, grid, dim3(64 * NW), lds, s, (const int8_t*)t.input, (const int8_t*)wptr,       \
                           t.weight_table, colsum, (uint8_t*)t.output, g, pg, sg, pad_byte, gp);                      \
    } while (0)
#define VPX_STREAM(TMW, NW, KS)                                                                                       \
    do {                                                                                                              \
        if (in_u8 && same_f) VPX_STREAM_W(true, TMW, true, NW, KS);                                                   \
        else if (in_u8) VPX_STREAM_W(true, TMW, false, NW, KS);                                                       \
        else if (same_f) VPX_STREAM_W(false, TMW, true, NW, KS);                                                      \
        else VPX_STREAM_W(false, TMW, false, NW, KS);                                                                 \
    } while (0)
                    // (a tile of one or two row blocks -- 7 x 7 planes -- would leave six of eight waves multiplying
                    // padding: four waves, one block each, a third of the LDS reads per weight slice)
                    if (ksplit_waves == 4) VPX_STREAM(1, 4, 4);
                    else if (ksplit_waves == 8) VPX_STREAM(1, 8, 4);
                    else if (ksplit_waves == 88) VPX_STREAM(1, 8, 8);
                    else if (pg.MT <= 4 / pg.nt) VPX_STREAM(1, 4, 0);
                    else if (per_wave <= 1) VPX_STREAM(1, 8, 0);
                    else if (per_wave <= 2) VPX_STREAM(2, 8, 0);
                    else VPX_STREAM(4, 8, 0);
#undef VPX_STREAM
#undef VPX_STREAM_W
                    VPX_HIP_CHECK(hipGetLastError());
                    *kernel_name = "nce_conv_stream";
                    return VPX_RESULT_SUCCESS;
                }
            }
        }
        // Fallback: activation fragments gathered from global memory; per-channel parameters come
        // from a small preparation kernel.
        void* ws = nullptr;
        rc = scratch(sizeof(ChanPrep) * (size_t)g.OC, &ws);
        if (rc) return rc;
        ChanPrep* prep = (ChanPrep*)ws;
        hipLaunchKernelGGL(nce_fold_kernel, dim3((unsigned)((g.OC + 3) / 4)), dim3(256), 0, s, (const int8_t*)wptr,
                           t.weight_table, prep, g.OC, Ktot, corr, ppe, out_f16 ? 15 : 0);
        VPX_HIP_CHECK(hipGetLastError());

        constexpr int BM = 256, BN = 64;
        // weight slice per staging round: whole taps while 64 rows of them fit 64 KiB, else 1024 channels of one tap
        const int icc = g.IC <= 1024 ? (int)g.IC : 1024;
        int tc = g.IC <= 1024 ? (int)(1024 / g.IC) : 1;
        if (tc > g.KY * g.KX) tc = g.KY * g.KX;
        const size_t lds = (size_t)BN * tc * icc;
        const dim3 grid((unsigned)((Mtot + BM - 1) / BM), (unsigned)((g.OC + BN - 1) / BN));
        const int pad_byte = t.zp_in & 0xff;
        const int swz = icc % 64 == 0 ? 1 : 0;
#define VPX_CONV(U8, SGN)                                                                                            \
    do {                                                                                                             \
        auto kern = nce_conv_mfma<BM, BN, U8, SGN>;                                                                  \
        rc = set_dyn_lds(kern, lds);                                                                                 \
        if (rc) return rc;                                                                                           \
        hipLaunchKernelGGL(kern, grid, dim3(256), lds, s, (const int8_t*)t.input, (const int8_t*)wptr, prep,    \
                           (uint8_t*)t.output, g, pad_byte, swz, tc, icc, pf);                                       \
    } while (0)
        if (out_f16 && in_u8) VPX_CONV(true, OUT_F16);
        else if (out_f16) VPX_CONV(false, OUT_F16);
        else if (in_u8 && out_signed) VPX_CONV(true, OUT_I8);
        else if (in_u8) VPX_CONV(true, OUT_U8);
        else if (out_signed) VPX_CONV(false, OUT_I8);
        else VPX_CONV(false, OUT_U8);
#undef VPX_CONV
        VPX_HIP_CHECK(hipGetLastError());
        *kernel_name = "nce_conv_mfma";
        return VPX_RESULT_SUCCESS;
    }

    if (allow_mfma && mfma_ok && aligned && g.IC % 16 == 0 && g.IC % 32 != 0 && ((Ktot + 31) / 32 * 32 + 16) * 64 <= 64 * 1024) {
        const int corr = in_u8 ? 128 - t.zp_in : -t.zp_in;
        PpeFast pf{};
        pf.zp_out = t.zp_out;
        pf.f16_lo = ppe.f16_lo;
        pf.f16_hi = ppe.f16_hi;
        const int tmin = out_signed ? -128 : 0, tmax = out_signed ? 127 : 255;
        pf.lo = ppe.clamp_lo > tmin ? ppe.clamp_lo : tmin;
        pf.hi = ppe.clamp_hi < tmax ? ppe.clamp_hi : tmax;
        if (pf.lo > tmax) pf.lo = tmax;
        if (pf.hi < tmin) pf.hi = tmin;
        if (pf.lo > pf.hi) pf.lo = pf.hi;
        int rc = rebias_weights();
        if (rc) return rc;
        pf.rowterm = rowterm;
        void* ws = nullptr;
        rc = scratch(sizeof(ChanPrep) * (size_t)g.OC, &ws);
        if (rc) return rc;
        ChanPrep* prep = (ChanPrep*)ws;
        hipLaunchKernelGGL(nce_fold_kernel, dim3((unsigned)((g.OC + 3) / 4)), dim3(256), 0, s, (const int8_t*)wptr,
                           t.weight_table, prep, g.OC, Ktot, corr, ppe, out_f16 ? 15 : 0);
        VPX_HIP_CHECK(hipGetLastError());
        const size_t lds = (size_t)64 * ((Ktot + 31) / 32 * 32 + 16);
        const dim3 grid((unsigned)((Mtot + 255) / 256), (unsigned)((g.OC + 63) / 64));
        const int pad_byte = t.zp_in & 0xff;
#define VPX_CONV16(U8, OUT)                                                                                           \
    hipLaunchKernelGGL((nce_conv_mfma16<U8, OUT>), grid, dim3(256), lds, s, (const int8_t*)t.input, (const int8_t*)wptr, prep, \
                       (uint8_t*)t.output, g, pad_byte, pf)
        if (in_u8 && out_f16) VPX_CONV16(true, OUT_F16);
        else if (in_u8) VPX_CONV16(true, OUT_U8);
        else if (out_f16) VPX_CONV16(false, OUT_F16);
        else VPX_CONV16(false, OUT_U8);
#undef VPX_CONV16
        VPX_HIP_CHECK(hipGetLastError());
        *kernel_name = "nce_conv_mfma16";
        return VPX_RESULT_SUCCESS;
    }

    const int64_t total = Mtot * g.OC;
    VPX_REQUIRE((total + 255) / 256 < (1ll << 31), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "NCE task: output of %lld elements exceeds the launch limit",
                (long long)total);
    const dim3 grid((unsigned)((total + 255) / 256));
#define VPX_NAIVE(IS, WS, OS)                                                                                        \
    hipLaunchKernelGGL((nce_conv_naive<IS, WS, OS>), grid, dim3(256), 0, s, (const uint8_t*)t.input,                 \
                       (const uint8_t*)t.weights, t.weight_table, (uint8_t*)t.output, g, t.zp_in, t.zp_w, ppe, total)
    const int sel = (in_u8 ? 0 : 4) | (w_u8 ? 0 : 2) | (out_signed ? 1 : 0);
    if (out_f16) {
        switch (sel >> 1) {
        case 0: VPX_NAIVE(false, false, OUT_F16); break;
        case 1: VPX_NAIVE(false, true, OUT_F16); break;
        case 2: VPX_NAIVE(true, false, OUT_F16); break;
        default: VPX_NAIVE(true, true, OUT_F16); break;
        }
    } else switch (sel) {
    case 0: VPX_NAIVE(false, false, OUT_U8); break;
    case 1: VPX_NAIVE(false, false, OUT_I8); break;
    case 2: VPX_NAIVE(false, true, OUT_U8); break;
    case 3: VPX_NAIVE(false, true, OUT_I8); break;
    case 4: VPX_NAIVE(true, false, OUT_U8); break;
    case 5: VPX_NAIVE(true, false, OUT_I8); break;
    case 6: VPX_NAIVE(true, true, OUT_U8); break;
    default: VPX_NAIVE(true, true, OUT_I8); break;
    }
#undef VPX_NAIVE
    VPX_HIP_CHECK(hipGetLastError());
    *kernel_name = "nce_conv_naive";
    return VPX_RESULT_SUCCESS;
}

}  // namespace vpx
