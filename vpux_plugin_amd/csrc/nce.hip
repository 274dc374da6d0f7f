// NCE cluster task on CDNA4: 8-bit convolution / matmul with int32 accumulation on the i8 MFMA
// units and the integer PPE fused into the epilogue.
//
// Device paths (chosen by vpx_nce_task):
//   nce_gemm_mfma  : 1x1 kernel, stride 1, no padding (this is how NCE.MatMul arrives): a plain
//                    A[M][K] x B[N][K]^T GEMM.  256x256 output tile per workgroup, K staged through
//                    double-buffered, XOR-swizzled LDS, v_mfma_i32_32x32x32_i8, 128x128 per wave.
//   nce_conv_mfma  : general KYxKX / stride / padding with IC a multiple of 32: implicit GEMM, the
//                    activation fragments are gathered from the NHWC tensor (no im2col buffer),
//                    the weights of the tile sit in LDS.
//   nce_conv_naive : any shape and any zero points, one output per lane.
//
// Zero points: the MFMA paths multiply raw bytes (u8 activations are re-biased to s8 by flipping
// the top bit) and add the missing term to the bias: acc_true = acc_raw + k * sum_k w[oc][k] with
// k = 128 - zp_in (u8) or -zp_in (i8); padded taps are filled with the byte that stands for the
// zero point so they contribute exactly 0, as the MPE does (runtime_dpu_parser_imports.cpp.inc:872-879).
#include <cstdlib>
#include <cstring>

#include "vpx_common.h"

namespace vpx {

int launch_nce(const vpx_nce_task_t& t, hipStream_t s, const char** kernel_name);

namespace {

typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
typedef int32_t i32x16 __attribute__((ext_vector_type(16)));

struct Ppe {
    int prelu_mult, prelu_shift, zp_out, clamp_lo, clamp_hi;
};

// Per output channel, unpacked from weight-table words 2 and 3 with the zero-point term folded in.
struct ChanParams {
    int bias, mult, shift, pad;
};

// Integer PPE in the order the compiler programs it (expand_dpu_config_invariant_ppe.cpp:322-380):
// bias add, scale multiply, [prelu multiply on negatives], one round-half-even over the combined
// right shift, zero point, clamp.
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

template <bool OUT_SIGNED>
__device__ __forceinline__ uint8_t saturate8(int r) {
    if (OUT_SIGNED) return (uint8_t)(int8_t)(r < -128 ? -128 : (r > 127 ? 127 : r));
    return (uint8_t)(r < 0 ? 0 : (r > 255 ? 255 : r));
}

// ---------------------------------------------------------------- per-channel parameter fold
// params[oc] = {bias + corr * sum_k w[oc][k], mult, shift}; one wavefront per output channel.
__global__ __launch_bounds__(256) void nce_fold_kernel(const int8_t* __restrict__ w, const int32_t* __restrict__ wt,
                                                       ChanParams* __restrict__ params, int64_t OC, int64_t K, int corr) {
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
        ChanParams c;
        c.bias = (int)((unsigned)wt[oc * 4 + 3] + (unsigned)(corr * sum));
        c.mult = (int)(int16_t)(w2 >> 16);
        c.shift = (int)((w2 >> 8) & 0xffu);
        c.pad = 0;
        params[oc] = c;
    }
}

// ---------------------------------------------------------------- naive path
struct ConvGeom {
    int64_t N, H, W, IC, OC, OH, OW;
    int KY, KX, SY, SX, PT, PL;
};

template <bool IN_SIGNED, bool W_SIGNED, bool OUT_SIGNED>
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
            const uint8_t* pi = in + ((n * g.H + iy) * g.W + ix) * g.IC;
            const uint8_t* pw = w + ((oc * g.KY + ky) * g.KX + kx) * g.IC;
            for (int64_t ic = 0; ic < g.IC; ic++) {
                const int a = IN_SIGNED ? (int)(int8_t)pi[ic] : (int)pi[ic];
                const int b = W_SIGNED ? (int)(int8_t)pw[ic] : (int)pw[ic];
                acc += (a - zp_in) * (b - zp_w);
            }
        }
    }
    const uint32_t w2 = (uint32_t)wt[oc * 4 + 2];
    ChanParams c{wt[oc * 4 + 3], (int)(int16_t)(w2 >> 16), (int)((w2 >> 8) & 0xffu), 0};
    out[idx] = saturate8<OUT_SIGNED>(ppe_requant(acc, c, ppe));
}

// ---------------------------------------------------------------- GEMM path
// LDS tile of ROWS x BK bytes; the 16-byte chunk c of row r is kept at chunk slot c ^ swz(r) so
// that the 16 lanes served together by a 128-bit LDS read hit 16 different bank groups.
template <int BK>
__device__ __forceinline__ int lds_offset(int row, int chunk) {
    constexpr int CPR = BK / 16;        // chunks per row
    constexpr int RPW = 16 / CPR;       // rows per 256-byte bank wrap
    return row * BK + ((chunk ^ ((row / RPW) % CPR)) << 4);
}

template <int BM, int BN, int BK, int WM, int WN, bool IN_U8, bool OUT_SIGNED>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * 64) void nce_gemm_mfma(
        const int8_t* __restrict__ A, const int8_t* __restrict__ B, const ChanParams* __restrict__ params,
        uint8_t* __restrict__ out, int64_t M, int64_t N, int64_t K, int tiles_m, int tiles_n, Ppe ppe) {
    constexpr int NT = (BM / WM) * (BN / WN) * 64;
    constexpr int CPR = BK / 16;
    constexpr int A_CHUNKS = BM * CPR / NT;  // 16-byte chunks per lane per K step
    constexpr int B_CHUNKS = BN * CPR / NT;
    constexpr int TM = WM / 32, TN = WN / 32;
    static_assert(BM * CPR % NT == 0 && BN * CPR % NT == 0, "tile does not split evenly over the lanes");

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* sA = smem;                  // [2][BM][BK]
    uint8_t* sB = smem + 2 * BM * BK;    // [2][BN][BK]

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

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm0 = (wave / (BN / WN)) * WM, wn0 = (wave % (BN / WN)) * WN;

    const int8_t* ga[A_CHUNKS];
    const int8_t* gb[B_CHUNKS];
    int la[A_CHUNKS], lb[B_CHUNKS];
#pragma unroll
    for (int i = 0; i < A_CHUNKS; i++) {
        const int cid = tid + NT * i, row = cid / CPR, c = cid % CPR;
        int64_t m = m0 + row;
        m = m < M ? m : M - 1;  // rows past the edge repeat the last one; their outputs are not stored
        ga[i] = A + m * K + c * 16;
        la[i] = lds_offset<BK>(row, c);
    }
#pragma unroll
    for (int i = 0; i < B_CHUNKS; i++) {
        const int cid = tid + NT * i, row = cid / CPR, c = cid % CPR;
        int64_t n = n0 + row;
        n = n < N ? n : N - 1;
        gb[i] = B + n * K + c * 16;
        lb[i] = lds_offset<BK>(row, c);
    }

    i32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

    i32x4 ra[A_CHUNKS], rb[B_CHUNKS];
    auto load_global = [&](int64_t k0) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; i++) {
            ra[i] = *reinterpret_cast<const i32x4*>(ga[i] + k0);
            if (IN_U8) ra[i] ^= (int32_t)0x80808080;
        }
#pragma unroll
        for (int i = 0; i < B_CHUNKS; i++) rb[i] = *reinterpret_cast<const i32x4*>(gb[i] + k0);
    };
    auto store_lds = [&](int buf) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; i++) *reinterpret_cast<i32x4*>(sA + buf * BM * BK + la[i]) = ra[i];
#pragma unroll
        for (int i = 0; i < B_CHUNKS; i++) *reinterpret_cast<i32x4*>(sB + buf * BN * BK + lb[i]) = rb[i];
    };

    const int nk = (int)(K / BK);
    load_global(0);
    store_lds(0);
    __syncthreads();
    for (int kt = 0; kt < nk; kt++) {
        const int buf = kt & 1;
        if (kt + 1 < nk) load_global((int64_t)(kt + 1) * BK);
        const uint8_t* pa = sA + buf * BM * BK;
        const uint8_t* pb = sB + buf * BN * BK;
#pragma unroll
        for (int kk = 0; kk < BK / 32; kk++) {
            i32x4 fa[TM], fb[TN];
            const int chunk = kk * 2 + (lane >> 5);
#pragma unroll
            for (int i = 0; i < TM; i++)
                fa[i] = *reinterpret_cast<const i32x4*>(pa + lds_offset<BK>(wm0 + i * 32 + (lane & 31), chunk));
#pragma unroll
            for (int j = 0; j < TN; j++)
                fb[j] = *reinterpret_cast<const i32x4*>(pb + lds_offset<BK>(wn0 + j * 32 + (lane & 31), chunk));
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk) store_lds(buf ^ 1);
        __syncthreads();
    }

    // Epilogue.  Accumulator register r of lane l is C[8*(r/4) + 4*(l/32) + r%4][l%32] of its 32x32 tile.
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int64_t n = n0 + wn0 + j * 32 + (lane & 31);
        if (n >= N) continue;
        const ChanParams cp = params[n];
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int64_t m = m0 + wm0 + i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
                if (m < M) out[m * N + n] = saturate8<OUT_SIGNED>(ppe_requant(acc[i][j][r], cp, ppe));
            }
        }
    }
}

// ---------------------------------------------------------------- implicit-GEMM convolution path
// Workgroup: BM output positions (flattened n, oy, ox) x BN output channels, 4 waves split BM.
// The weights of the BN channels, all taps, sit in LDS as [BN][KY*KX*IC] rows (swizzle as above
// on 64-byte granules, applied when a row is a whole number of them); activation fragments come straight from global memory, 16 bytes per lane.
template <int BM, int BN, bool IN_U8, bool OUT_SIGNED>
__global__ __launch_bounds__(256) void nce_conv_mfma(const int8_t* __restrict__ in, const int8_t* __restrict__ w,
                                                     const ChanParams* __restrict__ params, uint8_t* __restrict__ out,
                                                     ConvGeom g, int pad_byte, int swz, Ppe ppe) {
    constexpr int WM = BM / 4;
    constexpr int TM = WM / 32, TN = BN / 32;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];  // [BN][Ktot]
    const int64_t Ktot = (int64_t)g.KY * g.KX * g.IC;
    const int64_t Mtot = g.N * g.OH * g.OW;
    const int64_t m0 = (int64_t)blockIdx.x * BM;
    const int64_t oc0 = (int64_t)blockIdx.y * BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    // stage the weights: row = local output channel, 16-byte chunks, chunk index xor-ed with (row>>2)&3
    const int64_t chunks_per_row = Ktot / 16;
    for (int64_t cid = tid; cid < BN * chunks_per_row; cid += 256) {
        const int row = (int)(cid / chunks_per_row);
        const int64_t c = cid % chunks_per_row;
        int64_t oc = oc0 + row;
        oc = oc < g.OC ? oc : g.OC - 1;
        const i32x4 q = *reinterpret_cast<const i32x4*>(w + oc * Ktot + c * 16);
        const int64_t cs = swz ? ((c & ~3ll) | ((c ^ (row >> 2)) & 3)) : c;
        *reinterpret_cast<i32x4*>(smem + row * Ktot + cs * 16) = q;
    }
    __syncthreads();

    // positions of this lane's rows
    int64_t base_n[TM];
    int oy[TM], ox[TM];
    bool live[TM];
#pragma unroll
    for (int i = 0; i < TM; i++) {
        int64_t m = m0 + wave * WM + i * 32 + (lane & 31);
        live[i] = m < Mtot;
        m = live[i] ? m : Mtot - 1;
        ox[i] = (int)(m % g.OW);
        oy[i] = (int)((m / g.OW) % g.OH);
        base_n[i] = (m / (g.OW * g.OH)) * g.H * g.W * g.IC;
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
    for (int ky = 0; ky < g.KY; ky++) {
        for (int kx = 0; kx < g.KX; kx++) {
            const int8_t* pin[TM];
            bool inside[TM];
#pragma unroll
            for (int i = 0; i < TM; i++) {
                const int iy = oy[i] * g.SY + ky - g.PT;
                const int ix = ox[i] * g.SX + kx - g.PL;
                inside[i] = iy >= 0 && iy < g.H && ix >= 0 && ix < g.W;
                pin[i] = in + base_n[i] + ((int64_t)(inside[i] ? iy : 0) * g.W + (inside[i] ? ix : 0)) * g.IC + kgroup * 16;
            }
            const int64_t ktap = (int64_t)(ky * g.KX + kx) * g.IC;
            for (int64_t ic = 0; ic < g.IC; ic += 32) {
                i32x4 fa[TM], fb[TN];
#pragma unroll
                for (int i = 0; i < TM; i++) {
                    i32x4 q = *reinterpret_cast<const i32x4*>(pin[i] + ic);
                    if (!inside[i]) q = i32x4{pad32, pad32, pad32, pad32};
                    if (IN_U8) q ^= (int32_t)0x80808080;
                    fa[i] = q;
                }
                const int64_t c = (ktap + ic) / 16 + kgroup;
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const int row = j * 32 + (lane & 31);
                    const int64_t cs = swz ? ((c & ~3ll) | ((c ^ (row >> 2)) & 3)) : c;
                    fb[j] = *reinterpret_cast<const i32x4*>(smem + row * Ktot + cs * 16);
                }
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
            }
        }
    }

#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int64_t oc = oc0 + j * 32 + (lane & 31);
        if (oc >= g.OC) continue;
        const ChanParams cp = params[oc];
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int64_t m = m0 + wave * WM + i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
                if (m < Mtot) out[m * g.OC + oc] = saturate8<OUT_SIGNED>(ppe_requant(acc[i][j][r], cp, ppe));
            }
        }
    }
}

template <class KernelT>
int set_dyn_lds(KernelT kernel, size_t bytes) {
    if (bytes > 64 * 1024) {
        VPX_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
    }
    return VPX_RESULT_SUCCESS;
}

}  // namespace

int launch_nce(const vpx_nce_task_t& t, hipStream_t s, const char** kernel_name) {
    const bool in_u8 = t.input_type == VPX_NN_U8, w_u8 = t.weights_type == VPX_NN_U8,
               out_signed = t.output_type == VPX_NN_I8;
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
    switch (t.ppe.mode) {
    case VPX_PPE_NOOP: ppe.prelu_mult = 1; ppe.prelu_shift = 0; break;
    case VPX_PPE_LRELU:
    case VPX_PPE_LRELUX: ppe.prelu_mult = 0; ppe.prelu_shift = 0; break;
    case VPX_PPE_LPRELU: ppe.prelu_mult = t.ppe.lrelu_mult; ppe.prelu_shift = t.ppe.lrelu_shift; break;
    default: return fail(VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "NCE task: PPE mode %d is not an integer-pipeline mode", t.ppe.mode);
    }

    const int64_t Mtot = g.N * g.OH * g.OW;
    const int64_t Ktot = (int64_t)g.KY * g.KX * g.IC;
    if (Mtot == 0 || g.OC == 0) return VPX_RESULT_SUCCESS;

    const bool zp_in_ok = in_u8 ? (t.zp_in >= 0 && t.zp_in <= 255) : (t.zp_in >= -128 && t.zp_in <= 127);
    const bool mfma_ok = !w_u8 && t.zp_w == 0 && zp_in_ok && Mtot < (1ll << 31) && g.OC < (1ll << 31);
    const bool is_gemm = g.KY == 1 && g.KX == 1 && g.SY == 1 && g.SX == 1 && t.kernel_padding[0] == 0 &&
                         t.kernel_padding[1] == 0 && t.kernel_padding[2] == 0 && t.kernel_padding[3] == 0;
    const bool aligned = ((reinterpret_cast<uintptr_t>(t.input) | reinterpret_cast<uintptr_t>(t.weights)) & 15) == 0;
    // VPX_NCE_KERNEL=naive|conv restricts the choice to the slower, more general paths (used by tests
    // to check the device paths against each other).
    const char* force = std::getenv("VPX_NCE_KERNEL");
    const bool allow_gemm = !force || !*force;
    const bool allow_mfma = allow_gemm || std::strcmp(force, "conv") == 0;

    const bool use_gemm = allow_gemm && is_gemm && g.IC % 64 == 0;
    if (allow_mfma && mfma_ok && aligned && (use_gemm || (g.IC % 32 == 0 && 64 * Ktot <= 128 * 1024))) {
        void* ws = nullptr;
        int rc = get_workspace(s, sizeof(ChanParams) * (size_t)g.OC, &ws);
        if (rc) return rc;
        ChanParams* params = (ChanParams*)ws;
        const int corr = in_u8 ? 128 - t.zp_in : -t.zp_in;
        hipLaunchKernelGGL(nce_fold_kernel, dim3((unsigned)((g.OC + 3) / 4)), dim3(256), 0, s, (const int8_t*)t.weights,
                           t.weight_table, params, g.OC, Ktot, corr);
        VPX_HIP_CHECK(hipGetLastError());

        if (use_gemm) {
            constexpr int BM = 256, BN = 256, BK = 64, WM = 128, WN = 128;
            const int tiles_m = (int)((Mtot + BM - 1) / BM), tiles_n = (int)((g.OC + BN - 1) / BN);
            const int per_xcd = (tiles_m * tiles_n + 7) / 8;
            const size_t lds = 2 * (BM + BN) * BK;
            const dim3 grid((unsigned)(per_xcd * 8)), block((BM / WM) * (BN / WN) * 64);
#define VPX_GEMM(U8, SGN)                                                                                            \
    do {                                                                                                             \
        auto kern = nce_gemm_mfma<BM, BN, BK, WM, WN, U8, SGN>;                                                      \
        rc = set_dyn_lds(kern, lds);                                                                                 \
        if (rc) return rc;                                                                                           \
        hipLaunchKernelGGL(kern, grid, block, lds, s, (const int8_t*)t.input, (const int8_t*)t.weights, params,      \
                           (uint8_t*)t.output, Mtot, g.OC, g.IC, tiles_m, tiles_n, ppe);                            \
    } while (0)
            if (in_u8 && out_signed) VPX_GEMM(true, true);
            else if (in_u8) VPX_GEMM(true, false);
            else if (out_signed) VPX_GEMM(false, true);
            else VPX_GEMM(false, false);
#undef VPX_GEMM
            VPX_HIP_CHECK(hipGetLastError());
            *kernel_name = "nce_gemm_mfma";
            return VPX_RESULT_SUCCESS;
        }

        constexpr int BM = 256, BN = 64;
        const size_t lds = (size_t)BN * Ktot;
        const dim3 grid((unsigned)((Mtot + BM - 1) / BM), (unsigned)((g.OC + BN - 1) / BN));
        const int pad_byte = t.zp_in & 0xff;
        const int swz = Ktot % 64 == 0 ? 1 : 0;
#define VPX_CONV(U8, SGN)                                                                                            \
    do {                                                                                                             \
        auto kern = nce_conv_mfma<BM, BN, U8, SGN>;                                                                  \
        rc = set_dyn_lds(kern, lds);                                                                                 \
        if (rc) return rc;                                                                                           \
        hipLaunchKernelGGL(kern, grid, dim3(256), lds, s, (const int8_t*)t.input, (const int8_t*)t.weights, params,  \
                           (uint8_t*)t.output, g, pad_byte, swz, ppe);                                                  \
    } while (0)
        if (in_u8 && out_signed) VPX_CONV(true, true);
        else if (in_u8) VPX_CONV(true, false);
        else if (out_signed) VPX_CONV(false, true);
        else VPX_CONV(false, false);
#undef VPX_CONV
        VPX_HIP_CHECK(hipGetLastError());
        *kernel_name = "nce_conv_mfma";
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
    switch (sel) {
    case 0: VPX_NAIVE(false, false, false); break;
    case 1: VPX_NAIVE(false, false, true); break;
    case 2: VPX_NAIVE(false, true, false); break;
    case 3: VPX_NAIVE(false, true, true); break;
    case 4: VPX_NAIVE(true, false, false); break;
    case 5: VPX_NAIVE(true, false, true); break;
    case 6: VPX_NAIVE(true, true, false); break;
    default: VPX_NAIVE(true, true, true); break;
    }
#undef VPX_NAIVE
    VPX_HIP_CHECK(hipGetLastError());
    *kernel_name = "nce_conv_naive";
    return VPX_RESULT_SUCCESS;
}

}  // namespace vpx
