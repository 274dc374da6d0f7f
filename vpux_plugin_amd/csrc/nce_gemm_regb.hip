// nce_gemm_regb: A[M][K] x B[N][K]^T with the PPE fused, for a short K (64, 128 or 256) and many rows -- the 1x1
// layers of a network's early stages, where a row of the result costs more vector work in the PPE than matrix work and
// the tile kernel (nce_gemm.hip) is all prologue and epilogue.
//
// No workgroup barrier after the set-up, and neither operand goes through LDS.  A wave owns CBW blocks of 64 output
// channels for the whole launch and keeps their weights in registers (CBW x 4 x K/64 fragments of
// `v_mfma_i32_16x16x64_i8`, 64 registers at most); it walks blocks of 16 rows: one 16-byte load per lane and 64 of K
// straight from global memory (the 16 rows of a block are one contiguous piece when K = 64), then per channel block
// 4 x K/64 MFMAs that start from the bias and the short PPE.  The loads run kPrefetch blocks ahead of the arithmetic.
//
// The weights are the FIRST operand of the MFMA: the product is the transposed block, channels down and rows of the
// matrix across, so a lane's four accumulators of a tile are four channels of one row -- the bytes of a dword of the
// output as it lies in memory, no transpose.  Row i of tile j is channel 16*(i/4) + 4*j + i%4 of its block: lane
// (row n16, quarter c4) then holds channels 16*c4 .. 16*c4+15 of row n16 in its four result dwords.
// The PPE factors of a lane's sixteen channels per block come from a table in LDS that the workgroup prepares once
// (one channel per thread); in registers they would be 32 to 64 per block.
//
// Output: the wave collects its 16 rows x CBW x 64 bytes in an LDS tile of its own and writes them as whole pieces of
// rows, neighbouring lanes neighbouring 16-byte pieces (measured at [401408 x 64] . [64 x 256]: 64-byte pieces of
// 256-byte rows, one per lane quarter, 34 us; a row per sixteen lanes 28 us).
//
// Work is dealt by wave.  The four waves of a workgroup serve GW different groups of CBW channel blocks (4 / GW row
// streams each): with GW > 1 the waves that share a row block are neighbours, so its rows come from memory once.  A
// workgroup's index modulo the number of its kind picks the channels; wave s of those that share them takes row blocks
// s, s + S, ...
#include "nce_common.h"

namespace vpx {
namespace nce {
namespace {

constexpr int kRegbWaves = 4;

// Waves per SIMD the register budget is cut for (512 registers / 4, 3, 2 waves): the launch is bound by the memory
// system and by vector instructions, both of which want waves.
constexpr int regb_waves_per_simd(bool same_f, int ks, int cbw) {
    const int wregs = ks * cbw * 16;  // registers of weights
    return wregs == 16 ? 4 : (wregs == 32 ? (same_f && ks == 1 ? 4 : 3) : (same_f && ks <= 2 ? 3 : 2));
}

template <bool SAME_F, int KS, int CBW, int GW>
__global__ __launch_bounds__(64 * kRegbWaves) __attribute__((amdgpu_waves_per_eu(regb_waves_per_simd(SAME_F, KS, CBW)))) void nce_gemm_regb(
    const int8_t* __restrict__ A, const int8_t* __restrict__ B, const int32_t* __restrict__ wt, uint8_t* __restrict__ out, int64_t M, int N,
    int64_t lda, int64_t ldc, GemmPpe ppe, int supers, int sign_flip) {
    constexpr int K = KS * 64, NCH = CBW * 64, RSW = kRegbWaves / GW, TCH = GW * NCH;
    static_assert(TCH <= 64 * kRegbWaves, "one thread prepares one channel");
    constexpr int kPrefetch = KS * CBW >= 4 ? (KS == 1 ? 2 : 1) : (KS == 1 ? 3 : 2);  // row blocks ahead; (kPrefetch + 1) x KS x 4 registers
    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int gw = w / RSW, super = (int)blockIdx.x % supers;
    const int stream = ((int)blockIdx.x / supers) * RSW + w % RSW, streams = ((int)gridDim.x / supers) * RSW;
    const int n16 = lane & 15, c4 = lane >> 4;
    const int n0 = (super * GW + gw) * NCH;  // this wave's first channel
    const int tb = gw * NCH;                 // ... and its place in the workgroup's tables

    // ---- this wave's weights and their column sums.  Fragment (cbl, j): row n16 of tile j of block cbl, 16 of K per quarter.
    i32x4 wb[CBW][4][KS];
    int colsum[CBW][4];
#pragma unroll
    for (int cbl = 0; cbl < CBW; cbl++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            int ch = n0 + cbl * 64 + (n16 >> 2) * 16 + j * 4 + (n16 & 3);
            ch = ch < N ? ch : N - 1;  // channels past the end repeat the last one (never stored)
            int sum = 0;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                wb[cbl][j][ks] = *reinterpret_cast<const i32x4*>(B + (int64_t)ch * K + ks * 64 + c4 * 16);
#pragma unroll
                for (int q = 0; q < 4; q++) sum = __builtin_amdgcn_sdot4(wb[cbl][j][ks][q], 0x01010101, sum, false);
            }
            if (ppe.corr != 0) {  // the four lanes that hold a channel's K sit 16 lanes apart
                sum += __shfl_xor(sum, 16);
                sum += __shfl_xor(sum, 32);
            }
            colsum[cbl][j] = sum;  // of row n16 of tile j
        }

    // ---- PPE parameters: thread t prepares channel t of the workgroup's TCH into tables in LDS
    __shared__ double s_fpos[TCH], s_fneg[TCH];
    __shared__ __attribute__((aligned(16))) int s_bias[TCH];
    __shared__ int s_w2[TCH], s_sum[TCH];
    if (ppe.corr != 0 && c4 == 0) {  // (waves that serve the same channels write the same sums)
#pragma unroll
        for (int cbl = 0; cbl < CBW; cbl++)
#pragma unroll
            for (int j = 0; j < 4; j++) s_sum[tb + cbl * 64 + (n16 >> 2) * 16 + j * 4 + (n16 & 3)] = colsum[cbl][j];
    }
    __syncthreads();
    bool clip = false;
    if (tid < TCH) {
        int ch = super * TCH + tid;
        ch = ch < N ? ch : N - 1;
        const int sum = ppe.corr != 0 ? s_sum[tid] : 0;
        const uint32_t w2 = (uint32_t)wt[ch * 4 + 2];
        const ChanPrep c = ppe_prepare((int)(int16_t)(w2 >> 16), (int)((w2 >> 8) & 0xffu), (int)((unsigned)wt[ch * 4 + 3] + (unsigned)(ppe.corr * sum)),
                                       ppe.prelu_mult, ppe.prelu_shift);
        clip = c.bmax_pos != 0x7fffffff || c.bmax_neg != 0x7fffffff;
        s_fpos[tid] = c.f_pos;
        s_fneg[tid] = c.f_neg;
        s_bias[tid] = c.bias;
        s_w2[tid] = (int)w2;
    }
    __shared__ int s_general;
    if (tid == 0) s_general = 0;
    __syncthreads();
    const PpePack pk = make_ppe_pack(ppe.zp_out, ppe.lo, ppe.hi, ppe.out_signed != 0);
    // the short PPE serves slopes in [0, 1] (ReLU, LeakyReLU), an even zero-point offset and scales up to 1/2
    const bool slope_ok = SAME_F || (ppe.prelu_mult >= 0 && (ppe.prelu_shift >= 31 || ppe.prelu_mult <= (1 << ppe.prelu_shift)));
    if ((__builtin_amdgcn_ballot_w64(clip) != 0 || pk.odd != 0 || !slope_ok) && lane == 0) s_general = 1;
    __syncthreads();
    const bool general = s_general != 0;  // (one answer for the workgroup)
    const int32_t* const rt = ppe.rowterm;
    const int nblk = (int)((M + 15) >> 4);

    auto fetch = [&](int b, i32x4 (&a)[KS]) {
        int64_t row = (int64_t)b * 16 + n16;
        row = row < M ? row : M - 1;
        const int8_t* src = A + row * lda + c4 * 16;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) a[ks] = *reinterpret_cast<const i32x4*>(src + ks * 64);
    };
    // the sums of channel block cbl of a row block: from the bias (short PPE) or from zero, the row term added
    auto multiply = [&](int cbl, const i32x4 (&f)[KS], int rowterm, i32x4 (&acc)[4], bool from_bias) {
#pragma unroll
        for (int j = 0; j < 4; j++)
            acc[j] = from_bias ? *reinterpret_cast<const i32x4*>(&s_bias[tb + cbl * 64 + c4 * 16 + j * 4]) : i32x4{0, 0, 0, 0};
#pragma unroll
        for (int ks = 0; ks < KS; ks++)
#pragma unroll
            for (int j = 0; j < 4; j++) acc[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wb[cbl][j][ks], f[ks], acc[j], 0, 0, 0);
        if (rt) {
#pragma unroll
            for (int j = 0; j < 4; j++) acc[j] += rowterm;
        }
    };
    // The wave's tile: 16 rows of NCH bytes, padded to 2 mod 4 sixteen-byte pieces per row (the 16-row x 4-piece pattern
    // of a wave's writes without bank conflicts).  Lane L then writes piece L % PPR of row L / PPR, + 64 / PPR rows per step.
    // (the host sends layers here whose output rows are a fixed pitch apart, 16-byte aligned, N a multiple of 16)
    constexpr int kTileStride = NCH + 32, PPR = NCH / 16, RPS = 64 / PPR;
    __shared__ __attribute__((aligned(16))) uint8_t s_tile[kRegbWaves][16 * kTileStride];
    uint8_t* const tile_w = &s_tile[w][n16 * kTileStride + c4 * 16];
    const uint8_t* const tile_r = &s_tile[w][(lane / PPR) * kTileStride + (lane % PPR) * 16];
    const int64_t col = n0 + (lane % PPR) * 16;
    auto write_out = [&](int b) {
#pragma unroll
        for (int i = 0; i < 16 / RPS; i++) {
            const i32x4 v = *reinterpret_cast<const i32x4*>(tile_r + i * RPS * kTileStride);  // (LDS serves a wave's accesses in order)
            const int64_t m = (int64_t)b * 16 + i * RPS + lane / PPR;
            if (m < M && col < N) __builtin_nontemporal_store(v, reinterpret_cast<i32x4*>(out + (m * ldc + col)));
        }
    };
    auto one_block = [&](int b, const i32x4 (&a)[KS], auto general_c) {
        constexpr bool GENERAL = decltype(general_c)::value;
        i32x4 f[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ks++) f[ks] = a[ks] ^ sign_flip;  // unsigned input: the top bit of every byte
        const int rowterm = rt ? rt[(int64_t)b * 16 + n16] : 0;  // (padded past the last row: an edge block may read ahead)
#pragma unroll
        for (int cbl = 0; cbl < CBW; cbl++) {
            i32x4 acc[4];
            multiply(cbl, f, rowterm, acc, !GENERAL);
            if constexpr (GENERAL) {
                // Every PPE setting, in the integer form the compiler programs.  Rare (scales above 1/2, odd zero
                // points, slopes above one) and long: one copy of the arithmetic walks the sixteen sums through LDS.
                __shared__ int sums[kRegbWaves][16][64];
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int r = 0; r < 4; r++) sums[w][j * 4 + r][lane] = acc[j][r];
                const Ppe p{ppe.prelu_mult, ppe.prelu_shift, ppe.zp_out, ppe.lo, ppe.hi, 0.f, 0.f};
#pragma unroll 1
                for (int i = 0; i < 16; i++) {  // channel n0 + 64 * cbl + 16 * c4 + i
                    const uint32_t w2 = (uint32_t)s_w2[tb + cbl * 64 + c4 * 16 + i];
                    const ChanParams c{s_bias[tb + cbl * 64 + c4 * 16 + i], (int)(int16_t)(w2 >> 16), (int)((w2 >> 8) & 0xffu)};
                    tile_w[cbl * 64 + i] = (uint8_t)ppe_requant(sums[w][i][lane], c, p);
                }
            } else {
                i32x4 o;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    unsigned v = 0;
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const int ci = tb + cbl * 64 + c4 * 16 + j * 4 + r;
                        v |= ppe_one_biased<!SAME_F>(acc[j][r], s_fpos[ci], SAME_F ? 0.0 : s_fneg[ci], pk) << (8 * r);
                    }
                    o[j] = (int)(v ^ pk.flip);
                }
                *reinterpret_cast<i32x4*>(tile_w + cbl * 64) = o;
            }
        }
        write_out(b);
    };
    if (general) {  // (nothing fetched ahead)
        for (int b = stream; b < nblk; b += streams) {
            i32x4 a[KS];
            fetch(b, a);
            one_block(b, a, std::true_type{});
        }
    } else {
        i32x4 a[kPrefetch + 1][KS];
#pragma unroll
        for (int p = 0; p < kPrefetch; p++)
            if (stream + p * streams < nblk) fetch(stream + p * streams, a[p]);
        for (int b = stream; b < nblk; b += (kPrefetch + 1) * streams) {
#pragma unroll
            for (int p = 0; p <= kPrefetch; p++) {
                const int bb = b + p * streams;
                if (bb >= nblk) break;
                if (bb + kPrefetch * streams < nblk) fetch(bb + kPrefetch * streams, a[(p + kPrefetch) % (kPrefetch + 1)]);
                one_block(bb, a[p], std::false_type{});
            }
        }
    }
}

}  // namespace

// The shape of the work: `cbw` 64-channel blocks per wave, `gw` groups of them per workgroup.
// cbw: as many as keep the weights within 64 registers and divide the number of blocks -- whole pieces of output rows
// per store -- where the rows are many enough for units of that size to fill the waves evenly (about six row blocks per
// wave: [401408 x 64] . [64 x 256] 30.5 us with four blocks per wave, 34.1 with one; [100352 x 64] . [64 x 256] 11.8
// against 10.2 us); else one.  gw: as many groups as the workgroup's four waves and 256 table entries hold and the
// number of groups divides by.
void gemm_regb_shape(int64_t M, int64_t N, int64_t K, int cus, bool widest, int* cbw_out, int* gw_out) {
    const int64_t cb_total = (N + 63) / 64;
    int cbw = K == 64 ? 4 : (K == 128 ? 2 : 1);
    while (cb_total % cbw) cbw /= 2;
    const int64_t streams = (int64_t)cus * 3 * kRegbWaves / (cb_total / cbw);
    if ((M + 15) / 16 < 6 * streams && !widest) cbw = 1;
    const int64_t groups = cb_total / cbw;
    int gw = 4 / cbw;
    while (groups % gw) gw /= 2;
    *cbw_out = cbw;
    *gw_out = gw;
}

// Workgroups (of one wave per SIMD) a compute unit holds at once.
int gemm_regb_workgroups_per_cu(bool same_f, int64_t K, int cbw) { return regb_waves_per_simd(same_f, (int)(K / 64), cbw); }

int launch_gemm_regb(const GemmLaunch& a, int cbw, int gw, int workgroups, hipStream_t s) {
    const int supers = (int)((a.N + 63) / 64) / cbw / gw;
    const bool same_f = a.ppe.prelu_mult == 1 && a.ppe.prelu_shift == 0;
    const int ks = (int)(a.K / 64);
    const int sign_flip = a.in_u8 ? (int)0x80808080 : 0;
#define VPX_REGB(SAME, KS, CBW, GW)                                                                                  \
    hipLaunchKernelGGL((nce_gemm_regb<SAME, KS, CBW, GW>), dim3((unsigned)workgroups), dim3(64 * kRegbWaves), 0, s, a.A, a.B,   \
                       a.wt, a.out, a.M, (int)a.N, a.rows.lda, a.dst.sw, a.ppe, supers, sign_flip)
#define VPX_REGB_G(SAME, KS, CBW)                                                                                    \
    do {                                                                                                             \
        if (gw == 1) VPX_REGB(SAME, KS, CBW, 1);                                                                     \
        else if (gw == 2 && CBW <= 2) VPX_REGB(SAME, KS, (CBW <= 2 ? CBW : 1), 2);                                   \
        else if (gw == 4 && CBW == 1) VPX_REGB(SAME, KS, 1, 4);                                                      \
        else return VPX_RESULT_ERROR_UNKNOWN;                                                                        \
    } while (0)
#define VPX_REGB_K(SAME)                                                                                             \
    do {                                                                                                             \
        if (ks == 1 && cbw == 4) VPX_REGB_G(SAME, 1, 4);                                                             \
        else if (ks == 1 && cbw == 2) VPX_REGB_G(SAME, 1, 2);                                                        \
        else if (ks == 1 && cbw == 1) VPX_REGB_G(SAME, 1, 1);                                                        \
        else if (ks == 2 && cbw == 2) VPX_REGB_G(SAME, 2, 2);                                                        \
        else if (ks == 2 && cbw == 1) VPX_REGB_G(SAME, 2, 1);                                                        \
        else if (ks == 4 && cbw == 1) VPX_REGB_G(SAME, 4, 1);                                                        \
        else return VPX_RESULT_ERROR_UNSUPPORTED_FEATURE;                                                            \
    } while (0)
    if (supers < 1 || workgroups % supers != 0) return VPX_RESULT_ERROR_UNKNOWN;
    if (same_f) VPX_REGB_K(true); else VPX_REGB_K(false);
#undef VPX_REGB_K
#undef VPX_REGB_G
#undef VPX_REGB
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

}  // namespace nce
}  // namespace vpx
