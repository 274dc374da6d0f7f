// Convolutions of the NCE task with the input rows of a tile resident in LDS (64 output channels per workgroup):
//   nce_conv_regw   : 3x3 taps of 64 input channels: the weights of the 64 output channels in the registers of every wave.
//   nce_conv_tile   : KYxKX / stride / padding with 64 or 128 input channels: the weights in LDS beside the rows, every
//                     tap an LDS read.
//   nce_conv_stream : any multiple of 64 input channels: the weights pass through LDS a slice at a time.
#include "nce_common.h"

namespace vpx {
namespace nce {
namespace {

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
    // LDS strides of a pixel and of a weight row: a fragment read has sixteen lanes sixteen rows apart and four such
    // groups one 16-byte chunk apart, which LDS serves without bank conflicts when the row stride is 2 mod 4 chunks
    // (96 and 608 bytes; measured: 80 or 592 bytes take twice as long per read)
    constexpr int BN = 64, IC = 64, PS = IC + 32, NW = 8, NT = 64 * NW, TAPS = KY * KX, Ktot = TAPS * IC, WS = Ktot + 32;
    static_assert((PS / 16) % 4 == 2 && (WS / 16) % 4 == 2, "conflict-free fragment reads");
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* const wlds = smem;             // [64][Ktot + 32], rows in tile order
    uint8_t* const patch = smem + BN * WS;  // [PH*PW][IC + 32]
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

}  // namespace

int launch_conv_regw(const PatchLaunch& a, hipStream_t s) {
    int rc = VPX_RESULT_SUCCESS;
#define VPX_REGW(U8, SAME)                                                                                            \
    do {                                                                                                              \
        auto kern = nce_conv_regw<U8, SAME, 3, 3>;                                                                    \
        rc = set_dyn_lds(kern, a.lds);                                                                                \
        if (rc) return rc;                                                                                            \
        hipLaunchKernelGGL(kern, a.grid, dim3(512), a.lds, s, a.in, a.w, a.wt, a.out, a.g, a.pg, a.pad_byte, a.ppe);  \
    } while (0)
    if (a.in_u8 && a.same_f) VPX_REGW(true, true);
    else if (a.in_u8) VPX_REGW(true, false);
    else if (a.same_f) VPX_REGW(false, true);
    else VPX_REGW(false, false);
#undef VPX_REGW
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

// per_wave: row blocks of 32 positions a wave takes (the template's TMW is the next of 2, 4, 7); ics = IC / 64;
// waves: 4 or 8 per workgroup
int launch_conv_tile(const PatchLaunch& a, int per_wave, int ics, int waves, hipStream_t s) {
    int rc = VPX_RESULT_SUCCESS;
    const int nw = waves;
#define VPX_TILE_W(U8, TMW, SAME, ICS, NW)                                                                            \
    do {                                                                                                              \
        auto kern = nce_conv_tile<U8, TMW, SAME, ICS, NW>;                                                            \
        rc = set_dyn_lds(kern, a.lds);                                                                                \
        if (rc) return rc;                                                                                            \
        hipLaunchKernelGGL(kern, a.grid, dim3(64 * NW), a.lds, s, a.in, a.w, a.wt, a.out, a.g, a.pg, a.pad_byte, a.ppe); \
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
        if (a.in_u8 && a.same_f) VPX_TILE_I(true, TMW, true);                                                         \
        else if (a.in_u8) VPX_TILE_I(true, TMW, false);                                                               \
        else if (a.same_f) VPX_TILE_I(false, TMW, true);                                                              \
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
    return VPX_RESULT_SUCCESS;
}

// ksplit_waves: 0, or the K-split form (4: four waves; 8: eight waves, four shares; 88: eight waves, eight shares);
// per_wave: row blocks per wave of the eight-wave form
int launch_conv_stream(const PatchLaunch& a, int ksplit_waves, int per_wave, hipStream_t s) {
    int rc = VPX_RESULT_SUCCESS;
#define VPX_STREAM_W(U8, TMW, SAME, NW, KS)                                                                           \
    do {                                                                                                              \
        auto kern = nce_conv_stream<U8, TMW, SAME, NW, KS>;                                                           \
        rc = set_dyn_lds(kern, a.lds);                                                                                \
        if (rc) return rc;                                                                                            \
        hipLaunchKernelGGL(kern, a.grid, dim3(64 * NW), a.lds, s, a.in, a.w, a.wt, a.colsum, a.out, a.g, a.pg, a.sg,   \
                           a.pad_byte, a.ppe);                                                                        \
    } while (0)
#define VPX_STREAM(TMW, NW, KS)                                                                                       \
    do {                                                                                                              \
        if (a.in_u8 && a.same_f) VPX_STREAM_W(true, TMW, true, NW, KS);                                               \
        else if (a.in_u8) VPX_STREAM_W(true, TMW, false, NW, KS);                                                     \
        else if (a.same_f) VPX_STREAM_W(false, TMW, true, NW, KS);                                                    \
        else VPX_STREAM_W(false, TMW, false, NW, KS);                                                                 \
    } while (0)
    // (a tile of one or two row blocks -- 7 x 7 planes -- would leave six of eight waves multiplying
    // padding: four waves, one block each, a third of the LDS reads per weight slice)
    if (ksplit_waves == 4) VPX_STREAM(1, 4, 4);
    else if (ksplit_waves == 8) VPX_STREAM(1, 8, 4);
    else if (ksplit_waves == 88) VPX_STREAM(1, 8, 8);
    else if (a.pg.MT <= 4 / a.pg.nt) VPX_STREAM(1, 4, 0);
    else if (per_wave <= 1) VPX_STREAM(1, 8, 0);
    else if (per_wave <= 2) VPX_STREAM(2, 8, 0);
    else VPX_STREAM(4, 8, 0);
#undef VPX_STREAM
#undef VPX_STREAM_W
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

}  // namespace nce
}  // namespace vpx
