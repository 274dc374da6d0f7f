// nce_conv_rows16: the row-patch convolution kernel of the NCE task, for channel counts that are a multiple of 16 but
// not of 64 (stem layers; the 32 / 96 / 160-channel layers of mobile networks).
#include "nce_common.h"

namespace vpx {
namespace nce {
namespace {

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

}  // namespace

int launch_conv_rows16(const RowsLaunch& a, hipStream_t s) {
    int rc = VPX_RESULT_SUCCESS;
#define VPX_ROWS_T(U8, TNV, TMV, MULTIV)                                                                              \
    do {                                                                                                              \
        if (a.out_f16) {                                                                                              \
            auto kern = nce_conv_rows16<U8, TMV, TNV, MULTIV, true>;                                                  \
            rc = set_dyn_lds(kern, a.lds);                                                                            \
            if (rc) return rc;                                                                                        \
            hipLaunchKernelGGL(kern, a.grid, dim3(512), a.lds, s, a.in, a.w, a.wt, a.out, a.g, a.rg, a.pad_byte, a.ppe); \
        } else {                                                                                                      \
            auto kern = nce_conv_rows16<U8, TMV, TNV, MULTIV, false>;                                                 \
            rc = set_dyn_lds(kern, a.lds);                                                                            \
            if (rc) return rc;                                                                                        \
            hipLaunchKernelGGL(kern, a.grid, dim3(512), a.lds, s, a.in, a.w, a.wt, a.out, a.g, a.rg, a.pad_byte, a.ppe); \
        }                                                                                                             \
    } while (0)
#define VPX_ROWS(U8, TNV)                                                                                             \
    do {                                                                                                              \
        if (a.tm == 4 && a.multi) VPX_ROWS_T(U8, TNV, 4, true);                                                       \
        else if (a.tm == 4) VPX_ROWS_T(U8, TNV, 4, false);                                                            \
        else if (a.multi) VPX_ROWS_T(U8, TNV, 2, true);                                                               \
        else VPX_ROWS_T(U8, TNV, 2, false);                                                                           \
    } while (0)
    if (a.bn == 128) {  // (TM = 2 only: eight accumulator tiles a wave)
        if (a.in_u8 && a.multi) VPX_ROWS_T(true, 4, 2, true);
        else if (a.in_u8) VPX_ROWS_T(true, 4, 2, false);
        else if (a.multi) VPX_ROWS_T(false, 4, 2, true);
        else VPX_ROWS_T(false, 4, 2, false);
    } else if (a.in_u8 && a.bn == 32) VPX_ROWS(true, 1);
    else if (a.in_u8) VPX_ROWS(true, 2);
    else if (a.bn == 32) VPX_ROWS(false, 1);
    else VPX_ROWS(false, 2);
#undef VPX_ROWS
#undef VPX_ROWS_T
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

}  // namespace nce
}  // namespace vpx
