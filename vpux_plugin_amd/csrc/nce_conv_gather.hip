// The general convolution kernels of the NCE task: activation fragments gathered from global memory.
//   nce_conv_mfma   : IC a multiple of 32, any size: weights staged a K slice at a time.
//   nce_conv_mfma16 : IC a multiple of 16 only (stem layers), K up to 1008: two taps may share an MFMA step.
//   nce_conv_naive  : any shape and any zero points, one output per lane, 64-bit integer PPE.
// and the small kernels that prepare per-channel parameters for them.
#include "nce_common.h"

namespace vpx {
namespace nce {
namespace {

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

}  // namespace

int launch_fold(const int8_t* w, const int32_t* wt, ChanPrep* prep, int64_t OC, int64_t K, int corr, const Ppe& ppe, int shift_sub,
                hipStream_t s) {
    hipLaunchKernelGGL(nce_fold_kernel, dim3((unsigned)((OC + 3) / 4)), dim3(256), 0, s, w, wt, prep, OC, K, corr, ppe, shift_sub);
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

int launch_colsum(const int8_t* w, int32_t* colsum, int64_t OC, int64_t K, hipStream_t s) {
    hipLaunchKernelGGL(nce_colsum_kernel, dim3((unsigned)((OC + 3) / 4)), dim3(256), 0, s, w, colsum, OC, K);
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

int launch_conv_mfma(const int8_t* in, const int8_t* w, const ChanPrep* prep, uint8_t* out, const ConvGeom& g, int pad_byte,
                     const PpeFast& pf, bool in_u8, int out_kind, hipStream_t s) {
    constexpr int BM = 256, BN = 64;
    const int64_t Mtot = g.N * g.OH * g.OW;
    // weight slice per staging round: whole taps while 64 rows of them fit 64 KiB, else 1024 channels of one tap
    const int icc = g.IC <= 1024 ? (int)g.IC : 1024;
    int tc = g.IC <= 1024 ? (int)(1024 / g.IC) : 1;
    if (tc > g.KY * g.KX) tc = g.KY * g.KX;
    const size_t lds = (size_t)BN * tc * icc;
    const dim3 grid((unsigned)((Mtot + BM - 1) / BM), (unsigned)((g.OC + BN - 1) / BN));
    const int swz = icc % 64 == 0 ? 1 : 0;
    int rc = VPX_RESULT_SUCCESS;
#define VPX_CONV(U8, SGN)                                                                                            \
    do {                                                                                                             \
        auto kern = nce_conv_mfma<BM, BN, U8, SGN>;                                                                  \
        rc = set_dyn_lds(kern, lds);                                                                                 \
        if (rc) return rc;                                                                                           \
        hipLaunchKernelGGL(kern, grid, dim3(256), lds, s, in, w, prep, out, g, pad_byte, swz, tc, icc, pf);          \
    } while (0)
    const bool out_f16 = out_kind == OUT_F16, out_signed = out_kind == OUT_I8;
    if (out_f16 && in_u8) VPX_CONV(true, OUT_F16);
    else if (out_f16) VPX_CONV(false, OUT_F16);
    else if (in_u8 && out_signed) VPX_CONV(true, OUT_I8);
    else if (in_u8) VPX_CONV(true, OUT_U8);
    else if (out_signed) VPX_CONV(false, OUT_I8);
    else VPX_CONV(false, OUT_U8);
#undef VPX_CONV
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

int launch_conv_mfma16(const int8_t* in, const int8_t* w, const ChanPrep* prep, uint8_t* out, const ConvGeom& g, int pad_byte,
                       const PpeFast& pf, bool in_u8, int out_kind, hipStream_t s) {
    const int64_t Mtot = g.N * g.OH * g.OW, Ktot = (int64_t)g.KY * g.KX * g.IC;
    const size_t lds = (size_t)64 * ((Ktot + 31) / 32 * 32 + 16);
    const dim3 grid((unsigned)((Mtot + 255) / 256), (unsigned)((g.OC + 63) / 64));
    const bool out_f16 = out_kind == OUT_F16;
#define VPX_CONV16(U8, OUT)                                                                                           \
    hipLaunchKernelGGL((nce_conv_mfma16<U8, OUT>), grid, dim3(256), lds, s, in, w, prep, out, g, pad_byte, pf)
    // (the PPE's clamp window is already inside the storage range, so signed and unsigned bytes share a kernel)
    if (in_u8 && out_f16) VPX_CONV16(true, OUT_F16);
    else if (in_u8) VPX_CONV16(true, OUT_U8);
    else if (out_f16) VPX_CONV16(false, OUT_F16);
    else VPX_CONV16(false, OUT_U8);
#undef VPX_CONV16
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

int launch_conv_naive(const uint8_t* in, const uint8_t* w, const int32_t* wt, uint8_t* out, const ConvGeom& g, int zp_in, int zp_w,
                      const Ppe& ppe, bool in_u8, bool w_u8, int out_kind, hipStream_t s) {
    const int64_t total = g.N * g.OH * g.OW * g.OC;
    VPX_REQUIRE((total + 255) / 256 < (1ll << 31), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "NCE task: output of %lld elements exceeds the launch limit",
                (long long)total);
    const dim3 grid((unsigned)((total + 255) / 256));
    const bool out_f16 = out_kind == OUT_F16, out_signed = out_kind == OUT_I8;
#define VPX_NAIVE(IS, WS, OS)                                                                                        \
    hipLaunchKernelGGL((nce_conv_naive<IS, WS, OS>), grid, dim3(256), 0, s, in, w, wt, out, g, zp_in, zp_w, ppe, total)
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
    return VPX_RESULT_SUCCESS;
}

}  // namespace nce
}  // namespace vpx
