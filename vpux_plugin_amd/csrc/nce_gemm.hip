// nce_gemm_mfma: 1x1 kernel, no padding (this is how NCE.MatMul arrives; a stride picks rows from the input): a plain
// A[M][K] x B[N][K]^T GEMM.  256 x 256 (or 128 x 128) output tile per workgroup, v_mfma_i32_32x32x32_i8, K panels from
// global memory straight into XOR-swizzled LDS (global_load_lds, no register staging), four buffers, the integer PPE
// fused into the epilogue.
#include "nce_common.h"

namespace vpx {
namespace nce {
namespace {


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
//
// PP (eight waves, large tile, K a multiple of four panels): the two waves of a SIMD take turns.  While one runs the
// sixteen MFMAs of a panel back to back at raised priority, the other issues everything else it has to -- the twelve
// fragment reads of its next panel, its four panel loads, the column sums -- and at a workgroup barrier they swap,
// twice per panel.  (With both waves running the same interleaved stream their loads and reads fall on the same
// moments and the MFMA pipe waits for both.)
template <bool IN_U8, int OUT, int NW, int TILE = 256, bool SHORTK = false, bool PP = false>
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
    // Waves w and w + 4 share a SIMD.  Half-steps are counted from 0; in half-step h the first four waves (the tile's upper
    // half) multiply panel h / 2 when h is even and do their memory work when it is odd, the other four the other way
    // round, one half-step behind.  Panel p sits in buffer p % 4, and its loads are issued three panels ahead: by the
    // lower waves in half-step 2 (p - 3), by the upper ones in 2 (p - 3) + 1; the buffer they write held panel p - 4, whose
    // last fragment reads were consumed by MFMAs two half-steps earlier.  Before the barrier that ends an even
    // half-step 2 k every wave waits for its own loads of panel k + 1, so behind that barrier the panel is complete.
    auto pingpong_loop = [&]() {
        static_assert(!PP || (NW == 8 && TILE == 256 && !SHORTK), "wave roles alternate on the eight-wave large tile");
        auto read_panel = [&](auto stage_c) {
#pragma unroll
            for (int kk = 0; kk < 2; kk++)
#pragma unroll
                for (int n = 0; n < TM + TN; n++) load_frag_static(stage_c, kk, kk, n);
        };
        auto dma_panel = [&](int p) {
#pragma unroll
            for (int d = 0; d < 2 * DMA_PER_WAVE; d++) dma_one(std::false_type{}, p, d);
        };
        auto mfma_panel = [&]() {
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(1);
#pragma unroll
            for (int kk = 0; kk < 2; kk++)
#pragma unroll
                for (int i = 0; i < TM; i++) {
                    i32x4 a = fa[kk][i];
                    if (IN_U8) a ^= (int32_t)0x80808080;  // u8 -> s8 (value - 128)
#pragma unroll
                    for (int j = 0; j < TN; j++) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, fb[kk][j], acc[i][j], 0, 0, 0);
                }
            __builtin_amdgcn_s_setprio(0);
            __builtin_amdgcn_sched_barrier(0);
        };
        auto sum_panel = [&]() {  // the column sums of B from the fragments of the panel just multiplied
#pragma unroll
            for (int kk = 0; kk < 2; kk++)
#pragma unroll
                for (int j = 0; j < TN; j++)
#pragma unroll
                    for (int d = 0; d < 4; d++) cs[j] = __builtin_amdgcn_sdot4(fb[kk][j][d], 0x01010101, cs[j], false);
            __builtin_amdgcn_sched_barrier(0);
        };
#pragma unroll
        for (int p = 0; p < NS - 1; p++) dma_panel(p);
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(4 * DMA_PER_WAVE) : "memory");  // panel 0 is in
        // (two loops, one per role: the same number of barriers in each)
        if (wm0 == 0) {
            read_panel(std::integral_constant<int, 0>{});
            auto one_panel = [&](auto u_c, int k) {
                constexpr int u = decltype(u_c)::value;
                mfma_panel();
                asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(2 * DMA_PER_WAVE) : "memory");  // this wave's share of panel k + 1 is in
                sum_panel();
                if (k + 1 < nk) read_panel(std::integral_constant<int, (u + 1) & (NS - 1)>{});
                dma_panel(k + NS - 1);
                asm volatile("s_barrier" ::: "memory");
            };
            for (int k = 0; k < nk; k += NS) {
                one_panel(std::integral_constant<int, 0>{}, k);
                one_panel(std::integral_constant<int, 1>{}, k + 1);
                one_panel(std::integral_constant<int, 2>{}, k + 2);
                one_panel(std::integral_constant<int, 3>{}, k + 3);
            }
        } else {
            auto one_panel = [&](auto u_c, int k) {
                read_panel(u_c);
                dma_panel(k + NS - 1);
                asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(4 * DMA_PER_WAVE) : "memory");  // likewise, with panel k + 3 just asked for
                mfma_panel();
                asm volatile("s_barrier" ::: "memory");
            };
            for (int k = 0; k < nk; k += NS) {
                one_panel(std::integral_constant<int, 0>{}, k);
                one_panel(std::integral_constant<int, 1>{}, k + 1);
                one_panel(std::integral_constant<int, 2>{}, k + 2);
                one_panel(std::integral_constant<int, 3>{}, k + 3);
            }
        }
    };
    if constexpr (PP) {
        pingpong_loop();
    } else {
        // (a matmul of at most three panels is all epilogue: there every wave sums its own columns and nothing is handed over)
        if (SHORTK || wm0 == 0) main_loop(std::true_type{});
        else main_loop(std::false_type{});
    }
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

}  // namespace

int launch_gemm_mfma(const GemmLaunch& a, hipStream_t s) {
    const int tile = a.tile, nw = tile == 128 ? 4 : a.waves;
    const bool out_f16 = a.out_kind == OUT_F16;
    const int tiles_m = (int)((a.M + tile - 1) / tile), tiles_n = (int)((a.N + tile - 1) / tile);
    const int per_xcd = (tiles_m * tiles_n + 7) / 8;
    const dim3 grid((unsigned)(per_xcd * 8), (unsigned)a.G), block(64 * nw);
    const int64_t nk = a.K / 64;
    const bool shortk = a.shortk;
    size_t lds = 4 * (size_t)(tile + tile) * 64;  // four K panels; the output staging tile reuses them
    if (shortk) {
        lds = (size_t)nk * (tile + tile) * 64;  // only the panels there are ...
        if (lds < (size_t)tile * kOutStride) lds = (size_t)tile * kOutStride;  // ... or the staging tile
    }
    lds += kGemmLdsHead;
    const int32_t* colsum = nullptr;  // the kernel sums the columns of B itself, from the fragments it reads
    int rc = VPX_RESULT_SUCCESS;
    // the form in which the waves of a SIMD take turns: K a whole number of panel-buffer rounds
    const bool pingpong = a.pingpong && tile == 256 && nw == 8 && nk % 4 == 0 && nk >= 4 && !out_f16;
#define VPX_GEMM_W(U8, SGN, NW, TILE, SHORTK)                                                                        \
    do {                                                                                                             \
        auto kern = nce_gemm_mfma<U8, SGN, NW, TILE, SHORTK>;                                                        \
        rc = set_dyn_lds(kern, lds);                                                                                 \
        if (rc) return rc;                                                                                           \
        hipLaunchKernelGGL(kern, grid, dim3(64 * NW), lds, s, a.A, a.B, a.wt, colsum, a.out, a.M, a.N, a.K, tiles_m,  \
                           tiles_n, a.ppe, a.rows, a.dst);                                                           \
    } while (0)
#define VPX_GEMM_PP(U8, SGN)                                                                                         \
    do {                                                                                                             \
        auto kern = nce_gemm_mfma<U8, SGN, 8, 256, false, true>;                                                     \
        rc = set_dyn_lds(kern, lds);                                                                                 \
        if (rc) return rc;                                                                                           \
        hipLaunchKernelGGL(kern, grid, dim3(512), lds, s, a.A, a.B, a.wt, colsum, a.out, a.M, a.N, a.K, tiles_m,      \
                           tiles_n, a.ppe, a.rows, a.dst);                                                           \
    } while (0)
#define VPX_GEMM(U8, SGN)                                                                                            \
    do {                                                                                                             \
        if (shortk) VPX_GEMM_W(U8, SGN, 4, 128, true);                                                               \
        else if (tile == 128) VPX_GEMM_W(U8, SGN, 4, 128, false);                                                    \
        else if (nw == 4) VPX_GEMM_W(U8, SGN, 4, 256, false);                                                        \
        else if (pingpong) VPX_GEMM_PP(U8, SGN);                                                                     \
        else VPX_GEMM_W(U8, SGN, 8, 256, false);                                                                     \
    } while (0)
    if (out_f16) {
        // fp16 output: the eight-wave 256-tile and the four-wave 128-tile forms only (the host passes waves = 8)
        if (a.in_u8) { if (tile == 128) VPX_GEMM_W(true, OUT_F16, 4, 128, false); else VPX_GEMM_W(true, OUT_F16, 8, 256, false); }
        else { if (tile == 128) VPX_GEMM_W(false, OUT_F16, 4, 128, false); else VPX_GEMM_W(false, OUT_F16, 8, 256, false); }
    }
    else if (a.in_u8 && a.out_kind == OUT_I8) VPX_GEMM(true, OUT_I8);
    else if (a.in_u8) VPX_GEMM(true, OUT_U8);
    else if (a.out_kind == OUT_I8) VPX_GEMM(false, OUT_I8);
    else VPX_GEMM(false, OUT_U8);
#undef VPX_GEMM
#undef VPX_GEMM_PP
#undef VPX_GEMM_W
    (void)block;
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

}  // namespace nce
}  // namespace vpx
