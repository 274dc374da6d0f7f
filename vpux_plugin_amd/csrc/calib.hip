// Calibration loop for the int8 MFMA roofline: what the part sustains on `v_mfma_i32_32x32x32_i8` before a
// single byte comes from global memory.  Not part of the NCE path; the bench runs it beside the matmul so
// that the matmul's fraction of peak can be read against the rate the silicon holds on the same kind of
// operands (the shader clock drops under dense int8 MFMA work on random data).
//
// One workgroup of eight waves per launch slot, two waves per SIMD as in nce_gemm_mfma, each wave a
// 128 x 64 register tile (eight accumulators of 32 x 32).  Per iteration a wave issues sixteen MFMAs
// (two K steps of 32); with `fragment_reads` it also reads the twelve 16-byte fragments those MFMAs
// consume from LDS, in the matmul kernel's swizzled layout and interleaving.
#include <hip/hip_runtime.h>

#include "vpx_common.h"

namespace vpx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kCalibThreads = 512;
constexpr int kCalibLds = 64 * 1024;

template <bool READS>
__global__ __launch_bounds__(kCalibThreads) void calib_mfma_i8_kernel(const v4i* __restrict__ operands, v4i* __restrict__ sink,
                                                                      int iters) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    for (int i = threadIdx.x; i < kCalibLds / 16; i += kCalibThreads) reinterpret_cast<v4i*>(smem)[i] = operands[i];
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane % 32, c = lane / 32;
    // rows of 64 bytes, 16-byte chunk c kept at slot c ^ ((r >> 2) & 3): conflict-free for 128-bit reads
    const char* p = smem + r * 64 + ((c ^ ((r >> 2) & 3)) << 4) + (wave & 3) * 2048;
    v16i acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < 16; j++) acc[i][j] = 0;
    v4i a[2][4], b[2][2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
#pragma unroll
        for (int i = 0; i < 4; i++) a[h][i] = *reinterpret_cast<const v4i*>(p + i * 8192 + h * 32);
#pragma unroll
        for (int j = 0; j < 2; j++) b[h][j] = *reinterpret_cast<const v4i*>(p + 32768 + j * 8192 + h * 32);
    }
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const int idx = i * 2 + j;
                    acc[idx] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[h][i], b[h][j], acc[idx], 0, 0, 0);
                    if (READS) {
                        // the other half's fragments, one read behind each of the first six MFMAs
                        if (idx < 4) a[h ^ 1][idx] = *reinterpret_cast<const v4i*>(p + idx * 8192 + ((it + h) & 1) * 32);
                        else if (idx < 6) b[h ^ 1][idx - 4] = *reinterpret_cast<const v4i*>(p + 32768 + (idx - 4) * 8192 + ((it + h) & 1) * 32);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
        }
    }
    v4i s = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < 16; j++) s[j & 3] += acc[i][j];
    sink[(size_t)blockIdx.x * kCalibThreads + threadIdx.x] = s;
}

// Does the vector ALU work of one wave run under the MFMAs of the other wave of its SIMD?  Eight waves, two per SIMD.
// A round is sixteen MFMAs for an MFMA wave and sixty-four instructions of one kind for a vector wave.
//   mode 0: every wave multiplies; 1: every wave runs the vector instructions; 2: waves 0-3 multiply and waves 4-7 (their
//   SIMD partners) run the vector instructions; 3: every wave does both, four vector instructions behind each MFMA.
// If the two kinds overlap, mode 2 takes as long as the longer of the two alone on one wave (half of mode 0 or 1).
enum { CO_FMA_F64 = 0, CO_FMA_F32, CO_ADD_U32, CO_MUL_LO_U32, CO_MAD_U64_U32, CO_CVT_F64_I32, CO_KINDS };

template <int KIND>
__device__ __forceinline__ void co_valu4(unsigned (&x)[8], unsigned long long (&y)[4], int base) {
#pragma unroll
    for (int u = 0; u < 4; u++) {
        const int i = (base + u) & 7, j = (base + u) & 3;
        if (KIND == CO_FMA_F64) asm volatile("v_fma_f64 %0, %0, %1, %1" : "+v"(y[j]) : "v"(y[(j + 1) & 3]));
        else if (KIND == CO_FMA_F32) asm volatile("v_fma_f32 %0, %0, %1, %1" : "+v"(x[i]) : "v"(x[(i + 1) & 7]));
        else if (KIND == CO_ADD_U32) asm volatile("v_add_u32 %0, %0, %1" : "+v"(x[i]) : "v"(x[(i + 1) & 7]));
        else if (KIND == CO_MUL_LO_U32) asm volatile("v_mul_lo_u32 %0, %0, %1" : "+v"(x[i]) : "v"(x[(i + 1) & 7]));
        else if (KIND == CO_MAD_U64_U32) asm volatile("v_mad_u64_u32 %0, vcc, %1, %2, %0" : "+v"(y[j]) : "v"(x[i]), "v"(x[(i + 1) & 7]) : "vcc");
        else asm volatile("v_cvt_f64_i32 %0, %1" : "=v"(y[j]) : "v"(x[i]));
    }
}

template <int KIND, bool WIDE>
__global__ __launch_bounds__(kCalibThreads) void calib_coissue_kernel(v4i* __restrict__ sink, int iters, int mode) {
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const bool do_mfma = mode == 0 || mode == 3 || (mode == 2 && wave < 4);
    const bool do_valu = mode == 1 || (mode == 2 && wave >= 4);
    v16i acc32[4];
    v4i acc16[8];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 16; j++) acc32[i][j] = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) acc16[i] = v4i{0, 0, 0, 0};
    const v4i a = {(int)threadIdx.x * 0x01030507, 0x11223344, (int)threadIdx.x, 0x7f7f7f7f}, b = {0x01020304, (int)threadIdx.x * 77, 0x55aa55aa, 3};
    unsigned x[8];
    unsigned long long y[4];
#pragma unroll
    for (int i = 0; i < 8; i++) x[i] = threadIdx.x * 2654435761u + i;
#pragma unroll
    for (int i = 0; i < 4; i++) y[i] = 0x3ff0000000000000ull + threadIdx.x + i;  // doubles near 1
    if (mode == 3) {
        for (int it = 0; it < iters; it++)
#pragma unroll
            for (int m = 0; m < 16; m++) {
                if (WIDE) acc32[m & 3] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc32[m & 3], 0, 0, 0);
                else acc16[m & 7] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc16[m & 7], 0, 0, 0);
                co_valu4<KIND>(x, y, 4 * m);
            }
    } else if (do_mfma) {
        for (int it = 0; it < iters; it++)
#pragma unroll
            for (int m = 0; m < 16; m++) {
                if (WIDE) acc32[m & 3] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc32[m & 3], 0, 0, 0);
                else acc16[m & 7] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc16[m & 7], 0, 0, 0);
            }
    } else if (do_valu) {
        for (int it = 0; it < iters; it++)
#pragma unroll
            for (int m = 0; m < 16; m++) co_valu4<KIND>(x, y, 4 * m);
    }
    v4i sres = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 16; j++) sres[j & 3] += acc32[i][j];
#pragma unroll
    for (int i = 0; i < 8; i++) sres += acc16[i];
#pragma unroll
    for (int i = 0; i < 8; i++) sres[i & 3] += (int)x[i];
#pragma unroll
    for (int i = 0; i < 4; i++) sres[i] += (int)(y[i] >> 20);
    sink[(size_t)blockIdx.x * kCalibThreads + threadIdx.x] = sres;
}

}  // namespace

int calib_coissue(int valu_kind, int wide_mfma, int mode, int iters, void* sink, hipStream_t s) {
    if (!sink || iters < 1 || valu_kind < 0 || valu_kind >= CO_KINDS || mode < 0 || mode > 3)
        return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT, "calib_coissue: null buffer, iters < 1, or an unknown kind / mode");
    int blocks = 0;
    if (const int rc = device_compute_units(&blocks)) return rc;
#define VPX_CO(K)                                                                                                      \
    case K:                                                                                                            \
        if (wide_mfma) hipLaunchKernelGGL((calib_coissue_kernel<K, true>), dim3(blocks), dim3(kCalibThreads), 0, s, static_cast<v4i*>(sink), iters, mode); \
        else hipLaunchKernelGGL((calib_coissue_kernel<K, false>), dim3(blocks), dim3(kCalibThreads), 0, s, static_cast<v4i*>(sink), iters, mode); \
        break
    switch (valu_kind) {
        VPX_CO(CO_FMA_F64);
        VPX_CO(CO_FMA_F32);
        VPX_CO(CO_ADD_U32);
        VPX_CO(CO_MUL_LO_U32);
        VPX_CO(CO_MAD_U64_U32);
    default:
        VPX_CO(CO_CVT_F64_I32);
    }
#undef VPX_CO
    if (hipGetLastError() != hipSuccess) return fail(VPX_RESULT_ERROR_UNKNOWN, "calib_coissue: launch failed");
    return VPX_RESULT_SUCCESS;
}

int calib_mfma_i8(const void* operands, void* sink, int iters, int fragment_reads, int64_t* ops, hipStream_t s) {
    if (!operands || !sink || iters < 1) return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT, "calib_mfma_i8: null buffer or iters < 1");
    int blocks = 0;
    if (const int rc = device_compute_units(&blocks)) return rc;
    if (blocks <= 0) return fail(VPX_RESULT_ERROR_UNKNOWN, "calib_mfma_i8: no compute units reported");
    if (const int fewer = tuning_calib_blocks(); fewer > 0 && fewer < blocks) blocks = fewer;
    const auto kernel = fragment_reads ? calib_mfma_i8_kernel<true> : calib_mfma_i8_kernel<false>;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kCalibLds) != hipSuccess)
        return fail(VPX_RESULT_ERROR_UNKNOWN, "calib_mfma_i8: cannot reserve 64 KiB of LDS");
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(kCalibThreads), kCalibLds, s, static_cast<const v4i*>(operands),
                       static_cast<v4i*>(sink), iters);
    if (hipGetLastError() != hipSuccess) return fail(VPX_RESULT_ERROR_UNKNOWN, "calib_mfma_i8: launch failed");
    // sixteen MFMAs of 2 * 32 * 32 * 32 operations per iteration and wave
    if (ops) *ops = (int64_t)iters * 16 * 65536 * (kCalibThreads / 64) * blocks;
    return VPX_RESULT_SUCCESS;
}

}  // namespace vpx
