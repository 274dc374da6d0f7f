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

}  // namespace

int calib_mfma_i8(const void* operands, void* sink, int iters, int fragment_reads, int64_t* ops, hipStream_t s) {
    if (!operands || !sink || iters < 1) return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT, "calib_mfma_i8: null buffer or iters < 1");
    int blocks = 0;
    if (const int rc = device_compute_units(&blocks)) return rc;
    if (blocks <= 0) return fail(VPX_RESULT_ERROR_UNKNOWN, "calib_mfma_i8: no compute units reported");
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
