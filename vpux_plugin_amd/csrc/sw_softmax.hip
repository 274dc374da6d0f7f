// ACT-SHAVE `softmax` / `softmaxFp32`: y = exp(x - max) / sum(exp(x - max)) along one axis,
// fp32 arithmetic inside, driven by the packed {axis, pad, dims, strides} parameters the compiler
// writes (src/vpux_compiler/src/dialect/VPUIP/transforms/passes/update_sw_kernel_params.cpp:36-147).
//
// Device paths:
//   rows_wave  : reduction axis is the innermost, contiguous one and a row fits the registers of one
//                wavefront (up to 4096 fp16 / 2048 fp32 values): one 64-lane wave owns a row, 128-bit
//                loads, max and sum by DPP/swizzle butterflies, single pass over HBM.  fp16 rows
//                without padding take rows_f16, the same scheme with about half the
//                instructions (packed-half maximum, mixed-precision fma); it also serves rows of
//                up to 32768 values (one workgroup per row) and rows that are not 16-byte aligned.
//   rows_block : innermost axis of any length or alignment: one workgroup per row, three passes.
//   slabs      : fp16 reduction over an outer axis of up to 1024 steps with contiguous inner
//                dimensions: the whole [axis x 512 columns] slab of a workgroup sits in registers.
//   lines      : any other reduction over an outer (strided) axis: one lane per line, lanes adjacent
//                along the innermost dimension so every step of the axis is a coalesced access.
#include <type_traits>

#include <cstdlib>

#include "vpx_common.h"

namespace vpx {

namespace {

typedef _Float16 half_t;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr float kLog2e = 1.4426950408889634f;

struct MaxOp {
    __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); }
};
struct SumOp {
    __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};

template <int CTRL>
__device__ __forceinline__ float dpp(float v) {
    const int i = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(i, i, CTRL, 0xf, 0xf, true));
}

// All-reduce over the 64 lanes of a wavefront; every lane returns the same value.
template <class Op>
__device__ __forceinline__ float wave_allreduce(float v, Op op) {
    v = op(v, dpp<0xB1>(v));   // quad_perm [1,0,3,2]
    v = op(v, dpp<0x4E>(v));   // quad_perm [2,3,0,1]
    v = op(v, dpp<0x141>(v));  // row_half_mirror: the other quad of each 8 lanes
    v = op(v, dpp<0x140>(v));  // row_mirror: the other half of each 16 lanes
    v = op(v, __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F)));  // lane ^ 16
    const float lo = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    const float hi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    return op(lo, hi);
}

__device__ __forceinline__ float fast_exp(float x) {
    return __builtin_amdgcn_exp2f(x * kLog2e);
}

struct RowMap {
    int nd;                       // outer dimensions (all but the axis)
    int64_t dims[VPX_MAX_ND_DIMS];
    int64_t in_stride[VPX_MAX_ND_DIMS];
    int64_t out_stride[VPX_MAX_ND_DIMS];
};

// The outermost dimension needs no division, and the host merges dimensions that are contiguous
// in both operands, so a compact tensor costs one multiplication per row.
__device__ __forceinline__ void row_offsets(const RowMap& m, int64_t row, int64_t& in_off, int64_t& out_off) {
    if (m.nd == 1) {
        in_off = row * m.in_stride[0];
        out_off = row * m.out_stride[0];
        return;
    }
    in_off = 0;
    out_off = 0;
    for (int d = 0; d + 1 < m.nd; d++) {
        const int64_t q = row / m.dims[d];
        const int64_t r = row - q * m.dims[d];
        row = q;
        in_off += r * m.in_stride[d];
        out_off += r * m.out_stride[d];
    }
    if (m.nd > 0) {
        in_off += row * m.in_stride[m.nd - 1];
        out_off += row * m.out_stride[m.nd - 1];
    }
}

template <typename T>
struct VecTraits;
template <>
struct VecTraits<half_t> {
    static constexpr int N = 8;
};
template <>
struct VecTraits<float> {
    static constexpr int N = 4;
};

// ---------------------------------------------------------------- rows_wave
// NV 128-bit vectors per lane; ROWS rows per wave in flight.  `valid` = axis length minus padding.
template <typename T, int NV, int ROWS>
__global__ __launch_bounds__(256) void softmax_rows_wave(const T* __restrict__ in, T* __restrict__ out, RowMap map,
                                                         int64_t rows, int len, int valid) {
    constexpr int N = VecTraits<T>::N;
    const int lane = threadIdx.x & 63;
    // wave-uniform, so the row addressing below runs on the scalar unit
    const int64_t wave = (int64_t)blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t row0 = wave * ROWS;
    if (row0 >= rows) return;

    float x[ROWS][NV][N];
    int64_t ooff[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        const int64_t row = row0 + r < rows ? row0 + r : rows - 1;  // clamp: duplicates are not stored
        int64_t ioff;
        row_offsets(map, row, ioff, ooff[r]);
#pragma unroll
        for (int j = 0; j < NV; j++) {
            const int e0 = (j * 64 + lane) * N;
            if (e0 < len) {
                const u32x4 q = *reinterpret_cast<const u32x4*>(in + ioff + e0);
                const T* p = reinterpret_cast<const T*>(&q);
#pragma unroll
                for (int k = 0; k < N; k++) x[r][j][k] = e0 + k < valid ? (float)p[k] : -INFINITY;
            } else {
#pragma unroll
                for (int k = 0; k < N; k++) x[r][j][k] = -INFINITY;
            }
        }
    }
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        float m = -INFINITY;
#pragma unroll
        for (int j = 0; j < NV; j++)
#pragma unroll
            for (int k = 0; k < N; k++) m = fmaxf(m, x[r][j][k]);
        m = wave_allreduce(m, MaxOp{});
        const float mb = m * kLog2e;
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < NV; j++)
#pragma unroll
            for (int k = 0; k < N; k++) {
                // exp(x - m) as exp2(x*log2e - m*log2e); padded slots hold -inf and give 0
                const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(x[r][j][k], kLog2e, -mb));
                x[r][j][k] = e;
                s += e;
            }
        s = wave_allreduce(s, SumOp{});
        const float inv = 1.0f / s;
        if (row0 + r < rows) {
#pragma unroll
            for (int j = 0; j < NV; j++) {
                const int e0 = (j * 64 + lane) * N;
                if (e0 < len) {
                    u32x4 q;
                    T* p = reinterpret_cast<T*>(&q);
#pragma unroll
                    for (int k = 0; k < N; k++) p[k] = (T)(e0 + k < valid ? x[r][j][k] * inv : 0.f);
                    __builtin_nontemporal_store(q, reinterpret_cast<u32x4*>(out + ooff[r] + e0));
                }
            }
        }
    }
}

// fp16 rows without padding: the variant that serves the common case with the fewest
// instructions, because at one row per wave the kernel is otherwise bound by instruction issue,
// not by memory.  The maximum is taken on packed halves (exact); x*log2(e) - m*log2(e) is one
// mixed-precision fma that reads the half directly; the scaled result is rounded to half once.
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));

template <int CTRL>
__device__ __forceinline__ half2_t dpp_h2(half2_t v) {
    const int i = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(half2_t, __builtin_amdgcn_update_dpp(i, i, CTRL, 0xf, 0xf, true));
}

// LANES = 64: a wave owns ROWS rows (4 waves of a workgroup work independently);
// LANES = 256: the workgroup owns one row (rows of up to 32768 values), reductions cross LDS.
// MISALIGNED: rows start anywhere (odd lengths); the row is read through 16-byte-aligned vectors
// that may stick out at both ends -- those slots are masked to -inf, which makes them 0 after the
// exponential -- and the two ragged ends are stored value by value.  Input and output rows must
// be misaligned by the same amount.
template <int NV, int ROWS, int LANES, bool MISALIGNED, bool READ_ONCE>
__global__ __launch_bounds__(256) void softmax_rows_f16(const half_t* __restrict__ in, half_t* __restrict__ out,
                                                        RowMap map, int64_t rows, int len) {
    static_assert(LANES == 64 || (LANES == 256 && ROWS == 1), "a workgroup-wide row comes alone");
    __shared__ float red[2][4];
    const int lane = LANES == 64 ? (threadIdx.x & 63) : threadIdx.x;
    const int64_t unit = LANES == 64 ? (int64_t)blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) : blockIdx.x;
    const int64_t row0 = unit * ROWS;
    if (row0 >= rows) return;

    half8_t h[ROWS][NV];
    int64_t ooff[ROWS];
    int mis[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        const int64_t row = row0 + r < rows ? row0 + r : rows - 1;  // clamp: duplicates are not stored
        int64_t ioff;
        row_offsets(map, row, ioff, ooff[r]);
        mis[r] = MISALIGNED ? (int)((reinterpret_cast<uintptr_t>(in + ioff) >> 1) & 7) : 0;
        const half_t* src = in + ioff - mis[r];
        const int end = len + mis[r];
#pragma unroll
        for (int j = 0; j < NV; j++) {
            const int e0 = (j * LANES + lane) * 8;
            if (e0 < end) {
                // (a tensor beyond the caches is marked read-once on its way in: [8,16,512,512] 0.69 -> 0.72 of the HBM
                // peak when nothing of it is cached; smaller ones keep the plain load, which finds what the last kernel left)
                if constexpr (READ_ONCE) h[r][j] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(src + e0));
                else h[r][j] = *reinterpret_cast<const half8_t*>(src + e0);
                if (MISALIGNED && (e0 < mis[r] || e0 + 8 > end)) {
#pragma unroll
                    for (int k = 0; k < 8; k++)
                        if (e0 + k < mis[r] || e0 + k >= end) h[r][j][k] = (half_t)-INFINITY;
                }
            } else {
#pragma unroll
                for (int k = 0; k < 8; k++) h[r][j][k] = (half_t)-INFINITY;
            }
        }
    }
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        half8_t m8 = h[r][0];
#pragma unroll
        for (int j = 1; j < NV; j++) m8 = __builtin_elementwise_max(m8, h[r][j]);
        const half4_t m4 = __builtin_elementwise_max(__builtin_shufflevector(m8, m8, 0, 1, 2, 3),
                                                     __builtin_shufflevector(m8, m8, 4, 5, 6, 7));
        half2_t m2 = __builtin_elementwise_max(__builtin_shufflevector(m4, m4, 0, 1), __builtin_shufflevector(m4, m4, 2, 3));
        m2 = __builtin_elementwise_max(m2, dpp_h2<0xB1>(m2));
        m2 = __builtin_elementwise_max(m2, dpp_h2<0x4E>(m2));
        m2 = __builtin_elementwise_max(m2, dpp_h2<0x141>(m2));
        m2 = __builtin_elementwise_max(m2, dpp_h2<0x140>(m2));
        m2 = __builtin_elementwise_max(
                m2, __builtin_bit_cast(half2_t, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, m2), 0x401F)));
        const half2_t lo = __builtin_bit_cast(half2_t, __builtin_amdgcn_readlane(__builtin_bit_cast(int, m2), 0));
        const half2_t hi = __builtin_bit_cast(half2_t, __builtin_amdgcn_readlane(__builtin_bit_cast(int, m2), 32));
        m2 = __builtin_elementwise_max(lo, hi);
        float m = fmaxf((float)m2[0], (float)m2[1]);
        if (LANES == 256) {
            if ((threadIdx.x & 63) == 0) red[0][threadIdx.x >> 6] = m;
            __syncthreads();
            m = fmaxf(fmaxf(red[0][0], red[0][1]), fmaxf(red[0][2], red[0][3]));
        }
        const float nmb = -m * kLog2e;

        float e[NV][8];
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < NV; j++)
#pragma unroll
            for (int k = 0; k < 8; k++) {
                e[j][k] = __builtin_amdgcn_exp2f(__builtin_fmaf((float)h[r][j][k], kLog2e, nmb));
                s += e[j][k];
            }
        s = wave_allreduce(s, SumOp{});
        if (LANES == 256) {
            if ((threadIdx.x & 63) == 0) red[1][threadIdx.x >> 6] = s;
            __syncthreads();
            s = (red[1][0] + red[1][1]) + (red[1][2] + red[1][3]);
        }
        const float inv = __builtin_amdgcn_rcpf(s);  // 1 ulp, far inside the tolerance of the fp16 result
        if (row0 + r < rows) {
            half_t* dst = out + ooff[r] - mis[r];
            const int end = len + mis[r];
#pragma unroll
            for (int j = 0; j < NV; j++) {
                const int e0 = (j * LANES + lane) * 8;
                if (e0 < end) {
                    u32x4 q;
                    half_t* qh = reinterpret_cast<half_t*>(&q);
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        const half2_t v = {(half_t)(e[j][2 * k] * inv), (half_t)(e[j][2 * k + 1] * inv)};
                        q[k] = __builtin_bit_cast(uint32_t, v);
                    }
                    if (!MISALIGNED || (e0 >= mis[r] && e0 + 8 <= end)) {
                        __builtin_nontemporal_store(q, reinterpret_cast<u32x4*>(dst + e0));
                    } else {
#pragma unroll
                        for (int k = 0; k < 8; k++)
                            if (e0 + k >= mis[r] && e0 + k < end) dst[e0 + k] = qh[k];
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------- rows_block
__device__ __forceinline__ float block_allreduce_max(float v, float* smem) {
    v = wave_allreduce(v, MaxOp{});
    const int w = threadIdx.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) smem[w] = v;
    __syncthreads();
    return fmaxf(fmaxf(smem[0], smem[1]), fmaxf(smem[2], smem[3]));
}
__device__ __forceinline__ float block_allreduce_sum(float v, float* smem) {
    v = wave_allreduce(v, SumOp{});
    const int w = threadIdx.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) smem[w] = v;
    __syncthreads();
    return (smem[0] + smem[1]) + (smem[2] + smem[3]);
}

template <typename T>
__global__ __launch_bounds__(256) void softmax_rows_block(const T* __restrict__ in, T* __restrict__ out, RowMap map,
                                                          int64_t len, int64_t valid, int64_t in_es, int64_t out_es) {
    __shared__ float smem[4];
    int64_t ioff, ooff;
    row_offsets(map, blockIdx.x, ioff, ooff);
    const T* px = in + ioff;
    T* py = out + ooff;
    float m = -INFINITY;
    for (int64_t i = threadIdx.x; i < valid; i += 256) m = fmaxf(m, (float)px[i * in_es]);
    m = block_allreduce_max(m, smem);
    float s = 0.f;
    for (int64_t i = threadIdx.x; i < valid; i += 256) s += fast_exp((float)px[i * in_es] - m);
    s = block_allreduce_sum(s, smem);
    const float inv = 1.0f / s;
    for (int64_t i = threadIdx.x; i < len; i += 256)
        py[i * out_es] = (T)(i < valid ? fast_exp((float)px[i * in_es] - m) * inv : 0.f);
}

// ---------------------------------------------------------------- lines (outer axis)
template <typename T>
__global__ __launch_bounds__(256) void softmax_lines(const T* __restrict__ in, T* __restrict__ out, RowMap map,
                                                     int64_t lines, int64_t len, int64_t valid, int64_t in_as,
                                                     int64_t out_as) {
    const int64_t line = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (line >= lines) return;
    int64_t ioff, ooff;
    row_offsets(map, line, ioff, ooff);
    const T* px = in + ioff;
    T* py = out + ooff;
    // one pass keeps a running maximum and a sum rescaled whenever the maximum grows
    float m = -INFINITY, s = 0.f;
    for (int64_t a = 0; a < valid; a++) {
        const float v = (float)px[a * in_as];
        const float nm = fmaxf(m, v);
        if (nm > -INFINITY) s = s * fast_exp(m - nm) + fast_exp(v - nm);
        m = nm;
    }
    const float inv = 1.0f / s;
    for (int64_t a = 0; a < len; a++)
        py[a * out_as] = (T)(a < valid ? fast_exp((float)px[a * in_as] - m) * inv : 0.f);
}

// ---------------------------------------------------------------- slabs (outer axis, fp16)
// Reduction over an outer axis whose inner dimensions are contiguous: the tensor is
// [outer][axis L][inner I].  A tile is every step of the axis x 64*VEC adjacent inner positions of
// one outer index; lane l owns VEC adjacent columns, so each step of the axis is one contiguous
// access of the wave.  KW waves share a tile, wave w taking steps w, w+KW, ...; all values of the
// tile stay in registers (packed halves) between the single read and the single write, column
// maxima and sums of the KW waves meet in LDS.  The exponential is evaluated twice (for the sum and
// for the result) instead of keeping fp32 copies, which would not fit the registers.
template <int VEC, int KW, int SMAX>
__global__ __launch_bounds__(KW == 1 ? 256 : 64 * KW) void softmax_slab_f16(const half_t* __restrict__ in,
                                                                           half_t* __restrict__ out, RowMap outer_map,
                                                                           int64_t tiles, int tiles_per_outer, int L, int I,
                                                                           int64_t in_as, int64_t out_as) {
    typedef _Float16 hvec __attribute__((ext_vector_type(VEC)));
    typedef float fvec __attribute__((ext_vector_type(VEC)));
    __shared__ hvec smax[KW == 1 ? 1 : KW][64];
    __shared__ fvec ssum[KW == 1 ? 1 : KW][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t tile = KW == 1 ? (int64_t)blockIdx.x * 4 + wave : blockIdx.x;
    if (tile >= tiles) return;
    const int kw = KW == 1 ? 0 : wave;  // which share of the axis this wave takes
    const int64_t outer = tile / tiles_per_outer;
    const int col = (int)(tile - outer * tiles_per_outer) * 64 * VEC + lane * VEC;
    int64_t ioff, ooff;
    row_offsets(outer_map, outer, ioff, ooff);
    const bool live = col < I;
    const half_t* src = in + ioff + col;
    half_t* dst = out + ooff + col;

    hvec h[SMAX];
    hvec m;
#pragma unroll
    for (int k = 0; k < VEC; k++) m[k] = (half_t)-INFINITY;
#pragma unroll
    for (int i = 0; i < SMAX; i++) {
        const int a = kw + KW * i;
        h[i] = m;  // -inf
        if (live && a < L) h[i] = *reinterpret_cast<const hvec*>(src + a * in_as);
    }
#pragma unroll
    for (int i = 0; i < SMAX; i++) m = __builtin_elementwise_max(m, h[i]);
    if (KW > 1) {
        smax[kw][lane] = m;
        __syncthreads();
#pragma unroll
        for (int w = 0; w < KW; w++) m = __builtin_elementwise_max(m, smax[w][lane]);
    }
    fvec nmb, sum;
#pragma unroll
    for (int k = 0; k < VEC; k++) {
        nmb[k] = -(float)m[k] * kLog2e;
        sum[k] = 0.f;
    }
#pragma unroll
    for (int i = 0; i < SMAX; i++)
#pragma unroll
        for (int k = 0; k < VEC; k++) sum[k] += __builtin_amdgcn_exp2f(__builtin_fmaf((float)h[i][k], kLog2e, nmb[k]));
    if (KW > 1) {
        ssum[kw][lane] = sum;
        __syncthreads();
#pragma unroll
        for (int k = 0; k < VEC; k++) sum[k] = 0.f;
#pragma unroll
        for (int w = 0; w < KW; w++) sum += ssum[w][lane];  // same order in every wave
    }
    fvec inv;
#pragma unroll
    for (int k = 0; k < VEC; k++) {
        inv[k] = __builtin_amdgcn_rcpf(sum[k]);
        // hide the value's origin: otherwise the exponents of the summation pass are kept for reuse, one
        // fp32 register per value, which is exactly what does not fit
        asm volatile("" : "+v"(nmb[k]));
    }
#pragma unroll
    for (int i = 0; i < SMAX; i++) {
        const int a = kw + KW * i;
        if (live && a < L) {
            hvec r;
#pragma unroll
            for (int k = 0; k < VEC; k++)
                r[k] = (half_t)(__builtin_amdgcn_exp2f(__builtin_fmaf((float)h[i][k], kLog2e, nmb[k])) * inv[k]);
            __builtin_nontemporal_store(r, reinterpret_cast<hvec*>(dst + a * out_as));
        }
    }
}

// Packed, aligned fp16 rows of 8, 16, 32, 64, 128 or 256 values: T = len / 8 adjacent lanes hold a row, one 128-bit
// word each, so a wavefront's accesses are one contiguous run, and the row's maximum and sum cross the T lanes by DPP
// (and one 16-lane swap for the longest).
template <int T>
__global__ __launch_bounds__(256) void softmax_tiny_rows_f16(const half_t* __restrict__ in, half_t* __restrict__ out, int64_t n_vec) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (v >= n_vec) return;  // n_vec is a multiple of T and so is 256: a row's lanes leave together
    const u32x4 q = reinterpret_cast<const u32x4*>(in)[v];
    const half_t* h = reinterpret_cast<const half_t*>(&q);
    float x[8];
    float m = -INFINITY;
#pragma unroll
    for (int k = 0; k < 8; k++) {
        x[k] = (float)h[k];
        m = fmaxf(m, x[k]);
    }
    auto across = [](float a, auto op) {
        if (T >= 2) a = op(a, dpp<0xB1>(a));
        if (T >= 4) a = op(a, dpp<0x4E>(a));
        if (T >= 8) a = op(a, dpp<0x141>(a));
        if (T >= 16) a = op(a, dpp<0x140>(a));
        if (T >= 32) a = op(a, __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, a), 0x401F)));  // lane ^ 16
        return a;
    };
    m = across(m, [](float a, float b) { return fmaxf(a, b); });
    const float nmb = -m * kLog2e;
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < 8; k++) {
        x[k] = __builtin_amdgcn_exp2f(__builtin_fmaf(x[k], kLog2e, nmb));
        s += x[k];
    }
    s = across(s, [](float a, float b) { return a + b; });
    const float inv = 1.0f / s;
    u32x4 o;
    half_t* ho = reinterpret_cast<half_t*>(&o);
#pragma unroll
    for (int k = 0; k < 8; k++) ho[k] = (half_t)(x[k] * inv);
    __builtin_nontemporal_store(o, reinterpret_cast<u32x4*>(out) + v);
}

// Many short fp16 rows that follow one another in memory (rows of 32 ... 1024 values, any length: 197 as well as
// 64): a workgroup takes a run of whole rows of about 4096 values, moves it between global memory and LDS in aligned
// 128-bit words whatever the row length (values of neighbouring rows that share its first and last word are read
// too, never written), and every half-wavefront handles one row at a time with the row's values in registers.
constexpr int kShortRow = 1024;
constexpr int kShortChunk = 4096;
// All-reduce over the 32 lanes of half a wavefront: four DPP steps and one 16-lane swap, which all stay inside the half.
template <class Op>
__device__ __forceinline__ float half_wave_allreduce(float v, Op op) {
    v = op(v, dpp<0xB1>(v));
    v = op(v, dpp<0x4E>(v));
    v = op(v, dpp<0x141>(v));
    v = op(v, dpp<0x140>(v));
    return op(v, __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F)));
}
__device__ __forceinline__ float half_wave_max(float v) {
    return half_wave_allreduce(v, [](float a, float b) { return fmaxf(a, b); });
}
__device__ __forceinline__ float half_wave_sum(float v) {
    return half_wave_allreduce(v, [](float a, float b) { return a + b; });
}
template <int K>  // values per lane: a row has at most 32 K
__global__ __launch_bounds__(256) void softmax_short_rows_f16(const half_t* __restrict__ in, half_t* __restrict__ out, int64_t rows,
                                                              int len, int per_wg) {
    __shared__ __attribute__((aligned(16))) half_t buf[kShortChunk + 16];
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const int64_t r0 = (int64_t)blockIdx.x * per_wg;
    const int nr = rows - r0 < per_wg ? (int)(rows - r0) : per_wg;
    const int64_t e0 = r0 * len, e1 = e0 + (int64_t)nr * len, total = rows * len;
    const int64_t a0 = e0 & ~7ll;
    const int words = (int)((e1 - a0 + 7) >> 3);
    for (int w = threadIdx.x; w < words; w += 256) {
        const int64_t at = a0 + (int64_t)w * 8;
        if (at + 8 <= total) {
            *reinterpret_cast<u32x4*>(buf + w * 8) = *reinterpret_cast<const u32x4*>(in + at);
        } else {
            for (int k = 0; k < 8; k++) buf[w * 8 + k] = at + k < total ? in[at + k] : (half_t)0.f;
        }
    }
    __syncthreads();
    const int lane = threadIdx.x & 31, team = threadIdx.x >> 5;
    for (int r = team; r < nr; r += 8) {  // uniform per half-wavefront
        half_t* x = buf + (int)(e0 - a0) + r * len;
        float v[K];
        float m = -INFINITY;
#pragma unroll
        for (int k = 0; k < K; k++) {
            const int i = lane + 32 * k;
            v[k] = i < len ? (float)x[i] : -INFINITY;
            m = fmaxf(m, v[k]);
        }
        m = half_wave_max(m);
        const float nmb = -m * kLog2e;
        float sum = 0.f;
#pragma unroll
        for (int k = 0; k < K; k++) {
            v[k] = __builtin_amdgcn_exp2f(__builtin_fmaf(v[k], kLog2e, nmb));  // exp2(-inf) = 0 for the slots past the row
            sum += v[k];
        }
        const float inv = 1.0f / half_wave_sum(sum);
#pragma unroll
        for (int k = 0; k < K; k++) {
            const int i = lane + 32 * k;
            if (i < len) x[i] = (half_t)(v[k] * inv);
        }
    }
    __syncthreads();
    for (int w = threadIdx.x; w < words; w += 256) {
        const int64_t at = a0 + (int64_t)w * 8;
        if (at >= e0 && at + 8 <= e1) {
            __builtin_nontemporal_store(*reinterpret_cast<const u32x4*>(buf + w * 8), reinterpret_cast<u32x4*>(out + at));
        } else {
            for (int k = 0; k < 8; k++)
                if (at + k >= e0 && at + k < e1) out[at + k] = buf[w * 8 + k];
        }
    }
}

// fp16 rows of up to 76 800 values (a 50 257- or 65 536-entry vocabulary), aligned: the row stays in the LDS of one
// 1024-lane workgroup, so memory is read once: maximum on the way in, the sum of exponentials and the quotients
// from LDS.
constexpr int kLdsRowMax = 76800;
__global__ __launch_bounds__(1024) void softmax_lds_rows_f16(const half_t* __restrict__ in, half_t* __restrict__ out, RowMap map, int len) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    extern __shared__ __attribute__((aligned(16))) u32x4 row[];
    __shared__ float red[16];
    int64_t ioff, ooff;
    row_offsets(map, blockIdx.x, ioff, ooff);
    const u32x4* px = reinterpret_cast<const u32x4*>(in + ioff);
    u32x4* py = reinterpret_cast<u32x4*>(out + ooff);
    const int nvec = len / 8, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float m = -INFINITY;
    for (int v = threadIdx.x; v < nvec; v += 1024) {
        const u32x4 q = px[v];
        row[v] = q;
        const half_t* h = reinterpret_cast<const half_t*>(&q);
#pragma unroll
        for (int k = 0; k < 8; k++) m = fmaxf(m, (float)h[k]);
    }
    m = wave_allreduce(m, [](float a, float b) { return fmaxf(a, b); });
    if (lane == 0) red[wave] = m;
    __syncthreads();
    m = red[0];
#pragma unroll
    for (int w = 1; w < 16; w++) m = fmaxf(m, red[w]);
    const float nmb = -m * kLog2e;
    float s = 0.f;
    for (int v = threadIdx.x; v < nvec; v += 1024) {
        const u32x4 q = row[v];
        const half_t* h = reinterpret_cast<const half_t*>(&q);
#pragma unroll
        for (int k = 0; k < 8; k++) s += __builtin_amdgcn_exp2f(__builtin_fmaf((float)h[k], kLog2e, nmb));
    }
    s = wave_allreduce(s, [](float a, float b) { return a + b; });
    __syncthreads();
    if (lane == 0) red[wave] = s;
    __syncthreads();
    s = 0.f;
#pragma unroll
    for (int w = 0; w < 16; w++) s += red[w];
    const float inv = 1.0f / s;
    for (int v = threadIdx.x; v < nvec; v += 1024) {
        const u32x4 q = row[v];
        const half_t* h = reinterpret_cast<const half_t*>(&q);
        u32x4 o;
        half_t* ho = reinterpret_cast<half_t*>(&o);
#pragma unroll
        for (int k = 0; k < 8; k++) ho[k] = (half_t)(__builtin_amdgcn_exp2f(__builtin_fmaf((float)h[k], kLog2e, nmb)) * inv);
        __builtin_nontemporal_store(o, py + v);
    }
}

// Rows longer than the registers of a workgroup hold (a vocabulary of 128 K entries): one workgroup of 1024 lanes per
// row, a first pass that keeps a running maximum and a sum rescaled to it per lane (128-bit loads where the row is
// aligned), and a second pass over the row -- by then in L2 -- that writes the quotients.
template <typename T>
__global__ __launch_bounds__(1024) void softmax_long_rows(const T* __restrict__ in, T* __restrict__ out, RowMap map, int64_t len,
                                                          int64_t valid) {
    __shared__ float red_m[16], red_s[16];
    int64_t ioff, ooff;
    row_offsets(map, blockIdx.x, ioff, ooff);
    const T* px = in + ioff;
    T* py = out + ooff;
    constexpr int N = VecTraits<T>::N;
    typedef uint32_t Vec __attribute__((ext_vector_type(4)));  // 16 bytes: eight fp16 or four fp32 values
    const bool vec = valid % N == 0 && (reinterpret_cast<uintptr_t>(px) & 15) == 0 && (reinterpret_cast<uintptr_t>(py) & 15) == 0;
    float m = -INFINITY, s = 0.f;
    auto push = [&](float x) {
        if (x > m) {
            s *= fast_exp(m - x);  // exp(-inf) = 0 on the first value
            m = x;
        }
        s += fast_exp(x - m);
    };
    if (vec) {
        for (int64_t i = (int64_t)threadIdx.x * N; i < valid; i += 1024 * N) {
            const Vec q = *reinterpret_cast<const Vec*>(px + i);
            const T* e = reinterpret_cast<const T*>(&q);
            float lm = (float)e[0];
#pragma unroll
            for (int k = 1; k < N; k++) lm = fmaxf(lm, (float)e[k]);
            if (lm > m) {
                s *= fast_exp(m - lm);
                m = lm;
            }
#pragma unroll
            for (int k = 0; k < N; k++) s += fast_exp((float)e[k] - m);
        }
    } else {
        for (int64_t i = threadIdx.x; i < valid; i += 1024) push((float)px[i]);
    }
    // combine the lanes: maximum first, then the sums rescaled to it
    float wm = m;
    for (int o = 32; o > 0; o >>= 1) wm = fmaxf(wm, __shfl_xor(wm, o, 64));
    float ws = m == -INFINITY ? 0.f : s * fast_exp(m - wm);
    for (int o = 32; o > 0; o >>= 1) ws += __shfl_xor(ws, o, 64);
    if ((threadIdx.x & 63) == 0) {
        red_m[threadIdx.x >> 6] = wm;
        red_s[threadIdx.x >> 6] = ws;
    }
    __syncthreads();
    float M = red_m[0];
    for (int w = 1; w < 16; w++) M = fmaxf(M, red_m[w]);
    float S = 0.f;
    for (int w = 0; w < 16; w++) S += red_m[w] == -INFINITY ? 0.f : red_s[w] * fast_exp(red_m[w] - M);
    const float inv = 1.0f / S;
    if (vec) {
        for (int64_t i = (int64_t)threadIdx.x * N; i < valid; i += 1024 * N) {
            const Vec q = *reinterpret_cast<const Vec*>(px + i);
            const T* e = reinterpret_cast<const T*>(&q);
            Vec y;
            T* ye = reinterpret_cast<T*>(&y);
#pragma unroll
            for (int k = 0; k < N; k++) ye[k] = (T)(fast_exp((float)e[k] - M) * inv);
            *reinterpret_cast<Vec*>(py + i) = y;
        }
    } else {
        for (int64_t i = threadIdx.x; i < valid; i += 1024) py[i] = (T)(fast_exp((float)px[i] - M) * inv);
    }
    for (int64_t i = valid + threadIdx.x; i < len; i += 1024) py[i] = (T)0.f;  // padded tail, as the other kernels write it
}

// Softmax over an outer axis that is too long for the register slabs: a workgroup of 16 wavefronts takes VEC x 64
// adjacent columns of the contiguous inner run, its wavefronts split the steps of the axis and keep, per column, a
// running maximum and a sum rescaled to it; they meet in LDS, and a second pass over the same steps -- by then in
// cache -- writes the quotients.  `om` maps the dimensions above the axis.
template <typename T, int VEC>
__global__ __launch_bounds__(1024) void softmax_cols(const T* __restrict__ in, T* __restrict__ out, RowMap om, int tiles_per_outer,
                                                     int64_t len, int64_t valid, int64_t inner, int64_t in_as, int64_t out_as) {
    constexpr int KW = 16;
    __shared__ float sm[KW][64 * VEC], ss[KW][64 * VEC];
    typedef T Vec __attribute__((ext_vector_type(VEC)));
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t outer = blockIdx.x / tiles_per_outer;
    const int64_t c0 = (int64_t)(blockIdx.x % tiles_per_outer) * (64 * VEC) + lane * VEC;
    const bool live = c0 < inner;  // inner is a multiple of VEC
    int64_t ioff = 0, ooff = 0;
    if (om.nd > 0) row_offsets(om, outer, ioff, ooff);
    const T* px = in + ioff + (live ? c0 : 0);
    T* py = out + ooff + (live ? c0 : 0);
    float m[VEC], s[VEC];
#pragma unroll
    for (int k = 0; k < VEC; k++) {
        m[k] = -INFINITY;
        s[k] = 0.f;
    }
    // eight steps at a time: their loads are in flight together, and the running sum is rescaled once per eight
    constexpr int B = 8;
    for (int64_t a0 = wave; a0 < valid; a0 += KW * B) {
        Vec q[B];
#pragma unroll
        for (int j = 0; j < B; j++) {
            const int64_t a = a0 + (int64_t)j * KW;
            if (a < valid) q[j] = *reinterpret_cast<const Vec*>(px + a * in_as);
        }
#pragma unroll
        for (int k = 0; k < VEC; k++) {
            float nm = m[k];
#pragma unroll
            for (int j = 0; j < B; j++)
                if (a0 + (int64_t)j * KW < valid) nm = fmaxf(nm, (float)q[j][k]);
            if (nm > -INFINITY) {
                float acc = s[k] * fast_exp(m[k] - nm);
#pragma unroll
                for (int j = 0; j < B; j++)
                    if (a0 + (int64_t)j * KW < valid) acc += fast_exp((float)q[j][k] - nm);
                s[k] = acc;
            }
            m[k] = nm;
        }
    }
#pragma unroll
    for (int k = 0; k < VEC; k++) {
        sm[wave][lane * VEC + k] = m[k];
        ss[wave][lane * VEC + k] = s[k];
    }
    __syncthreads();
    float inv[VEC];
#pragma unroll
    for (int k = 0; k < VEC; k++) {
        float M = sm[0][lane * VEC + k];
        for (int w = 1; w < KW; w++) M = fmaxf(M, sm[w][lane * VEC + k]);
        float S = 0.f;
        for (int w = 0; w < KW; w++) {
            const float mw = sm[w][lane * VEC + k];
            S += mw == -INFINITY ? 0.f : ss[w][lane * VEC + k] * fast_exp(mw - M);
        }
        m[k] = M;
        inv[k] = 1.0f / S;
    }
    if (!live) return;
    for (int64_t a0 = wave; a0 < len; a0 += KW * B) {
        Vec q[B];
#pragma unroll
        for (int j = 0; j < B; j++) {
            const int64_t a = a0 + (int64_t)j * KW;
            if (a < valid) q[j] = *reinterpret_cast<const Vec*>(px + a * in_as);
        }
#pragma unroll
        for (int j = 0; j < B; j++) {
            const int64_t a = a0 + (int64_t)j * KW;
            if (a >= len) break;
            Vec y;
#pragma unroll
            for (int k = 0; k < VEC; k++) y[k] = a < valid ? (T)(fast_exp((float)q[j][k] - m[k]) * inv[k]) : (T)0.f;
            *reinterpret_cast<Vec*>(py + a * out_as) = y;
        }
    }
}

template <typename T, int NV, int ROWS>
void launch_rows_wave(const T* in, T* out, const RowMap& map, int64_t rows, int len, int valid, hipStream_t s) {
    const int64_t waves = (rows + ROWS - 1) / ROWS;
    const unsigned blocks = (unsigned)((waves + 3) / 4);
    hipLaunchKernelGGL((softmax_rows_wave<T, NV, ROWS>), dim3(blocks), dim3(256), 0, s, in, out, map, rows, len, valid);
}

template <typename T>
int softmax_typed(const SoftmaxPlan& p, const T* in, T* out, hipStream_t s) {
    constexpr int N = VecTraits<T>::N;
    const int ax = p.axis;
    const int64_t len = p.dims[ax];
    const int64_t valid = len - p.pad;
    VPX_REQUIRE(valid > 0, VPX_RESULT_ERROR_INVALID_ARGUMENT, "softmax: padSize %d leaves no element on an axis of %lld",
                p.pad, (long long)len);
    RowMap map{};
    int64_t rows = 1;
    for (int d = 0; d < p.nd; d++) {
        if (d == ax) continue;
        rows *= p.dims[d];
        if (p.dims[d] == 1) continue;
        const int k = map.nd - 1;
        if (k >= 0 && p.in_stride[d] == map.dims[k] * map.in_stride[k] &&
            p.out_stride[d] == map.dims[k] * map.out_stride[k]) {
            map.dims[k] *= p.dims[d];  // contiguous with the previous one in both operands: one dimension
            continue;
        }
        map.dims[map.nd] = p.dims[d];
        map.in_stride[map.nd] = p.in_stride[d];
        map.out_stride[map.nd] = p.out_stride[d];
        map.nd++;
    }
    if (rows == 0 || len == 0) return VPX_RESULT_SUCCESS;
    VPX_REQUIRE(rows < (1ll << 31), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "softmax: %lld rows exceed the launch limit",
                (long long)rows);

    const bool inner = ax == 0 && p.in_stride[0] == 1 && p.out_stride[0] == 1;
    if (inner && std::is_same<T, half_t>::value && valid == len && len <= 256 * 8 * 16) {
        // fp16 rows without padding: registers hold the row; rows need not be 16-byte aligned as long as
        // input and output rows are misaligned alike
        const half_t* hin = reinterpret_cast<const half_t*>(in);
        half_t* hout = reinterpret_cast<half_t*>(out);
        bool aligned = len % 8 == 0 && (reinterpret_cast<uintptr_t>(in) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
        bool same_mis = ((reinterpret_cast<uintptr_t>(in) ^ reinterpret_cast<uintptr_t>(out)) & 15) == 0;
        for (int d = 0; d < map.nd; d++) {
            if (map.dims[d] == 1) continue;
            aligned = aligned && map.in_stride[d] % 8 == 0 && map.out_stride[d] % 8 == 0;
            same_mis = same_mis && (map.in_stride[d] - map.out_stride[d]) % 8 == 0;
        }
        // short rows, one after another in memory: runs of rows through LDS, half a wavefront per row
        const bool packed = map.nd == 0 || (map.nd == 1 && map.in_stride[0] == len && map.out_stride[0] == len);
        const bool base16 = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
        if (packed && base16 && (len == 8 || len == 16 || len == 32 || len == 64 || len == 128 || len == 256) && rows * (len / 8) < (1ll << 39)) {
            const int64_t n_vec = rows * (len / 8);
            const dim3 grid((unsigned)((n_vec + 255) / 256));
#define VPX_TINY(T) hipLaunchKernelGGL(softmax_tiny_rows_f16<T>, grid, dim3(256), 0, s, hin, hout, n_vec)
            if (len == 8) VPX_TINY(1);
            else if (len == 16) VPX_TINY(2);
            else if (len == 32) VPX_TINY(4);
            else if (len == 64) VPX_TINY(8);
            else if (len == 128) VPX_TINY(16);
            else VPX_TINY(32);
#undef VPX_TINY
            VPX_HIP_CHECK(hipGetLastError());
            return VPX_RESULT_SUCCESS;
        }
        if (packed && rows >= 64 && (len < 256 || (len % 8 != 0 && len <= 384)) && base16) {  // one wavefront per row idles lanes below 256 values
            const int per_wg = (int)(kShortChunk / len);
            const dim3 grid((unsigned)((rows + per_wg - 1) / per_wg));
#define VPX_SHORT(K) hipLaunchKernelGGL(softmax_short_rows_f16<K>, grid, dim3(256), 0, s, hin, hout, rows, (int)len, per_wg)
            if (len <= 32) VPX_SHORT(1);
            else if (len <= 64) VPX_SHORT(2);
            else if (len <= 128) VPX_SHORT(4);
            else if (len <= 256) VPX_SHORT(8);
            else VPX_SHORT(12);
#undef VPX_SHORT
            VPX_HIP_CHECK(hipGetLastError());
            return VPX_RESULT_SUCCESS;
        }
        if (aligned || same_mis) {
            const int l = (int)len;
            const bool once = rows * len >= (16ll << 20);  // 32 MB of input and more: read-once loads (aligned rows)
            const int span = aligned ? l : l + 7;  // aligned vectors a misaligned row can touch
            const dim3 block(256);
            const dim3 gw((unsigned)((rows + 3) / 4)), gb((unsigned)rows);
#define VPX_SM(NV, ROWS, LANES, GRID)                                                                                 \
    do {                                                                                                              \
        if (aligned && once) hipLaunchKernelGGL((softmax_rows_f16<NV, ROWS, LANES, false, true>), GRID, block, 0, s, hin, hout, map, rows, l); \
        else if (aligned) hipLaunchKernelGGL((softmax_rows_f16<NV, ROWS, LANES, false, false>), GRID, block, 0, s, hin, hout, map, rows, l); \
        else hipLaunchKernelGGL((softmax_rows_f16<NV, ROWS, LANES, true, false>), GRID, block, 0, s, hin, hout, map, rows, l);         \
    } while (0)
            // short rows, many of them: two rows per wave keep more bytes in flight (measured best)
            if (span <= 512 && rows >= 16384) VPX_SM(1, 2, 64, dim3((unsigned)((rows + 7) / 8)));
            else if (span <= 512) VPX_SM(1, 1, 64, gw);
            else if (span <= 1024) VPX_SM(2, 1, 64, gw);
            else if (span <= 2048) VPX_SM(4, 1, 64, gw);
            else if (span <= 4096 && rows >= 1024) VPX_SM(8, 1, 64, gw);
            else if (span <= 4096) VPX_SM(2, 1, 256, gb);
            else if (span <= 8192) VPX_SM(4, 1, 256, gb);
            else if (span <= 16384) VPX_SM(8, 1, 256, gb);
            else VPX_SM(16, 1, 256, gb);
#undef VPX_SM
            VPX_HIP_CHECK(hipGetLastError());
            return VPX_RESULT_SUCCESS;
        }
    }
    if (inner) {
        bool vec_ok = len % N == 0 && (reinterpret_cast<uintptr_t>(in) & 15) == 0 &&
                      (reinterpret_cast<uintptr_t>(out) & 15) == 0 && len <= 64 * N * 8;
        for (int d = 0; d < map.nd && vec_ok; d++)
            vec_ok = map.dims[d] == 1 || (map.in_stride[d] % N == 0 && map.out_stride[d] % N == 0);
        if (vec_ok) {
            const int l = (int)len, v = (int)valid;
            const int64_t per = 64 * N;
            // general form (fp32, padded axis)
            if (len <= per) launch_rows_wave<T, 1, 1>(in, out, map, rows, l, v, s);
            else if (len <= 2 * per) launch_rows_wave<T, 2, 1>(in, out, map, rows, l, v, s);
            else if (len <= 4 * per) launch_rows_wave<T, 4, 1>(in, out, map, rows, l, v, s);
            else launch_rows_wave<T, 8, 1>(in, out, map, rows, l, v, s);
            VPX_HIP_CHECK(hipGetLastError());
            return VPX_RESULT_SUCCESS;
        }
    }
    if (inner && std::is_same<T, half_t>::value && valid == len && len % 8 == 0 && len <= kLdsRowMax && rows >= 64 &&
        ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0) {
        bool al = true;
        for (int d = 0; d < map.nd; d++) al = al && (map.dims[d] == 1 || (map.in_stride[d] % 8 == 0 && map.out_stride[d] % 8 == 0));
        if (al) {
            VPX_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(softmax_lds_rows_f16), hipFuncAttributeMaxDynamicSharedMemorySize,
                                              kLdsRowMax * 2));
            hipLaunchKernelGGL(softmax_lds_rows_f16, dim3((unsigned)rows), dim3(1024), (size_t)len * 2, s, reinterpret_cast<const half_t*>(in),
                               reinterpret_cast<half_t*>(out), map, (int)len);
            VPX_HIP_CHECK(hipGetLastError());
            return VPX_RESULT_SUCCESS;
        }
    }
    if (ax == 0 && p.in_stride[0] == 1 && p.out_stride[0] == 1 && len >= 2048) {
        hipLaunchKernelGGL(softmax_long_rows<T>, dim3((unsigned)rows), dim3(1024), 0, s, in, out, map, len, valid);
        VPX_HIP_CHECK(hipGetLastError());
        return VPX_RESULT_SUCCESS;
    }
    if (ax == 0) {
        hipLaunchKernelGGL(softmax_rows_block<T>, dim3((unsigned)rows), dim3(256), 0, s, in, out, map, len, valid,
                           p.in_stride[0], p.out_stride[0]);
        VPX_HIP_CHECK(hipGetLastError());
        return VPX_RESULT_SUCCESS;
    }
    // fp16, outer axis, contiguous inner dimension: register-resident slabs
    if (std::is_same<T, half_t>::value && valid == len && len <= 1024 && p.in_stride[0] == 1 && p.out_stride[0] == 1) {
        // inner = the dimensions below the axis, which must form one contiguous run in both operands
        int64_t inner = 1;
        bool ok = true;
        for (int d = 0; d < ax && ok; d++) {
            ok = p.dims[d] == 1 || (p.in_stride[d] == inner && p.out_stride[d] == inner);
            inner *= p.dims[d];
        }
        RowMap om{};
        int64_t outer = 1;
        for (int d = ax + 1; d < p.nd; d++) {
            outer *= p.dims[d];
            if (p.dims[d] == 1) continue;
            om.dims[om.nd] = p.dims[d];
            om.in_stride[om.nd] = p.in_stride[d];
            om.out_stride[om.nd] = p.out_stride[d];
            om.nd++;
        }
        const int64_t in_as = p.in_stride[ax], out_as = p.out_stride[ax];
        auto aligned_to = [&](int vec) {
            bool a = inner % vec == 0 && in_as % vec == 0 && out_as % vec == 0 &&
                     (reinterpret_cast<uintptr_t>(in) % (2 * vec)) == 0 && (reinterpret_cast<uintptr_t>(out) % (2 * vec)) == 0;
            for (int d = 0; d < om.nd; d++) a = a && om.in_stride[d] % vec == 0 && om.out_stride[d] % vec == 0;
            return a;
        };
        // 128 halves per lane (64 registers): 16, 32 or 64 steps of 8, 4 or 2 columns, times 1, 4 or 16 waves
        // the widest vector the axis length allows; when that leaves fewer tiles than compute units, the narrowest
        // (measured: [32,256,56,56] over the channels 25.4 us with 8 values per lane, 29.2 with 4, 21.3 with 2)
        int vec = 0;
        if (len <= 256 && aligned_to(8)) vec = 8;
        else if (len <= 512 && aligned_to(4)) vec = 4;
        else if (aligned_to(2)) vec = 2;
        if (vec > 2 && outer * ((inner + 64 * vec - 1) / (64 * vec)) < 256 && aligned_to(2)) vec = 2;
        if (ok && vec != 0 && inner < (1ll << 31)) {
            const half_t* hin = reinterpret_cast<const half_t*>(in);
            half_t* hout = reinterpret_cast<half_t*>(out);
            const int tpo = (int)((inner + 64 * vec - 1) / (64 * vec));
            const int64_t tiles = outer * tpo;
            VPX_REQUIRE(tiles < (1ll << 31), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "softmax: %lld tiles exceed the launch limit",
                        (long long)tiles);
            const int L = (int)len, I = (int)inner;
#define VPX_SLAB(VEC, KW, SMAX, GRID, BLOCK)                                                                          \
    hipLaunchKernelGGL((softmax_slab_f16<VEC, KW, SMAX>), dim3((unsigned)(GRID)), dim3(BLOCK), 0, s, hin, hout, om,     \
                       tiles, tpo, L, I, in_as, out_as)
            if (vec == 8 && L <= 16) VPX_SLAB(8, 1, 16, (tiles + 3) / 4, 256);
            else if (vec == 8 && L <= 64) VPX_SLAB(8, 4, 16, tiles, 256);
            else if (vec == 8) VPX_SLAB(8, 16, 16, tiles, 1024);
            else if (vec == 4 && L <= 32) VPX_SLAB(4, 1, 32, (tiles + 3) / 4, 256);
            else if (vec == 4 && L <= 128) VPX_SLAB(4, 4, 32, tiles, 256);
            else if (vec == 4) VPX_SLAB(4, 16, 32, tiles, 1024);
            else if (L <= 64) VPX_SLAB(2, 1, 64, (tiles + 3) / 4, 256);
            else if (L <= 256) VPX_SLAB(2, 4, 64, tiles, 256);
            else VPX_SLAB(2, 16, 64, tiles, 1024);
#undef VPX_SLAB
            VPX_HIP_CHECK(hipGetLastError());
            return VPX_RESULT_SUCCESS;
        }
    }
    // outer axis, contiguous inner run of at least 64 columns: wavefronts along the axis, lanes along the columns
    if (ax > 0 && p.in_stride[0] == 1 && p.out_stride[0] == 1 && len >= 32) {
        int64_t inner = 1;
        bool ok = true;
        for (int d = 0; d < ax && ok; d++) {
            ok = p.dims[d] == 1 || (p.in_stride[d] == inner && p.out_stride[d] == inner);
            inner *= p.dims[d];
        }
        RowMap om{};
        int64_t outer = 1;
        for (int d = ax + 1; d < p.nd; d++) {
            outer *= p.dims[d];
            if (p.dims[d] == 1) continue;
            om.dims[om.nd] = p.dims[d];
            om.in_stride[om.nd] = p.in_stride[d];
            om.out_stride[om.nd] = p.out_stride[d];
            om.nd++;
        }
        const int64_t in_as = p.in_stride[ax], out_as = p.out_stride[ax];
        auto aligned_to = [&](int vec) {
            const size_t bytes = sizeof(T) * (size_t)vec;
            bool a = inner % vec == 0 && in_as % vec == 0 && out_as % vec == 0 && (reinterpret_cast<uintptr_t>(in) % bytes) == 0 &&
                     (reinterpret_cast<uintptr_t>(out) % bytes) == 0;
            for (int d = 0; d < om.nd; d++) a = a && om.in_stride[d] % vec == 0 && om.out_stride[d] % vec == 0;
            return a;
        };
        if (ok && inner >= 64) {
            // the widest vector that still leaves a workgroup for every compute unit
            int vec = 1;
            for (int v = 16 / (int)sizeof(T); v > 1; v /= 2)
                if (aligned_to(v) && outer * ((inner + 64 * v - 1) / (64 * v)) >= 256) {
                    vec = v;
                    break;
                }
            const int64_t tpo = (inner + 64 * vec - 1) / (64 * vec);
            VPX_REQUIRE(outer * tpo < (1ll << 31), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "softmax: %lld tiles exceed the launch limit",
                        (long long)(outer * tpo));
            const dim3 grid((unsigned)(outer * tpo));
#define VPX_COLS(V) hipLaunchKernelGGL((softmax_cols<T, V>), grid, dim3(1024), 0, s, in, out, om, (int)tpo, len, valid, inner, in_as, out_as)
            if (vec == 8) {
                if constexpr (sizeof(T) == 2) VPX_COLS(8);
            } else if (vec == 4) VPX_COLS(4);
            else if (vec == 2) VPX_COLS(2);
            else VPX_COLS(1);
#undef VPX_COLS
            VPX_HIP_CHECK(hipGetLastError());
            return VPX_RESULT_SUCCESS;
        }
    }
    const unsigned blocks = (unsigned)((rows + 255) / 256);
    hipLaunchKernelGGL(softmax_lines<T>, dim3(blocks), dim3(256), 0, s, in, out, map, rows, len, valid, p.in_stride[ax],
                       p.out_stride[ax]);
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

// ---------------------------------------------------------------- bounded dynamic shapes
// The compiler leaves a softmax over a tensor whose shape is only bounded at compile time two parameter words -- [axis,
// padSize] and [SoftmaxModeDynamic, rank] (update_sw_kernel_params.cpp:48-55) -- and the kernel takes the shape from the
// memrefs' dims and strides in memory when it runs.  Here: one workgroup per row of the BOUND shape (every combination
// of the other coordinates); each reads the live dims, leaves if its row lies outside them, and otherwise walks the
// axis three times with the strides it finds (in bits, as MemRefData holds them).  Elements outside the live shape are
// not touched, and a live dimension larger than its bound is cut to the bound.  The last `pad` positions of the axis
// are written as zeros, as in the static kernels.
struct DynDims {
    const int32_t* dims;      // live dims of the input, innermost first (device memory)
    const int64_t* in_bits;   // live strides of the input, bits
    const int64_t* out_bits;  // live strides of the output, bits
    int nd, axis, pad, elem_bits;
    int32_t bound[VPX_MAX_ND_DIMS];  // the dims the blob holds: a live dimension is never taken to be larger
};

template <typename T>
__global__ __launch_bounds__(256) void softmax_dynamic_kernel(const T* __restrict__ in, T* __restrict__ out, DynDims dd) {
    __shared__ float smem[4];
    // the row's coordinates over the live dims (the axis left out), innermost first
    int64_t r = blockIdx.x, ioff = 0, ooff = 0, len = 1;
    bool inside = true;
    for (int d = 0; d < dd.nd; d++) {
        const int64_t live = dd.dims[d];
        const int64_t n = live < dd.bound[d] ? live : dd.bound[d];  // (the buffers were sized for the bound)
        if (d == dd.axis) {
            len = n;
            continue;
        }
        if (n <= 0) {
            inside = false;
            break;
        }
        const int64_t c = r % n;
        r /= n;
        ioff += c * (dd.in_bits[d] / dd.elem_bits);
        ooff += c * (dd.out_bits[d] / dd.elem_bits);
    }
    if (!inside || r != 0) return;  // (wave-uniform: the row is the workgroup's)
    const int64_t in_es = dd.in_bits[dd.axis] / dd.elem_bits, out_es = dd.out_bits[dd.axis] / dd.elem_bits;
    const int64_t valid = len - dd.pad > 0 ? len - dd.pad : 0;
    const T* px = in + ioff;
    T* py = out + ooff;
    float m = -INFINITY;
    for (int64_t i = threadIdx.x; i < valid; i += 256) m = fmaxf(m, (float)px[i * in_es]);
    m = block_allreduce_max(m, smem);
    float sum = 0.f;
    for (int64_t i = threadIdx.x; i < valid; i += 256) sum += fast_exp((float)px[i * in_es] - m);
    sum = block_allreduce_sum(sum, smem);
    const float inv = 1.0f / sum;
    for (int64_t i = threadIdx.x; i < len; i += 256)
        py[i * out_es] = (T)(i < valid ? fast_exp((float)px[i * in_es] - m) * inv : 0.f);
}

}  // namespace

int launch_softmax_dynamic(const MemRef& in, const MemRef& out, int axis, int pad, hipStream_t s) {
    VPX_REQUIRE(in.live_dims && in.live_strides && out.live_strides, VPX_RESULT_ERROR_INVALID_NULL_HANDLE,
                "softmax: a dynamic shape needs its live dims and strides in device memory");
    int64_t rows = 1;
    for (int d = 0; d < in.nd; d++)
        if (d != axis) rows *= in.dims[d];  // the bound shape
    VPX_REQUIRE(rows < (1ll << 31), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "softmax: %lld rows in the bound shape exceed the launch limit",
                (long long)rows);
    if (rows == 0 || in.dims[axis] == 0) return VPX_RESULT_SUCCESS;
    DynDims dd{in.live_dims, in.live_strides, out.live_strides, in.nd, axis, pad, in.elem_bits, {}};
    for (int d = 0; d < in.nd; d++) dd.bound[d] = (int32_t)in.dims[d];
    if (in.dtype == VPX_NN_FP16) {
        hipLaunchKernelGGL(softmax_dynamic_kernel<half_t>, dim3((unsigned)rows), dim3(256), 0, s, (const half_t*)in.data, (half_t*)out.data, dd);
    } else if (in.dtype == VPX_NN_FP32) {
        hipLaunchKernelGGL(softmax_dynamic_kernel<float>, dim3((unsigned)rows), dim3(256), 0, s, (const float*)in.data, (float*)out.data, dd);
    } else {
        return fail(VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "softmax: element type %s is not implemented", dtype_name(in.dtype));
    }
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

int launch_softmax(const SoftmaxPlan& p, uint32_t dtype, const void* in, void* out, hipStream_t s) {
    VPX_REQUIRE(p.nd >= 1 && p.nd <= VPX_MAX_ND_DIMS && p.axis >= 0 && p.axis < p.nd, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                "softmax: axis %d outside a tensor of rank %d", p.axis, p.nd);
    if (dtype == VPX_NN_FP16) return softmax_typed<half_t>(p, (const half_t*)in, (half_t*)out, s);
    if (dtype == VPX_NN_FP32) return softmax_typed<float>(p, (const float*)in, (float*)out, s);
    return fail(VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "softmax: element type %s is not implemented", dtype_name(dtype));
}

}  // namespace vpx
