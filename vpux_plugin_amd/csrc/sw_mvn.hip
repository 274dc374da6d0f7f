// ACT-SHAVE `mvn1`: per normalisation group, y = (x - mean) / sqrt(var + eps) (eps inside the
// square root) or x - mean; group = (C,H,W) of one batch element when across_channels, else (H,W)
// of one channel (VPU.MVN, src/vpux_compiler/tblgen/vpux/compiler/dialect/VPU/ops.td:3600-3652).
//
// Statistics are fp32.  Each workgroup owns one 4096-element chunk of a group, keeps it in
// registers, computes the chunk's mean and centred sum of squares exactly in two register passes
// and publishes {count, mean, M2}.  Chunks of a group are merged with the pairwise update of
// Chan et al. in a fixed tree order, so results do not depend on scheduling.  This is the
// decomposition the compiler itself uses when a group does not fit local memory
// (MVN1Sum -> MVN1MeanVar -> MVN1Normalize,
// src/vpux_compiler/src/NPU37XX/dialect/VPU/transforms/passes/decompose_mvn.cpp:82-129), with
// centred partial sums instead of raw sum / sum of squares.
//
// Two launches on purpose.  A single launch whose workgroups keep their chunk in registers and
// meet at a device-wide barrier (arrival counter + bounded wait) was built and measured: on this
// part the barrier alone costs about 30 us (device-scope atomics from 1024 workgroups on 8 dies
// meet in memory, not in a cache), against about 3 us for a launch boundary, and the second read
// of the input comes from L2 / Infinity Cache anyway.
#include <atomic>

#include "vpx_common.h"

namespace vpx {

namespace {

typedef _Float16 half_t;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kVecPerThread = 2;                           // 128-bit loads per lane
constexpr int kChunk = kThreads * kVecPerThread * 8;       // fp16 elements per workgroup
constexpr int kMergeInKernel = 256;                        // most chunks per group merged inside the normalise kernel

struct Moments {
    float n, mean, m2;
};

// A published record: 16 bytes, so that it moves as one access.
struct __attribute__((aligned(16))) Record {
    float n, mean, m2, pad;
};
__device__ __forceinline__ Moments unpack(const Record& r) {
    return Moments{r.n, r.mean, r.m2};
}

// Chan/Golub/LeVeque pairwise combination of two sample sets.
__device__ __forceinline__ Moments merge(Moments a, Moments b) {
    const float n = a.n + b.n;
    if (n == 0.f) return Moments{0.f, 0.f, 0.f};
    const float d = b.mean - a.mean;
    const float w = b.n * __builtin_amdgcn_rcpf(n);  // 1 ulp; the same everywhere, so still deterministic
    Moments r;
    r.n = n;
    r.mean = a.mean + d * w;
    r.m2 = a.m2 + b.m2 + d * d * a.n * w;
    return r;
}

template <int CTRL>
__device__ __forceinline__ float dppf(float v) {
    const int i = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(i, i, CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float swz16(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));
}
__device__ __forceinline__ float lane_bcast(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

__device__ __forceinline__ float wave_sum(float v) {
    v += dppf<0xB1>(v);
    v += dppf<0x4E>(v);
    v += dppf<0x141>(v);
    v += dppf<0x140>(v);
    v += swz16(v);
    return lane_bcast(v, 0) + lane_bcast(v, 32);
}

template <class Shuffle>
__device__ __forceinline__ Moments merge_with(Moments m, Shuffle sh) {
    return merge(m, Moments{sh(m.n), sh(m.mean), sh(m.m2)});
}

// Combines the moments held by the 64 lanes of a wavefront in a fixed butterfly order.  The
// pairwise update is not exactly commutative, so lanes may end a few ulps apart: lane 0's value
// is taken for all.
__device__ __forceinline__ Moments wave_merge(Moments m) {
    m = merge_with(m, [](float v) { return dppf<0xB1>(v); });
    m = merge_with(m, [](float v) { return dppf<0x4E>(v); });
    m = merge_with(m, [](float v) { return dppf<0x141>(v); });
    m = merge_with(m, [](float v) { return dppf<0x140>(v); });
    m = merge_with(m, [](float v) { return swz16(v); });
    const Moments lo{lane_bcast(m.n, 0), lane_bcast(m.mean, 0), lane_bcast(m.m2, 0)};
    const Moments hi{lane_bcast(m.n, 32), lane_bcast(m.mean, 32), lane_bcast(m.m2, 32)};
    return merge(lo, hi);
}

struct Chunk {
    float x[kVecPerThread][8];
    int cnt;  // valid elements held by this lane
};

template <bool ALIGNED>
__device__ __forceinline__ void load_chunk(const half_t* __restrict__ g, int64_t base, int64_t size, Chunk& c) {
    c.cnt = 0;
#pragma unroll
    for (int j = 0; j < kVecPerThread; j++) {
        const int64_t e0 = base + (int64_t)(j * kThreads + threadIdx.x) * 8;
        if (ALIGNED && e0 + 8 <= size) {
            const u32x4 q = *reinterpret_cast<const u32x4*>(g + e0);
            const half_t* p = reinterpret_cast<const half_t*>(&q);
#pragma unroll
            for (int k = 0; k < 8; k++) c.x[j][k] = (float)p[k];
            c.cnt += 8;
        } else {
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const bool ok = e0 + k < size;
                c.x[j][k] = ok ? (float)g[ok ? e0 + k : 0] : 0.f;
                c.cnt += ok ? 1 : 0;
            }
        }
    }
}

// Chunk statistics.  Each wavefront finds the mean and centred sum of squares of its own 1024
// elements with lane shuffles only; the four results meet in local memory once and every lane
// merges them in the same order.  Padded slots hold 0 and are excluded through the counts.
__device__ __forceinline__ Moments chunk_moments(const Chunk& c, int64_t base, int64_t size, Moments* smem) {
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < kVecPerThread; j++)
#pragma unroll
        for (int k = 0; k < 8; k++) s += c.x[j][k];
    const float n = wave_sum((float)c.cnt);
    const float mean = n > 0.f ? wave_sum(s) / n : 0.f;
    float q = 0.f;
#pragma unroll
    for (int j = 0; j < kVecPerThread; j++)
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const int64_t e = base + (int64_t)(j * kThreads + threadIdx.x) * 8 + k;
            const float d = c.x[j][k] - mean;
            q += e < size ? d * d : 0.f;
        }
    q = wave_sum(q);
    if ((threadIdx.x & 63) == 0) smem[threadIdx.x >> 6] = Moments{n, mean, q};
    __syncthreads();
    return merge(merge(smem[0], smem[1]), merge(smem[2], smem[3]));
}

template <bool ALIGNED>
__device__ __forceinline__ void store_chunk(half_t* __restrict__ g, int64_t base, int64_t size, const Chunk& c,
                                            float mean, float inv) {
#pragma unroll
    for (int j = 0; j < kVecPerThread; j++) {
        const int64_t e0 = base + (int64_t)(j * kThreads + threadIdx.x) * 8;
        if (ALIGNED && e0 + 8 <= size) {
            u32x4 q;
            half_t* p = reinterpret_cast<half_t*>(&q);
#pragma unroll
            for (int k = 0; k < 8; k++) p[k] = (half_t)((c.x[j][k] - mean) * inv);
            __builtin_nontemporal_store(q, reinterpret_cast<u32x4*>(g + e0));
        } else {
#pragma unroll
            for (int k = 0; k < 8; k++)
                if (e0 + k < size) g[e0 + k] = (half_t)((c.x[j][k] - mean) * inv);
        }
    }
}

__device__ __forceinline__ float inv_std(Moments m, bool normalize_variance, float eps) {
    return normalize_variance ? 1.0f / __builtin_sqrtf(m.m2 / m.n + eps) : 1.0f;
}

// Fixed-order merge of up to 256 published partials of one group.  Every wavefront does the
// whole merge on its own (lane l folds partials l, l+64, l+128, l+192 in sequence -- a wave reads
// 64 consecutive records at a time --, then the butterfly), so all wavefronts of all workgroups get
// the same bits.  `get(i)` returns partial i.
template <class Get>
__device__ __forceinline__ Moments merge_partials(Get get, int chunks) {
    const int lane = threadIdx.x & 63;
    Moments acc{0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < kMergeInKernel / 64; k++) {
        const int i = k * 64 + lane;
        if (i < chunks) acc = merge(acc, get(i));
    }
    return wave_merge(acc);
}

// Fixed-order tree merge of one partial per lane of the workgroup; every lane returns the total.
__device__ __forceinline__ Moments block_merge(Moments m, Moments* smem) {
    __syncthreads();
    smem[threadIdx.x] = m;
    __syncthreads();
    for (int step = kThreads / 2; step > 0; step >>= 1) {
        if ((int)threadIdx.x < step) smem[threadIdx.x] = merge(smem[threadIdx.x], smem[threadIdx.x + step]);
        __syncthreads();
    }
    return smem[0];
}

// One workgroup per (group, chunk).  MODE 0: the group is a single chunk, normalise at once.
// MODE 1: publish the chunk's moments.  MODE 2: merge the group's published moments (all of them
// when `merged` is null, else read the finished result) and normalise.
template <int MODE, bool ALIGNED>
__global__ __launch_bounds__(kThreads) void mvn_chunk_kernel(const half_t* __restrict__ in, half_t* __restrict__ out,
                                                             int64_t group_size, int chunks, Record* partial,
                                                             const Record* merged, int normalize_variance, float eps) {
    __shared__ Moments red[4];
    const int64_t group = blockIdx.x / chunks;
    const int chunk = blockIdx.x % chunks;
    const int64_t base = (int64_t)chunk * kChunk;
    const half_t* gin = in + group * group_size;
    Chunk c;
    load_chunk<ALIGNED>(gin, base, group_size, c);
    if (MODE == 0) {
        const Moments m = chunk_moments(c, base, group_size, red);
        store_chunk<ALIGNED>(out + group * group_size, base, group_size, c, m.mean, inv_std(m, normalize_variance, eps));
    } else if (MODE == 1) {
        const Moments m = chunk_moments(c, base, group_size, red);
        if (threadIdx.x == 0) partial[blockIdx.x] = Record{m.n, m.mean, m.m2, 0.f};
    } else {
        const Record* mine = partial + group * chunks;
        const Moments total = merged ? unpack(merged[group]) : merge_partials([&](int i) { return unpack(mine[i]); }, chunks);
        store_chunk<ALIGNED>(out + group * group_size, base, group_size, c, total.mean,
                             inv_std(total, normalize_variance, eps));
    }
}

// Groups with more than kMergeInKernel chunks: one workgroup per group folds its partials.
__global__ __launch_bounds__(kThreads) void mvn_merge_kernel(const Record* partial, Record* merged, int chunks) {
    __shared__ Moments tree[kThreads];
    const int64_t group = blockIdx.x;
    Moments acc{0.f, 0.f, 0.f};
    // lane t folds chunks t, t+256, ... in order, then the lanes are merged by the fixed tree
    for (int c = threadIdx.x; c < chunks; c += kThreads) acc = merge(acc, unpack(partial[group * chunks + c]));
    const Moments total = block_merge(acc, tree);
    if (threadIdx.x == 0) merged[group] = Record{total.n, total.mean, total.m2, 0.f};
}

// Many short groups that follow one another in memory (per-channel statistics of small planes, 14 x 14 or 7 x 7; rows
// of a few hundred values): a workgroup takes a run of whole groups of about kSmallChunk values, moves it between
// global memory and LDS in aligned 128-bit words whatever the group length (the values of neighbouring groups that
// share its first and last word are read too, but never written), and half-wavefronts normalise one group each in LDS:
// sum, centred sum of squares, scale -- three passes over at most kSmallGroup values.
constexpr int kSmallGroup = 1024;   // longest group this form takes
constexpr int kSmallChunk = 4096;   // values per workgroup, at most
__device__ __forceinline__ float half_wave_sum(float v) {
    v += dppf<0xB1>(v);
    v += dppf<0x4E>(v);
    v += dppf<0x141>(v);
    v += dppf<0x140>(v);
    return v + swz16(v);
}
template <int K>  // values per lane: a group has at most 32 K
__global__ __launch_bounds__(kThreads) void mvn_small_groups_kernel(const half_t* __restrict__ in, half_t* __restrict__ out,
                                                                    int64_t groups, int len, int per_wg, int normalize_variance,
                                                                    int eps_mode, float eps) {
    __shared__ __attribute__((aligned(16))) half_t buf[kSmallChunk + 16];
    const int64_t g0 = (int64_t)blockIdx.x * per_wg;
    const int ng = groups - g0 < per_wg ? (int)(groups - g0) : per_wg;
    const int64_t e0 = g0 * len, e1 = e0 + (int64_t)ng * len, total = groups * len;
    const int64_t a0 = e0 & ~7ll;                  // first aligned word that holds a value of the run
    const int words = (int)((e1 - a0 + 7) >> 3);
    for (int w = threadIdx.x; w < words; w += kThreads) {
        const int64_t at = a0 + (int64_t)w * 8;
        if (at + 8 <= total) {
            *reinterpret_cast<u32x4*>(buf + w * 8) = *reinterpret_cast<const u32x4*>(in + at);
        } else {
            for (int k = 0; k < 8; k++) buf[w * 8 + k] = at + k < total ? in[at + k] : (half_t)0.f;
        }
    }
    __syncthreads();
    const int lane = threadIdx.x & 31, team = threadIdx.x >> 5;
    const float n = (float)len;
    for (int g = team; g < ng; g += kThreads / 32) {   // uniform per half-wavefront
        half_t* x = buf + (int)(e0 - a0) + g * len;
        float v[K];  // the lane's values stay in registers between the passes
        float sum = 0.f;
#pragma unroll
        for (int k = 0; k < K; k++) {
            const int i = lane + 32 * k;
            v[k] = i < len ? (float)x[i] : 0.f;
            sum += v[k];
        }
        const float mean = half_wave_sum(sum) / n;
        float q = 0.f;
#pragma unroll
        for (int k = 0; k < K; k++) {
            const float d = v[k] - mean;
            q += lane + 32 * k < len ? d * d : 0.f;
        }
        const float inv = !normalize_variance ? 1.0f
                          : (eps_mode == 0 ? 1.0f / __builtin_sqrtf(half_wave_sum(q) / n + eps) : 1.0f / (__builtin_sqrtf(half_wave_sum(q) / n) + eps));
#pragma unroll
        for (int k = 0; k < K; k++) {
            const int i = lane + 32 * k;
            if (i < len) x[i] = (half_t)((v[k] - mean) * inv);
        }
    }
    __syncthreads();
    for (int w = threadIdx.x; w < words; w += kThreads) {
        const int64_t at = a0 + (int64_t)w * 8;
        if (at >= e0 && at + 8 <= e1) {
            __builtin_nontemporal_store(*reinterpret_cast<const u32x4*>(buf + w * 8), reinterpret_cast<u32x4*>(out + at));
        } else {
            for (int k = 0; k < 8; k++)
                if (at + k >= e0 && at + k < e1) out[at + k] = buf[w * 8 + k];
        }
    }
}

// Groups of a few thousand to some 75 000 values (112 x 112 or 224 x 224 planes), many of them: one workgroup of
// 1024 lanes keeps its whole group in LDS, so the tensor is read once and written once where the chunked form reads
// it twice.  Sum on the way in, centred sum of squares and the scaled values from LDS.
constexpr int kLdsGroupMax = 76800;  // values: 150 KiB of the 160 KiB a compute unit has
__global__ __launch_bounds__(1024) void mvn_lds_group_kernel(const half_t* __restrict__ in, half_t* __restrict__ out, int64_t len,
                                                             int normalize_variance, int eps_mode, float eps) {
    extern __shared__ __attribute__((aligned(16))) u32x4 grp[];
    __shared__ float red[16];
    const half_t* px = in + (int64_t)blockIdx.x * len;
    half_t* py = out + (int64_t)blockIdx.x * len;
    const int nvec = (int)(len / 8), lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    auto block_sum = [&](float v) {
        v = wave_sum(v);
        __syncthreads();
        if (lane == 0) red[wave] = v;
        __syncthreads();
        float t = 0.f;
#pragma unroll
        for (int w = 0; w < 16; w++) t += red[w];
        return t;
    };
    float sum = 0.f;
    for (int v = threadIdx.x; v < nvec; v += 1024) {
        const u32x4 q = reinterpret_cast<const u32x4*>(px)[v];
        grp[v] = q;
        const half_t* h = reinterpret_cast<const half_t*>(&q);
#pragma unroll
        for (int k = 0; k < 8; k++) sum += (float)h[k];
    }
    const float n = (float)len;
    const float mean = block_sum(sum) / n;
    float sq = 0.f;
    for (int v = threadIdx.x; v < nvec; v += 1024) {
        const u32x4 q = grp[v];
        const half_t* h = reinterpret_cast<const half_t*>(&q);
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const float d = (float)h[k] - mean;
            sq += d * d;
        }
    }
    const float var = block_sum(sq) / n;
    const float inv = !normalize_variance ? 1.0f : (eps_mode == 0 ? 1.0f / __builtin_sqrtf(var + eps) : 1.0f / (__builtin_sqrtf(var) + eps));
    for (int v = threadIdx.x; v < nvec; v += 1024) {
        const u32x4 q = grp[v];
        const half_t* h = reinterpret_cast<const half_t*>(&q);
        u32x4 o;
        half_t* ho = reinterpret_cast<half_t*>(&o);
#pragma unroll
        for (int k = 0; k < 8; k++) ho[k] = (half_t)(((float)h[k] - mean) * inv);
        __builtin_nontemporal_store(o, reinterpret_cast<u32x4*>(py) + v);
    }
}
static bool lds_groups_ok(const half_t* in, const half_t* out, int64_t groups, int64_t len) {
    return len > kChunk && len <= kLdsGroupMax && len % 8 == 0 && groups >= 128 && groups < (1ll << 31) &&
           ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
}
static int launch_lds_groups(const half_t* in, half_t* out, int64_t groups, int64_t len, int nv, int eps_mode, float eps, hipStream_t s) {
    const size_t lds = (size_t)len * sizeof(half_t);
    // more than 64 KiB of dynamic LDS is an opt-in per device and function; asking again costs little
    VPX_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(mvn_lds_group_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      kLdsGroupMax * (int)sizeof(half_t)));
    hipLaunchKernelGGL(mvn_lds_group_kernel, dim3((unsigned)groups), dim3(1024), lds, s, in, out, len, nv, eps_mode, eps);
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

// Packed, aligned groups of 8, 16, ... 256 values (a power of two): T = len / 8 adjacent lanes hold a group, one
// 128-bit word each, and its sums cross the T lanes by DPP (one 16-lane swap for T = 32).
template <int T>
__global__ __launch_bounds__(kThreads) void mvn_tiny_groups_kernel(const half_t* __restrict__ in, half_t* __restrict__ out, int64_t n_vec,
                                                                   int normalize_variance, int eps_mode, float eps) {
    const int64_t v = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (v >= n_vec) return;  // n_vec is a multiple of T and so is the workgroup: a group's lanes leave together
    const u32x4 q = reinterpret_cast<const u32x4*>(in)[v];
    const half_t* h = reinterpret_cast<const half_t*>(&q);
    auto across = [](float a) {
        if (T >= 2) a += dppf<0xB1>(a);
        if (T >= 4) a += dppf<0x4E>(a);
        if (T >= 8) a += dppf<0x141>(a);
        if (T >= 16) a += dppf<0x140>(a);
        if (T >= 32) a += swz16(a);
        return a;
    };
    float x[8];
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < 8; k++) {
        x[k] = (float)h[k];
        sum += x[k];
    }
    constexpr float n = (float)(8 * T);
    const float mean = across(sum) / n;
    float sq = 0.f;
#pragma unroll
    for (int k = 0; k < 8; k++) {
        x[k] -= mean;
        sq += x[k] * x[k];
    }
    const float var = across(sq) / n;
    const float inv = !normalize_variance ? 1.0f : (eps_mode == 0 ? 1.0f / __builtin_sqrtf(var + eps) : 1.0f / (__builtin_sqrtf(var) + eps));
    u32x4 o;
    half_t* ho = reinterpret_cast<half_t*>(&o);
#pragma unroll
    for (int k = 0; k < 8; k++) ho[k] = (half_t)(x[k] * inv);
    __builtin_nontemporal_store(o, reinterpret_cast<u32x4*>(out) + v);
}
static bool tiny_groups_ok(const half_t* in, const half_t* out, int64_t groups, int64_t len) {
    return (len == 8 || len == 16 || len == 32 || len == 64 || len == 128 || len == 256) && groups * (len / 8) < (1ll << 39) &&
           ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
}
static int launch_tiny_groups(const half_t* in, half_t* out, int64_t groups, int64_t len, int nv, int eps_mode, float eps, hipStream_t s) {
    const int64_t n_vec = groups * (len / 8);
    const dim3 grid((unsigned)((n_vec + kThreads - 1) / kThreads));
#define VPX_TINY(T) hipLaunchKernelGGL(mvn_tiny_groups_kernel<T>, grid, dim3(kThreads), 0, s, in, out, n_vec, nv, eps_mode, eps)
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

// Whether the short-group form applies, and its launch.
static bool small_groups_ok(const half_t* in, const half_t* out, int64_t groups, int64_t len) {
    return len >= 1 && len <= kSmallGroup && groups >= 64 && ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0 &&
           (groups + (kSmallChunk / len) - 1) / (kSmallChunk / len) < (1ll << 31);
}
static int launch_small_groups(const half_t* in, half_t* out, int64_t groups, int64_t len, int nv, int eps_mode, float eps, hipStream_t s) {
    const int per_wg = (int)(kSmallChunk / len);
    const unsigned blocks = (unsigned)((groups + per_wg - 1) / per_wg);
#define VPX_SMALL(K) hipLaunchKernelGGL(mvn_small_groups_kernel<K>, dim3(blocks), dim3(kThreads), 0, s, in, out, groups, (int)len, per_wg, nv, eps_mode, eps)
    if (len <= 64) VPX_SMALL(2);
    else if (len <= 128) VPX_SMALL(4);
    else if (len <= 256) VPX_SMALL(8);
    else if (len <= 512) VPX_SMALL(16);
    else VPX_SMALL(32);
#undef VPX_SMALL
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

// position (counted from the innermost memory dimension) of logical dimension `logical`
int mem_pos_of(uint64_t order, int nd, int logical) {
    for (int i = 0; i < nd; i++)
        if ((int)((order >> (4 * i)) & 0xf) == logical + 1) return nd - 1 - i;
    return -1;
}

// ------------------------------------------------------------------------------------------------
// A few long groups in ONE launch, the tensor read once: as many workgroups as the device has compute units, each
// keeps a slice of one group in registers and publishes the slice's {mean, M2}, each word tagged, with write-through
// stores; the first wavefront then polls the records of ITS group (not of the whole grid) with loads that bypass the
// caches until every tag names this launch, merges them in a fixed order and hands the result to the other wavefronts,
// which normalise the slice from the registers.  No read-modify-write is involved: arrivals do not queue at a counter.
// The tag is the group's launch count + 1; the count lives in the zero-initialised sync area.  The wait is bounded: a
// workgroup that does not see its group complete in time (the others are not resident, e.g. the device is shared)
// computes the group's moments itself, slice by slice with the same arithmetic, so the result is the same bits and
// every wave exits.
constexpr int kFusedMaxVec = 16;           // 128-bit words per lane: slices of up to 32768 values
constexpr int kSyncStride = 64;            // words per group in the sync area: the launch count at +0, alone in its cache lines
constexpr int kFusedMaxGroups = 16;        // groups this form takes: each owns a fixed run of kMergeInKernel record slots, so a
                                           // slot only ever carries tags of its own group's launch count
constexpr size_t kSyncRecords = 4 * 1024;  // byte offset of the records in the sync area (the groups' counters before it)
static_assert(kFusedMaxGroups * kSyncStride * sizeof(unsigned) <= kSyncRecords &&
              kSyncRecords + sizeof(Record) * kFusedMaxGroups * kMergeInKernel <= kSyncBytes, "sync area layout");

// A published slice: two 64-bit words, {mean, tag} and {M2, tag}, each written and read as one access that goes
// through to memory (agent scope), so neither needs the other to be valid; the count of a slice follows from its index.
struct __attribute__((aligned(16))) Tagged {
    unsigned long long mean, m2;
};
__device__ __forceinline__ unsigned long long tagged(float v, unsigned tag) {
    return (unsigned long long)__builtin_bit_cast(unsigned, v) | ((unsigned long long)tag << 32);
}

template <int V>
struct Slice {
    u32x4 q[V];
    unsigned valid;  // bit j: word j lies inside the slice
};

template <int V>
__device__ __forceinline__ void load_slice(const half_t* __restrict__ g, int64_t base, int64_t end, Slice<V>& sl) {
    sl.valid = 0;
#pragma unroll
    for (int j = 0; j < V; j++) {
        const int64_t e0 = base + (int64_t)(j * kThreads + threadIdx.x) * 8;
        const bool ok = e0 < end;  // slices and groups are whole words
        sl.q[j] = ok ? *reinterpret_cast<const u32x4*>(g + e0) : u32x4{0, 0, 0, 0};
        sl.valid |= ok ? (1u << j) : 0u;
    }
}

// Moments of the slice held by the workgroup: per wavefront by lane shuffles (mean first, then centred squares),
// the four wavefronts' results merged in a fixed order by every lane.
// The slice as single-precision values (the conversion is exact): both passes of the moments and the normalisation
// read these, so every value is converted once.
template <int V>
struct SliceF {
    float f[V][8];
};
template <int V>
__device__ __forceinline__ void widen_slice(const Slice<V>& sl, SliceF<V>& w) {
#pragma unroll
    for (int j = 0; j < V; j++) {
        const half_t* p = reinterpret_cast<const half_t*>(&sl.q[j]);
#pragma unroll
        for (int k = 0; k < 8; k++) w.f[j][k] = (float)p[k];
    }
}

template <int V>
__device__ __forceinline__ Moments slice_moments(const SliceF<V>& w, unsigned valid, Moments* red) {
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < V; j++) {
#pragma unroll
        for (int k = 0; k < 8; k++) sum += w.f[j][k];
    }
    const float n = wave_sum((float)(8 * __builtin_popcount(valid)));
    const float mean = n > 0.f ? wave_sum(sum) / n : 0.f;
    float q = 0.f;
#pragma unroll
    for (int j = 0; j < V; j++) {
        float qj = 0.f;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const float d = w.f[j][k] - mean;
            qj += d * d;
        }
        q += (valid >> j) & 1u ? qj : 0.f;
    }
    q = wave_sum(q);
    __syncthreads();  // the previous use of `red` is over
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = Moments{n, mean, q};
    __syncthreads();
    return merge(merge(red[0], red[1]), merge(red[2], red[3]));
}

template <int V>
__global__ __launch_bounds__(kThreads) void mvn_fused_kernel(const half_t* __restrict__ in, half_t* __restrict__ out,
                                                             int64_t group_size, int wpg, int64_t slice, unsigned* sync,
                                                             int normalize_variance, float eps, unsigned long long spin_ticks) {
    __shared__ Moments red[4];
    __shared__ Moments others[kMergeInKernel];
    __shared__ Moments shared_total;
    __shared__ int complete;
    const int64_t group = blockIdx.x / wpg;
    const int part = blockIdx.x % wpg;
    const int lane = threadIdx.x & 63;
    unsigned* count = sync + group * kSyncStride;
    Tagged* mine = reinterpret_cast<Tagged*>(reinterpret_cast<char*>(sync) + kSyncRecords) + group * kMergeInKernel;
    unsigned tag = 0;
    if (wpg > 1 && threadIdx.x < 64) {
        tag = __hip_atomic_load(count, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;
        tag = tag == 0u ? 1u : tag;
    }
    const half_t* gin = in + group * group_size;
    const int64_t base = (int64_t)part * slice;
    const int64_t end = base + slice < group_size ? base + slice : group_size;
    Slice<V> sl;
    load_slice<V>(gin, base, end, sl);
    SliceF<V> wide;
    widen_slice<V>(sl, wide);
    Moments total = slice_moments<V>(wide, sl.valid, red);
    if (wpg > 1) {
        if (threadIdx.x < 64) {  // the first wavefront
            if (lane == 0) {
                __hip_atomic_store(&mine[part].mean, tagged(total.mean, tag), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(&mine[part].m2, tagged(total.m2, tag), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            const unsigned long long t0 = wall_clock64();
            unsigned long long rm[kMergeInKernel / 64], rq[kMergeInKernel / 64];
            bool ok;
            for (;;) {
                bool ready = true;
#pragma unroll
                for (int k = 0; k < kMergeInKernel / 64; k++) {
                    const int i = k * 64 + lane;
                    rm[k] = rq[k] = 0;
                    if (i < wpg) {
                        rm[k] = __hip_atomic_load(&mine[i].mean, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        rq[k] = __hip_atomic_load(&mine[i].m2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        ready = ready && (unsigned)(rm[k] >> 32) == tag && (unsigned)(rq[k] >> 32) == tag;
                    }
                }
                ok = __builtin_amdgcn_ballot_w64(!ready) == 0;
                if (ok || wall_clock64() - t0 >= spin_ticks) break;  // (pausing between polls measured slower)
            }
            if (ok) {
                Moments acc{0.f, 0.f, 0.f};
#pragma unroll
                for (int k = 0; k < kMergeInKernel / 64; k++) {
                    const int i = k * 64 + lane;
                    if (i < wpg) {
                        const int64_t b = (int64_t)i * slice;
                        const int64_t cnt = (b + slice < group_size ? b + slice : group_size) - b;
                        acc = merge(acc, Moments{(float)cnt, __builtin_bit_cast(float, (unsigned)rm[k]), __builtin_bit_cast(float, (unsigned)rq[k])});
                    }
                }
                const Moments t = wave_merge(acc);
                if (lane == 0) shared_total = t;
            }
            if (lane == 0) complete = ok ? 1 : 0;
        }
        __syncthreads();
        if (complete) {
            total = shared_total;
        } else {
            for (int p = 0; p < wpg; p++) {
                const int64_t b = (int64_t)p * slice;
                const int64_t e = b + slice < group_size ? b + slice : group_size;
                Slice<V> t;
                load_slice<V>(gin, b, e, t);
                SliceF<V> tw;
                widen_slice<V>(t, tw);
                const Moments mp = slice_moments<V>(tw, t.valid, red);
                if (threadIdx.x == 0) others[p] = mp;
            }
            __syncthreads();
            total = merge_partials([&](int i) { return others[i]; }, wpg);  // the order the first wavefront uses above
        }
        // The group's first workgroup advances the launch count, and it alone: stores of many workgroups to one word
        // queue up (64 of them cost 1.5 us here).  When its wait was met, every workgroup of the group has read the
        // count already (a record carries the tag only after its writer has); when its wait ran out, a workgroup that
        // starts even later reads the advanced count, publishes under the next tag, meets nobody and recomputes, like
        // everyone else in a launch that far apart.  A workgroup whose wait ran out withdraws its record (tag 0 is
        // never used), so that whichever tag the next launch uses, the slot is not taken for published until its
        // owner writes it again.
        if (threadIdx.x == 0) {
            if (part == 0) __hip_atomic_store(count, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (!complete) {
                __hip_atomic_store(&mine[part].mean, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(&mine[part].m2, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    const float mean = total.mean, inv = inv_std(total, normalize_variance, eps);
    half_t* gout = out + group * group_size;
#pragma unroll
    for (int j = 0; j < V; j++) {
        if (!((sl.valid >> j) & 1u)) continue;
        u32x4 r;
        half_t* o = reinterpret_cast<half_t*>(&r);
#pragma unroll
        for (int k = 0; k < 8; k++) o[k] = (half_t)((wide.f[j][k] - mean) * inv);
        __builtin_nontemporal_store(r, reinterpret_cast<u32x4*>(gout + base + (int64_t)(j * kThreads + threadIdx.x) * 8));
    }
}

// Takes the launch when the groups are few and the tensor fits the registers of one workgroup per compute unit.
// *done is set when the kernel was launched.
int launch_fused_groups(const half_t* in, half_t* out, int64_t groups, int64_t group_size, int nv, float eps, hipStream_t s,
                        bool* done) {
    *done = false;
    const int mode = tuning_mvn_fused();  // 0: never, 1: default, 2: spin limit 0 (every workgroup recomputes)
    if (mode == 0) return VPX_RESULT_SUCCESS;
    int cus = 0;
    int rc = device_compute_units(&cus);
    if (rc) return rc;
    if (groups > cus || groups > kFusedMaxGroups) return VPX_RESULT_SUCCESS;
    // In place (or any overlap of the two tensors): a workgroup whose wait runs out reads its whole group again, and by
    // then other workgroups may have stored their normalised slices over it.  The two-launch kernels finish every
    // read of the statistics before the first store, so overlapping tensors go there.
    {
        const uintptr_t ib = reinterpret_cast<uintptr_t>(in), ob = reinterpret_cast<uintptr_t>(out);
        const uintptr_t bytes = (uintptr_t)(groups * group_size) * sizeof(half_t);
        if (ib < ob + bytes && ob < ib + bytes) return VPX_RESULT_SUCCESS;
    }
    int64_t wpg = cus / groups;  // (two workgroups per compute unit measured 1.2 us slower at [4,256,64,64])
    if (wpg > kMergeInKernel) wpg = kMergeInKernel;
    const int64_t words = group_size / 8;
    const int64_t most = (words + kThreads - 1) / kThreads;  // at least one word per lane
    if (wpg > most) wpg = most;
    const int64_t slice = (words + wpg - 1) / wpg * 8;
    wpg = (group_size + slice - 1) / slice;  // no empty slices
    int v = 1;
    while (v < kFusedMaxVec && (int64_t)v * kThreads * 8 < slice) v *= 2;
    if ((int64_t)v * kThreads * 8 < slice) return VPX_RESULT_SUCCESS;
    void* sync = nullptr;
    rc = get_sync_area(s, &sync);
    if (rc) return rc;
    const unsigned long long spin = mode == 2 ? 0ull : 50000ull;  // 0.5 ms of the 100 MHz counter
    const dim3 grid((unsigned)(groups * wpg)), block(kThreads);
#define VPX_FUSED(V)                                                                                                  \
    hipLaunchKernelGGL((mvn_fused_kernel<V>), grid, block, 0, s, in, out, group_size, (int)wpg, slice, (unsigned*)sync, \
                       nv, eps, spin)
    switch (v) {
    case 1: VPX_FUSED(1); break;
    case 2: VPX_FUSED(2); break;
    case 4: VPX_FUSED(4); break;
    case 8: VPX_FUSED(8); break;
    default: VPX_FUSED(16); break;
    }
#undef VPX_FUSED
    VPX_HIP_CHECK(hipGetLastError());
    *done = true;
    return VPX_RESULT_SUCCESS;
}

template <bool ALIGNED>
int launch_groups(const half_t* in, half_t* out, int64_t groups, int64_t group_size, int nv, float eps, hipStream_t s) {
    const int64_t chunks64 = (group_size + kChunk - 1) / kChunk;
    VPX_REQUIRE(chunks64 * groups < (1ll << 31), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                "mvn1: %lld groups of %lld elements exceed the launch limit", (long long)groups, (long long)group_size);
    const int chunks = (int)chunks64;
    const unsigned blocks = (unsigned)(groups * chunks);
    if (ALIGNED && chunks > 1) {
        bool done = false;
        const int rc = launch_fused_groups(in, out, groups, group_size, nv, eps, s, &done);
        if (rc || done) return rc;
    }
    if (chunks == 1) {
        hipLaunchKernelGGL((mvn_chunk_kernel<0, ALIGNED>), dim3(blocks), dim3(kThreads), 0, s, in, out, group_size, 1,
                           (Record*)nullptr, (const Record*)nullptr, nv, eps);
        VPX_HIP_CHECK(hipGetLastError());
        return VPX_RESULT_SUCCESS;
    }
    void* ws = nullptr;
    const size_t need = sizeof(Record) * ((size_t)blocks + (size_t)groups);
    int rc = get_workspace(s, need, &ws);
    if (rc) return rc;
    Record* partial = (Record*)ws;
    Record* merged = partial + blocks;

    hipLaunchKernelGGL((mvn_chunk_kernel<1, ALIGNED>), dim3(blocks), dim3(kThreads), 0, s, in, out, group_size, chunks,
                       partial, (const Record*)nullptr, nv, eps);
    VPX_HIP_CHECK(hipGetLastError());
    const Record* use_merged = nullptr;
    if (chunks > kMergeInKernel) {
        hipLaunchKernelGGL(mvn_merge_kernel, dim3((unsigned)groups), dim3(kThreads), 0, s, partial, merged, chunks);
        VPX_HIP_CHECK(hipGetLastError());
        use_merged = merged;
    }
    hipLaunchKernelGGL((mvn_chunk_kernel<2, ALIGNED>), dim3(blocks), dim3(kThreads), 0, s, in, out, group_size, chunks,
                       partial, use_merged, nv, eps);
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}


// ------------------------------------------------------------------------------------------------
// The compiler's three-step decomposition of MVN-1 for tensors that do not fit local memory
// (src/vpux_compiler/src/NPU37XX/dialect/VPU/transforms/passes/decompose_mvn.cpp:82-129;
// operator definitions src/vpux_compiler/tblgen/vpux/compiler/dialect/VPU/ops.td:3659-3845):
//   mvn1_sum      x[N,C,H,W] -> f32 {sum, sum of squares} [N, C or 1, parts, 2 or 1], channel-minor
//   mvn1_mean_var those partial sums -> {mean, 1/sqrt(var + eps)} [N, C or 1, 1, 2 or 1]
//   mvn1_norm     x, {mean, 1/std} -> (x - mean) * 1/std
// `parts` (the output height of mvn1_sum) is the number of partial sums per group; a single call
// here splits the group's elements into that many consecutive ranges, so that their sum is the
// group's total whatever the count.

// fp32 value -> fp16, round to nearest even.  The empty asm keeps the compiler from folding the preceding
// multiply into a mixed-precision multiply that rounds the exact product once: the result is defined as
// the fp32 product rounded again.
__device__ __forceinline__ half_t round_f16(float v) {
    asm volatile("" : "+v"(v));
    return (half_t)v;
}

struct SumOut {
    float* out;
    int parts, out_w;
    int64_t out_c;
    __device__ __forceinline__ void put(int64_t group, int part, float s, float q) const {
        const int64_t n = group / out_c, c = group % out_c;
        float* o = out + ((n * parts + part) * out_w) * out_c + c;
        o[0] = s;
        if (out_w == 2) o[out_c] = q;
    }
};

__device__ __forceinline__ float2 add2(float2 a, float2 b) {
    return float2{a.x + b.x, a.y + b.y};
}

// One workgroup per (group, chunk) of a contiguous group: raw fp32 sum and sum of squares.
template <bool ALIGNED>
__global__ __launch_bounds__(kThreads) void mvn_sum_chunk_kernel(const half_t* __restrict__ in, int64_t group_size,
                                                                 int chunks, float2* __restrict__ partial, SumOut o,
                                                                 int direct) {
    __shared__ float2 red[4];
    const int64_t group = blockIdx.x / chunks;
    const int chunk = blockIdx.x % chunks;
    Chunk c;
    load_chunk<ALIGNED>(in + group * group_size, (int64_t)chunk * kChunk, group_size, c);
    float sum = 0.f, sq = 0.f;
#pragma unroll
    for (int j = 0; j < kVecPerThread; j++)
#pragma unroll
        for (int k = 0; k < 8; k++) {
            sum += c.x[j][k];
            sq += c.x[j][k] * c.x[j][k];
        }
    sum = wave_sum(sum);
    sq = wave_sum(sq);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = float2{sum, sq};
    __syncthreads();
    if (threadIdx.x == 0) {
        const float2 t = add2(add2(red[0], red[1]), add2(red[2], red[3]));
        if (direct) o.put(group, 0, t.x, t.y);
        else partial[blockIdx.x] = t;
    }
}

// One workgroup per (group, part): folds that part's chunk sums in a fixed order.
__global__ __launch_bounds__(kThreads) void mvn_sum_finish_kernel(const float2* __restrict__ partial, int chunks, SumOut o) {
    __shared__ float2 tree[kThreads];
    const int64_t group = blockIdx.x / o.parts;
    const int part = blockIdx.x % o.parts;
    const int c0 = (int)((int64_t)part * chunks / o.parts), c1 = (int)((int64_t)(part + 1) * chunks / o.parts);
    float2 acc{0.f, 0.f};
    for (int c = c0 + threadIdx.x; c < c1; c += kThreads) acc = add2(acc, partial[group * chunks + c]);
    tree[threadIdx.x] = acc;
    __syncthreads();
    for (int step = kThreads / 2; step > 0; step >>= 1) {
        if ((int)threadIdx.x < step) tree[threadIdx.x] = add2(tree[threadIdx.x], tree[threadIdx.x + step]);
        __syncthreads();
    }
    if (threadIdx.x == 0) o.put(group, part, tree[0].x, tree[0].y);
}

// Per-channel sums of a channel-minor layout: a workgroup takes 64 channels of one spatial range
// of one batch element (lane (r, c) walks positions r, r+4, ...).  With SHIFT the sums are of
// x - x[first position of the channel], which keeps the sum of squares free of cancellation when a
// channel's mean is far from zero (used where the variance is taken from these sums).
template <bool SHIFT>
__global__ __launch_bounds__(kThreads) void mvn_sum_cminor_kernel(const half_t* __restrict__ in, int64_t S, int64_t C,
                                                                  int subparts, int64_t cpad, float2* __restrict__ partial) {
    __shared__ float2 red[4][64];
    const int cl = threadIdx.x & 63, r = threadIdx.x >> 6;
    const int64_t ctiles = cpad / 64;
    const int64_t ct = blockIdx.x % ctiles;
    const int sp = (int)((blockIdx.x / ctiles) % subparts);
    const int64_t n = blockIdx.x / (ctiles * subparts);
    const int64_t s0 = sp * S / subparts, s1 = (sp + 1) * S / subparts;
    const int64_t c = ct * 64 + cl;
    float sum = 0.f, sq = 0.f;
    if (c < C) {
        const half_t* px = in + n * S * C + c;
        const float shift = SHIFT ? (float)px[0] : 0.f;
        for (int64_t i = s0 + r; i < s1; i += 4) {
            const float x = (float)px[i * C] - shift;
            sum += x;
            sq += x * x;
        }
    }
    red[r][cl] = float2{sum, sq};
    __syncthreads();
    if (r == 0) partial[(n * subparts + sp) * cpad + c] = add2(add2(red[0][cl], red[1][cl]), add2(red[2][cl], red[3][cl]));
}

// The same sums with eight adjacent channels per lane (channel counts that are a multiple of eight, up to 2048): a
// lane's 128-bit loads walk the positions of its channel octet, the workgroup's lanes cover 256 / (C / 8) positions
// at a time, and the lanes that share an octet meet in LDS.  Same partial layout as the kernel above.
template <bool SHIFT>
__global__ __launch_bounds__(kThreads) void mvn_sum_cminor8_kernel(const half_t* __restrict__ in, int64_t S, int64_t C,
                                                                   int subparts, int64_t cpad, float2* __restrict__ partial) {
    extern __shared__ float2 red8[];  // [slots][C]
    const int cv = (int)(C / 8), slots = kThreads / cv;
    const int sp = (int)(blockIdx.x % subparts);
    const int64_t n = blockIdx.x / subparts;
    const int64_t s0 = sp * S / subparts, s1 = (sp + 1) * S / subparts;
    const int slot = threadIdx.x / cv, oct = threadIdx.x % cv;
    float sum[8], sq[8];
#pragma unroll
    for (int k = 0; k < 8; k++) sum[k] = sq[k] = 0.f;
    if (slot < slots) {
        const half_t* px = in + n * S * C + oct * 8;
        float shift[8];
        {
            const u32x4 q = *reinterpret_cast<const u32x4*>(px);
            const half_t* h = reinterpret_cast<const half_t*>(&q);
#pragma unroll
            for (int k = 0; k < 8; k++) shift[k] = SHIFT ? (float)h[k] : 0.f;
        }
        for (int64_t i = s0 + slot; i < s1; i += slots) {
            const u32x4 q = *reinterpret_cast<const u32x4*>(px + i * C);
            const half_t* h = reinterpret_cast<const half_t*>(&q);
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const float x = (float)h[k] - shift[k];
                sum[k] += x;
                sq[k] += x * x;
            }
        }
#pragma unroll
        for (int k = 0; k < 8; k++) red8[(int64_t)slot * C + oct * 8 + k] = float2{sum[k], sq[k]};
    }
    __syncthreads();
    for (int c = threadIdx.x; c < C; c += kThreads) {
        float2 t = red8[c];
        for (int r = 1; r < slots; r++) t = add2(t, red8[(int64_t)r * C + c]);
        partial[(n * subparts + sp) * cpad + c] = t;
    }
}

// Launches whichever sum kernel fits; `subparts` spatial ranges per image, partials [N][subparts][cpad].
template <bool SHIFT>
static int launch_sum_cminor(const half_t* in, int64_t N, int64_t S, int64_t C, int64_t subparts, int64_t cpad, float2* partial,
                             hipStream_t s) {
    if (C % 8 == 0 && C >= 8 && C <= 2048 && (reinterpret_cast<uintptr_t>(in) & 15) == 0) {
        const int slots = kThreads / (int)(C / 8);
        const size_t lds = sizeof(float2) * (size_t)slots * (size_t)C;  // at most 16 KiB
        hipLaunchKernelGGL(mvn_sum_cminor8_kernel<SHIFT>, dim3((unsigned)(N * subparts)), dim3(kThreads), lds, s, in, S, C, (int)subparts,
                           cpad, partial);
    } else {
        hipLaunchKernelGGL(mvn_sum_cminor_kernel<SHIFT>, dim3((unsigned)(N * subparts * (cpad / 64))), dim3(kThreads), 0, s, in, S, C,
                           (int)subparts, cpad, partial);
    }
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

__global__ __launch_bounds__(kThreads) void mvn_sum_cminor_finish_kernel(const float2* __restrict__ partial, int64_t total,
                                                                         int64_t C, int64_t cpad, int subparts, int isplit,
                                                                         SumOut o) {
    const int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= total) return;
    const int64_t c = idx % C;
    const int part = (int)((idx / C) % o.parts);
    const int64_t n = idx / (C * o.parts);
    float2 acc{0.f, 0.f};
#pragma unroll 8
    for (int j = 0; j < isplit; j++) acc = add2(acc, partial[(n * subparts + part * isplit + j) * cpad + c]);
    o.put(n * C + c, part, acc.x, acc.y);
}

// mvn1 on a channel-minor layout with per-channel statistics: folds the shifted partial sums of one
// (n, c) and leaves {mean, 1/std} as fp32 in the layout mvn_norm_cminor_kernel reads.
__global__ __launch_bounds__(kThreads) void mvn_cminor_stats_kernel(const half_t* __restrict__ in, const float2* __restrict__ partial,
                                                                    float* __restrict__ stats, int64_t total, int64_t S, int64_t C,
                                                                    int64_t cpad, int subparts, int normalize_variance, float eps) {
    const int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= total) return;
    const int64_t c = idx % C, n = idx / C;
    float2 acc{0.f, 0.f};
#pragma unroll 8
    for (int j = 0; j < subparts; j++) acc = add2(acc, partial[(n * subparts + j) * cpad + c]);
    const float shift = (float)in[n * S * C + c];
    const float cnt = (float)S;
    const float m = acc.x / cnt;
    const float var = fmaxf(acc.y / cnt - m * m, 0.f);
    stats[(n * 2) * C + c] = shift + m;
    stats[(n * 2 + 1) * C + c] = normalize_variance ? 1.0f / __builtin_sqrtf(var + eps) : 1.0f;
}

// One lane per output statistic; the handful of partial sums is folded in double.
template <typename TO>
__global__ __launch_bounds__(kThreads) void mvn_mean_var_kernel(const float* __restrict__ sum, TO* __restrict__ out, int64_t N,
                                                                int64_t c_in, int parts, int in_w, int64_t out_c, int out_w,
                                                                int across, int64_t group_c, double count, float eps) {
    const int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= N * out_c) return;
    const int64_t n = idx / out_c, c = idx % out_c;
    int64_t c0 = 0, c1 = c_in;
    if (!across) {
        c0 = (c / group_c) * group_c;
        c1 = c0 + group_c < c_in ? c0 + group_c : c_in;
    }
    double s = 0.0, q = 0.0;
    for (int p = 0; p < parts; p++) {
        const float* row = sum + ((n * parts + p) * in_w) * c_in;
        for (int64_t ci = c0; ci < c1; ci++) {
            s += (double)row[ci];
            if (in_w == 2) q += (double)row[c_in + ci];
        }
    }
    const double mean = s / count;
    out[(n * out_w) * out_c + c] = (TO)(float)mean;
    if (out_w == 2) {
        double var = q / count - mean * mean;
        var = var > 0.0 ? var : 0.0;
        out[(n * out_w + 1) * out_c + c] = (TO)(float)(1.0 / __builtin_sqrt(var + (double)eps));
    }
}

// x and y in runs of `run` elements that share one statistic (a (n,c) plane, or a whole batch
// element when across channels): one workgroup per 2048-element piece of a run.
template <typename TS, bool ALIGNED>
__global__ __launch_bounds__(kThreads) void mvn_norm_runs_kernel(const half_t* __restrict__ in, half_t* __restrict__ out,
                                                                 const TS* __restrict__ mv, int64_t run, int pieces,
                                                                 int64_t rows_per_n, int64_t out_c, int out_w) {
    const int64_t row = blockIdx.x / pieces;
    const int piece = blockIdx.x % pieces;
    const int64_t n = row / rows_per_n, c = row % rows_per_n;  // rows_per_n = 1 when across channels
    const float mean = (float)mv[(n * out_w) * out_c + c];
    const float inv = out_w == 2 ? (float)mv[(n * out_w + 1) * out_c + c] : 1.0f;
    const int64_t e0 = (int64_t)piece * (kThreads * 8) + threadIdx.x * 8;
    const half_t* gi = in + row * run;
    half_t* go = out + row * run;
    if (ALIGNED && e0 + 8 <= run) {
        const u32x4 q = *reinterpret_cast<const u32x4*>(gi + e0);
        const half_t* p = reinterpret_cast<const half_t*>(&q);
        u32x4 y;
        half_t* py = reinterpret_cast<half_t*>(&y);
#pragma unroll
        for (int k = 0; k < 8; k++) py[k] = round_f16(((float)p[k] - mean) * inv);
        __builtin_nontemporal_store(y, reinterpret_cast<u32x4*>(go + e0));
    } else {
        for (int k = 0; k < 8; k++)
            if (e0 + k < run) go[e0 + k] = round_f16(((float)gi[e0 + k] - mean) * inv);
    }
}

// Channel-minor layout with per-channel statistics: element e of batch element n has channel e % C.
// VEC: the channel count is a multiple of 8 and everything is 16-byte aligned, so a lane's 8 elements are 8
// consecutive channels and their statistics two contiguous runs.
template <typename TS, bool VEC>
__global__ __launch_bounds__(kThreads) void mvn_norm_cminor_kernel(const half_t* __restrict__ in, half_t* __restrict__ out,
                                                                   const TS* __restrict__ mv, int64_t per_n, int64_t C,
                                                                   int pieces, int out_w) {
    const int64_t n = blockIdx.x / pieces;
    const int64_t e0 = (int64_t)(blockIdx.x % pieces) * (kThreads * 8) + threadIdx.x * 8;
    const TS* mean = mv + (n * out_w) * C;
    const TS* inv = mean + C;
    const half_t* gi = in + n * per_n;
    half_t* go = out + n * per_n;
    uint32_t c = (uint32_t)(e0 % C);
    if (VEC) {
        if (e0 >= per_n) return;
        const u32x4 q = *reinterpret_cast<const u32x4*>(gi + e0);
        const half_t* p = reinterpret_cast<const half_t*>(&q);
        TS m[8], iv[8];
        typedef uint32_t words_t __attribute__((ext_vector_type(sizeof(TS) * 2)));  // 8 statistics = 16 or 32 bytes
        *reinterpret_cast<words_t*>(m) = *reinterpret_cast<const words_t*>(mean + c);
        if (out_w == 2) *reinterpret_cast<words_t*>(iv) = *reinterpret_cast<const words_t*>(inv + c);
        u32x4 y;
        half_t* py = reinterpret_cast<half_t*>(&y);
#pragma unroll
        for (int k = 0; k < 8; k++) py[k] = round_f16(((float)p[k] - (float)m[k]) * (out_w == 2 ? (float)iv[k] : 1.0f));
        __builtin_nontemporal_store(y, reinterpret_cast<u32x4*>(go + e0));
        return;
    }
    for (int k = 0; k < 8; k++) {
        if (e0 + k < per_n) {
            const float i = out_w == 2 ? (float)inv[c] : 1.0f;
            go[e0 + k] = round_f16(((float)gi[e0 + k] - (float)mean[c]) * i);
        }
        c = c + 1 == (uint32_t)C ? 0 : c + 1;
    }
}

struct MvnShape {
    int64_t N, C, S;
    bool channel_minor;
};

int mvn_shape(const char* what, const MemRef& in, MvnShape& sh) {
    VPX_REQUIRE(in.nd == 4, VPX_RESULT_ERROR_INVALID_ARGUMENT, "%s: expects a 4-D tensor, got rank %d", what, in.nd);
    VPX_REQUIRE(in.order == VPX_ORDER_NCHW || in.order == VPX_ORDER_NCWH || in.order == VPX_ORDER_NHWC ||
                        in.order == VPX_ORDER_NWHC,
                VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "%s: unsupported order 0x%llx", what, (unsigned long long)in.order);
    VPX_REQUIRE(in.compact, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "%s: only compact tensors are supported", what);
    const int pn = mem_pos_of(in.order, 4, 0), pc = mem_pos_of(in.order, 4, 1);
    VPX_REQUIRE(pn == 3, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "%s: batch must be the outermost dimension", what);
    sh.N = in.dims[pn];
    sh.C = in.dims[pc];
    sh.S = sh.N * sh.C ? in.numel() / (sh.N * sh.C) : 0;
    sh.channel_minor = pc != 2;
    return VPX_RESULT_SUCCESS;
}

// Logical [N, C, H, W] of a 4-D channel-minor (NHWC) statistics tensor.
int stats_shape(const char* what, const MemRef& m, int64_t dims[4]) {
    VPX_REQUIRE(m.nd == 4 && m.order == VPX_ORDER_NHWC && m.compact, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                "%s: the statistics tensor must be a compact 4-D NHWC tensor", what);
    for (int l = 0; l < 4; l++) dims[l] = m.dims[mem_pos_of(m.order, 4, l)];
    return VPX_RESULT_SUCCESS;
}


// ------------------------------------------------------------------------------------------------
// mvn6: OpenVINO MVN-6 over an arbitrary set of axes with the eps inside or outside the square
// root, and the compiler's fused `* scale + bias` (VPU.MVN6,
// src/vpux_compiler/tblgen/vpux/compiler/dialect/VPU/ops.td:3850-3900;
// src/vpux_compiler/src/dialect/IE/transforms/passes/fuse_mvn6_scale_bias.cpp).  A row is one
// combination of the kept (not normalised) coordinates.

struct Mvn6Geom {
    int nk, nr;
    int32_t kdim[kMaxDims], rdim[kMaxDims];
    int64_t k_in[kMaxDims], k_out[kMaxDims], k_sc[kMaxDims], k_bi[kMaxDims];
    int64_t r_in[kMaxDims], r_out[kMaxDims], r_sc[kMaxDims], r_bi[kMaxDims];
    int64_t rows;
    uint32_t row_len;
    int sc_along_row, bi_along_row;  // contiguous-row kernels: 1 = the operand has the row's elements, 0 = one value per row
};

struct RowBase {
    int64_t in, out, sc, bi;
};

__device__ __forceinline__ RowBase row_base(const Mvn6Geom& g, int64_t row) {
    RowBase b{0, 0, 0, 0};
    uint32_t r = (uint32_t)row;  // the host keeps the row count below 2^31
    for (int d = 0; d < g.nk; d++) {
        const bool last = d == g.nk - 1;  // what is left indexes the outermost kept dimension: no division
        const int64_t c = last ? r : r % (uint32_t)g.kdim[d];
        if (!last) r /= (uint32_t)g.kdim[d];
        b.in += c * g.k_in[d];
        b.out += c * g.k_out[d];
        b.sc += c * g.k_sc[d];
        b.bi += c * g.k_bi[d];
    }
    return b;
}

__device__ __forceinline__ float mvn6_inv(float var, int normalize_variance, int eps_mode, float eps) {
    if (!normalize_variance) return 1.0f;
    return eps_mode == 0 ? 1.0f / __builtin_sqrtf(var + eps) : 1.0f / (__builtin_sqrtf(var) + eps);
}

// Sum over the TEAM lanes that share a row: half a wavefront, a wavefront, or the whole workgroup.
template <int TEAM>
__device__ __forceinline__ float team_sum(float v, float* smem) {
    if (TEAM == 32) {  // the row operations and the 16-lane swap stay inside each half
        v += dppf<0xB1>(v);
        v += dppf<0x4E>(v);
        v += dppf<0x141>(v);
        v += dppf<0x140>(v);
        return v + swz16(v);
    }
    v = wave_sum(v);
    if (TEAM == 64) return v;
    // one barrier: each sum of a workgroup's lifetime has four slots of its own
    if ((threadIdx.x & 63) == 0) smem[threadIdx.x >> 6] = v;
    __syncthreads();
    return (smem[0] + smem[1]) + (smem[2] + smem[3]);
}

// Rows that are contiguous in memory and a multiple of 8 long: the row lives in the registers of half a
// wavefront (TEAM = 32, eight rows per workgroup), of a wavefront (64) or of the workgroup (256).
constexpr int kMvn6MaxRegRow = 16384;  // longest row a workgroup keeps in registers (64 values per lane)
template <int TEAM, int VPT, int RPT = 1>  // RPT: consecutive rows a team walks, keeping a scale / bias that runs along the row in registers
__global__ __launch_bounds__(kThreads) void mvn6_rows_kernel(const half_t* __restrict__ in, half_t* __restrict__ out,
                                                             const half_t* __restrict__ sc, const half_t* __restrict__ bi,
                                                             Mvn6Geom g, int normalize_variance, int eps_mode, float eps) {
    __shared__ float red[8];
    static_assert(TEAM != 256 || RPT == 1, "the workgroup-wide sums have slots for one row");
    const int t = (int)(threadIdx.x % TEAM);
    const int64_t row0 = ((int64_t)blockIdx.x * (kThreads / TEAM) + threadIdx.x / TEAM) * RPT;
    // scale and bias that run along the row (and do not depend on it): loaded once for the RPT rows
    u32x4 scv[VPT], biv[VPT];
    if (RPT > 1) {
#pragma unroll
        for (int j = 0; j < VPT; j++) {
            const uint32_t e0 = (uint32_t)(j * TEAM + t) * 8;
            if (e0 < g.row_len) {
                if (sc) scv[j] = *reinterpret_cast<const u32x4*>(sc + e0);
                if (bi) biv[j] = *reinterpret_cast<const u32x4*>(bi + e0);
            }
        }
    }
#pragma unroll 1
    for (int rr = 0; rr < RPT; rr++) {
    int64_t row = row0 + rr;
    const bool live = row < g.rows;  // uniform per team; dead teams skip memory only
    if (!live) row = 0;
    const RowBase b = row_base(g, row);
    float x[VPT][8];
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < VPT; j++) {
        const uint32_t e0 = (uint32_t)(j * TEAM + t) * 8;
        if (live && e0 < g.row_len) {
            const u32x4 q = *reinterpret_cast<const u32x4*>(in + b.in + e0);
            const half_t* p = reinterpret_cast<const half_t*>(&q);
#pragma unroll
            for (int k = 0; k < 8; k++) {
                x[j][k] = (float)p[k];
                sum += x[j][k];
            }
        } else {
#pragma unroll
            for (int k = 0; k < 8; k++) x[j][k] = 0.f;
        }
    }
    const float n = (float)g.row_len;
    const float mean = team_sum<TEAM>(sum, red) / n;
    float q = 0.f;
#pragma unroll
    for (int j = 0; j < VPT; j++) {
        const uint32_t e0 = (uint32_t)(j * TEAM + t) * 8;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const float d = x[j][k] - mean;
            q += e0 < g.row_len ? d * d : 0.f;
        }
    }
    const float var = team_sum<TEAM>(q, red + 4) / n;
    const float inv = mvn6_inv(var, normalize_variance, eps_mode, eps);
    const float sc_row = sc && !g.sc_along_row ? (float)sc[b.sc] : 1.0f;
    const float bi_row = bi && !g.bi_along_row ? (float)bi[b.bi] : 0.0f;
#pragma unroll
    for (int j = 0; j < VPT; j++) {
        const uint32_t e0 = (uint32_t)(j * TEAM + t) * 8;
        if (!(live && e0 < g.row_len)) continue;
        float y[8];
#pragma unroll
        for (int k = 0; k < 8; k++) y[k] = (x[j][k] - mean) * inv;
        if (sc) {
            if (g.sc_along_row) {
                const u32x4 v = RPT > 1 ? scv[j] : *reinterpret_cast<const u32x4*>(sc + b.sc + e0);
                const half_t* p = reinterpret_cast<const half_t*>(&v);
#pragma unroll
                for (int k = 0; k < 8; k++) y[k] *= (float)p[k];
            } else {
#pragma unroll
                for (int k = 0; k < 8; k++) y[k] *= sc_row;
            }
        }
        if (bi) {
            if (g.bi_along_row) {
                const u32x4 v = RPT > 1 ? biv[j] : *reinterpret_cast<const u32x4*>(bi + b.bi + e0);
                const half_t* p = reinterpret_cast<const half_t*>(&v);
#pragma unroll
                for (int k = 0; k < 8; k++) y[k] += (float)p[k];
            } else {
#pragma unroll
                for (int k = 0; k < 8; k++) y[k] += bi_row;
            }
        }
        u32x4 o;
        half_t* po = reinterpret_cast<half_t*>(&o);
#pragma unroll
        for (int k = 0; k < 8; k++) po[k] = (half_t)y[k];
        __builtin_nontemporal_store(o, reinterpret_cast<u32x4*>(out + b.out + e0));
    }
    }
}

struct ElemOff {
    int64_t in, out, sc, bi;
};
__device__ __forceinline__ ElemOff elem_off(const Mvn6Geom& g, uint32_t e) {
    ElemOff o{0, 0, 0, 0};
    for (int d = 0; d < g.nr; d++) {
        const uint32_t c = e % (uint32_t)g.rdim[d];
        e /= (uint32_t)g.rdim[d];
        o.in += c * g.r_in[d];
        o.out += c * g.r_out[d];
        o.sc += c * g.r_sc[d];
        o.bi += c * g.r_bi[d];
    }
    return o;
}

// The innermost dimension is kept and contiguous (normalising over channels of a channel-major tensor,
// say): a workgroup takes P adjacent positions of it, so that every access covers a contiguous run, and
// splits the reduced elements over its 256 / P lane groups (group r walks elements r, r + G, ...; three
// passes, the later ones from cache).  Smaller P gives more workgroups when the tensor has few positions.
template <int P>
__global__ __launch_bounds__(kThreads) void mvn6_inner_kernel(const half_t* __restrict__ in, half_t* __restrict__ out,
                                                              const half_t* __restrict__ sc, const half_t* __restrict__ bi,
                                                              Mvn6Geom g, int normalize_variance, int eps_mode, float eps) {
    constexpr int G = kThreads / P;
    __shared__ float red[G][P];
    const int cl = threadIdx.x % P;
    const uint32_t r = P == 64 ? (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x / P)) : threadIdx.x / P;
    const int64_t tiles = (g.kdim[0] + P - 1) / P;
    int64_t o = blockIdx.x / tiles;
    const int64_t i0 = (blockIdx.x % tiles) * P + cl;
    const bool ok = i0 < g.kdim[0];
    RowBase b{0, 0, 0, 0};
    for (int d = 1; d < g.nk; d++) {
        const int64_t c = o % g.kdim[d];
        o /= g.kdim[d];
        b.in += c * g.k_in[d];
        b.out += c * g.k_out[d];
        b.sc += c * g.k_sc[d];
        b.bi += c * g.k_bi[d];
    }
    const int64_t i = ok ? i0 : 0;
    b.in += i * g.k_in[0];
    b.out += i * g.k_out[0];
    b.sc += i * g.k_sc[0];
    b.bi += i * g.k_bi[0];
    const float n = (float)g.row_len;
    const auto total = [&](float v) {
        __syncthreads();
        red[r][cl] = v;
        __syncthreads();
        float t = 0.f;
#pragma unroll
        for (int k = 0; k < G; k++) t += red[k][cl];
        return t;
    };
    float sum = 0.f;
    for (uint32_t e = r; e < g.row_len; e += G) sum += (float)in[b.in + elem_off(g, e).in];
    const float mean = total(sum) / n;
    float q = 0.f;
    if (normalize_variance)
        for (uint32_t e = r; e < g.row_len; e += G) {
            const float d = (float)in[b.in + elem_off(g, e).in] - mean;
            q += d * d;
        }
    const float var = total(q) / n;
    const float inv = mvn6_inv(var, normalize_variance, eps_mode, eps);
    if (!ok) return;
    for (uint32_t e = r; e < g.row_len; e += G) {
        const ElemOff off = elem_off(g, e);
        float y = ((float)in[b.in + off.in] - mean) * inv;
        if (sc) y *= (float)sc[b.sc + off.sc];
        if (bi) y += (float)bi[b.bi + off.bi];
        out[b.out + off.out] = (half_t)y;
    }
}

// Any layout, any row length: one workgroup per row, three passes over the row (the second and
// third come from cache).
__global__ __launch_bounds__(kThreads) void mvn6_generic_kernel(const half_t* __restrict__ in, half_t* __restrict__ out,
                                                                const half_t* __restrict__ sc, const half_t* __restrict__ bi,
                                                                Mvn6Geom g, int normalize_variance, int eps_mode, float eps) {
    __shared__ float red[8];
    const RowBase b = row_base(g, blockIdx.x);
    float sum = 0.f;
    for (uint32_t e = threadIdx.x; e < g.row_len; e += kThreads) sum += (float)in[b.in + elem_off(g, e).in];
    const float n = (float)g.row_len;
    const float mean = team_sum<256>(sum, red) / n;
    float q = 0.f;
    if (normalize_variance)
        for (uint32_t e = threadIdx.x; e < g.row_len; e += kThreads) {
            const float d = (float)in[b.in + elem_off(g, e).in] - mean;
            q += d * d;
        }
    const float var = team_sum<256>(q, red + 4) / n;
    const float inv = mvn6_inv(var, normalize_variance, eps_mode, eps);
    for (uint32_t e = threadIdx.x; e < g.row_len; e += kThreads) {
        const ElemOff o = elem_off(g, e);
        float y = ((float)in[b.in + o.in] - mean) * inv;
        if (sc) y *= (float)sc[b.sc + o.sc];
        if (bi) y += (float)bi[b.bi + o.bi];
        out[b.out + o.out] = (half_t)y;
    }
}


// mvn1 with per-channel statistics on a channel-minor layout: shifted partial sums over spatial ranges,
// a fold to {mean, 1/std}, then the element-wise pass.
int launch_channel_minor(const half_t* in, half_t* out, int64_t N, int64_t S, int64_t C, int nv, float eps, hipStream_t s) {
    const int64_t ctiles = (C + 63) / 64, cpad = ctiles * 64;
    // spatial ranges per image: enough workgroups to fill the chip (the eight-channel kernel has no channel tiles)
    const bool octets = C % 8 == 0 && C >= 8 && C <= 2048 && (reinterpret_cast<uintptr_t>(in) & 15) == 0;
    const int64_t per_range = octets ? N : N * ctiles;
    int64_t subparts = ((octets ? 2048 : 1024) + per_range - 1) / per_range;
    if (subparts > S / 64) subparts = S / 64;
    if (subparts < 1) subparts = 1;
    const int64_t per_n = S * C, piece = kThreads * 8, pieces = (per_n + piece - 1) / piece;
    VPX_REQUIRE(N * subparts * ctiles < (1ll << 31) && N * pieces < (1ll << 31) && C < (1ll << 31), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                "mvn1: tensor exceeds the launch limit");
    void* ws = nullptr;
    const size_t partial_bytes = sizeof(float2) * (size_t)(N * subparts * cpad);
    int rc = get_workspace(s, partial_bytes + sizeof(float) * (size_t)(N * 2 * C), &ws);
    if (rc) return rc;
    float2* partial = (float2*)ws;
    float* stats = (float*)((char*)ws + partial_bytes);
    rc = launch_sum_cminor<true>(in, N, S, C, subparts, cpad, partial, s);
    if (rc) return rc;
    hipLaunchKernelGGL(mvn_cminor_stats_kernel, dim3((unsigned)((N * C + kThreads - 1) / kThreads)), dim3(kThreads), 0, s, in,
                       (const float2*)partial, stats, N * C, S, C, cpad, (int)subparts, nv, eps);
    VPX_HIP_CHECK(hipGetLastError());
    const bool vec = C % 8 == 0 && ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0 &&
                     (reinterpret_cast<uintptr_t>(stats) & 31) == 0;
    if (vec)
        hipLaunchKernelGGL((mvn_norm_cminor_kernel<float, true>), dim3((unsigned)(N * pieces)), dim3(kThreads), 0, s, in, out,
                           (const float*)stats, per_n, C, (int)pieces, 2);
    else
        hipLaunchKernelGGL((mvn_norm_cminor_kernel<float, false>), dim3((unsigned)(N * pieces)), dim3(kThreads), 0, s, in, out,
                           (const float*)stats, per_n, C, (int)pieces, 2);
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

}  // namespace

int launch_mvn(const MemRef& in, const MemRef& out, bool across_channels, bool normalize_variance, float eps,
               hipStream_t s) {
    VPX_REQUIRE(in.dtype == VPX_NN_FP16 && out.dtype == VPX_NN_FP16, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                "mvn1: only FP16 input/output is implemented, got %s -> %s", dtype_name(in.dtype), dtype_name(out.dtype));
    VPX_REQUIRE(in.nd == 4 && out.nd == 4, VPX_RESULT_ERROR_INVALID_ARGUMENT, "mvn1: expects 4-D tensors, got rank %d",
                in.nd);
    VPX_REQUIRE(in.order == out.order, VPX_RESULT_ERROR_INVALID_ARGUMENT, "mvn1: input and output layouts differ");
    // Same layouts as the reference kernel (sw_kernel.cpp:946-953); compact operands only.
    VPX_REQUIRE(in.order == VPX_ORDER_NCHW || in.order == VPX_ORDER_NCWH || in.order == VPX_ORDER_NHWC ||
                        in.order == VPX_ORDER_NWHC,
                VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "mvn1: unsupported order 0x%llx", (unsigned long long)in.order);
    VPX_REQUIRE(in.compact && out.compact, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "mvn1: only compact tensors are supported");
    for (int d = 0; d < 4; d++)
        VPX_REQUIRE(in.dims[d] == out.dims[d], VPX_RESULT_ERROR_INVALID_ARGUMENT, "mvn1: input and output shapes differ");
    const int pn = mem_pos_of(in.order, 4, 0), pc = mem_pos_of(in.order, 4, 1);
    VPX_REQUIRE(pn == 3, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "mvn1: batch must be the outermost dimension");
    const int64_t N = in.dims[pn], C = in.dims[pc];
    const int64_t total = in.numel();
    if (total == 0) return VPX_RESULT_SUCCESS;
    const int64_t S = total / (N * C);
    const half_t* pi = (const half_t*)in.data;
    half_t* po = (half_t*)out.data;
    const int nv = normalize_variance ? 1 : 0;
    {   // in place is served (every kernel reads a value before it stores that value's result); any other overlap is not
        const uintptr_t ib = reinterpret_cast<uintptr_t>(pi), ob = reinterpret_cast<uintptr_t>(po);
        const uintptr_t bytes = (uintptr_t)total * sizeof(half_t);
        VPX_REQUIRE(ib == ob || ib + bytes <= ob || ob + bytes <= ib, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                    "mvn1: input and output overlap without being the same tensor");
    }

    int64_t groups, group_size;
    if (across_channels) {
        groups = N;
        group_size = C * S;
    } else if (pc == 2) {  // channel-major: each (n,c) plane is contiguous
        groups = N * C;
        group_size = S;
    } else {  // channel-minor layout, per-channel statistics
        return launch_channel_minor(pi, po, N, S, C, nv, eps, s);
    }
    if (tiny_groups_ok(pi, po, groups, group_size)) return launch_tiny_groups(pi, po, groups, group_size, nv, 0, eps, s);
    if (small_groups_ok(pi, po, groups, group_size)) return launch_small_groups(pi, po, groups, group_size, nv, 0, eps, s);
    if (lds_groups_ok(pi, po, groups, group_size)) return launch_lds_groups(pi, po, groups, group_size, nv, 0, eps, s);
    const bool aligned = group_size % 8 == 0 && (reinterpret_cast<uintptr_t>(pi) & 15) == 0 &&
                         (reinterpret_cast<uintptr_t>(po) & 15) == 0;
    return aligned ? launch_groups<true>(pi, po, groups, group_size, nv, eps, s)
                   : launch_groups<false>(pi, po, groups, group_size, nv, eps, s);
}

int launch_mvn_sum(const MemRef& in, const MemRef& out, bool across_channels, bool normalize_variance, hipStream_t s) {
    VPX_REQUIRE(in.dtype == VPX_NN_FP16 && out.dtype == VPX_NN_FP32, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                "mvn1_sum: FP16 input and FP32 sums are implemented, got %s -> %s", dtype_name(in.dtype), dtype_name(out.dtype));
    MvnShape sh;
    int rc = mvn_shape("mvn1_sum", in, sh);
    if (rc) return rc;
    int64_t od[4];
    rc = stats_shape("mvn1_sum", out, od);
    if (rc) return rc;
    const int64_t out_c = across_channels ? 1 : sh.C;
    const int out_w = normalize_variance ? 2 : 1;
    VPX_REQUIRE(od[0] == sh.N && od[1] == out_c && od[2] >= 1 && od[3] == out_w, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                "mvn1_sum: output shape [%lld,%lld,%lld,%lld] does not match [%lld,%lld,parts,%d]", (long long)od[0],
                (long long)od[1], (long long)od[2], (long long)od[3], (long long)sh.N, (long long)out_c, out_w);
    VPX_REQUIRE(od[2] <= 4096, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "mvn1_sum: %lld partial sums per group", (long long)od[2]);
    if (in.numel() == 0) return VPX_RESULT_SUCCESS;
    const SumOut o{(float*)out.data, (int)od[2], out_w, out_c};
    const half_t* pi = (const half_t*)in.data;

    if (!across_channels && sh.channel_minor) {
        const int64_t ctiles = (sh.C + 63) / 64, cpad = ctiles * 64;
        // enough spatial ranges to spread over the device, at least 64 positions each
        int64_t isplit = (1024 + sh.N * ctiles * o.parts - 1) / (sh.N * ctiles * o.parts);
        const int64_t most = sh.S / (64 * (int64_t)o.parts);
        if (isplit > most) isplit = most;
        if (isplit < 1) isplit = 1;
        const int64_t subparts = isplit * o.parts;
        const int64_t blocks = sh.N * subparts * ctiles, total = sh.N * o.parts * sh.C;
        VPX_REQUIRE(blocks < (1ll << 31) && total < (1ll << 31) * kThreads, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                    "mvn1_sum: tensor exceeds the launch limit");
        void* ws = nullptr;
        rc = get_workspace(s, sizeof(float2) * (size_t)(sh.N * subparts * cpad), &ws);
        if (rc) return rc;
        rc = launch_sum_cminor<false>(pi, sh.N, sh.S, sh.C, subparts, cpad, (float2*)ws, s);
        if (rc) return rc;
        hipLaunchKernelGGL(mvn_sum_cminor_finish_kernel, dim3((unsigned)((total + kThreads - 1) / kThreads)), dim3(kThreads), 0,
                           s, (const float2*)ws, total, sh.C, cpad, (int)subparts, (int)isplit, o);
        VPX_HIP_CHECK(hipGetLastError());
        return VPX_RESULT_SUCCESS;
    }

    const int64_t groups = across_channels ? sh.N : sh.N * sh.C;
    const int64_t group_size = across_channels ? sh.C * sh.S : sh.S;
    const int64_t chunks64 = (group_size + kChunk - 1) / kChunk;
    VPX_REQUIRE(chunks64 * groups < (1ll << 31) && groups * o.parts < (1ll << 31), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                "mvn1_sum: %lld groups of %lld elements exceed the launch limit", (long long)groups, (long long)group_size);
    const int chunks = (int)chunks64;
    const bool direct = chunks == 1 && o.parts == 1;
    void* ws = nullptr;
    if (!direct) {
        rc = get_workspace(s, sizeof(float2) * (size_t)(groups * chunks), &ws);
        if (rc) return rc;
    }
    const bool aligned = group_size % 8 == 0 && (reinterpret_cast<uintptr_t>(pi) & 15) == 0;
    const dim3 grid((unsigned)(groups * chunks));
    if (aligned)
        hipLaunchKernelGGL((mvn_sum_chunk_kernel<true>), grid, dim3(kThreads), 0, s, pi, group_size, chunks, (float2*)ws, o,
                           direct ? 1 : 0);
    else
        hipLaunchKernelGGL((mvn_sum_chunk_kernel<false>), grid, dim3(kThreads), 0, s, pi, group_size, chunks, (float2*)ws, o,
                           direct ? 1 : 0);
    VPX_HIP_CHECK(hipGetLastError());
    if (!direct) {
        hipLaunchKernelGGL(mvn_sum_finish_kernel, dim3((unsigned)(groups * o.parts)), dim3(kThreads), 0, s, (const float2*)ws,
                           chunks, o);
        VPX_HIP_CHECK(hipGetLastError());
    }
    return VPX_RESULT_SUCCESS;
}

int launch_mvn_mean_var(const MemRef& sum, const MemRef& out, const int64_t orig_shape[4], bool across_channels,
                        bool normalize_variance, int64_t group_c, float eps, hipStream_t s) {
    VPX_REQUIRE(sum.dtype == VPX_NN_FP32 && (out.dtype == VPX_NN_FP16 || out.dtype == VPX_NN_FP32),
                VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "mvn1_mean_var: FP32 sums and FP16/FP32 output are implemented, got %s -> %s",
                dtype_name(sum.dtype), dtype_name(out.dtype));
    int64_t id[4], od[4];
    int rc = stats_shape("mvn1_mean_var", sum, id);
    if (rc) return rc;
    rc = stats_shape("mvn1_mean_var", out, od);
    if (rc) return rc;
    for (int i = 0; i < 4; i++)
        VPX_REQUIRE(orig_shape[i] >= 1, VPX_RESULT_ERROR_INVALID_ARGUMENT, "mvn1_mean_var: orig_shape[%d] = %lld", i,
                    (long long)orig_shape[i]);
    const int64_t N = orig_shape[0], C = orig_shape[1];
    const int64_t out_c = across_channels ? 1 : C;
    const int out_w = normalize_variance ? 2 : 1;
    VPX_REQUIRE(id[0] == N && id[3] >= out_w && id[3] <= 2 && id[1] == out_c, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                "mvn1_mean_var: sums of shape [%lld,%lld,%lld,%lld] do not fit the original shape [%lld,%lld,..] (%s channels)",
                (long long)id[0], (long long)id[1], (long long)id[2], (long long)id[3], (long long)N, (long long)C,
                across_channels ? "across" : "per");
    VPX_REQUIRE(od[0] == N && od[1] == out_c && od[2] == 1 && od[3] == out_w, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                "mvn1_mean_var: output shape [%lld,%lld,%lld,%lld] does not match [%lld,%lld,1,%d]", (long long)od[0],
                (long long)od[1], (long long)od[2], (long long)od[3], (long long)N, (long long)out_c, out_w);
    VPX_REQUIRE(group_c >= 1 && C % group_c == 0, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                "mvn1_mean_var: %lld channels per group does not divide %lld channels", (long long)group_c, (long long)C);
    VPX_REQUIRE(eps >= 0.f, VPX_RESULT_ERROR_INVALID_ARGUMENT, "mvn1_mean_var: eps must not be negative, got %g", (double)eps);
    const double count = (double)orig_shape[2] * (double)orig_shape[3] * (double)(across_channels ? C : group_c);
    const dim3 grid((unsigned)((N * out_c + kThreads - 1) / kThreads));
    if (out.dtype == VPX_NN_FP16)
        hipLaunchKernelGGL((mvn_mean_var_kernel<half_t>), grid, dim3(kThreads), 0, s, (const float*)sum.data, (half_t*)out.data, N,
                           id[1], (int)id[2], (int)id[3], out_c, out_w, across_channels ? 1 : 0, group_c, count, eps);
    else
        hipLaunchKernelGGL((mvn_mean_var_kernel<float>), grid, dim3(kThreads), 0, s, (const float*)sum.data, (float*)out.data, N,
                           id[1], (int)id[2], (int)id[3], out_c, out_w, across_channels ? 1 : 0, group_c, count, eps);
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

template <typename TS>
static int mvn_norm_impl(const MemRef& in, const MemRef& mv, const MemRef& out, const MvnShape& sh, bool across_channels, int out_w,
                         hipStream_t s) {
    const half_t* pi = (const half_t*)in.data;
    half_t* po = (half_t*)out.data;
    const TS* pm = (const TS*)mv.data;
    const int64_t piece = kThreads * 8;
    if (!across_channels && sh.channel_minor) {
        const int64_t per_n = sh.S * sh.C;
        const int64_t pieces = (per_n + piece - 1) / piece;
        VPX_REQUIRE(sh.N * pieces < (1ll << 31) && sh.C < (1ll << 31), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                    "mvn1_norm: tensor exceeds the launch limit");
        const bool vec = sh.C % 8 == 0 && ((reinterpret_cast<uintptr_t>(pi) | reinterpret_cast<uintptr_t>(po)) & 15) == 0 &&
                         (reinterpret_cast<uintptr_t>(pm) & 31) == 0;
        if (vec)
            hipLaunchKernelGGL((mvn_norm_cminor_kernel<TS, true>), dim3((unsigned)(sh.N * pieces)), dim3(kThreads), 0, s, pi, po, pm,
                               per_n, sh.C, (int)pieces, out_w);
        else
            hipLaunchKernelGGL((mvn_norm_cminor_kernel<TS, false>), dim3((unsigned)(sh.N * pieces)), dim3(kThreads), 0, s, pi, po, pm,
                               per_n, sh.C, (int)pieces, out_w);
        VPX_HIP_CHECK(hipGetLastError());
        return VPX_RESULT_SUCCESS;
    }
    const int64_t rows = across_channels ? sh.N : sh.N * sh.C;
    const int64_t run = across_channels ? sh.C * sh.S : sh.S;
    const int64_t pieces = (run + piece - 1) / piece;
    VPX_REQUIRE(rows * pieces < (1ll << 31), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "mvn1_norm: tensor exceeds the launch limit");
    const bool aligned = run % 8 == 0 && (reinterpret_cast<uintptr_t>(pi) & 15) == 0 && (reinterpret_cast<uintptr_t>(po) & 15) == 0;
    const int64_t rows_per_n = across_channels ? 1 : sh.C;
    const int64_t out_c = across_channels ? 1 : sh.C;
    const dim3 grid((unsigned)(rows * pieces));
    if (aligned)
        hipLaunchKernelGGL((mvn_norm_runs_kernel<TS, true>), grid, dim3(kThreads), 0, s, pi, po, pm, run, (int)pieces, rows_per_n,
                           out_c, out_w);
    else
        hipLaunchKernelGGL((mvn_norm_runs_kernel<TS, false>), grid, dim3(kThreads), 0, s, pi, po, pm, run, (int)pieces, rows_per_n,
                           out_c, out_w);
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

int launch_mvn_norm(const MemRef& in, const MemRef& mean_var, const MemRef& out, bool across_channels, bool normalize_variance,
                    hipStream_t s) {
    VPX_REQUIRE(in.dtype == VPX_NN_FP16 && out.dtype == VPX_NN_FP16, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                "mvn1_norm: only FP16 input/output is implemented, got %s -> %s", dtype_name(in.dtype), dtype_name(out.dtype));
    VPX_REQUIRE(mean_var.dtype == VPX_NN_FP16 || mean_var.dtype == VPX_NN_FP32, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                "mvn1_norm: statistics must be FP16 or FP32, got %s", dtype_name(mean_var.dtype));
    MvnShape sh;
    int rc = mvn_shape("mvn1_norm", in, sh);
    if (rc) return rc;
    VPX_REQUIRE(out.nd == 4 && out.order == in.order && out.compact, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                "mvn1_norm: output must be a compact tensor of the input's layout");
    for (int d = 0; d < 4; d++)
        VPX_REQUIRE(in.dims[d] == out.dims[d], VPX_RESULT_ERROR_INVALID_ARGUMENT, "mvn1_norm: input and output shapes differ");
    int64_t md[4];
    rc = stats_shape("mvn1_norm", mean_var, md);
    if (rc) return rc;
    const int out_w = normalize_variance ? 2 : 1;
    VPX_REQUIRE(md[0] == sh.N && md[1] == (across_channels ? 1 : sh.C) && md[2] == 1 && md[3] == out_w,
                VPX_RESULT_ERROR_INVALID_ARGUMENT, "mvn1_norm: statistics of shape [%lld,%lld,%lld,%lld] do not match [%lld,%lld,1,%d]",
                (long long)md[0], (long long)md[1], (long long)md[2], (long long)md[3], (long long)sh.N,
                (long long)(across_channels ? 1 : sh.C), out_w);
    if (in.numel() == 0) return VPX_RESULT_SUCCESS;
    if (mean_var.dtype == VPX_NN_FP16) return mvn_norm_impl<half_t>(in, mean_var, out, sh, across_channels, out_w, s);
    return mvn_norm_impl<float>(in, mean_var, out, sh, across_channels, out_w, s);
}

namespace {

// How an optional operand varies along a row whose reduced dimensions have element strides `stride`:
// 1 = laid out like the contiguous row, 0 = constant along the row, -1 = neither.
int along_row(bool present, const int32_t* rdim, const int64_t* stride, int nr) {
    if (!present) return 0;
    bool constant = true, full = true;
    int64_t expect = 1;
    for (int d = 0; d < nr; d++) {
        if (stride[d] != 0) constant = false;
        if (stride[d] != expect) full = false;
        expect *= rdim[d];
    }
    return constant ? 0 : (full ? 1 : -1);
}

bool aligned_rows(const void* p, const int64_t* kstride, int nk) {
    if (reinterpret_cast<uintptr_t>(p) & 15) return false;
    for (int d = 0; d < nk; d++)
        if (kstride[d] % 8 != 0) return false;
    return true;
}

}  // namespace

int launch_mvn6(const MemRef& in, const MemRef* scale, const MemRef* bias, const MemRef& out, bool normalize_variance, int eps_mode,
                float eps, const int64_t* mem_axes, int n_axes, hipStream_t s) {
    VPX_REQUIRE(in.dtype == VPX_NN_FP16 && out.dtype == VPX_NN_FP16, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                "mvn6: only FP16 input/output is implemented, got %s -> %s", dtype_name(in.dtype), dtype_name(out.dtype));
    VPX_REQUIRE(in.nd == out.nd && in.nd <= kMaxDims, VPX_RESULT_ERROR_INVALID_ARGUMENT, "mvn6: ranks %d / %d (at most %d)", in.nd,
                out.nd, kMaxDims);
    for (int d = 0; d < in.nd; d++)
        VPX_REQUIRE(in.dims[d] == out.dims[d], VPX_RESULT_ERROR_INVALID_ARGUMENT, "mvn6: input and output shapes differ");
    VPX_REQUIRE(eps_mode == 0 || eps_mode == 1, VPX_RESULT_ERROR_INVALID_ARGUMENT, "mvn6: unknown eps mode %d", eps_mode);
    VPX_REQUIRE(eps >= 0.f, VPX_RESULT_ERROR_INVALID_ARGUMENT, "mvn6: eps must not be negative, got %g", (double)eps);
    VPX_REQUIRE(n_axes >= 1 && n_axes <= in.nd, VPX_RESULT_ERROR_INVALID_ARGUMENT, "mvn6: %d axes for rank %d", n_axes, in.nd);
    bool reduced[kMaxDims] = {};
    for (int i = 0; i < n_axes; i++) {
        VPX_REQUIRE(mem_axes[i] >= 0 && mem_axes[i] < in.nd && !reduced[mem_axes[i]], VPX_RESULT_ERROR_INVALID_ARGUMENT,
                    "mvn6: axis %lld is outside rank %d or repeated", (long long)mem_axes[i], in.nd);
        reduced[mem_axes[i]] = true;
    }
    const MemRef* extra[2] = {scale, bias};
    for (const MemRef* m : extra) {
        if (!m) continue;
        VPX_REQUIRE(m->dtype == VPX_NN_FP16 && m->nd == in.nd, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                    "mvn6: scale / bias must be FP16 tensors of the input's rank");
        for (int d = 0; d < in.nd; d++)
            VPX_REQUIRE(m->dims[d] == in.dims[d] || m->dims[d] == 1, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                        "mvn6: scale / bias dimension %d is %lld, input has %lld", d, (long long)m->dims[d], (long long)in.dims[d]);
    }
    if (in.numel() == 0) return VPX_RESULT_SUCCESS;

    Mvn6Geom g{};
    int64_t row_len = 1;
    g.rows = 1;
    bool innermost = true;   // the reduced dimensions are the innermost ones
    bool inner_kept = false;  // the innermost dimension (of more than one element) is kept
    for (int d = 0; d < in.nd; d++) {
        if (in.dims[d] == 1) continue;
        if (g.nk + g.nr == 0) inner_kept = !reduced[d];
        const int64_t ssc = scale && scale->dims[d] != 1 ? scale->strides[d] : 0;
        const int64_t sbi = bias && bias->dims[d] != 1 ? bias->strides[d] : 0;
        if (reduced[d]) {
            if (g.nk > 0) innermost = false;
            g.rdim[g.nr] = (int32_t)in.dims[d];
            g.r_in[g.nr] = in.strides[d];
            g.r_out[g.nr] = out.strides[d];
            g.r_sc[g.nr] = ssc;
            g.r_bi[g.nr] = sbi;
            g.nr++;
            row_len *= in.dims[d];
        } else {
            g.kdim[g.nk] = (int32_t)in.dims[d];
            g.k_in[g.nk] = in.strides[d];
            g.k_out[g.nk] = out.strides[d];
            g.k_sc[g.nk] = ssc;
            g.k_bi[g.nk] = sbi;
            g.nk++;
            g.rows *= in.dims[d];
        }
    }
    // Kept dimensions that every operand walks as one (stride of the outer = stride x extent of the inner) fold
    // into one, so a packed tensor's rows are found without a division.
    for (int d = 0; d + 1 < g.nk;) {
        const int64_t e = g.kdim[d];
        if (g.k_in[d + 1] == g.k_in[d] * e && g.k_out[d + 1] == g.k_out[d] * e && g.k_sc[d + 1] == g.k_sc[d] * e &&
            g.k_bi[d + 1] == g.k_bi[d] * e && e * g.kdim[d + 1] < (1ll << 31)) {
            g.kdim[d] = (int32_t)(e * g.kdim[d + 1]);
            for (int k = d + 1; k + 1 < g.nk; k++) {
                g.kdim[k] = g.kdim[k + 1];
                g.k_in[k] = g.k_in[k + 1];
                g.k_out[k] = g.k_out[k + 1];
                g.k_sc[k] = g.k_sc[k + 1];
                g.k_bi[k] = g.k_bi[k + 1];
            }
            g.nk--;
        } else {
            d++;
        }
    }
    VPX_REQUIRE(row_len < (1ll << 31) && g.rows < (1ll << 31), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                "mvn6: %lld rows of %lld elements exceed the launch limit", (long long)g.rows, (long long)row_len);
    g.row_len = (uint32_t)row_len;
    const half_t* pi = (const half_t*)in.data;
    half_t* po = (half_t*)out.data;
    const half_t* ps = scale ? (const half_t*)scale->data : nullptr;
    const half_t* pb = bias ? (const half_t*)bias->data : nullptr;
    const int nv = normalize_variance ? 1 : 0;

    // Long contiguous rows of a compact tensor, eps inside the root, no scale or bias: the chunked two-launch
    // scheme of mvn1 (a row is a group there).
    if (innermost && row_len > kMvn6MaxRegRow && !scale && !bias && in.compact && out.compact && lds_groups_ok(pi, po, g.rows, row_len))
        return launch_lds_groups(pi, po, g.rows, row_len, nv, eps_mode, eps, s);
    if (innermost && row_len > kMvn6MaxRegRow && !scale && !bias && eps_mode == 0 && in.compact && out.compact) {
        const bool aligned = row_len % 8 == 0 && ((reinterpret_cast<uintptr_t>(pi) | reinterpret_cast<uintptr_t>(po)) & 15) == 0;
        return aligned ? launch_groups<true>(pi, po, g.rows, row_len, nv, eps, s) : launch_groups<false>(pi, po, g.rows, row_len, nv, eps, s);
    }
    // Short contiguous rows whose length is not a multiple of eight (7 x 7 planes, rows of 100): runs of whole rows
    // per workgroup, as for mvn1's short groups.
    if (innermost && !scale && !bias && in.compact && out.compact && tiny_groups_ok(pi, po, g.rows, row_len))
        return launch_tiny_groups(pi, po, g.rows, row_len, nv, eps_mode, eps, s);
    if (innermost && row_len % 8 != 0 && !scale && !bias && in.compact && out.compact && small_groups_ok(pi, po, g.rows, row_len))
        return launch_small_groups(pi, po, g.rows, row_len, nv, eps_mode, eps, s);
    bool fast = innermost && row_len % 8 == 0 && row_len <= kMvn6MaxRegRow;
    if (fast) {
        fast = along_row(true, g.rdim, g.r_in, g.nr) == 1 && along_row(true, g.rdim, g.r_out, g.nr) == 1;
        g.sc_along_row = along_row(scale != nullptr, g.rdim, g.r_sc, g.nr);
        g.bi_along_row = along_row(bias != nullptr, g.rdim, g.r_bi, g.nr);
        fast = fast && g.sc_along_row >= 0 && g.bi_along_row >= 0 && aligned_rows(pi, g.k_in, g.nk) && aligned_rows(po, g.k_out, g.nk);
        if (fast && scale && g.sc_along_row) fast = aligned_rows(ps, g.k_sc, g.nk);
        if (fast && bias && g.bi_along_row) fast = aligned_rows(pb, g.k_bi, g.nk);
    }
    if (fast) {
#define VPX_MVN6_ROWS(TEAM, VPT) \
    hipLaunchKernelGGL((mvn6_rows_kernel<TEAM, VPT>), dim3((unsigned)((g.rows + kThreads / TEAM - 1) / (kThreads / TEAM))), \
                       dim3(kThreads), 0, s, pi, po, ps, pb, g, nv, eps_mode, eps)
        // A scale / bias shared by all rows stays in registers while a team walks 2 or 4 consecutive rows, as long
        // as that leaves 4096 workgroups (two rounds of the chip) or more.
        bool shared_rows = (scale && g.sc_along_row) || (bias && g.bi_along_row);
        for (int d = 0; d < g.nk; d++)
            if ((scale && g.sc_along_row && g.k_sc[d] != 0) || (bias && g.bi_along_row && g.k_bi[d] != 0)) shared_rows = false;
        const bool half768 = shared_rows && row_len == 768;  // 32 lanes x 3 words, none idle: pays with scale / bias
        const int team = row_len <= 256 || half768 ? 32 : 64;
        const int64_t team_rows = g.rows / (kThreads / team);
        const int rpt = !shared_rows ? 1 : team_rows >= 4 * 4096 ? 4 : team_rows >= 2 * 4096 ? 2 : 1;
#define VPX_MVN6_ROWS_R(TEAM, VPT, RPT) \
    hipLaunchKernelGGL((mvn6_rows_kernel<TEAM, VPT, RPT>), dim3((unsigned)((g.rows + RPT * kThreads / TEAM - 1) / (RPT * kThreads / TEAM))), \
                       dim3(kThreads), 0, s, pi, po, ps, pb, g, nv, eps_mode, eps)
#define VPX_MVN6_SHORT(TEAM, VPT)                   \
    do {                                            \
        if (rpt == 4) VPX_MVN6_ROWS_R(TEAM, VPT, 4); \
        else if (rpt == 2) VPX_MVN6_ROWS_R(TEAM, VPT, 2); \
        else VPX_MVN6_ROWS(TEAM, VPT);              \
    } while (0)
        if (row_len <= 256) VPX_MVN6_SHORT(32, 1);
        else if (row_len <= 512) VPX_MVN6_SHORT(64, 1);
        else if (half768) VPX_MVN6_SHORT(32, 3);
        else if (row_len <= 1024) VPX_MVN6_SHORT(64, 2);
        else if (row_len <= 1536) VPX_MVN6_SHORT(64, 3);
        else if (row_len <= 2048) VPX_MVN6_SHORT(64, 4);
        else if (row_len <= 2560) VPX_MVN6_SHORT(64, 5);
        else if (row_len > 2560 && row_len <= 3072) VPX_MVN6_SHORT(64, 6);
        else if (row_len <= 2048) VPX_MVN6_ROWS(256, 1);
        else if (row_len <= 4096) VPX_MVN6_ROWS(256, 2);  // one wavefront per 4096-element row measured 9 % slower
        else if (row_len <= 6144) VPX_MVN6_ROWS(256, 3);
        else if (row_len <= 8192) VPX_MVN6_ROWS(256, 4);
        else if (row_len <= 10240) VPX_MVN6_ROWS(256, 5);
        else if (row_len <= 12288) VPX_MVN6_ROWS(256, 6);
        else if (row_len <= 14336) VPX_MVN6_ROWS(256, 7);
        else VPX_MVN6_ROWS(256, 8);
#undef VPX_MVN6_ROWS
#undef VPX_MVN6_ROWS_R
#undef VPX_MVN6_SHORT
    } else if (inner_kept && g.k_in[0] == 1 && g.k_out[0] == 1) {
        const int64_t outer = g.rows / g.kdim[0];
        const auto blocks = [&](int p) { return outer * ((g.kdim[0] + p - 1) / p); };
        if (blocks(64) >= 512)
            hipLaunchKernelGGL(mvn6_inner_kernel<64>, dim3((unsigned)blocks(64)), dim3(kThreads), 0, s, pi, po, ps, pb, g, nv, eps_mode, eps);
        else if (blocks(32) >= 512)
            hipLaunchKernelGGL(mvn6_inner_kernel<32>, dim3((unsigned)blocks(32)), dim3(kThreads), 0, s, pi, po, ps, pb, g, nv, eps_mode, eps);
        else
            hipLaunchKernelGGL(mvn6_inner_kernel<16>, dim3((unsigned)blocks(16)), dim3(kThreads), 0, s, pi, po, ps, pb, g, nv, eps_mode, eps);
    } else {
        hipLaunchKernelGGL(mvn6_generic_kernel, dim3((unsigned)g.rows), dim3(kThreads), 0, s, pi, po, ps, pb, g, nv, eps_mode, eps);
    }
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

}  // namespace vpx
