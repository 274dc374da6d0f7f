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

// Per-channel statistics of a channel-minor layout (NHWC / NWHC): element (n,s,c) at
// n*S*C + s*C + c.  A workgroup takes 64 channels of one batch element; lane (r, c) walks the
// spatial positions r, r+4, ... so that every access covers 64 adjacent channels.
__global__ __launch_bounds__(kThreads) void mvn_channel_minor_kernel(const half_t* __restrict__ in,
                                                                     half_t* __restrict__ out, int64_t S, int64_t C,
                                                                     int normalize_variance, float eps) {
    __shared__ float red[4][64];
    const int cl = threadIdx.x & 63, r = threadIdx.x >> 6;
    const int64_t ctiles = (C + 63) / 64;
    const int64_t n = blockIdx.x / ctiles;
    const int64_t c = (blockIdx.x % ctiles) * 64 + cl;
    const bool ok = c < C;
    const half_t* px = in + n * S * C + c;
    half_t* py = out + n * S * C + c;
    float s = 0.f;
    if (ok)
        for (int64_t i = r; i < S; i += 4) s += (float)px[i * C];
    red[r][cl] = s;
    __syncthreads();
    const float mean = ((red[0][cl] + red[1][cl]) + (red[2][cl] + red[3][cl])) / (float)S;
    __syncthreads();
    float q = 0.f;
    if (ok)
        for (int64_t i = r; i < S; i += 4) {
            const float d = (float)px[i * C] - mean;
            q += d * d;
        }
    red[r][cl] = q;
    __syncthreads();
    const float var = ((red[0][cl] + red[1][cl]) + (red[2][cl] + red[3][cl])) / (float)S;
    const float inv = normalize_variance ? 1.0f / __builtin_sqrtf(var + eps) : 1.0f;
    if (ok)
        for (int64_t i = r; i < S; i += 4) py[i * C] = (half_t)(((float)px[i * C] - mean) * inv);
}

// position (counted from the innermost memory dimension) of logical dimension `logical`
int mem_pos_of(uint64_t order, int nd, int logical) {
    for (int i = 0; i < nd; i++)
        if ((int)((order >> (4 * i)) & 0xf) == logical + 1) return nd - 1 - i;
    return -1;
}

template <bool ALIGNED>
int launch_groups(const half_t* in, half_t* out, int64_t groups, int64_t group_size, int nv, float eps, hipStream_t s) {
    const int64_t chunks64 = (group_size + kChunk - 1) / kChunk;
    VPX_REQUIRE(chunks64 * groups < (1ll << 31), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                "mvn1: %lld groups of %lld elements exceed the launch limit", (long long)groups, (long long)group_size);
    const int chunks = (int)chunks64;
    const unsigned blocks = (unsigned)(groups * chunks);
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

    int64_t groups, group_size;
    if (across_channels) {
        groups = N;
        group_size = C * S;
    } else if (pc == 2) {  // channel-major: each (n,c) plane is contiguous
        groups = N * C;
        group_size = S;
    } else {  // channel-minor layout, per-channel statistics
        const int64_t ctiles = (C + 63) / 64;
        VPX_REQUIRE(N * ctiles < (1ll << 31), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "mvn1: tensor exceeds the launch limit");
        hipLaunchKernelGGL(mvn_channel_minor_kernel, dim3((unsigned)(N * ctiles)), dim3(kThreads), 0, s, pi, po, S, C, nv,
                           eps);
        VPX_HIP_CHECK(hipGetLastError());
        return VPX_RESULT_SUCCESS;
    }
    const bool aligned = group_size % 8 == 0 && (reinterpret_cast<uintptr_t>(pi) & 15) == 0 &&
                         (reinterpret_cast<uintptr_t>(po) & 15) == 0;
    return aligned ? launch_groups<true>(pi, po, groups, group_size, nv, eps, s)
                   : launch_groups<false>(pi, po, groups, group_size, nv, eps, s);
}

}  // namespace vpx
