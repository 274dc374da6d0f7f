// Streaming ACT-SHAVE kernels: convert, eltwise_*, fake_quantize, quantize, dequantize.
//
// All of them are HBM-bound maps.  The fast path views compact operands as flat arrays and moves
// 128 bits per lane per access, several independent accesses in flight per lane; a strided /
// broadcasting path covers sub-views and NUMPY broadcast one element per lane.
#include "vpx_common.h"

namespace vpx {

namespace {

typedef _Float16 half_t;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <int BYTES>
struct Words;
template <>
struct Words<4> {
    typedef uint32_t type;
};
template <>
struct Words<8> {
    typedef u32x2 type;
};
template <>
struct Words<16> {
    typedef u32x4 type;
};

// N elements of T moved by one 32/64/128-bit access per lane.  Adjacent lanes touch adjacent
// words, so a wavefront's access is one contiguous run; the wider operand of a kernel gets the
// 128-bit form.  Stores are non-temporal (results are not re-read); loads are ordinary, which
// measures faster than non-temporal loads on this memory system.
template <typename T, int N>
struct Pack {
    typedef typename Words<sizeof(T) * N>::type W;
    W q;
    __device__ __forceinline__ T get(int k) const { return reinterpret_cast<const T*>(&q)[k]; }
    __device__ __forceinline__ void set(int k, T v) { reinterpret_cast<T*>(&q)[k] = v; }
    __device__ __forceinline__ void load(const T* base, int64_t v) { q = reinterpret_cast<const W*>(base)[v]; }
    __device__ __forceinline__ void store(T* base, int64_t v) const {
        __builtin_nontemporal_store(q, reinterpret_cast<W*>(base) + v);
    }
};

constexpr int kBlock = 256;
constexpr int kUnroll = 4;

// fp32 -> fp16 with the exact behaviour of vpux::type::float16
// (src/vpux_utils/src/core/type/float16.cpp:30-108): round to nearest even; a NaN keeps its sign
// and top ten payload bits (at least one set); and a value below 2^-15 whose mantissa is at least
// 0x7ff000 rounds as if it were doubled (the exponent bump of the reference's first rounding step
// leaks into its subnormal branch, :74-107).
__device__ __forceinline__ half_t f32_to_f16(float f) {
    const uint32_t bits = __builtin_bit_cast(uint32_t, f);
    const uint32_t e = bits & 0x7f800000u;
    const bool doubled = e != 0 && e <= (111u << 23) && (bits & 0x7fffffu) >= 0x7ff000u;
    half_t h = (half_t)(doubled ? f * 2.0f : f);
    if (__builtin_isnan(f)) {
        uint32_t payload = (bits & 0x7fffffu) >> 13;
        payload = payload ? payload : 1u;
        const uint16_t hb = (uint16_t)(((bits >> 16) & 0x8000u) | 0x7c00u | payload);
        h = __builtin_bit_cast(half_t, hb);
    }
    return h;
}

// vpux::fakeQuantize, src/vpux_compiler/src/utils/quantization.cpp:995-1003 (fp32, round half away)
__device__ __forceinline__ float fq_f32(float x, float ilo, float ihi, float olo, float ohi, float lm1) {
    const float q = roundf((x - ilo) / (ihi - ilo) * lm1) / lm1 * (ohi - olo) + olo;
    return x <= ilo ? olo : (x > ihi ? ohi : q);
}

template <typename T>
__device__ __forceinline__ T narrow(float r);
template <>
__device__ __forceinline__ half_t narrow<half_t>(float r) {
    return f32_to_f16(r);
}
template <>
__device__ __forceinline__ float narrow<float>(float r) {
    return r;
}

// ---------------------------------------------------------------- flat streaming skeleton
// F provides: static constexpr int VEC; void vec(int64_t v) (elements [v*VEC, v*VEC+VEC)); void one(int64_t i).
template <class F, int BLOCK, int UNROLL>
__global__ __launch_bounds__(BLOCK) void stream_kernel(F f, int64_t n_vec, int64_t n) {
    const int64_t block0 = (int64_t)blockIdx.x * (BLOCK * UNROLL);
    if (block0 + BLOCK * UNROLL <= n_vec) {
        f.template vecs<UNROLL>(block0 + threadIdx.x, BLOCK);
    } else {
        for (int u = 0; u < UNROLL; u++) {
            const int64_t v = block0 + u * BLOCK + threadIdx.x;
            if (v < n_vec) f.template vecs<1>(v, 0);
        }
    }
    // ragged tail, fewer than VEC elements
    if (blockIdx.x == gridDim.x - 1) {
        const int64_t i = n_vec * F::VEC + threadIdx.x;
        if (i < n) f.one(i);
    }
}

template <class F>
int launch_stream(const F& f, int64_t n, hipStream_t s) {
    if (n <= 0) return VPX_RESULT_SUCCESS;
    const int64_t n_vec = n / F::VEC;
    // A tensor too small to give every compute unit several full-size workgroups is latency-bound:
    // fewer vectors per lane, and in the end single-wave workgroups, spread it over more units.
    const int tier = n_vec >= (int64_t)kBlock * kUnroll * 2048 ? 2 : (n_vec >= (int64_t)kBlock * 1024 ? 1 : 0);
    const int64_t per_block = tier == 2 ? kBlock * kUnroll : (tier == 1 ? kBlock : 64);
    int64_t blocks = (n_vec + per_block - 1) / per_block;
    if (blocks < 1) blocks = 1;
    VPX_REQUIRE(blocks < (1ll << 31), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "tensor of %lld elements is too large",
                (long long)n);
    const dim3 grid((unsigned)blocks);
    if (tier == 2) hipLaunchKernelGGL((stream_kernel<F, kBlock, kUnroll>), grid, dim3(kBlock), 0, s, f, n_vec, n);
    else if (tier == 1) hipLaunchKernelGGL((stream_kernel<F, kBlock, 1>), grid, dim3(kBlock), 0, s, f, n_vec, n);
    else hipLaunchKernelGGL((stream_kernel<F, 64, 1>), grid, dim3(64), 0, s, f, n_vec, n);
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

// A unary map from TI to TO; Fn is a stateless-or-small functor applied per element in fp32.
template <typename TI, typename TO, int VEC_, class Fn>
struct UnaryMap {
    static constexpr int VEC = VEC_;
    const TI* __restrict__ in;
    TO* __restrict__ out;
    Fn fn;
    template <int U>
    __device__ __forceinline__ void vecs(int64_t v0, int64_t step) const {
        Pack<TI, VEC> x[U];
#pragma unroll
        for (int u = 0; u < U; u++) x[u].load(in, v0 + u * step);
#pragma unroll
        for (int u = 0; u < U; u++) {
            Pack<TO, VEC> y;
#pragma unroll
            for (int k = 0; k < VEC; k++) y.set(k, fn(x[u].get(k)));
            y.store(out, v0 + u * step);
        }
    }
    __device__ __forceinline__ void one(int64_t i) const {
        out[i] = fn(in[i]);
    }
};

template <typename T, int VEC_, class Fn>
struct BinaryMap {
    static constexpr int VEC = VEC_;
    const T* __restrict__ a;
    const T* __restrict__ b;
    T* __restrict__ out;
    Fn fn;
    template <int U>
    __device__ __forceinline__ void vecs(int64_t v0, int64_t step) const {
        Pack<T, VEC> x[U], y[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            x[u].load(a, v0 + u * step);
            y[u].load(b, v0 + u * step);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            Pack<T, VEC> r;
#pragma unroll
            for (int k = 0; k < VEC; k++) r.set(k, fn(x[u].get(k), y[u].get(k)));
            r.store(out, v0 + u * step);
        }
    }
    __device__ __forceinline__ void one(int64_t i) const {
        out[i] = fn(a[i], b[i]);
    }
};

// ---------------------------------------------------------------- element functors
struct CvtF16F32 {
    __device__ __forceinline__ float operator()(half_t h) const { return (float)h; }
};
struct CvtF32F16 {
    __device__ __forceinline__ half_t operator()(float f) const { return f32_to_f16(f); }
};
template <typename T>
struct Copy {
    __device__ __forceinline__ T operator()(T v) const { return v; }
};

// float16 arithmetic = fp32 operation, then one rounding (include/vpux/utils/core/type/float16.hpp:123-150)
template <typename T, int OP>
struct EltFn {
    __device__ __forceinline__ T operator()(T x, T y) const {
        const float a = (float)x, b = (float)y;
        float r;
        if (OP == ELT_ADD) r = a + b;
        else if (OP == ELT_SUB) r = a - b;
        else if (OP == ELT_MUL) r = a * b;
        else if (OP == ELT_MIN) r = fminf(a, b);
        else if (OP == ELT_MAX) r = fmaxf(a, b);
        else r = a / b;
        return narrow<T>(r);
    }
};

struct FqFn {
    const half_t* ilo;
    const half_t* ihi;
    const half_t* olo;
    const half_t* ohi;
    float lm1;
    __device__ __forceinline__ half_t operator()(half_t x) const {
        return f32_to_f16(fq_f32((float)x, (float)*ilo, (float)*ihi, (float)*olo, (float)*ohi, lm1));
    }
};

// createQuantizeFn, src/vpux_compiler/src/dialect/const/attributes/quantize.cpp:91-106
template <typename TI, typename TQ>
struct QuantFn {
    float in_min, in_max, qmin, qmax, lm1;
    __device__ __forceinline__ TQ operator()(TI x) const {
        return (TQ)(int)fq_f32((float)x, in_min, in_max, qmin, qmax, lm1);
    }
};

// vpux::dequantize, include/vpux/compiler/utils/quantization.hpp:208-210: double product -> float
// PLAIN: every nonzero result is at least 2^-14 in magnitude and finite, where the reference's
// float16 rounding is plain round-to-nearest-even, one conversion instruction.
template <typename TQ, typename TO, bool PLAIN>
struct DequantFn {
    double scale;
    int zp;
    __device__ __forceinline__ TO operator()(TQ q) const {
        const float r = (float)((double)((int)q - zp) * scale);
        if (PLAIN) return (TO)r;
        return narrow<TO>(r);
    }
};

// ---------------------------------------------------------------- strided / broadcast path
template <int NOPS>
__device__ __forceinline__ void nd_offsets(const NdIndex& ix, int64_t lin, int64_t off[NOPS]) {
#pragma unroll
    for (int o = 0; o < NOPS; o++) off[o] = 0;
    for (int d = 0; d < ix.nd; d++) {
        const int64_t q = lin / ix.dims[d];
        const int64_t r = lin - q * ix.dims[d];
        lin = q;
#pragma unroll
        for (int o = 0; o < NOPS; o++) off[o] += r * ix.stride[o][d];
    }
}

template <typename TI, typename TO, class Fn>
__global__ __launch_bounds__(kBlock) void nd_unary_kernel(const TI* in, TO* out, Fn fn, NdIndex ix, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    int64_t off[2];
    nd_offsets<2>(ix, i, off);
    out[off[1]] = fn(in[off[0]]);
}

template <typename T, class Fn>
__global__ __launch_bounds__(kBlock) void nd_binary_kernel(const T* a, const T* b, T* out, Fn fn, NdIndex ix,
                                                           int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    int64_t off[3];
    nd_offsets<3>(ix, i, off);
    out[off[2]] = fn(a[off[0]], b[off[1]]);
}

// fake_quantize with limits that broadcast along some dimensions (per-channel and the like)
__global__ __launch_bounds__(kBlock) void nd_fq_kernel(const half_t* in, half_t* out, const half_t* ilo,
                                                       const half_t* ihi, const half_t* olo, const half_t* ohi,
                                                       NdIndex io, NdIndex lim, float lm1, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    int64_t off[2], lo[4];
    nd_offsets<2>(io, i, off);
    nd_offsets<4>(lim, i, lo);
    out[off[1]] = f32_to_f16(fq_f32((float)in[off[0]], (float)ilo[lo[0]], (float)ihi[lo[1]], (float)olo[lo[2]],
                                    (float)ohi[lo[3]], lm1));
}

int grid_1d(int64_t n, unsigned* blocks) {
    const int64_t b = (n + kBlock - 1) / kBlock;
    VPX_REQUIRE(b < (1ll << 31), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "tensor of %lld elements is too large",
                (long long)n);
    *blocks = (unsigned)(b < 1 ? 1 : b);
    return VPX_RESULT_SUCCESS;
}

// Fill operand `slot` of an NdIndex from a memref that must broadcast onto `out`.
int fill_index(NdIndex& ix, int slot, const MemRef& m, const MemRef& out, const char* what) {
    VPX_REQUIRE(out.nd <= kMaxDims, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                "%s: rank %d exceeds the %d dimensions the strided path handles", what, out.nd, kMaxDims);
    VPX_REQUIRE(m.nd == out.nd || m.numel() == 1, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                "%s: rank %d does not match the output rank %d", what, m.nd, out.nd);
    ix.nd = out.nd;
    for (int d = 0; d < out.nd; d++) {
        ix.dims[d] = (int32_t)out.dims[d];
        if (m.numel() == 1) {
            ix.stride[slot][d] = 0;
            continue;
        }
        VPX_REQUIRE(m.dims[d] == out.dims[d] || m.dims[d] == 1, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                    "%s: dimension %d of size %lld cannot broadcast to %lld", what, d, (long long)m.dims[d],
                    (long long)out.dims[d]);
        ix.stride[slot][d] = m.dims[d] == 1 ? 0 : m.strides[d];
    }
    return VPX_RESULT_SUCCESS;
}

bool same_shape(const MemRef& a, const MemRef& b) {
    if (a.nd != b.nd) return false;
    for (int d = 0; d < a.nd; d++)
        if (a.dims[d] != b.dims[d]) return false;
    return true;
}

bool aligned16(const void* p) {
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

}  // namespace

// ---------------------------------------------------------------- convert
template <typename TI, typename TO, class Fn>
static int convert_impl(const MemRef& in, const MemRef& out, Fn fn, hipStream_t s) {
    const int64_t n = out.numel();
    if (in.compact && out.compact && aligned16(in.data) && aligned16(out.data)) {
        constexpr int VEC = 16 / (sizeof(TI) > sizeof(TO) ? sizeof(TI) : sizeof(TO));
        UnaryMap<TI, TO, VEC, Fn> f{(const TI*)in.data, (TO*)out.data, fn};
        return launch_stream(f, n, s);
    }
    NdIndex ix{};
    int rc = fill_index(ix, 0, in, out, "convert input");
    if (rc) return rc;
    rc = fill_index(ix, 1, out, out, "convert output");
    if (rc) return rc;
    unsigned blocks;
    rc = grid_1d(n, &blocks);
    if (rc) return rc;
    if (n == 0) return VPX_RESULT_SUCCESS;
    hipLaunchKernelGGL((nd_unary_kernel<TI, TO, Fn>), dim3(blocks), dim3(kBlock), 0, s, (const TI*)in.data,
                       (TO*)out.data, fn, ix, n);
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

int launch_convert(const MemRef& in, const MemRef& out, hipStream_t s) {
    VPX_REQUIRE(same_shape(in, out), VPX_RESULT_ERROR_INVALID_ARGUMENT, "convert: input and output shapes differ");
    if (in.dtype == VPX_NN_FP16 && out.dtype == VPX_NN_FP32) return convert_impl<half_t, float>(in, out, CvtF16F32{}, s);
    if (in.dtype == VPX_NN_FP32 && out.dtype == VPX_NN_FP16) return convert_impl<float, half_t>(in, out, CvtF32F16{}, s);
    if (in.dtype == out.dtype && in.elem_bits == 16) return convert_impl<uint16_t, uint16_t>(in, out, Copy<uint16_t>{}, s);
    if (in.dtype == out.dtype && in.elem_bits == 32) return convert_impl<uint32_t, uint32_t>(in, out, Copy<uint32_t>{}, s);
    if (in.dtype == out.dtype && in.elem_bits == 8) return convert_impl<uint8_t, uint8_t>(in, out, Copy<uint8_t>{}, s);
    return fail(VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "convert: %s -> %s is not implemented", dtype_name(in.dtype),
                dtype_name(out.dtype));
}

// ---------------------------------------------------------------- eltwise
template <typename T, int OP>
static int eltwise_impl(const MemRef& a, const MemRef& b, const MemRef& out, hipStream_t s) {
    const int64_t n = out.numel();
    typedef EltFn<T, OP> Fn;
    if (a.compact && b.compact && out.compact && same_shape(a, out) && same_shape(b, out) && aligned16(a.data) &&
        aligned16(b.data) && aligned16(out.data)) {
        BinaryMap<T, 16 / sizeof(T), Fn> f{(const T*)a.data, (const T*)b.data, (T*)out.data, Fn{}};
        return launch_stream(f, n, s);
    }
    NdIndex ix{};
    int rc = fill_index(ix, 0, a, out, "eltwise input 1");
    if (rc) return rc;
    rc = fill_index(ix, 1, b, out, "eltwise input 2");
    if (rc) return rc;
    rc = fill_index(ix, 2, out, out, "eltwise output");
    if (rc) return rc;
    unsigned blocks;
    rc = grid_1d(n, &blocks);
    if (rc) return rc;
    if (n == 0) return VPX_RESULT_SUCCESS;
    hipLaunchKernelGGL((nd_binary_kernel<T, Fn>), dim3(blocks), dim3(kBlock), 0, s, (const T*)a.data, (const T*)b.data,
                       (T*)out.data, Fn{}, ix, n);
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

template <typename T>
static int eltwise_dispatch(int op, const MemRef& a, const MemRef& b, const MemRef& out, hipStream_t s) {
    switch (op) {
    case ELT_ADD: return eltwise_impl<T, ELT_ADD>(a, b, out, s);
    case ELT_SUB: return eltwise_impl<T, ELT_SUB>(a, b, out, s);
    case ELT_MUL: return eltwise_impl<T, ELT_MUL>(a, b, out, s);
    case ELT_MIN: return eltwise_impl<T, ELT_MIN>(a, b, out, s);
    case ELT_MAX: return eltwise_impl<T, ELT_MAX>(a, b, out, s);
    case ELT_DIV: return eltwise_impl<T, ELT_DIV>(a, b, out, s);
    default: return fail(VPX_RESULT_ERROR_INVALID_ARGUMENT, "eltwise: unknown operation %d", op);
    }
}

int launch_eltwise(int op, const MemRef& a, const MemRef& b, const MemRef& out, hipStream_t s) {
    VPX_REQUIRE(a.dtype == b.dtype && a.dtype == out.dtype, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                "eltwise: operand types differ (%s, %s -> %s)", dtype_name(a.dtype), dtype_name(b.dtype),
                dtype_name(out.dtype));
    if (out.dtype == VPX_NN_FP16) return eltwise_dispatch<half_t>(op, a, b, out, s);
    if (out.dtype == VPX_NN_FP32) return eltwise_dispatch<float>(op, a, b, out, s);
    return fail(VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "eltwise: element type %s is not implemented",
                dtype_name(out.dtype));
}

// ---------------------------------------------------------------- fake_quantize
int launch_fake_quantize(const MemRef& in, const MemRef lims[4], const MemRef& out, int64_t levels, hipStream_t s) {
    // Only FP16 in/out, like the reference kernel (sw_kernel.cpp:1156-1157).
    VPX_REQUIRE(in.dtype == VPX_NN_FP16 && out.dtype == VPX_NN_FP16, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                "fake_quantize: only FP16 input/output is supported, got %s -> %s", dtype_name(in.dtype),
                dtype_name(out.dtype));
    for (int k = 0; k < 4; k++)
        VPX_REQUIRE(lims[k].dtype == VPX_NN_FP16, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                    "fake_quantize: limit %d must be FP16, got %s", k, dtype_name(lims[k].dtype));
    VPX_REQUIRE(levels >= 2, VPX_RESULT_ERROR_INVALID_ARGUMENT, "fake_quantize: levels must be at least 2, got %lld",
                (long long)levels);
    VPX_REQUIRE(same_shape(in, out), VPX_RESULT_ERROR_INVALID_ARGUMENT, "fake_quantize: input and output shapes differ");
    const int64_t n = out.numel();
    const float lm1 = (float)levels - 1.0f;
    const bool per_tensor =
            lims[0].numel() == 1 && lims[1].numel() == 1 && lims[2].numel() == 1 && lims[3].numel() == 1;
    if (per_tensor && in.compact && out.compact && aligned16(in.data) && aligned16(out.data)) {
        FqFn fn{(const half_t*)lims[0].data, (const half_t*)lims[1].data, (const half_t*)lims[2].data,
                (const half_t*)lims[3].data, lm1};
        UnaryMap<half_t, half_t, 8, FqFn> f{(const half_t*)in.data, (half_t*)out.data, fn};
        return launch_stream(f, n, s);
    }
    NdIndex io{}, lim{};
    int rc = fill_index(io, 0, in, out, "fake_quantize input");
    if (rc) return rc;
    rc = fill_index(io, 1, out, out, "fake_quantize output");
    if (rc) return rc;
    for (int k = 0; k < 4; k++) {
        rc = fill_index(lim, k, lims[k], out, "fake_quantize limit");
        if (rc) return rc;
    }
    unsigned blocks;
    rc = grid_1d(n, &blocks);
    if (rc) return rc;
    if (n == 0) return VPX_RESULT_SUCCESS;
    hipLaunchKernelGGL(nd_fq_kernel, dim3(blocks), dim3(kBlock), 0, s, (const half_t*)in.data, (half_t*)out.data,
                       (const half_t*)lims[0].data, (const half_t*)lims[1].data, (const half_t*)lims[2].data,
                       (const half_t*)lims[3].data, io, lim, lm1, n);
    VPX_HIP_CHECK(hipGetLastError());
    return VPX_RESULT_SUCCESS;
}

// ---------------------------------------------------------------- quantize / dequantize
template <typename TI, typename TQ>
static int quantize_impl(const MemRef& in, const MemRef& out, double scale, int64_t zp, int64_t qmin, int64_t qmax,
                         hipStream_t s) {
    // Limits of the FakeQuantize the reference quantizer is built from (quantize.cpp:91-96).
    QuantFn<TI, TQ> fn;
    fn.in_min = (float)((double)(qmin - zp) * scale);
    fn.in_max = (float)((double)(qmax - zp) * scale);
    fn.qmin = (float)qmin;
    fn.qmax = (float)qmax;
    fn.lm1 = (float)(qmax - qmin + 1) - 1.0f;
    return convert_impl<TI, TQ>(in, out, fn, s);
}

int launch_quantize(const MemRef& in, const MemRef& out, double scale, int64_t zp, hipStream_t s) {
    VPX_REQUIRE(same_shape(in, out), VPX_RESULT_ERROR_INVALID_ARGUMENT, "quantize: input and output shapes differ");
    VPX_REQUIRE(scale > 0.0, VPX_RESULT_ERROR_INVALID_ARGUMENT, "quantize: scale must be positive, got %g", scale);
    if (in.dtype == VPX_NN_FP16 && out.dtype == VPX_NN_U8) return quantize_impl<half_t, uint8_t>(in, out, scale, zp, 0, 255, s);
    if (in.dtype == VPX_NN_FP16 && out.dtype == VPX_NN_I8) return quantize_impl<half_t, int8_t>(in, out, scale, zp, -128, 127, s);
    if (in.dtype == VPX_NN_FP32 && out.dtype == VPX_NN_U8) return quantize_impl<float, uint8_t>(in, out, scale, zp, 0, 255, s);
    if (in.dtype == VPX_NN_FP32 && out.dtype == VPX_NN_I8) return quantize_impl<float, int8_t>(in, out, scale, zp, -128, 127, s);
    return fail(VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "quantize: %s -> %s is not implemented", dtype_name(in.dtype),
                dtype_name(out.dtype));
}

int launch_dequantize(const MemRef& in, const MemRef& out, double scale, int64_t zp, hipStream_t s) {
    VPX_REQUIRE(same_shape(in, out), VPX_RESULT_ERROR_INVALID_ARGUMENT, "dequantize: input and output shapes differ");
    const int z = (int)zp;
    const bool plain = __builtin_isfinite(scale) && __builtin_fabs(scale) >= 0x1p-14 && __builtin_fabs(scale) < 64.0;
    if (in.dtype == VPX_NN_U8 && out.dtype == VPX_NN_FP16)
        return plain ? convert_impl<uint8_t, half_t>(in, out, DequantFn<uint8_t, half_t, true>{scale, z}, s)
                     : convert_impl<uint8_t, half_t>(in, out, DequantFn<uint8_t, half_t, false>{scale, z}, s);
    if (in.dtype == VPX_NN_I8 && out.dtype == VPX_NN_FP16)
        return plain ? convert_impl<int8_t, half_t>(in, out, DequantFn<int8_t, half_t, true>{scale, z}, s)
                     : convert_impl<int8_t, half_t>(in, out, DequantFn<int8_t, half_t, false>{scale, z}, s);
    if (in.dtype == VPX_NN_U8 && out.dtype == VPX_NN_FP32)
        return convert_impl<uint8_t, float>(in, out, DequantFn<uint8_t, float, true>{scale, z}, s);
    if (in.dtype == VPX_NN_I8 && out.dtype == VPX_NN_FP32)
        return convert_impl<int8_t, float>(in, out, DequantFn<int8_t, float, true>{scale, z}, s);
    return fail(VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "dequantize: %s -> %s is not implemented", dtype_name(in.dtype),
                dtype_name(out.dtype));
}

}  // namespace vpx
