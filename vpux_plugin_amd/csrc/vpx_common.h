// Shared host/device helpers of the execution library.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "vpx_runtime.h"

namespace vpx {

// ---- error channel -------------------------------------------------------------------------
std::string& last_error();
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

#define VPX_HIP_CHECK(expr)                                                                              \
    do {                                                                                                 \
        hipError_t _e = (expr);                                                                          \
        if (_e != hipSuccess)                                                                            \
            return ::vpx::fail(_e == hipErrorOutOfMemory ? VPX_RESULT_ERROR_OUT_OF_MEMORY                \
                                                         : VPX_RESULT_ERROR_UNKNOWN,                     \
                               "%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, __LINE__); \
    } while (0)

#define VPX_REQUIRE(cond, code, ...)                   \
    do {                                               \
        if (!(cond)) return ::vpx::fail(code, __VA_ARGS__); \
    } while (0)

// ---- tensor views parsed from a params blob ---------------------------------------------------
constexpr int kMaxDims = 8;  // deepest rank the strided kernels accept

struct MemRef {
    void* data = nullptr;
    uint32_t dtype = VPX_NN_UNDEFINED;
    uint64_t order = 0;
    int nd = 0;
    int64_t dims[VPX_MAX_ND_DIMS] = {};     // innermost first
    int64_t strides[VPX_MAX_ND_DIMS] = {};  // in elements, innermost first
    int elem_bits = 0;
    bool compact = false;
    // A memref whose MemRefData says isStatic = 0 (a bounded dynamic shape): dims / strides above are the bounds the blob
    // holds; the live ones sit in device memory (int32 dims, int64 strides in bits, innermost first), where the producer
    // of the shape wrote them, and only a kernel can read them.
    const int32_t* live_dims = nullptr;
    const int64_t* live_strides = nullptr;

    int64_t numel() const {
        int64_t n = 1;
        for (int i = 0; i < nd; i++) n *= dims[i];
        return n;
    }
};

inline int dtype_bits(uint32_t t) {
    switch (t) {
    case VPX_NN_FP32:
    case VPX_NN_I32:
    case VPX_NN_U32: return 32;
    case VPX_NN_FP16:
    case VPX_NN_BF16:
    case VPX_NN_I16:
    case VPX_NN_U16: return 16;
    case VPX_NN_U8:
    case VPX_NN_I8: return 8;
    case VPX_NN_FP64:
    case VPX_NN_I64:
    case VPX_NN_U64: return 64;
    default: return 0;
    }
}

const char* dtype_name(uint32_t t);

// Device-side view for the generic strided kernels.
struct NdIndex {
    int nd;
    int32_t dims[kMaxDims];     // output dims, innermost first
    int64_t stride[4][kMaxDims];  // element strides of up to 4 operands (0 where broadcast)
};

// Library-owned scratch memory, one buffer per (device, stream): calls on one stream are ordered,
// so they can share it; calls on different streams get different buffers.
int get_workspace(hipStream_t stream, size_t bytes, void** out);
// A small area of zero-initialised counters per (device, stream handle) for kernels whose workgroups meet inside a
// launch; a kernel that uses it leaves every word zero again.
constexpr size_t kSyncBytes = 128 * 1024;
int get_sync_area(hipStream_t stream, void** out);
// Compute units of the current device (cached per device).
int device_compute_units(int* out);
// True while the calling thread is inside the entry point that may not allocate: get_workspace() then hands out the
// fixed scratch array (at most VPX_NOALLOC_SCRATCH_BYTES), and launchers must not call hipMalloc for caches of their own.
bool noalloc_call();
// Frees the per-axis quantization tables cached for (device, stream); the caller has drained the stream.
int release_axis_tables(int dev, hipStream_t stream);

// Register-only int8 MFMA loop over every compute unit (calibration of the MFMA roofline); *ops = operations enqueued.
int calib_mfma_i8(const void* operands, void* sink, int iters, int fragment_reads, int64_t* ops, hipStream_t s);
int calib_coissue(int valu_kind, int wide_mfma, int mode, int iters, void* sink, hipStream_t s);

// Dispatch override for tests and tuning (knob names are those of the VPX_* environment variables, read once).
int set_tuning(const char* knob, const char* value);
// VPX_MVN_FUSED: 0 = never take the one-launch MVN kernel, 1 = default, 2 = its workgroups do not wait for each other
// (every one recomputes the group's moments: the path a workgroup takes when the others are not resident)
int tuning_mvn_fused();
// VPX_CALIB_BLOCKS: workgroups of the MFMA calibration loop (0: one per compute unit); fewer leave compute units free
// for whatever another stream launches beside it
int tuning_calib_blocks();

// ---- kernel launchers (defined in the .hip files) ------------------------------------------
int launch_convert(const MemRef& in, const MemRef& out, hipStream_t s);
int launch_eltwise(int op, const MemRef& a, const MemRef& b, const MemRef& out, hipStream_t s);
int launch_fake_quantize(const MemRef& in, const MemRef lims[4], const MemRef& out, int64_t levels, hipStream_t s);
int launch_quantize(const MemRef& in, const MemRef& out, double scale, int64_t zp, hipStream_t s);
int launch_dequantize(const MemRef& in, const MemRef& out, double scale, int64_t zp, hipStream_t s);
// per-axis forms: n scales / zero points along the dimension of size n (see the definition for how it is chosen)
int launch_quantize_per_axis(const MemRef& in, const MemRef& out, const double* scales, const int64_t* zps, int64_t n,
                             hipStream_t s);
int launch_dequantize_per_axis(const MemRef& in, const MemRef& out, const double* scales, const int64_t* zps, int64_t n,
                               hipStream_t s);

struct SoftmaxPlan {
    int axis;  // index into dims (innermost first)
    int pad;
    int nd;
    int64_t dims[VPX_MAX_ND_DIMS];
    int64_t in_stride[VPX_MAX_ND_DIMS];
    int64_t out_stride[VPX_MAX_ND_DIMS];
};
int launch_softmax(const SoftmaxPlan& p, uint32_t dtype, const void* in, void* out, hipStream_t s);
// bounded dynamic shapes (SoftmaxModeDynamic): the live dims and strides are read on the device; `axis` counts from the
// innermost dimension of the memrefs as they are (no packing)
int launch_softmax_dynamic(const MemRef& in, const MemRef& out, int axis, int pad, hipStream_t s);

int launch_mvn(const MemRef& in, const MemRef& out, bool across_channels, bool normalize_variance, float eps,
               hipStream_t s);

// whole-tensor range -> one scale and zero point -> u8 values (ONNX DynamicQuantizeLinear arithmetic)
int launch_dynamic_quantize(const MemRef& in, const MemRef& out, const MemRef& scale, const MemRef& zp, hipStream_t s);

// y = (q - zp) * scale with tensor scale / zero point that broadcast onto the input; zp may be null
int launch_dynamic_dequantize(const MemRef& in, const MemRef& scale, const MemRef* zp, const MemRef& out, hipStream_t s);

// MVN-1 decomposition (mvn1_sum -> mvn1_mean_var -> mvn1_norm)
int launch_mvn_sum(const MemRef& in, const MemRef& out, bool across_channels, bool normalize_variance, hipStream_t s);
int launch_mvn_mean_var(const MemRef& sum, const MemRef& out, const int64_t orig_shape[4], bool across_channels,
                        bool normalize_variance, int64_t group_c, float eps, hipStream_t s);
int launch_mvn_norm(const MemRef& in, const MemRef& mean_var, const MemRef& out, bool across_channels, bool normalize_variance,
                    hipStream_t s);

// mem_axes: normalised dimensions counted from the innermost memory dimension; scale / bias may be null
int launch_mvn6(const MemRef& in, const MemRef* scale, const MemRef* bias, const MemRef& out, bool normalize_variance, int eps_mode,
                float eps, const int64_t* mem_axes, int n_axes, hipStream_t s);

enum EltOp { ELT_ADD = 0, ELT_SUB, ELT_MUL, ELT_MIN, ELT_MAX, ELT_DIV, ELT_PRELU };

// Unary activations; p0 / p1 are the kernel's float attributes in the order the compiler serialises them.
enum ActOp {
    ACT_RELU = 0,
    ACT_LEAKY_RELU,   // p0 = negative slope
    ACT_CLAMP,        // p0 = min, p1 = max
    ACT_NEGATIVE,
    ACT_ABS,
    ACT_HSWISH,
    ACT_HSIGMOID,
    ACT_HARDSIGMOID,  // p0 = alpha, p1 = beta
    ACT_SIGMOID,
    ACT_TANH,
    ACT_EXP,
    ACT_SQRT,
    ACT_LOG,
    ACT_FLOOR,
    ACT_CEIL,
    ACT_SIGN,
    ACT_ELU,          // p0 = alpha
    ACT_SELU,         // p0 = alpha, p1 = lambda
    ACT_SWISH,        // p0 = beta
    ACT_MISH,
    ACT_SOFTPLUS,
    ACT_GELU,
    ACT_ERF,
    ACT_COUNT
};
int launch_activation(int op, float p0, float p1, const MemRef& in, const MemRef& out, hipStream_t s);

}  // namespace vpx
