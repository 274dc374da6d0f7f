// C ABI of the execution library: blob parsing, validation, dispatch, error text, scratch memory.
#include <atomic>
#include <cmath>
#include <cstring>
#include <map>
#include <mutex>
#include <utility>
#include <vector>

#include "vpx_common.h"

namespace vpx {

int launch_nce(const vpx_nce_task_t& t, hipStream_t s, const char** kernel_name);

std::string& last_error() {
    static thread_local std::string text;
    return text;
}

int fail(int code, const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    last_error() = buf;
    return code;
}

const char* dtype_name(uint32_t t) {
    static const char* names[] = {"FP64", "FP32", "FP16", "FP8", "U64", "U32", "U16", "U8",  "I64",
                                  "I32",  "I16",  "I8",   "I4",  "I2",  "BIN", "BF16", "UNDEFINED", "U4"};
    return t < sizeof(names) / sizeof(names[0]) ? names[t] : "?";
}

// ---- scratch memory ---------------------------------------------------------------------------
// Two providers behind get_workspace():
//  * a grown-on-demand block per (device, stream handle), allocated with hipMalloc (vpx_workspace_reserve sizes it
//    ahead of time; vpx_workspace_release frees it).  Growing is refused while the stream is capturing.
//  * a fixed array in device memory for the entry point that may not allocate (vpx_sw_kernel_launch_noalloc).
namespace {
struct Scratch {
    void* ptr = nullptr;
    size_t size = 0;
    std::vector<void*> retired;  // outgrown blocks: work already queued may still use them, freed on release
    void* sync = nullptr;        // kSyncBytes of counters for kernels whose workgroups meet inside one launch
};
std::mutex g_ws_mutex;
std::map<std::pair<int, hipStream_t>, Scratch> g_ws;

// The fixed scratch array.  Its name is a host-side handle, not a device address: host code uses the per-device
// address that hipGetSymbolAddress returns (each device holds its own copy of the array).
// (the counters of the allocation-free entry point sit behind the bytes get_workspace() hands out; device arrays
// start as zeros)
static __device__ __align__(256) unsigned char scratch[VPX_NOALLOC_SCRATCH_BYTES + kSyncBytes];
constexpr int kMaxDevices = 64;
void* g_static_scratch[kMaxDevices] = {};  // guarded by g_ws_mutex
thread_local bool t_noalloc = false;

bool stream_is_capturing(hipStream_t stream) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &st) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return st != hipStreamCaptureStatusNone;
}

int grow_workspace(Scratch& sc, hipStream_t stream, size_t bytes) {
    if (sc.size >= bytes) return VPX_RESULT_SUCCESS;
    VPX_REQUIRE(!stream_is_capturing(stream), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                "the stream is capturing and its scratch block (%zu bytes) is smaller than the %zu bytes this launch needs: "
                "call vpx_workspace_reserve before the capture, or use vpx_sw_kernel_launch_noalloc",
                sc.size, bytes);
    size_t want = 64 * 1024;
    while (want < bytes) want *= 2;
    void* p = nullptr;
    VPX_HIP_CHECK(hipMalloc(&p, want));
    if (sc.ptr) sc.retired.push_back(sc.ptr);
    sc.ptr = p;
    sc.size = want;
    return VPX_RESULT_SUCCESS;
}

// Device address of the fixed scratch array on the current device (looked up once per device).
int static_scratch_address(void** out) {
    int dev = 0;
    VPX_HIP_CHECK(hipGetDevice(&dev));
    VPX_REQUIRE(dev >= 0 && dev < kMaxDevices, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "device ordinal %d is beyond the %d this library tracks",
                dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    if (!g_static_scratch[dev]) {
        void* p = nullptr;
        VPX_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        VPX_REQUIRE(p != nullptr, VPX_RESULT_ERROR_UNKNOWN, "hipGetSymbolAddress returned a null address for the scratch array");
        g_static_scratch[dev] = p;
    }
    *out = g_static_scratch[dev];
    return VPX_RESULT_SUCCESS;
}
}  // namespace

bool noalloc_call() {
    return t_noalloc;
}

int get_workspace(hipStream_t stream, size_t bytes, void** out) {
    if (t_noalloc) {
        VPX_REQUIRE(bytes <= (size_t)VPX_NOALLOC_SCRATCH_BYTES, VPX_RESULT_ERROR_OUT_OF_MEMORY,
                    "this launch needs %zu bytes of scratch memory; the allocation-free entry point holds %zu", bytes,
                    (size_t)VPX_NOALLOC_SCRATCH_BYTES);
        return static_scratch_address(out);
    }
    int dev = 0;
    VPX_HIP_CHECK(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    Scratch& sc = g_ws[std::make_pair(dev, stream)];
    const int rc = grow_workspace(sc, stream, bytes);
    if (rc) return rc;
    *out = sc.ptr;
    return VPX_RESULT_SUCCESS;
}

// Counters that start as zeros and that every kernel using them leaves as zeros (the last workgroup through resets
// them), so launches on one stream can share them without a clearing pass.  One area per (device, stream handle),
// allocated and cleared on first need; nothing else is ever written there.
int get_sync_area(hipStream_t stream, void** out) {
    if (t_noalloc) {
        void* base = nullptr;
        const int rc = static_scratch_address(&base);
        if (rc) return rc;
        *out = (char*)base + VPX_NOALLOC_SCRATCH_BYTES;
        return VPX_RESULT_SUCCESS;
    }
    int dev = 0;
    VPX_HIP_CHECK(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    Scratch& sc = g_ws[std::make_pair(dev, stream)];
    if (!sc.sync) {
        VPX_REQUIRE(!stream_is_capturing(stream), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                    "the stream is capturing and has no counter area yet: call vpx_workspace_reserve before the capture, "
                    "or use vpx_sw_kernel_launch_noalloc");
        void* p = nullptr;
        VPX_HIP_CHECK(hipMalloc(&p, kSyncBytes));
        const hipError_t e = hipMemsetAsync(p, 0, kSyncBytes, stream);
        if (e != hipSuccess) {
            (void)hipFree(p);
            VPX_HIP_CHECK(e);
        }
        sc.sync = p;
    }
    *out = sc.sync;
    return VPX_RESULT_SUCCESS;
}

int device_compute_units(int* out) {
    static std::atomic<int> cached[kMaxDevices];
    int dev = 0;
    VPX_HIP_CHECK(hipGetDevice(&dev));
    int v = dev >= 0 && dev < kMaxDevices ? cached[dev].load() : 0;
    if (v == 0) {
        VPX_HIP_CHECK(hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev));
        if (dev >= 0 && dev < kMaxDevices) cached[dev].store(v);
    }
    *out = v;
    return VPX_RESULT_SUCCESS;
}

int workspace_reserve(hipStream_t stream, size_t bytes) {
    void* sync = nullptr;
    const int rc = get_sync_area(stream, &sync);
    if (rc) return rc;
    int dev = 0;
    VPX_HIP_CHECK(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    return grow_workspace(g_ws[std::make_pair(dev, stream)], stream, bytes);
}

int workspace_release(hipStream_t stream) {
    VPX_REQUIRE(!stream_is_capturing(stream), VPX_RESULT_ERROR_INVALID_ARGUMENT, "the stream is capturing: its scratch memory cannot be released");
    // work already queued may still read or write the blocks
    VPX_HIP_CHECK(hipStreamSynchronize(stream));
    int dev = 0;
    VPX_HIP_CHECK(hipGetDevice(&dev));
    // Everything the stream holds is freed whatever an individual hipFree returns; the first failure is reported.
    hipError_t first = hipSuccess;
    const auto release = [&first](void* p) {
        if (!p) return;
        const hipError_t e = hipFree(p);
        if (e != hipSuccess && first == hipSuccess) first = e;
    };
    {
        std::lock_guard<std::mutex> lock(g_ws_mutex);
        const auto it = g_ws.find(std::make_pair(dev, stream));
        if (it != g_ws.end()) {
            Scratch sc = it->second;
            g_ws.erase(it);
            for (void* p : sc.retired) release(p);
            release(sc.ptr);
            release(sc.sync);
        }
    }
    const int rc = release_axis_tables(dev, stream);
    VPX_HIP_CHECK(first);
    return rc;
}

// ---- blob parsing -----------------------------------------------------------------------------
namespace {

constexpr int kMaxMemRefs = VPX_MAX_KERNEL_INPUTS + VPX_MAX_KERNEL_OUTPUTS;

// The operands of one launch, on the caller's stack: a launch allocates nothing on the heap.
struct Args {
    MemRef mem[kMaxMemRefs];
    int n_mem = 0;
    const uint8_t* attrs = nullptr;
    size_t attrs_size = 0;
};

bool is_compact(const MemRef& m) {
    int64_t expect = 1;
    for (int d = 0; d < m.nd; d++) {
        if (m.dims[d] != 1 && m.strides[d] != expect) return false;
        expect *= m.dims[d];
    }
    return true;
}

int parse_blob(const char* entry, int n_in, int n_out, const void* params, size_t params_size,
               const vpx_memref_addr_t* addrs, uint32_t num_addrs, bool dynamic_ok, Args& a) {
    const int n_mem = n_in + n_out;
    VPX_REQUIRE(n_mem <= kMaxMemRefs, VPX_RESULT_ERROR_INVALID_ARGUMENT, "%s: %d operands, at most %d are supported", entry, n_mem, kMaxMemRefs);
    VPX_REQUIRE((int)num_addrs == n_mem, VPX_RESULT_ERROR_INVALID_ARGUMENT, "%s: expects %d memref addresses (%d in, %d out), got %u",
                entry, n_mem, n_in, n_out, num_addrs);
    VPX_REQUIRE(params_size >= (size_t)n_mem * sizeof(vpx_memref_data_t), VPX_RESULT_ERROR_INVALID_ARGUMENT,
                "%s: params blob of %zu bytes cannot hold %d MemRefData records", entry, params_size, n_mem);
    const uint8_t* p = (const uint8_t*)params;
    a.n_mem = n_mem;
    size_t tail = 0;
    bool tail_needed = false;
    for (int i = 0; i < n_mem; i++) {
        vpx_memref_data_t md;
        memcpy(&md, p + (size_t)i * sizeof(md), sizeof(md));
        MemRef& m = a.mem[i];
        VPX_REQUIRE(md.numDims >= 1 && md.numDims <= VPX_MAX_ND_DIMS, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                    "%s: memref %d has %u dimensions (1..%d allowed)", entry, i, md.numDims, VPX_MAX_ND_DIMS);
        m.nd = (int)md.numDims;
        m.dtype = md.dataType;
        m.order = md.dimsOrder;
        m.elem_bits = dtype_bits(md.dataType);
        VPX_REQUIRE(m.elem_bits > 0, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "%s: memref %d has unsupported data type %s (%u)", entry, i,
                    dtype_name(md.dataType), md.dataType);
        VPX_REQUIRE((addrs[i].dims == nullptr) == (addrs[i].strides == nullptr), VPX_RESULT_ERROR_INVALID_ARGUMENT,
                    "%s: memref %d must give both dims and strides or neither", entry, i);
        if (md.isStatic == 0) {
            // bounded dynamic shape: the side pointers are device memory with the live values, the blob holds the bounds
            VPX_REQUIRE(dynamic_ok, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                        "%s: memref %d has a dynamic shape (isStatic = 0), which only softmax / softmaxFp32 take", entry, i);
            VPX_REQUIRE(addrs[i].dims != nullptr, VPX_RESULT_ERROR_INVALID_NULL_HANDLE,
                        "%s: memref %d has a dynamic shape: its dims and strides must point at the live values in device memory", entry, i);
            m.live_dims = addrs[i].dims;
            m.live_strides = addrs[i].strides;
        }
        m.data = addrs[i].data;
        tail += (size_t)m.nd * (sizeof(int32_t) + sizeof(int64_t));
        if (addrs[i].dims == nullptr || md.isStatic == 0) tail_needed = true;  // (a dynamic shape's bounds are in the blob)
    }
    size_t body = params_size - (size_t)n_mem * sizeof(vpx_memref_data_t);
    if (tail_needed) {
        VPX_REQUIRE(body >= tail, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                    "%s: params blob of %zu bytes has no room for the %zu bytes of dims/strides it must end with", entry,
                    params_size, tail);
        body -= tail;
    }
    a.attrs = p + (size_t)n_mem * sizeof(vpx_memref_data_t);
    a.attrs_size = body;

    // tail: input dims | input strides | output dims | output strides (kernel_params.cpp:56-71)
    const uint8_t* t = a.attrs + body;
    const uint8_t* in_dims = t;
    size_t in_nd = 0, out_nd = 0;
    for (int i = 0; i < n_in; i++) in_nd += a.mem[i].nd;
    for (int i = n_in; i < n_mem; i++) out_nd += a.mem[i].nd;
    const uint8_t* in_strides = in_dims + in_nd * 4;
    const uint8_t* out_dims = in_strides + in_nd * 8;
    const uint8_t* out_strides = out_dims + out_nd * 4;
    size_t di = 0, dout = 0;
    for (int i = 0; i < n_mem; i++) {
        MemRef& m = a.mem[i];
        const bool is_in = i < n_in;
        size_t& cursor = is_in ? di : dout;
        for (int d = 0; d < m.nd; d++) {
            int32_t dim;
            int64_t stride_bits;
            if (addrs[i].dims && m.live_dims == nullptr) {
                dim = addrs[i].dims[d];
                stride_bits = addrs[i].strides[d];
            } else {
                memcpy(&dim, (is_in ? in_dims : out_dims) + (cursor + d) * 4, 4);
                memcpy(&stride_bits, (is_in ? in_strides : out_strides) + (cursor + d) * 8, 8);
            }
            VPX_REQUIRE(dim >= 0, VPX_RESULT_ERROR_INVALID_ARGUMENT, "%s: memref %d dimension %d is negative (%d)", entry, i, d, dim);
            VPX_REQUIRE(stride_bits >= 0 && stride_bits % m.elem_bits == 0, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                        "%s: memref %d stride %lld bits is not a multiple of the %d-bit element", entry, i,
                        (long long)stride_bits, m.elem_bits);
            m.dims[d] = dim;
            m.strides[d] = stride_bits / m.elem_bits;
        }
        cursor += m.nd;
        m.compact = is_compact(m);
        VPX_REQUIRE(m.data != nullptr || m.numel() == 0, VPX_RESULT_ERROR_INVALID_NULL_HANDLE,
                    "%s: memref %d has a null data address", entry, i);
    }
    return VPX_RESULT_SUCCESS;
}

template <typename T>
bool read_attr(const Args& a, size_t offset, T* out) {
    if (offset + sizeof(T) > a.attrs_size) return false;
    memcpy(out, a.attrs + offset, sizeof(T));
    return true;
}

float half_bits_to_float(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
    float mag;
    if (e == 0) mag = std::ldexp((float)m, -24);
    else if (e == 31) mag = m ? NAN : INFINITY;
    else mag = std::ldexp((float)(m | 0x400u), (int)e - 25);
    return sign ? -mag : mag;
}

// quantize / dequantize attributes: int64 n, then n scales and n zero points, both as packed
// floating-point values of the non-quantized operand's type (sw_kernel.cpp:97-163).
int read_quant_params(const char* entry, const Args& a, uint32_t float_type, std::vector<double>& scales,
                      std::vector<int64_t>& zps) {
    int64_t n = 0;
    VPX_REQUIRE(read_attr(a, 0, &n), VPX_RESULT_ERROR_INVALID_ARGUMENT, "%s: params blob has no quantization parameters", entry);
    VPX_REQUIRE(n >= 1 && n <= (1 << 24), VPX_RESULT_ERROR_INVALID_ARGUMENT, "%s: quantization parameter count is %lld", entry,
                (long long)n);
    const int per_word = float_type == VPX_NN_FP16 ? 4 : 2;
    const size_t words = (size_t)((n + per_word - 1) / per_word);
    scales.resize((size_t)n);
    zps.resize((size_t)n);
    for (int64_t i = 0; i < n; i++) {
        uint64_t sw = 0, zw = 0;
        const size_t word = (size_t)(i / per_word), slot = (size_t)(i % per_word);
        VPX_REQUIRE(read_attr(a, 8 + word * 8, &sw) && read_attr(a, 8 + (words + word) * 8, &zw), VPX_RESULT_ERROR_INVALID_ARGUMENT,
                    "%s: params blob is too short for %lld scales and zero points", entry, (long long)n);
        float sf, zf;
        if (float_type == VPX_NN_FP16) {
            sf = half_bits_to_float((uint16_t)((sw >> (16 * slot)) & 0xffffu));
            zf = half_bits_to_float((uint16_t)((zw >> (16 * slot)) & 0xffffu));
        } else {
            const uint32_t sb = (uint32_t)(sw >> (32 * slot)), zb = (uint32_t)(zw >> (32 * slot));
            memcpy(&sf, &sb, 4);
            memcpy(&zf, &zb, 4);
        }
        scales[(size_t)i] = (double)sf;
        zps[(size_t)i] = (int64_t)std::llround(zf);
    }
    return VPX_RESULT_SUCCESS;
}

// Restatement of the compiler's softmax parameter packing for callers that pass the first form
// (axis counted from the innermost memory dimension, padSize): drop unit dimensions, fuse
// dimensions outer to the axis whose strides allow it (update_sw_kernel_params.cpp:73-101).
void plan_from_memrefs(const MemRef& in, const MemRef& out, int64_t axis, int64_t pad, SoftmaxPlan& p) {
    p.nd = 0;
    int new_axis = 0;
    for (int d = 0; d < in.nd; d++) {
        if (in.dims[d] == 1 && d != axis && in.nd > 1) continue;
        if (d == axis) new_axis = p.nd;
        p.dims[p.nd] = in.dims[d];
        p.in_stride[p.nd] = in.strides[d];
        p.out_stride[p.nd] = out.strides[d];
        p.nd++;
    }
    if (p.nd == 0) {
        p.dims[0] = in.dims[0];
        p.in_stride[0] = in.strides[0];
        p.out_stride[0] = out.strides[0];
        p.nd = 1;
        new_axis = 0;
    }
    for (int i = p.nd - 2; i > new_axis; i--) {
        if (p.in_stride[i + 1] == p.in_stride[i] * p.dims[i] && p.out_stride[i + 1] == p.out_stride[i] * p.dims[i]) {
            p.dims[i] *= p.dims[i + 1];
            for (int j = i + 1; j < p.nd - 1; j++) {
                p.dims[j] = p.dims[j + 1];
                p.in_stride[j] = p.in_stride[j + 1];
                p.out_stride[j] = p.out_stride[j + 1];
            }
            p.nd--;
        }
    }
    p.axis = new_axis;
    p.pad = (int)pad;
}

int run_softmax(const char* entry, const Args& a, hipStream_t s) {
    const MemRef& in = a.mem[0];
    const MemRef& out = a.mem[1];
    VPX_REQUIRE(in.dtype == out.dtype, VPX_RESULT_ERROR_INVALID_ARGUMENT, "%s: input %s and output %s types differ", entry,
                dtype_name(in.dtype), dtype_name(out.dtype));
    const uint32_t want = strcmp(entry, "softmaxFp32") == 0 ? VPX_NN_FP32 : VPX_NN_FP16;
    VPX_REQUIRE(in.dtype == want, VPX_RESULT_ERROR_INVALID_ARGUMENT, "%s: expects %s tensors, got %s", entry, dtype_name(want),
                dtype_name(in.dtype));
    VPX_REQUIRE(in.nd == out.nd, VPX_RESULT_ERROR_INVALID_ARGUMENT, "%s: input and output ranks differ", entry);
    for (int d = 0; d < in.nd; d++)
        VPX_REQUIRE(in.dims[d] == out.dims[d], VPX_RESULT_ERROR_INVALID_ARGUMENT, "%s: input and output shapes differ", entry);
    uint64_t w0 = 0, w1 = 0;
    VPX_REQUIRE(read_attr(a, 0, &w0) && read_attr(a, 8, &w1), VPX_RESULT_ERROR_INVALID_ARGUMENT,
                "%s: params blob has no axis / padSize attributes", entry);
    SoftmaxPlan p{};
    if ((w1 >> 32) == 0) {
        // first form: int64 axis, int64 padSize
        VPX_REQUIRE(in.live_dims == nullptr && out.live_dims == nullptr, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                    "%s: memrefs with isStatic = 0 need the dynamic-shape form of the parameters", entry);
        const int64_t axis = (int64_t)w0, pad = (int64_t)w1;
        VPX_REQUIRE(axis >= 0 && axis < in.nd, VPX_RESULT_ERROR_INVALID_ARGUMENT, "%s: axis %lld outside rank %d", entry,
                    (long long)axis, in.nd);
        VPX_REQUIRE(pad >= 0 && pad < in.dims[axis], VPX_RESULT_ERROR_INVALID_ARGUMENT, "%s: padSize %lld does not fit axis of %lld",
                    entry, (long long)pad, (long long)in.dims[axis]);
        plan_from_memrefs(in, out, axis, pad, p);
    } else {
        // packed form
        const int64_t axis = (int64_t)(w0 & 0xffffffffu), pad = (int64_t)(w0 >> 32);
        const int64_t mode = (int64_t)(w1 & 0xffffffffu), nd = (int64_t)(w1 >> 32);
        if (mode == VPX_SOFTMAX_DYNAMIC) {
            // [axis, padSize], [SoftmaxModeDynamic, rank] and nothing else (update_sw_kernel_params.cpp:48-55): the shape is
            // whatever the memrefs' dims and strides in device memory say when the kernel runs
            VPX_REQUIRE(in.live_dims != nullptr && out.live_dims != nullptr, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                        "%s: dynamic-shape parameters need memrefs with isStatic = 0 and their live dims / strides in device memory", entry);
            VPX_REQUIRE(nd == in.nd && axis >= 0 && axis < nd, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                        "%s: dynamic-shape parameters name axis %lld of %lld dimensions, the memrefs have %d", entry, (long long)axis,
                        (long long)nd, in.nd);
            VPX_REQUIRE(pad >= 0 && pad < (1ll << 31), VPX_RESULT_ERROR_INVALID_ARGUMENT, "%s: padSize %lld", entry, (long long)pad);
            return launch_softmax_dynamic(in, out, (int)axis, (int)pad, s);
        }
        VPX_REQUIRE(in.live_dims == nullptr && out.live_dims == nullptr, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                    "%s: memrefs with isStatic = 0 need the dynamic-shape form of the parameters", entry);
        VPX_REQUIRE(mode >= 1 && mode <= 3, VPX_RESULT_ERROR_INVALID_ARGUMENT, "%s: unknown mode %lld", entry, (long long)mode);
        VPX_REQUIRE(nd >= 1 && nd <= VPX_MAX_ND_DIMS && axis < nd, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                    "%s: packed parameters name axis %lld of %lld dimensions", entry, (long long)axis, (long long)nd);
        p.nd = (int)nd;
        p.axis = (int)axis;
        p.pad = (int)pad;
        int64_t count = 1;
        for (int d = 0; d < p.nd; d++) {
            uint64_t wd = 0, ws = 0;
            VPX_REQUIRE(read_attr(a, 16 + (size_t)d * 16, &wd) && read_attr(a, 24 + (size_t)d * 16, &ws),
                        VPX_RESULT_ERROR_INVALID_ARGUMENT, "%s: packed parameters end before dimension %d", entry, d);
            p.dims[d] = (int64_t)(wd & 0xffffffffu);
            p.in_stride[d] = (int64_t)(ws & 0xffffffffu);
            p.out_stride[d] = (int64_t)(ws >> 32);
            count *= p.dims[d];
        }
        VPX_REQUIRE(count == in.numel(), VPX_RESULT_ERROR_INVALID_ARGUMENT,
                    "%s: packed dimensions cover %lld elements but the tensor has %lld", entry, (long long)count,
                    (long long)in.numel());
        VPX_REQUIRE(pad >= 0 && pad < p.dims[p.axis], VPX_RESULT_ERROR_INVALID_ARGUMENT, "%s: padSize %lld does not fit axis of %lld",
                    entry, (long long)pad, (long long)p.dims[p.axis]);
    }
    return launch_softmax(p, in.dtype, in.data, out.data, s);
}

struct Entry {
    const char* name;
    int n_in, n_out;
    int kind;  // dispatch tag
    int op;
    int n_float_attrs = 0;  // K_ACT: 32-bit float attributes that follow the memrefs
};

enum { K_CONVERT, K_ELTWISE, K_FQ, K_QUANT, K_DEQUANT, K_MVN, K_SOFTMAX, K_ACT, K_MVN_SUM, K_MVN_MEAN_VAR, K_MVN_NORM, K_MVN6, K_DYN_DEQUANT, K_DYN_QUANT };

const Entry kEntries[] = {
        {"convert", 1, 1, K_CONVERT, 0},
        {"eltwise_add", 2, 1, K_ELTWISE, ELT_ADD},
        {"eltwise_sub", 2, 1, K_ELTWISE, ELT_SUB},
        {"eltwise_mul", 2, 1, K_ELTWISE, ELT_MUL},
        {"eltwise_min", 2, 1, K_ELTWISE, ELT_MIN},
        {"eltwise_max", 2, 1, K_ELTWISE, ELT_MAX},
        {"eltwise_div", 2, 1, K_ELTWISE, ELT_DIV},
        {"fake_quantize", 5, 1, K_FQ, 0},
        {"quantize", 1, 1, K_QUANT, 0},
        {"dequantize", 1, 1, K_DEQUANT, 0},
        {"mvn1", 1, 1, K_MVN, 0},
        {"mvn1_sum", 1, 1, K_MVN_SUM, 0},
        {"mvn1_mean_var", 1, 1, K_MVN_MEAN_VAR, 0},
        {"mvn1_norm", 2, 1, K_MVN_NORM, 0},
        {"dynamic_quantize", 1, 3, K_DYN_QUANT, 0},  // outputs: values, scale, zero point (sw_kernel.cpp:1177-1179)
        {"dynamic_dequantize", -1, 1, K_DYN_DEQUANT, 0},  // input, scale, optional zero point; list ends at an INT64_MAX word
        {"mvn6", -1, 1, K_MVN6, 0},  // input, optional scale, optional bias; the memref list ends at an INT64_MIN word
        {"softmax", 1, 1, K_SOFTMAX, 0},
        {"softmaxFp32", 1, 1, K_SOFTMAX, 0},
        // activations (sw_kernel.cpp:650-941, 1266-1285, 1689-1845); float attributes in serialisation order
        {"prelu_fp16", 2, 1, K_ELTWISE, ELT_PRELU},
        {"activation_relu", 1, 1, K_ACT, ACT_RELU, 0},
        {"leaky_relu_fp16", 1, 1, K_ACT, ACT_LEAKY_RELU, 1},
        {"activation_clamp", 1, 1, K_ACT, ACT_CLAMP, 2},
        {"activation_negative", 1, 1, K_ACT, ACT_NEGATIVE, 0},
        {"activation_abs", 1, 1, K_ACT, ACT_ABS, 0},
        {"activation_hswish", 1, 1, K_ACT, ACT_HSWISH, 0},
        {"activation_hsigmoid", 1, 1, K_ACT, ACT_HSIGMOID, 0},
        {"activation_hardsigmoid", 1, 1, K_ACT, ACT_HARDSIGMOID, 2},
        {"activation_sigmoid", 1, 1, K_ACT, ACT_SIGMOID, 0},
        {"activation_tanh", 1, 1, K_ACT, ACT_TANH, 0},
        {"activation_exp", 1, 1, K_ACT, ACT_EXP, 0},
        {"activation_sqrt", 1, 1, K_ACT, ACT_SQRT, 0},
        {"activation_log", 1, 1, K_ACT, ACT_LOG, 0},
        {"activation_floor", 1, 1, K_ACT, ACT_FLOOR, 0},
        {"activation_ceil", 1, 1, K_ACT, ACT_CEIL, 0},
        {"activation_sign", 1, 1, K_ACT, ACT_SIGN, 0},
        {"activation_elu", 1, 1, K_ACT, ACT_ELU, 1},
        {"activation_selu", 1, 1, K_ACT, ACT_SELU, 2},
        {"activation_swish", 1, 1, K_ACT, ACT_SWISH, 1},
        {"activation_mish", 1, 1, K_ACT, ACT_MISH, 0},
        {"activation_softplus", 1, 1, K_ACT, ACT_SOFTPLUS, 0},
        {"activation_gelu", 1, 1, K_ACT, ACT_GELU, 0},
        {"activation_erf", 1, 1, K_ACT, ACT_ERF, 0},
};
constexpr uint32_t kNumEntries = sizeof(kEntries) / sizeof(kEntries[0]);

const Entry* find_entry(const char* name) {
    // callers pass the same string again and again: the last pointer's entry is checked first (one comparison)
    thread_local const char* last_name = nullptr;
    thread_local const Entry* last_entry = nullptr;
    if (name == last_name && last_entry != nullptr && strcmp(last_entry->name, name) == 0) return last_entry;
    for (uint32_t i = 0; i < kNumEntries; i++)
        if (strcmp(kEntries[i].name, name) == 0) {
            last_name = name;
            last_entry = &kEntries[i];
            return last_entry;
        }
    return nullptr;
}

thread_local const char* g_last_nce_kernel = "";

}  // namespace
}  // namespace vpx

using namespace vpx;

extern "C" {

const char* vpx_get_last_error(void) {
    return last_error().c_str();
}

uint32_t vpx_get_version(void) {
    return (0u << 16) | 1u;
}

int vpx_sw_kernel_supported(const char* entry) {
    return entry && find_entry(entry) ? 1 : 0;
}

uint32_t vpx_sw_kernel_count(void) {
    return kNumEntries;
}

const char* vpx_sw_kernel_name(uint32_t i) {
    return i < kNumEntries ? kEntries[i].name : nullptr;
}

static int sw_kernel_launch(const char* entry, const void* params, size_t params_size, const vpx_memref_addr_t* addrs,
                            uint32_t num_addrs, void* stream) {
    VPX_REQUIRE(entry != nullptr, VPX_RESULT_ERROR_INVALID_NULL_HANDLE, "kernel entry name is null");
    VPX_REQUIRE(params != nullptr, VPX_RESULT_ERROR_INVALID_NULL_HANDLE, "%s: params blob is null", entry);
    VPX_REQUIRE(addrs != nullptr, VPX_RESULT_ERROR_INVALID_NULL_HANDLE, "%s: memref address table is null", entry);
    const Entry* e = find_entry(entry);
    VPX_REQUIRE(e != nullptr, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "software kernel '%s' is not implemented", entry);
    Args a;
    int n_in = e->n_in;
    if (n_in < 0) {
        // optional operands: count MemRefData records up to the marker word (INT64_MIN, sw_kernel.cpp:164-185) or
        // the delimiter (INT64_MAX, sw_runtime_kernels/kernels/inc/common_types.h:141-151)
        int n_mem = 0;
        int64_t head = 0;
        while ((size_t)(n_mem + 1) * sizeof(vpx_memref_data_t) <= params_size && n_mem <= 4) {
            memcpy(&head, (const uint8_t*)params + (size_t)n_mem * sizeof(vpx_memref_data_t), 8);
            if (head == INT64_MIN || head == INT64_MAX) break;
            n_mem++;
        }
        VPX_REQUIRE((head == INT64_MIN || head == INT64_MAX) && n_mem >= 2 && n_mem <= 4, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                    "%s: the memref list must hold 2..4 records and end at the marker word", entry);
        n_in = n_mem - e->n_out;
    }
    int rc = parse_blob(entry, n_in, e->n_out, params, params_size, addrs, num_addrs, e->kind == K_SOFTMAX, a);
    if (rc) return rc;
    hipStream_t s = (hipStream_t)stream;
    switch (e->kind) {
    case K_CONVERT: return launch_convert(a.mem[0], a.mem[1], s);
    case K_ELTWISE: return launch_eltwise(e->op, a.mem[0], a.mem[1], a.mem[2], s);
    case K_FQ: {
        int64_t levels = 0;
        VPX_REQUIRE(read_attr(a, 0, &levels), VPX_RESULT_ERROR_INVALID_ARGUMENT, "fake_quantize: params blob has no levels attribute");
        return launch_fake_quantize(a.mem[0], &a.mem[1], a.mem[5], levels, s);
    }
    case K_QUANT: {
        thread_local std::vector<double> scales;  // (their storage is kept from launch to launch)
        thread_local std::vector<int64_t> zps;
        rc = read_quant_params(entry, a, a.mem[0].dtype, scales, zps);
        if (rc) return rc;
        if (scales.size() == 1) return launch_quantize(a.mem[0], a.mem[1], scales[0], zps[0], s);
        return launch_quantize_per_axis(a.mem[0], a.mem[1], scales.data(), zps.data(), (int64_t)scales.size(), s);
    }
    case K_DEQUANT: {
        thread_local std::vector<double> scales;  // (their storage is kept from launch to launch)
        thread_local std::vector<int64_t> zps;
        rc = read_quant_params(entry, a, a.mem[1].dtype, scales, zps);
        if (rc) return rc;
        if (scales.size() == 1) return launch_dequantize(a.mem[0], a.mem[1], scales[0], zps[0], s);
        return launch_dequantize_per_axis(a.mem[0], a.mem[1], scales.data(), zps.data(), (int64_t)scales.size(), s);
    }
    case K_MVN: {
        int64_t across = 0, normvar = 0;
        float eps = 0.f;
        VPX_REQUIRE(read_attr(a, 0, &across) && read_attr(a, 8, &normvar) && read_attr(a, 16, &eps),
                    VPX_RESULT_ERROR_INVALID_ARGUMENT, "mvn1: params blob is too short for {acrossChannels, normalizeVariance, eps}");
        VPX_REQUIRE(eps >= 0.f, VPX_RESULT_ERROR_INVALID_ARGUMENT, "mvn1: eps must not be negative, got %g", (double)eps);
        return launch_mvn(a.mem[0], a.mem[1], across != 0, normvar != 0, eps, s);
    }
    case K_MVN_SUM:
    case K_MVN_NORM: {
        // {acrossChannels, normalizeVariance} (sw_kernel.cpp:964-968, 982-986)
        int64_t across = 0, normvar = 0;
        VPX_REQUIRE(read_attr(a, 0, &across) && read_attr(a, 8, &normvar), VPX_RESULT_ERROR_INVALID_ARGUMENT,
                    "%s: params blob is too short for {acrossChannels, normalizeVariance}", entry);
        if (e->kind == K_MVN_SUM) return launch_mvn_sum(a.mem[0], a.mem[1], across != 0, normvar != 0, s);
        return launch_mvn_norm(a.mem[0], a.mem[1], a.mem[2], across != 0, normvar != 0, s);
    }
    case K_MVN_MEAN_VAR: {
        // {origShape[4], acrossChannels, normalizeVariance, groupC, eps} (sw_kernel.cpp:969-981)
        int64_t shape[4] = {0, 0, 0, 0}, across = 0, normvar = 0, group_c = 0;
        float eps = 0.f;
        bool ok = true;
        for (int i = 0; i < 4; i++) ok = ok && read_attr(a, (size_t)i * 8, &shape[i]);
        ok = ok && read_attr(a, 32, &across) && read_attr(a, 40, &normvar) && read_attr(a, 48, &group_c) && read_attr(a, 56, &eps);
        VPX_REQUIRE(ok, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                    "mvn1_mean_var: params blob is too short for {origShape[4], acrossChannels, normalizeVariance, groupC, eps}");
        return launch_mvn_mean_var(a.mem[0], a.mem[1], shape, across != 0, normvar != 0, group_c, eps, s);
    }
    case K_DYN_QUANT: return launch_dynamic_quantize(a.mem[0], a.mem[1], a.mem[2], a.mem[3], s);
    case K_DYN_DEQUANT: {
        VPX_REQUIRE(a.n_mem == 3 || a.n_mem == 4, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                    "dynamic_dequantize: expects input, scale, an optional zero point and the output, got %d memrefs", a.n_mem);
        const bool has_zp = a.n_mem == 4;
        return launch_dynamic_dequantize(a.mem[0], a.mem[1], has_zp ? &a.mem[2] : nullptr, a.mem[has_zp ? 3 : 2], s);
    }
    case K_MVN6: {
        // {marker, io mask}, normalizeVariance, epsMode, eps, numAxes, memAxes[numAxes] (sw_kernel.cpp:987-1004)
        int64_t marker = 0, mask = 0, normvar = 0, eps_mode = 0, n_axes = 0;
        float eps = 0.f;
        VPX_REQUIRE(read_attr(a, 0, &marker) && read_attr(a, 8, &mask) && read_attr(a, 16, &normvar) && read_attr(a, 24, &eps_mode) &&
                            read_attr(a, 32, &eps) && read_attr(a, 36, &n_axes),
                    VPX_RESULT_ERROR_INVALID_ARGUMENT, "mvn6: params blob is too short for its attributes");
        VPX_REQUIRE((mask & 9) == 9 && (mask & ~15ll) == 0 && 2 + ((mask >> 1) & 1) + ((mask >> 2) & 1) == (int64_t)a.n_mem,
                    VPX_RESULT_ERROR_INVALID_ARGUMENT, "mvn6: operand mask 0x%llx does not describe %d memrefs",
                    (unsigned long long)mask, a.n_mem);
        VPX_REQUIRE(n_axes >= 1 && n_axes <= VPX_MAX_ND_DIMS, VPX_RESULT_ERROR_INVALID_ARGUMENT, "mvn6: %lld axes", (long long)n_axes);
        int64_t axes[VPX_MAX_ND_DIMS];
        for (int64_t i = 0; i < n_axes; i++)
            VPX_REQUIRE(read_attr(a, 44 + (size_t)i * 8, &axes[i]), VPX_RESULT_ERROR_INVALID_ARGUMENT,
                        "mvn6: params blob ends before axis %lld", (long long)i);
        int next = 1;
        const MemRef* scale = (mask & 2) ? &a.mem[next++] : nullptr;
        const MemRef* bias = (mask & 4) ? &a.mem[next++] : nullptr;
        return launch_mvn6(a.mem[0], scale, bias, a.mem[next], normvar != 0, (int)eps_mode, eps, axes, (int)n_axes, s);
    }
    case K_SOFTMAX: return run_softmax(entry, a, s);
    case K_ACT: {
        float p[2] = {0.f, 0.f};
        for (int i = 0; i < e->n_float_attrs; i++)
            VPX_REQUIRE(read_attr(a, (size_t)i * 4, &p[i]), VPX_RESULT_ERROR_INVALID_ARGUMENT,
                        "%s: params blob is too short for %d float attributes", entry, e->n_float_attrs);
        return launch_activation(e->op, p[0], p[1], a.mem[0], a.mem[1], s);
    }
    default: return fail(VPX_RESULT_ERROR_UNKNOWN, "%s: no dispatcher", entry);
    }
}

int vpx_sw_kernel_launch(const char* entry, const void* params, size_t params_size, const vpx_memref_addr_t* addrs,
                         uint32_t num_addrs, void* stream) {
    last_error().clear();
    return sw_kernel_launch(entry, params, size_t(params_size), addrs, num_addrs, stream);
}

int vpx_sw_kernel_launch_noalloc(const char* entry, const void* params, size_t params_size, const vpx_memref_addr_t* addrs,
                                 uint32_t num_addrs, void* stream) {
    last_error().clear();
    // set-up, once per device: the device address of the fixed scratch array
    void* fixed = nullptr;
    const int rc = static_scratch_address(&fixed);
    if (rc) return rc;
    struct Mode {
        Mode() { t_noalloc = true; }
        ~Mode() { t_noalloc = false; }
    } mode;  // get_workspace() hands out `fixed` instead of allocating while this call runs on this thread
    return sw_kernel_launch(entry, params, params_size, addrs, num_addrs, stream);
}

int vpx_nce_task(const vpx_nce_task_t* t, void* stream) {
    last_error().clear();
    VPX_REQUIRE(t != nullptr, VPX_RESULT_ERROR_INVALID_NULL_HANDLE, "NCE task descriptor is null");
    VPX_REQUIRE(t->task_type == VPX_NCE_CONV || t->task_type == VPX_NCE_ELTWISE, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                "NCE task type %d is not implemented (CONV and ELTWISE only)", t->task_type);
    const bool eltwise = t->task_type == VPX_NCE_ELTWISE;
    VPX_REQUIRE(t->input && t->weights && (eltwise || t->weight_table) && t->output, VPX_RESULT_ERROR_INVALID_NULL_HANDLE,
                "NCE task: input, weights%s and output must all be set", eltwise ? " (second input)" : ", weight_table");
    if (eltwise) {
        VPX_REQUIRE(t->eltwise_type == VPX_ELTWISE_ADD || t->eltwise_type == VPX_ELTWISE_SUBTRACT, VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                    "NCE eltwise type %d is not implemented (ADD and SUBTRACT only)", t->eltwise_type);
        VPX_REQUIRE(t->OC == t->IC, VPX_RESULT_ERROR_INVALID_ARGUMENT, "NCE eltwise: OC %lld differs from IC %lld",
                    (long long)t->OC, (long long)t->IC);
        // input multipliers are unsigned 16-bit registers, the output shift has 6 bits (quantization.cpp:466-473)
        VPX_REQUIRE(t->ppe.in1_quant_mult >= 0 && t->ppe.in1_quant_mult <= 65535 && t->ppe.in2_quant_mult >= 0 &&
                            t->ppe.in2_quant_mult <= 65535 && t->ppe.quant_shift >= 0 && t->ppe.quant_shift <= 63 &&
                            t->ppe.quant_mult >= -32768 && t->ppe.quant_mult <= 32767,
                    VPX_RESULT_ERROR_INVALID_ARGUMENT,
                    "NCE eltwise: multipliers %d, %d, %d / shift %d outside the register ranges", t->ppe.in1_quant_mult,
                    t->ppe.in2_quant_mult, t->ppe.quant_mult, t->ppe.quant_shift);
        VPX_REQUIRE(t->zp_in >= -128 && t->zp_in <= 255 && t->zp_w >= -128 && t->zp_w <= 255 && t->zp_out >= -(1 << 20) &&
                            t->zp_out <= (1 << 20),
                    VPX_RESULT_ERROR_INVALID_ARGUMENT, "NCE eltwise: zero point out of range");
    }
    VPX_REQUIRE(t->groups >= 0 && (t->groups <= 1 || !eltwise), VPX_RESULT_ERROR_INVALID_ARGUMENT,
                "NCE task: groups = %d (CONV tasks take 0, 1 or more; ELTWISE tasks 0 or 1)", t->groups);
    const auto is8 = [](int32_t ty) { return ty == VPX_NN_U8 || ty == VPX_NN_I8; };
    const bool f16_out = t->output_type == VPX_NN_FP16;
    VPX_REQUIRE(is8(t->input_type) && is8(t->weights_type) && (is8(t->output_type) || f16_out), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                "NCE task: U8/I8 input and weights with a U8/I8 or FP16 output are implemented (got %s, %s, %s)",
                dtype_name((uint32_t)t->input_type), dtype_name((uint32_t)t->weights_type), dtype_name((uint32_t)t->output_type));
    // a float output has no zero point (setupQuantInFloatOut programs none, runtime_dpu_parser_imports.cpp.inc:546-574)
    VPX_REQUIRE(!f16_out || t->zp_out == 0, VPX_RESULT_ERROR_INVALID_ARGUMENT, "NCE task: an FP16 output takes no zero point (got %d)",
                t->zp_out);
    VPX_REQUIRE(t->N >= 0 && t->H >= 0 && t->W >= 0 && t->IC > 0 && t->OC >= 0, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                "NCE task: invalid shape N=%lld H=%lld W=%lld IC=%lld OC=%lld", (long long)t->N, (long long)t->H,
                (long long)t->W, (long long)t->IC, (long long)t->OC);
    VPX_REQUIRE(t->kernel_size[0] >= 1 && t->kernel_size[1] >= 1 && t->kernel_strides[0] >= 1 && t->kernel_strides[1] >= 1,
                VPX_RESULT_ERROR_INVALID_ARGUMENT, "NCE task: kernel size and strides must be positive");
    for (int i = 0; i < 4; i++)
        VPX_REQUIRE(t->kernel_padding[i] >= 0, VPX_RESULT_ERROR_INVALID_ARGUMENT, "NCE task: negative padding");
    // (for an FP16 output clamp_high packs two fp16 bounds and clamp_low is not used)
    VPX_REQUIRE(f16_out || t->ppe.clamp_low <= t->ppe.clamp_high, VPX_RESULT_ERROR_INVALID_ARGUMENT,
                "NCE task: clamp_low %d exceeds clamp_high %d", t->ppe.clamp_low, t->ppe.clamp_high);
    // prelu multiplier is an unsigned 11-bit field, prelu shift 5 bits (runtime_dpu_parser_imports.cpp.inc:411-417)
    if (t->ppe.mode == VPX_PPE_LPRELU)
        VPX_REQUIRE(t->ppe.lrelu_mult >= 0 && t->ppe.lrelu_mult < 2048 && t->ppe.lrelu_shift >= 0 && t->ppe.lrelu_shift < 32,
                    VPX_RESULT_ERROR_INVALID_ARGUMENT, "NCE task: lrelu_mult %d / lrelu_shift %d outside the 11-bit / 5-bit fields",
                    t->ppe.lrelu_mult, t->ppe.lrelu_shift);
    const char* name = "";
    const int rc = launch_nce(*t, (hipStream_t)stream, &name);
    if (rc == VPX_RESULT_SUCCESS) g_last_nce_kernel = name;
    return rc;
}

int vpx_workspace_reserve(void* stream, size_t bytes) {
    last_error().clear();
    return workspace_reserve(static_cast<hipStream_t>(stream), bytes);
}

int vpx_workspace_release(void* stream) {
    last_error().clear();
    return workspace_release(static_cast<hipStream_t>(stream));
}

int vpx_set_tuning(const char* knob, const char* value) {
    last_error().clear();
    return set_tuning(knob, value);
}

int vpx_calib_mfma_i8(const void* operands, void* sink, int iters, int fragment_reads, int64_t* ops, void* stream) {
    last_error().clear();
    return calib_mfma_i8(operands, sink, iters, fragment_reads, ops, static_cast<hipStream_t>(stream));
}

int vpx_calib_coissue(int valu_kind, int wide_mfma, int mode, int iters, void* sink, void* stream) {
    last_error().clear();
    return calib_coissue(valu_kind, wide_mfma, mode, iters, sink, static_cast<hipStream_t>(stream));
}

const char* vpx_nce_last_kernel(void) {
    return g_last_nce_kernel;
}

}  // extern "C"
