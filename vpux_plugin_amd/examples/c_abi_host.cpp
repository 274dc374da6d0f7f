// A C++ host that drives the library through its C ABI alone: no Python, no PyTorch.
// It plays the part the reference's runtime plays for a compiled network: it owns the buffers,
// serialises the kernel parameters the way the compiler does, and enqueues
//   (1) a `softmax` ACT-SHAVE kernel (fp16, last axis), and
//   (2) an NCE matmul with the integer PPE followed by `dequantize`,
// checking both against straightforward host arithmetic, and
//   (3) times what a call costs the host: 10 000 launches each of an empty kernel through hipLaunchKernelGGL, of
//       `fake_quantize` ([1,64,56,56] fp16, per tensor) and of an NCE convolution ([32,56,56,64] -> 64, 3 x 3), on the
//       same buffers, in batches of 500 with the stream drained between batches (the clock runs while calls are
//       enqueued, not while the GPU catches up).
// Exit code 0 = all checks passed.
//
// Build (the library leaves the HIP runtime to the process, so the host links it):
//   hipcc -O2 -std=c++17 -I include vpux_plugin_amd/examples/c_abi_host.cpp -L vpux_plugin_amd -lvpx_amd
//         -Wl,-rpath,$PWD/vpux_plugin_amd -o c_abi_host
#include <hip/hip_runtime.h>

#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <random>
#include <vector>

#include "vpx_compiler_utils.h"
#include "vpx_runtime.h"
#include "vpx_sw_params.h"

#define HIP_OK(x)                                                                                   \
    do {                                                                                            \
        hipError_t e_ = (x);                                                                        \
        if (e_ != hipSuccess) {                                                                     \
            std::fprintf(stderr, "%s failed: %s\n", #x, hipGetErrorString(e_));                      \
            return 2;                                                                               \
        }                                                                                           \
    } while (0)
#define VPX_OK(x)                                                                                   \
    do {                                                                                            \
        int r_ = (x);                                                                               \
        if (r_ != VPX_RESULT_SUCCESS) {                                                             \
            std::fprintf(stderr, "%s failed (%d): %s\n", #x, r_, vpx_get_last_error());              \
            return 3;                                                                               \
        }                                                                                           \
    } while (0)

static std::vector<uint8_t> make_blob(const std::vector<vpx_tensor_desc_t>& in, const std::vector<vpx_tensor_desc_t>& out,
                                      const void* attrs, size_t attrs_size) {
    size_t size = 0;
    vpx_create_kernel_params(in.data(), (uint32_t)in.size(), out.data(), (uint32_t)out.size(), attrs, attrs_size, nullptr, &size);
    std::vector<uint8_t> blob(size);
    vpx_create_kernel_params(in.data(), (uint32_t)in.size(), out.data(), (uint32_t)out.size(), attrs, attrs_size, blob.data(), &size);
    return blob;
}

// an empty kernel with the argument block of a typical launch (seven pointers and three words)
struct EmptyArgs {
    const void* p[7];
    int64_t n[3];
};
__global__ void empty_kernel(EmptyArgs a, int64_t n_vec, int64_t n) {
    if (n < 0) *(int64_t*)a.p[0] = n_vec;  // (never: keeps the arguments alive)
}

// microseconds of host time per call of `call`, over `batches` batches of `per_batch` calls
template <class F>
static double host_us_per_call(F&& call, hipStream_t stream, int batches = 20, int per_batch = 500) {
    for (int i = 0; i < 50; i++) call();
    (void)hipStreamSynchronize(stream);
    double total = 0;
    for (int b = 0; b < batches; b++) {
        const auto t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < per_batch; i++) call();
        const auto t1 = std::chrono::steady_clock::now();
        (void)hipStreamSynchronize(stream);
        total += std::chrono::duration<double, std::micro>(t1 - t0).count();
    }
    return total / ((double)batches * per_batch);
}

int main() {
    std::mt19937 rng(7);
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    int failures = 0;

    // ---------------------------------------------------------------- softmax, fp16 [64][1000], last axis
    {
        const int rows = 64, len = 1000;
        std::normal_distribution<float> dist(0.f, 3.f);
        std::vector<uint16_t> x((size_t)rows * len), y(x.size());
        for (auto& v : x) v = vpx_float_to_half_bits(dist(rng));
        void *dx, *dy;
        HIP_OK(hipMalloc(&dx, x.size() * 2));
        HIP_OK(hipMalloc(&dy, y.size() * 2));
        HIP_OK(hipMemcpy(dx, x.data(), x.size() * 2, hipMemcpyHostToDevice));
        const int32_t dims[2] = {len, rows};               // innermost first
        const int64_t strides_bits[2] = {16, 16 * len};
        const int64_t dims64[2] = {len, rows}, strides_el[2] = {1, len};
        vpx_tensor_desc_t t{2, dims, strides_bits, VPX_NN_FP16, VPX_ORDER_NC, VPX_LOC_DDR};
        uint64_t words[2 + 2 * 16];
        uint32_t n_words = 0;
        VPX_OK(vpx_generate_softmax_attr(2, dims64, strides_el, strides_el, /*axis=*/0, /*pad=*/0, words, &n_words));
        const std::vector<uint8_t> blob = make_blob({t}, {t}, words, n_words * 8);
        const vpx_memref_addr_t addrs[2] = {{dx, nullptr, nullptr}, {dy, nullptr, nullptr}};
        VPX_OK(vpx_sw_kernel_launch("softmax", blob.data(), blob.size(), addrs, 2, stream));
        HIP_OK(hipStreamSynchronize(stream));
        HIP_OK(hipMemcpy(y.data(), dy, y.size() * 2, hipMemcpyDeviceToHost));
        double worst = 0;
        for (int r = 0; r < rows; r++) {
            double m = -1e30, s = 0;
            for (int i = 0; i < len; i++) m = std::fmax(m, (double)vpx_half_bits_to_float(x[(size_t)r * len + i]));
            for (int i = 0; i < len; i++) s += std::exp((double)vpx_half_bits_to_float(x[(size_t)r * len + i]) - m);
            for (int i = 0; i < len; i++) {
                const double want = std::exp((double)vpx_half_bits_to_float(x[(size_t)r * len + i]) - m) / s;
                const double got = vpx_half_bits_to_float(y[(size_t)r * len + i]);
                worst = std::fmax(worst, std::fabs(got - want) / std::fmax(want, 6.1e-5));
            }
        }
        std::printf("softmax [%d][%d]: worst relative error %.2e (fp16 result)\n", rows, len, worst);
        if (worst > 2e-3) failures++;
        HIP_OK(hipFree(dx));
        HIP_OK(hipFree(dy));
    }

    // ---------------------------------------------------------------- NCE matmul + PPE, then dequantize
    {
        const int M = 300, K = 256, N = 520;
        std::uniform_int_distribution<int> d8(-128, 127), dw(-127, 127), dm(1 << 14, (1 << 15) - 1), db(-1000, 1000);
        std::vector<int8_t> a((size_t)M * K), b((size_t)N * K), q((size_t)M * N);
        for (auto& v : a) v = (int8_t)d8(rng);
        for (auto& v : b) v = (int8_t)dw(rng);
        std::vector<int32_t> wt((size_t)N * 4), mult(N), shift(N), bias(N);
        for (int n = 0; n < N; n++) {
            mult[n] = dm(rng);
            shift[n] = 22 + n % 3;
            bias[n] = db(rng);
            wt[(size_t)n * 4 + 0] = 0;           // weights pointer: an NPU address, ignored
            wt[(size_t)n * 4 + 1] = 0xFFFFFF;    // sparsity pointer: dense
            wt[(size_t)n * 4 + 2] = vpx_wt_get_scale((uint8_t)shift[n], (int16_t)mult[n]);
            wt[(size_t)n * 4 + 3] = bias[n];
        }
        const int zp_a = 3;
        void *da, *db_, *dwt, *dq, *dy;
        HIP_OK(hipMalloc(&da, a.size()));
        HIP_OK(hipMalloc(&db_, b.size()));
        HIP_OK(hipMalloc(&dwt, wt.size() * 4));
        HIP_OK(hipMalloc(&dq, q.size()));
        HIP_OK(hipMalloc(&dy, q.size() * 2));
        HIP_OK(hipMemcpy(da, a.data(), a.size(), hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(db_, b.data(), b.size(), hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(dwt, wt.data(), wt.size() * 4, hipMemcpyHostToDevice));
        vpx_nce_task_t t{};
        t.task_type = VPX_NCE_CONV;
        t.input = da; t.weights = db_; t.weight_table = (const int32_t*)dwt; t.output = dq;
        t.input_type = t.weights_type = t.output_type = VPX_NN_I8;
        t.N = 1; t.H = M; t.W = 1; t.IC = K; t.OC = N;
        t.kernel_size[0] = t.kernel_size[1] = t.kernel_strides[0] = t.kernel_strides[1] = 1;
        t.zp_in = zp_a;
        t.ppe.mode = VPX_PPE_LPRELU;
        t.ppe.clamp_low = -128; t.ppe.clamp_high = 127;
        t.ppe.lrelu_mult = 1638; t.ppe.lrelu_shift = 14;   // LeakyReLU 0.1
        VPX_OK(vpx_nce_task(&t, stream));
        std::printf("NCE matmul dispatched to %s\n", vpx_nce_last_kernel());

        const int32_t dims[2] = {N, M};
        const int64_t sb8[2] = {8, 8 * N}, sb16[2] = {16, 16 * N};
        vpx_tensor_desc_t tq{2, dims, sb8, VPX_NN_I8, VPX_ORDER_NC, VPX_LOC_DDR}, ty{2, dims, sb16, VPX_NN_FP16, VPX_ORDER_NC, VPX_LOC_DDR};
        const double scale = 0.05;
        const int64_t zp = 0;
        uint64_t qwords[3];
        uint32_t nq = 0;
        VPX_OK(vpx_get_quant_params_attr(&scale, &zp, 1, VPX_NN_FP16, qwords, &nq));
        const std::vector<uint8_t> blob = make_blob({tq}, {ty}, qwords, nq * 8);
        const vpx_memref_addr_t addrs[2] = {{dq, nullptr, nullptr}, {dy, nullptr, nullptr}};
        VPX_OK(vpx_sw_kernel_launch("dequantize", blob.data(), blob.size(), addrs, 2, stream));
        HIP_OK(hipStreamSynchronize(stream));
        std::vector<uint16_t> y(q.size());
        HIP_OK(hipMemcpy(q.data(), dq, q.size(), hipMemcpyDeviceToHost));
        HIP_OK(hipMemcpy(y.data(), dy, y.size() * 2, hipMemcpyDeviceToHost));

        // integer pipeline on the host: bias, multiply, PReLU on negatives, one round-half-even shift, clamp
        long mismatches = 0;
        const float shipped_scale = vpx_half_bits_to_float(vpx_float_to_half_bits((float)scale));
        for (int m = 0; m < M; m++)
            for (int n = 0; n < N; n++) {
                int64_t acc = 0;
                for (int k = 0; k < K; k++) acc += (int64_t)(a[(size_t)m * K + k] - zp_a) * b[(size_t)n * K + k];
                int64_t tv = (acc + bias[n]) * mult[n];
                int s = shift[n];
                if (tv < 0) {
                    tv *= 1638;
                    s += 14;
                }
                const int64_t fl = tv >> s, rem = tv - (fl << s), half = (int64_t)1 << (s - 1);
                int64_t r = fl + ((rem > half || (rem == half && (fl & 1))) ? 1 : 0);
                r = r < -128 ? -128 : (r > 127 ? 127 : r);
                const size_t i = (size_t)m * N + n;
                if (q[i] != (int8_t)r) mismatches++;
                if (y[i] != vpx_float_to_half_bits((float)((double)q[i] * (double)shipped_scale))) mismatches++;
            }
        std::printf("matmul %dx%dx%d + PPE + dequantize: %ld mismatches (bit-exact expected)\n", M, K, N, mismatches);
        if (mismatches) failures++;
    }

    // ---------------------------------------------------------------- what a call costs the host
    {
        const EmptyArgs ea{};
        const double bare = host_us_per_call([&] { hipLaunchKernelGGL(empty_kernel, dim3(196), dim3(256), 0, stream, ea, (int64_t)1, (int64_t)1); }, stream);

        // FakeQuantize fp16 NCHW [1,64,56,56], per tensor, 256 levels
        const size_t n_fq = (size_t)64 * 56 * 56;
        void *fx, *fy, *frange;
        HIP_OK(hipMalloc(&fx, n_fq * 2));
        HIP_OK(hipMalloc(&fy, n_fq * 2));
        HIP_OK(hipMalloc(&frange, 4 * 2));
        HIP_OK(hipMemset(fx, 0, n_fq * 2));
        const uint16_t range[4] = {vpx_float_to_half_bits(-4.f), vpx_float_to_half_bits(4.f), vpx_float_to_half_bits(-4.f), vpx_float_to_half_bits(4.f)};
        HIP_OK(hipMemcpy(frange, range, sizeof(range), hipMemcpyHostToDevice));
        const int32_t xd[4] = {56, 56, 64, 1}, od[4] = {1, 1, 1, 1};
        const int64_t xs[4] = {16, 16 * 56, 16 * 56 * 56, 16 * 56 * 56 * 64}, os[4] = {16, 16, 16, 16};
        vpx_tensor_desc_t tx{4, xd, xs, VPX_NN_FP16, VPX_ORDER_NCHW, VPX_LOC_DDR}, t1{4, od, os, VPX_NN_FP16, VPX_ORDER_NCHW, VPX_LOC_DDR};
        const int64_t levels = 256;
        const std::vector<uint8_t> fq_blob = make_blob({tx, t1, t1, t1, t1}, {tx}, &levels, 8);
        const vpx_memref_addr_t fq_addrs[6] = {{fx, nullptr, nullptr},
                                               {(uint16_t*)frange + 0, nullptr, nullptr},
                                               {(uint16_t*)frange + 1, nullptr, nullptr},
                                               {(uint16_t*)frange + 2, nullptr, nullptr},
                                               {(uint16_t*)frange + 3, nullptr, nullptr},
                                               {fy, nullptr, nullptr}};
        VPX_OK(vpx_sw_kernel_launch("fake_quantize", fq_blob.data(), fq_blob.size(), fq_addrs, 6, stream));
        const double fq = host_us_per_call([&] { (void)vpx_sw_kernel_launch("fake_quantize", fq_blob.data(), fq_blob.size(), fq_addrs, 6, stream); }, stream);

        // NCE convolution u8 [32,56,56,64] -> 64 channels, 3 x 3, pad 1
        const size_t n_in = (size_t)32 * 56 * 56 * 64, n_w = (size_t)64 * 9 * 64;
        void *ci, *cw, *cwt, *co;
        HIP_OK(hipMalloc(&ci, n_in));
        HIP_OK(hipMalloc(&cw, n_w));
        HIP_OK(hipMalloc(&cwt, 64 * 16));
        HIP_OK(hipMalloc(&co, n_in));
        HIP_OK(hipMemset(ci, 0x80, n_in));
        HIP_OK(hipMemset(cw, 1, n_w));
        std::vector<int32_t> cwt_h(64 * 4);
        for (int n = 0; n < 64; n++) {
            cwt_h[n * 4 + 0] = 0;
            cwt_h[n * 4 + 1] = 0xFFFFFF;
            cwt_h[n * 4 + 2] = vpx_wt_get_scale(22, (int16_t)20000);
            cwt_h[n * 4 + 3] = 100;
        }
        HIP_OK(hipMemcpy(cwt, cwt_h.data(), cwt_h.size() * 4, hipMemcpyHostToDevice));
        vpx_nce_task_t c{};
        c.task_type = VPX_NCE_CONV;
        c.input = ci; c.weights = cw; c.weight_table = (const int32_t*)cwt; c.output = co;
        c.input_type = VPX_NN_U8; c.weights_type = VPX_NN_I8; c.output_type = VPX_NN_U8;
        c.N = 32; c.H = 56; c.W = 56; c.IC = 64; c.OC = 64;
        c.kernel_size[0] = c.kernel_size[1] = 3;
        c.kernel_strides[0] = c.kernel_strides[1] = 1;
        c.kernel_padding[0] = c.kernel_padding[1] = c.kernel_padding[2] = c.kernel_padding[3] = 1;
        c.zp_in = 128;
        c.ppe.mode = VPX_PPE_LRELU;
        c.ppe.clamp_low = 0; c.ppe.clamp_high = 255;
        c.ppe.lrelu_mult = 1; c.ppe.lrelu_shift = 0;
        VPX_OK(vpx_nce_task(&c, stream));
        const char* conv_kernel = vpx_nce_last_kernel();
        const double conv = host_us_per_call([&] { (void)vpx_nce_task(&c, stream); }, stream, 20, 100);
        std::printf("host time per call: empty kernel through hipLaunchKernelGGL %.2f us; vpx_sw_kernel_launch(fake_quantize) %.2f us "
                    "(+%.2f); vpx_nce_task(%s) %.2f us (+%.2f)\n", bare, fq, fq - bare, conv_kernel, conv, conv - bare);
    }
    std::printf(failures ? "FAILED\n" : "OK\n");
    return failures ? 1 : 0;
}
