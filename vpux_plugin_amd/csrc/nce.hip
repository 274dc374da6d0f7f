// NCE cluster task on CDNA4: the dispatcher from a vpx_nce_task_t to a device kernel, the tuning knobs, the operand
// views and the small kernels that prepare a weight zero point.  The kernels live in nce_gemm.hip, nce_gemm_regb.hip, nce_conv_patch.hip,
// nce_conv_rows.hip, nce_conv_gather.hip and nce_eltwise.hip; nce_common.h says what each serves.
#include <mutex>
#include <set>

#include "nce_common.h"

namespace vpx {

int launch_nce(const vpx_nce_task_t& t, hipStream_t s, const char** kernel_name);

namespace nce {

// Kernels that may ask for more than 64 KiB of dynamic LDS are given the largest size any launch of them uses,
// once per (device, kernel): the attribute is then never changed again, so concurrent launches that want
// different sizes cannot undo each other's setting.
namespace {
std::mutex g_lds_mutex;
std::set<std::pair<int, const void*>> g_lds_done;
}  // namespace

int set_dyn_lds_attribute(const void* fn) {
    int dev = 0;
    VPX_HIP_CHECK(hipGetDevice(&dev));
    // the kernel this thread launched last needs no lock and no search
    thread_local int last_dev = -1;
    thread_local const void* last_fn = nullptr;
    if (dev == last_dev && fn == last_fn) return VPX_RESULT_SUCCESS;
    std::lock_guard<std::mutex> lock(g_lds_mutex);
    if (!g_lds_done.count({dev, fn})) {
        VPX_HIP_CHECK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxDynLds));
        g_lds_done.insert({dev, fn});
    }
    last_dev = dev;
    last_fn = fn;
    return VPX_RESULT_SUCCESS;
}

int operand_view(const int64_t st[4], int64_t N, int64_t H, int64_t W, int64_t C, const char* what, View* v) {
    if ((st[0] | st[1] | st[2] | st[3]) == 0) {
        *v = View{H * W * C, W * C, C, true, 2, N * H * W * C};
        return VPX_RESULT_SUCCESS;
    }
    VPX_REQUIRE(st[3] == 1, VPX_RESULT_ERROR_INVALID_ARGUMENT, "NCE task: the %s's channel stride is %lld; channels must be contiguous (1)", what,
                (long long)st[3]);
    VPX_REQUIRE(st[0] >= 0 && st[1] >= 0 && st[2] >= 0, VPX_RESULT_ERROR_INVALID_ARGUMENT, "NCE task: the %s has a negative stride", what);
    const int64_t ext_w = (W - 1) * st[2] + C;
    VPX_REQUIRE(W <= 1 || st[2] >= C, VPX_RESULT_ERROR_INVALID_ARGUMENT, "NCE task: the %s's W stride %lld is below its %lld channels", what,
                (long long)st[2], (long long)C);
    VPX_REQUIRE(H <= 1 || st[1] >= ext_w, VPX_RESULT_ERROR_INVALID_ARGUMENT, "NCE task: the %s's H stride %lld is below the %lld elements a row spans",
                what, (long long)st[1], (long long)ext_w);
    const int64_t ext_h = (H - 1) * st[1] + ext_w;
    VPX_REQUIRE(N <= 1 || st[0] >= ext_h, VPX_RESULT_ERROR_INVALID_ARGUMENT, "NCE task: the %s's N stride %lld is below the %lld elements an image spans",
                what, (long long)st[0], (long long)ext_h);
    int64_t sn = st[0], sh = st[1], sw = st[2];
    if (W <= 1) sw = H > 1 ? sh : (N > 1 ? sn : C);
    if (H <= 1) sh = N > 1 && W <= 1 ? sn : W * sw;
    if (N <= 1) sn = H * sh;
    v->sn = sn;
    v->sh = sh;
    v->sw = sw;
    v->flat = sh == W * sw ? (sn == H * sh ? 2 : 1) : 0;
    v->dense = v->flat == 2 && sw == C;
    v->span = (N > 0 && H > 0 && W > 0) ? (N - 1) * sn + (H - 1) * sh + (W - 1) * sw + C : 0;
    return VPX_RESULT_SUCCESS;
}


namespace {

// Weights with a zero point zw.  The MFMA kernels multiply signed bytes W = w - cw (cw = 128 for unsigned storage,
// re-biased into a scratch copy, else 0), so sum (a - za)(w - zw) lacks (cw - zw) * sum (a - za) over the taps
// inside the image: one value per output position, the same for all its channels.  Two small kernels prepare
// it: the channel sum of every input pixel, then the sum of those under each window times (cw - zw); the
// convolution kernels add the result to their accumulators before the PPE.  A 1x1, stride-1, unpadded layer
// (a matmul) needs only the first, which then applies the factor itself.
__global__ __launch_bounds__(256) void nce_pixel_sum_kernel(const uint8_t* __restrict__ in, int32_t* __restrict__ cs, int64_t pixels,
                                                            int IC, int lpp, int flip, int offset, int factor, ConvGeom g, int in_flat) {
    // lpp lanes (a power of two, at most 64) share a pixel; each sums 16-byte chunks
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t pixel = t / lpp;
    const int sub = (int)(t % lpp);
    unsigned sum = 0;
    if (pixel < pixels) {
        // (pixels are counted over the dense N x H x W grid; a view of a larger tensor has them isw / ish / isn apart)
        int64_t at = pixel * g.isw;
        if (!in_flat) {
            const int64_t hw = g.H * g.W, n = pixel / hw, rem = pixel - n * hw, y = rem / g.W;
            at = in_pos(g, n, y, rem - y * g.W);
        }
        const i32x4* row = reinterpret_cast<const i32x4*>(in + at);
        for (int c = sub; c < IC / 16; c += lpp) {
            const i32x4 q = row[c];
#pragma unroll
            for (int k = 0; k < 4; k++) sum = __builtin_amdgcn_sad_u8((unsigned)(q[k] ^ flip), 0u, sum);  // four bytes at once
        }
    }
    for (int o = lpp >> 1; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
    if (pixel < pixels && sub == 0) cs[pixel] = ((int)sum - offset) * factor;
}

__global__ __launch_bounds__(256) void nce_window_sum_kernel(const int32_t* __restrict__ cs, int32_t* __restrict__ rowterm, ConvGeom g,
                                                             int factor, int64_t total) {
    const int64_t m = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (m >= total) return;
    const int64_t ox = m % g.OW, oy = (m / g.OW) % g.OH, n = m / (g.OW * g.OH);
    int sum = 0;
    for (int ky = 0; ky < g.KY; ky++) {
        const int64_t iy = oy * g.SY + ky - g.PT;
        if (iy < 0 || iy >= g.H) continue;
        for (int kx = 0; kx < g.KX; kx++) {
            const int64_t ix = ox * g.SX + kx - g.PL;
            if (ix >= 0 && ix < g.W) sum += cs[(n * g.H + iy) * g.W + ix];
        }
    }
    rowterm[m] = sum * factor;
}

// u8 weights whose zero point is 128 (symmetric weights kept in unsigned storage) are the signed weights
// w - 128: one pass flips the top bit of every byte into a scratch copy and the signed kernels run on that.
__global__ __launch_bounds__(256) void nce_weights_to_s8_kernel(const i32x4* __restrict__ in, i32x4* __restrict__ out, int64_t n_vec) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n_vec; i += (int64_t)gridDim.x * 256) out[i] = in[i] ^ (int32_t)0x80808080;
}


Tuning g_tuning;
std::once_flag g_tuning_once;

bool set_knob(const char* knob, const char* value) {
    const char* v = value ? value : "";
    if (!std::strcmp(knob, "VPX_NCE_KERNEL")) {
        g_tuning.nce_kernel = !std::strcmp(v, "naive") ? NCE_NAIVE : (!std::strcmp(v, "gather") ? NCE_GATHER : (!std::strcmp(v, "conv") ? NCE_CONV : NCE_AUTO));
    } else if (!std::strcmp(knob, "VPX_GEMM_TILE")) {
        g_tuning.gemm_tile = *v ? (std::atoi(v) == 128 ? 128 : 256) : 0;
    } else if (!std::strcmp(knob, "VPX_GEMM_WAVES")) {
        g_tuning.gemm_waves = *v ? (std::atoi(v) == 4 ? 4 : 8) : 0;
    } else if (!std::strcmp(knob, "VPX_GEMM_REGB")) {
        g_tuning.gemm_regb = !std::strcmp(v, "on") ? 1 : (!std::strcmp(v, "wide") ? 2 : (!std::strcmp(v, "off") ? -1 : 0));
    } else if (!std::strcmp(knob, "VPX_GEMM_PINGPONG")) {
        g_tuning.gemm_pingpong = !std::strcmp(v, "on") ? 1 : 0;
    } else if (!std::strcmp(knob, "VPX_CONV_KERNEL")) {
        g_tuning.conv_stream = !std::strcmp(v, "stream") ? 2 : (!std::strcmp(v, "tile") ? 1 : (!std::strcmp(v, "regw") ? -1 : 0));
    } else if (!std::strcmp(knob, "VPX_CONV_ROWS")) {
        g_tuning.conv_rows = std::atoi(v) > 0 ? std::atoi(v) : 0;
    } else if (!std::strcmp(knob, "VPX_CONV_COLS")) {
        g_tuning.conv_cols = std::atoi(v) > 0 ? std::atoi(v) : 0;
    } else if (!std::strcmp(knob, "VPX_CONV_WAVES")) {
        g_tuning.conv_waves = std::atoi(v) == 4 ? 4 : 0;
    } else if (!std::strcmp(knob, "VPX_STREAM_KSPLIT")) {
        g_tuning.stream_ksplit = (!std::strcmp(v, "off") || !std::strcmp(v, "0")) ? 0 : 1;
    } else if (!std::strcmp(knob, "VPX_MVN_FUSED")) {
        g_tuning.mvn_fused = !std::strcmp(v, "off") ? 0 : (!std::strcmp(v, "nowait") ? 2 : 1);
    } else if (!std::strcmp(knob, "VPX_CALIB_BLOCKS")) {
        g_tuning.calib_blocks = std::atoi(v) > 0 ? std::atoi(v) : 0;
    } else {
        return false;
    }
    return true;
}


}  // namespace

const Tuning& tuning() {
    std::call_once(g_tuning_once, [] {
        for (const char* k : {"VPX_NCE_KERNEL", "VPX_GEMM_TILE", "VPX_GEMM_WAVES", "VPX_GEMM_REGB", "VPX_GEMM_PINGPONG", "VPX_CONV_KERNEL", "VPX_CONV_ROWS", "VPX_CONV_COLS", "VPX_CONV_WAVES", "VPX_STREAM_KSPLIT", "VPX_MVN_FUSED", "VPX_CALIB_BLOCKS"})
            if (const char* v = std::getenv(k)) set_knob(k, v);
    });
    return g_tuning;
}


}  // namespace nce

using namespace nce;

int tuning_mvn_fused() {
    return tuning().mvn_fused.load();
}

int tuning_calib_blocks() {
    return tuning().calib_blocks.load();
}

int set_tuning(const char* knob, const char* value) {
    (void)tuning();  // the environment is consulted before the first explicit setting, never after it
    VPX_REQUIRE(knob != nullptr, VPX_RESULT_ERROR_INVALID_NULL_HANDLE, "tuning knob name is null");
    VPX_REQUIRE(set_knob(knob, value), VPX_RESULT_ERROR_INVALID_ARGUMENT, "unknown tuning knob '%s'", knob);
    return VPX_RESULT_SUCCESS;
}

int launch_nce(const vpx_nce_task_t& t, hipStream_t s, const char** kernel_name) {
    const bool in_u8 = t.input_type == VPX_NN_U8, w_u8 = t.weights_type == VPX_NN_U8,
               out_signed = t.output_type == VPX_NN_I8, out_f16 = t.output_type == VPX_NN_FP16;
    ConvGeom g{};
    g.N = t.N; g.H = t.H; g.W = t.W; g.IC = t.IC; g.OC = t.OC;
    g.KY = t.kernel_size[0]; g.KX = t.kernel_size[1];
    g.SY = t.kernel_strides[0]; g.SX = t.kernel_strides[1];
    g.PL = t.kernel_padding[0]; g.PT = t.kernel_padding[2];
    g.OH = (t.H + t.kernel_padding[2] + t.kernel_padding[3] - g.KY) / g.SY + 1;
    g.OW = (t.W + t.kernel_padding[0] + t.kernel_padding[1] - g.KX) / g.SX + 1;
    VPX_REQUIRE(g.OH > 0 && g.OW > 0, VPX_RESULT_ERROR_INVALID_ARGUMENT, "NCE task: kernel %dx%d does not fit the padded input",
                g.KY, g.KX);

    Ppe ppe;
    ppe.zp_out = t.zp_out;
    ppe.clamp_lo = t.ppe.clamp_low;
    ppe.clamp_hi = t.ppe.clamp_high;
    ppe.f16_lo = -INFINITY;
    ppe.f16_hi = INFINITY;
    if (out_f16 && t.ppe.clamp_high != INT32_MAX) {
        // two fp16 bounds in one word, 0xllllhhhh (dialect/VPU/utils/ppe_utils.hpp:36-87); clamp_low is not used
        const auto half = [](uint32_t h) {
            const uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
            const float mag = e == 0 ? std::ldexp((float)m, -24) : (e == 31 ? (m ? NAN : INFINITY) : std::ldexp((float)(m | 0x400u), (int)e - 25));
            return (h & 0x8000u) ? -mag : mag;
        };
        const float lo = half(((uint32_t)t.ppe.clamp_high >> 16) & 0xffffu), hi = half((uint32_t)t.ppe.clamp_high & 0xffffu);
        if (!std::isnan(lo)) ppe.f16_lo = lo;
        if (!std::isnan(hi)) ppe.f16_hi = hi;
    }
    switch (t.ppe.mode) {
    case VPX_PPE_NOOP: ppe.prelu_mult = 1; ppe.prelu_shift = 0; break;
    case VPX_PPE_LRELU:
    case VPX_PPE_LRELUX: ppe.prelu_mult = 0; ppe.prelu_shift = 0; break;
    case VPX_PPE_LPRELU: ppe.prelu_mult = t.ppe.lrelu_mult; ppe.prelu_shift = t.ppe.lrelu_shift; break;
    default: return fail(VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "NCE task: PPE mode %d is not an integer-pipeline mode", t.ppe.mode);
    }

    if (t.task_type == VPX_NCE_ELTWISE) return launch_nce_eltwise(t, ppe, s, kernel_name);

    // A slope of zero (ReLU) is a clamp: the negative branch ends at the zero point whatever the accumulator, and rounding
    // is monotone, so the result is that of a layer without a PReLU stage held at or above the zero point before the
    // clamp (max, then min) -- the same layer with the lower bound raised to the zero point.  Every kernel's epilogue then
    // runs its one-factor form: no sign test, no second product.  (Integer outputs only: an fp16 zero keeps its sign.)
    if (!out_f16 && ppe.prelu_mult == 0) {
        ppe.prelu_mult = 1;
        ppe.prelu_shift = 0;
        if (ppe.clamp_lo < t.zp_out) ppe.clamp_lo = t.zp_out;
    }

    const int64_t Mtot = g.N * g.OH * g.OW;
    const int64_t Ktot = (int64_t)g.KY * g.KX * g.IC;
    if (Mtot == 0 || g.OC == 0) return VPX_RESULT_SUCCESS;

    // Input and output as views (dense unless the task gives strides); the weights are always dense.
    View vin, vout;
    {
        int rc = operand_view(t.input_strides, g.N, g.H, g.W, g.IC, "input", &vin);
        if (!rc) rc = operand_view(t.output_strides, g.N, g.OH, g.OW, g.OC, "output", &vout);
        if (rc) return rc;
        VPX_REQUIRE(t.groups <= 1 || (vin.dense && vout.dense), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE,
                    "NCE task: a grouped task takes dense operands (strides were given with groups = %d)", t.groups);
    }
    g.isn = vin.sn; g.ish = vin.sh; g.isw = vin.sw;
    g.osn = vout.sn; g.osh = vout.sh; g.osw = vout.sw;
    g.out_flat = vout.flat;
    g.out_bits = (unsigned)(reinterpret_cast<uintptr_t>(t.output) | (uintptr_t)((vout.sn | vout.sh | vout.sw) * (out_f16 ? 2 : 1)));
    const bool in_flat = vin.flat == 2;

    const bool zp_in_ok = in_u8 ? (t.zp_in >= 0 && t.zp_in <= 255) : (t.zp_in >= -128 && t.zp_in <= 127);
    // the fast epilogue adds the output zero point after limiting the scaled value to +-2^30
    const bool zp_out_ok = t.zp_out >= -(1 << 20) && t.zp_out <= (1 << 20);
    // Unsigned weights are re-biased by 128 into a signed scratch copy; what is left of the weight zero point
    // (wz_rest = 128 - zp_w, or -zp_w for signed storage) enters through one term per output position.
    const bool w_rebias = w_u8 && Ktot % 16 == 0;
    const bool zp_w_ok = w_u8 ? (t.zp_w >= 0 && t.zp_w <= 255) : (t.zp_w >= -128 && t.zp_w <= 127);
    const int wz_rest = (w_u8 ? 128 : 0) - t.zp_w;
    const bool mfma_ok = (!w_u8 || w_rebias) && zp_w_ok && zp_in_ok && zp_out_ok && Mtot < (1ll << 31) && g.OC < (1ll << 31) &&
                         (wz_rest == 0 || (g.IC % 16 == 0 && g.N * g.H * g.W < (1ll << 31) && g.IC < (1 << 23)));
    const bool is_1x1 = g.KY == 1 && g.KX == 1 && t.kernel_padding[0] == 0 && t.kernel_padding[1] == 0 &&
                        t.kernel_padding[2] == 0 && t.kernel_padding[3] == 0;
    const bool is_gemm = is_1x1 && g.SY == 1 && g.SX == 1;
    // a 1x1 layer with a stride, or whose input pixels are not evenly spaced (a window of a larger tensor), is a matmul
    // over rows picked from the input (one group, the view spanning less than 4 GiB)
    const bool picks_rows = !(is_gemm && in_flat);
    const bool is_strided_gemm = is_1x1 && picks_rows && t.groups <= 1 && vin.span < (1ll << 32);
    const bool is_flat_gemm = is_gemm && in_flat && vin.sw < (1ll << 23);
    // (the MFMA kernels read 16 bytes at a time from wherever a pixel starts)
    const bool aligned = ((reinterpret_cast<uintptr_t>(t.input) | reinterpret_cast<uintptr_t>(t.weights) |
                           (uintptr_t)(vin.sn | vin.sh | vin.sw)) & 15) == 0;
    // VPX_NCE_KERNEL=naive|gather|conv restricts the choice to the slower, more general paths (used by tests
    // to check the device paths against each other).
    const Tuning& knobs = tuning();
    const int force = knobs.nce_kernel.load();
    const bool allow_gemm = force == NCE_AUTO;
    const bool allow_lds = allow_gemm || force == NCE_CONV;
    const bool allow_mfma = allow_lds || force == NCE_GATHER;

    // A matmul tile wastes half (128 columns) or three quarters of its MFMAs on 64 output channels: such 1x1 layers go
    // to the convolution kernels, whose tiles are 64 channels wide (7.5 us against 9.5 us at [100352 x 64 x 64]), unless K
    // is long enough for the matmul kernel's deeper pipeline to make up for it (from 192 channels on: [100352 x 192 x 64]
    // 13.8 -> 11.1 us, [25088 x 512 x 64] 8.6 -> 7.5 us, [6272 x 1024 x 64] 11.1 -> 9.0 us; 128 channels: even).
    const int64_t gemm_tiles = ((Mtot + 255) / 256) * ((g.OC + 255) / 256);
    // A short K and many rows: the weights of 64-channel blocks stay in the registers of waves that walk blocks of 16
    // rows (nce_gemm_regb.hip; its units are 64 channels wide, so it serves the narrow layers too).  VPX_GEMM_REGB=on|
    // wide|off overrides.  Measured against the tile kernel (us, rotating buffers): [100352 x 64] . [64 x 256] 10.3 / 15.2,
    // [401408 x 64] . [64 x 256] 30.8 / 42.9, [100352 x 256] . [256 x 64] 12.3 / 17.6, [25088 x 64] . [64 x 256] 6.2 / 6.4;
    // about equal at K = 128 ([100352 x 128] . [128 x 256] 17.5 / 17.8, [25088 x 128] . [128 x 512] 10.3 / 10.5); behind it
    // at K = 256 with more than 64 channels ([25088 x 256] . [256 x 128] 8.9 / 8.0, [25088 x 256] . [256 x 512] 15.5 / 12.8).
    // Against the convolution kernels on 64 channels and fewer: [100352 x 64] . [64 x 64] 6.4 / 7.9, [100352 x 128] . [128 x 64]
    // 9.1 / 14.1, [401408 x 64] . [64 x 64] 14.4 / 30.3, [25088 x 64] . [64 x 64] 6.4 / 6.3.
    int regb_cbw = 0, regb_gw = 0;
    int64_t regb_wgs = 0;
    {
        const int regb_knob = knobs.gemm_regb.load();
        if (allow_gemm && is_flat_gemm && !out_f16 && t.groups <= 1 && (g.IC == 64 || g.IC == 128 || g.IC == 256) && regb_knob >= 0 &&
            Mtot < (1ll << 31) && vout.flat == 2 && g.OC % 16 == 0 && (g.out_bits & 15) == 0) {
            int cus = 0;
            const int rc = device_compute_units(&cus);
            if (rc) return rc;
            int cbw = 1, gw = 1;
            gemm_regb_shape(Mtot, g.OC, g.IC, cus, regb_knob == 2, &cbw, &gw);
            const int64_t nblk = (Mtot + 15) / 16;
            const int64_t supers = (g.OC + 63) / 64 / cbw / gw;  // workgroups come in multiples of this
            // workgroups of four waves, as many as are resident at once
            const bool same_f = ppe.prelu_mult == 1 && ppe.prelu_shift == 0;
            int64_t wgs = (int64_t)cus * gemm_regb_workgroups_per_cu(same_f, g.IC, cbw);
            wgs = (wgs + supers - 1) / supers * supers;
            const int64_t per_wg = 4 / gw, streams = wgs / supers * per_wg;  // row streams
            // units of 16 rows x 64 channels per wave: from one and a half on, three where the tile kernel is the alternative at K = 128
            const int64_t units = nblk * ((g.OC + 63) / 64), waves = wgs * 4;
            const bool pays = (g.OC <= 64 || g.IC == 64 ? 2 * units >= 3 * waves : units >= 3 * waves) && (g.IC < 256 || g.OC <= 64);
            if (regb_knob > 0 || pays) {
                if (nblk < streams) wgs = (nblk + per_wg - 1) / per_wg * supers;
                regb_cbw = cbw;
                regb_gw = gw;
                regb_wgs = wgs;
            }
        }
    }
    const bool use_gemm = allow_gemm && (is_flat_gemm || is_strided_gemm) && g.IC % 64 == 0 && g.IC < (1 << 24) &&
                          (g.OC > 64 || (g.OC > 48 && g.IC >= 192) || Mtot < 1024 || regb_cbw != 0);
    // VPU.NCE.MatMul's groups: one launch of the matmul kernel when it serves the shape (the preparation passes then
    // walk all groups' weights / activations as one tensor), else one task after the other on the stream.
    const int64_t G = t.groups > 1 ? t.groups : 1;
    const bool one_launch = G > 1 && allow_mfma && mfma_ok && aligned && use_gemm && (wz_rest == 0 || Mtot % 4 == 0) && G <= 65535 &&
                            G * g.OC < (1ll << 31) && G * Mtot < (1ll << 31);
    if (G > 1 && !one_launch) {
        const int64_t out_bytes = out_f16 ? 2 : 1;
        for (int64_t grp = 0; grp < G; grp++) {
            vpx_nce_task_t sub = t;
            sub.groups = 1;
            sub.input = (const char*)t.input + grp * g.N * g.H * g.W * g.IC;
            sub.weights = (const char*)t.weights + grp * g.OC * Ktot;
            sub.weight_table = t.weight_table + grp * g.OC * 4;
            sub.output = (char*)t.output + grp * Mtot * g.OC * out_bytes;
            const int rc = launch_nce(sub, s, kernel_name);
            if (rc) return rc;
        }
        return VPX_RESULT_SUCCESS;
    }
    const void* wptr = t.weights;  // the signed weights the MFMA kernels read
    size_t wofs = 0;               // scratch bytes taken by their re-biased copy
    const auto scratch = [&](size_t bytes, void** out) {
        void* base = nullptr;
        const int r = get_workspace(s, wofs + bytes, &base);
        *out = (char*)base + wofs;
        return r;
    };
    const int32_t* rowterm = nullptr;  // the per-position term of the weight zero point, when there is one
    const auto rebias_weights = [&]() -> int {
        // (G > 1 here only on the matmul path: all groups' weights and pixels are walked as one tensor)
        const size_t wbytes = w_rebias ? ((size_t)(G * g.OC) * (size_t)Ktot + 255) / 256 * 256 : 0;
        const int64_t pixels = G * g.N * g.H * g.W;
        const bool direct = is_gemm;  // every output position is one input pixel
        constexpr int64_t kRowPad = 32 * kPatchMaxMT + 256;  // edge tiles read past the last position
        const size_t rbytes = wz_rest != 0 ? (size_t)(G * Mtot + kRowPad + (direct ? 0 : pixels)) * sizeof(int32_t) : 0;
        if (wbytes + rbytes == 0) return VPX_RESULT_SUCCESS;
        void* base = nullptr;
        const int r = get_workspace(s, wbytes + (rbytes + 255) / 256 * 256, &base);
        if (r) return r;
        if (w_rebias) {
            const int64_t n_vec = G * g.OC * Ktot / 16;
            const int64_t blocks = (n_vec + 255) / 256;
            hipLaunchKernelGGL(nce_weights_to_s8_kernel, dim3((unsigned)(blocks < 4096 ? blocks : 4096)), dim3(256), 0, s,
                               (const i32x4*)t.weights, (i32x4*)base, n_vec);
            VPX_HIP_CHECK(hipGetLastError());
            wptr = base;
        }
        if (wz_rest != 0) {
            int32_t* rt = (int32_t*)((char*)base + wbytes);
            int32_t* cs = direct ? rt : rt + G * Mtot + kRowPad;
            int lpp = 1;
            while (lpp < g.IC / 16 && lpp < 64) lpp *= 2;
            const int64_t blocks = (pixels * lpp + 255) / 256;
            VPX_REQUIRE(blocks < (1ll << 31), VPX_RESULT_ERROR_UNSUPPORTED_FEATURE, "NCE task: input of %lld pixels exceeds the launch limit",
                        (long long)pixels);
            hipLaunchKernelGGL(nce_pixel_sum_kernel, dim3((unsigned)blocks), dim3(256), 0, s, (const uint8_t*)t.input, cs, pixels,
                               (int)g.IC, lpp, in_u8 ? 0 : (int)0x80808080, (int)((in_u8 ? 0 : 128) * g.IC + t.zp_in * g.IC),
                               direct ? wz_rest : 1, g, in_flat ? 1 : 0);
            VPX_HIP_CHECK(hipGetLastError());
            if (!direct) {
                hipLaunchKernelGGL(nce_window_sum_kernel, dim3((unsigned)((Mtot + 255) / 256)), dim3(256), 0, s, cs, rt, g, wz_rest, Mtot);
                VPX_HIP_CHECK(hipGetLastError());
            }
            rowterm = rt;
        }
        wofs = wbytes + (rbytes + 255) / 256 * 256;
        return VPX_RESULT_SUCCESS;
    };
    // Channel counts that are a multiple of 16 but not of 64 (stem layers; 32, 96, 160 ... channels): the row-patch kernel
    // where a band of input rows and the weights fit LDS together, else the gather kernels below.  (Multiples of 32 have a
    // gather kernel that takes any K: they come here while the weights leave most of LDS to the rows -- [32,112,112,32] ->
    // 64 3x3: 27 us against 64 us, [32,14,14,160] -> 320 1x1: 9 against 19.5; 5x5 x 96 channels, 154 KiB of weights: 183 against 47.)
    if (allow_lds && !use_gemm && mfma_ok && aligned && g.IC % 16 == 0 &&
        (g.IC % 32 != 0 || (g.IC % 64 != 0 && (g.OC <= 32 ? 32 : 64) * ((g.KY * g.KX * (g.IC / 16) + 1) / 2 * 32 + 16) <= 100 * 1024)) &&
        g.H * g.ish < (1ll << 31) &&
        g.N * g.OH < (1ll << 30) && g.OC < (1 << 24) && g.KY * g.KX * g.IC < (1 << 16)) {
        RowsGeom rg{};
        const int cpt = (int)g.IC / 16;
        rg.S = (g.KY * g.KX * cpt + 1) / 2;
        rg.WS = rg.S * 32 + 16;
        rg.m = g.SX * cpt;
        // bytes per patch row under CW output columns: m planes of chunks
        auto row_bytes = [&](int64_t CW) { return (((CW - 1) * g.SX + g.KX) * cpt + rg.m - 1) / rg.m * rg.m * 16; };
        // channels per workgroup: 128 where more than 64 are wanted, their weights are short (a quarter of LDS at most) and
        // blocks of 128 leave at most an eighth of the last one empty ([32,28,28,96] -> 576 1x1: 21.6 -> 16.4 us; 192 channels,
        // a third of two blocks empty: 21.7 -> 23.9 us, so those stay with blocks of 64)
        const bool wide = g.OC > 64 && 128 * (size_t)rg.WS <= 40 * 1024 && ((g.OC + 127) / 128 * 128 - g.OC) * 8 <= g.OC;
        const int bn = g.OC <= 32 ? 32 : (wide ? 128 : 64);
        const size_t fixed = bn * (size_t)rg.WS + bn * sizeof(ChanPrep) + 2 * bn * sizeof(int) + 16 + (size_t)(2 * rg.S + 3) / 4 * 16;
        auto need = [&](int64_t R, int64_t CW) { return fixed + (size_t)((R - 1) * g.SY + g.KY) * (size_t)row_bytes(CW); };
        int cus = 0;
        int rc = device_compute_units(&cus);
        if (rc) return rc;
        const int64_t ocb = (g.OC + bn - 1) / bn;
        const int64_t slots = cus / ocb > 0 ? cus / ocb : 1;  // workgroups per block of channels
        // Tile height and positions per wave block: the cheapest of all that fit, counted in MFMA time (32 clocks
        // each) plus the staging of the rows at about 64 bytes per clock; a workgroup's eight waves take a block each.
        const int S = rg.S;
        int best_r = 0, best_tm = 0;
        int64_t best_cw = 0;
        double best = 0;
        // (the whole width, or the width in 2 .. 32 column tiles: the rows under a band of a wide image do not fit LDS)
        for (int tx = 1; tx <= 32 && (tx == 1 || best_tm == 0 || g.OW / tx >= 64); tx++) {
            const int64_t CW = (g.OW + tx - 1) / tx, RB = row_bytes(CW);
            if (tx > 1 && (g.OW + CW - 1) / CW != tx) continue;
            for (int64_t R = 1; R <= g.OH && need(R, CW) <= kMaxDynLds; R++) {
                const int64_t ntiles = g.N * ((g.OH + R - 1) / R) * tx;
                const int64_t per_wg = (ntiles + slots - 1) / slots;
                for (int tm = 2; tm <= (bn == 128 ? 2 : 4); tm += 2) {
                    const int64_t blocks = (R * CW + 32 * tm - 1) / (32 * tm);
                    const double cost = (double)per_wg * ((double)((blocks + 7) / 8) * tm * (bn / 32) * (S * 32.0 + 400) * 2 +
                                                          (double)((R - 1) * g.SY + g.KY) * (double)RB / 64 + 1500);
                    if (best_tm == 0 || cost < best || (cost == best && (int)R == best_r && CW == best_cw)) {  // (a tie between the block sizes of one tile: the larger)
                        best = cost;
                        best_r = (int)R;
                        best_cw = CW;
                        best_tm = tm;
                    }
                }
            }
        }
        if (const int v = knobs.conv_rows.load()) {
            if (best_tm != 0 && v >= 1 && v <= g.OH && need(v, best_cw) <= kMaxDynLds) best_r = v;
        }
        if (const int v = knobs.conv_cols.load()) {
            if (best_tm != 0 && v >= 1 && v <= g.OW && need(best_r, v) <= kMaxDynLds) best_cw = v;
        }
        const int64_t RB = best_tm ? row_bytes(best_cw) : 0;
        if (best_tm != 0 && RB < (1 << 20) && g.N * ((g.OH + best_r - 1) / best_r) * ((g.OW + best_cw - 1) / best_cw) < (1ll << 30)) {
            const int corr = in_u8 ? 128 - t.zp_in : -t.zp_in;
            rc = rebias_weights();
            if (rc) return rc;
            const int tmin = out_signed ? -128 : 0, tmax = out_signed ? 127 : 255;
            int lo = ppe.clamp_lo > tmin ? ppe.clamp_lo : tmin, hi = ppe.clamp_hi < tmax ? ppe.clamp_hi : tmax;
            if (lo > tmax) lo = tmax;
            if (hi < tmin) hi = tmin;
            if (lo > hi) lo = hi;
            auto fd = [](int64_t d) { return FastDiv{(uint32_t)d, (uint32_t)(((1ull << 32) + (uint64_t)d - 1) / (uint64_t)d)}; };
            const int tiles_y = (int)((g.OH + best_r - 1) / best_r), tiles_x = (int)((g.OW + best_cw - 1) / best_cw);
            rg.R = best_r;
            rg.CW = (int)best_cw;
            rg.PH = (best_r - 1) * g.SY + g.KY;
            rg.RB = (int)RB;
            rg.plane = (int)(RB / 16 / rg.m);
            rg.row_chunks = (int)(((best_cw - 1) * g.SX + g.KX) * cpt);
            rg.ntiles = (int)(g.N * tiles_y * tiles_x);
            rg.tiles_y = fd(tiles_y);
            rg.tiles_x = fd(tiles_x);
            rg.cw = fd(best_cw);
            rg.ow = fd(g.OW);
            rg.rc = fd(rg.row_chunks);
            rg.cpp = fd(cpt);
            rg.kc = fd(2 * rg.S);
            rg.fm = fd(rg.m);
            rg.rin = fd(g.KX * cpt);
            const size_t lds = need(best_r, best_cw);
            const int64_t per_wg = (rg.ntiles + slots - 1) / slots;
            const dim3 grid((unsigned)((rg.ntiles + per_wg - 1) / per_wg), (unsigned)ocb);
            GemmPpe gp{ppe.prelu_mult, ppe.prelu_shift, corr, t.zp_out, lo, hi, out_signed ? 1 : 0, rowterm, ppe.f16_lo, ppe.f16_hi, out_f16 ? 1 : 0};
            const int pad_byte = t.zp_in & 0xff;
            RowsLaunch rl{(const int8_t*)t.input, (const int8_t*)wptr, t.weight_table, (uint8_t*)t.output, g, rg, pad_byte, gp,
                          in_u8, out_f16, per_wg > 1, bn, best_tm, grid, lds};
            rc = launch_conv_rows16(rl, s);
            if (rc) return rc;
            *kernel_name = "nce_conv_rows16";
            return VPX_RESULT_SUCCESS;
        }
    }

    if (allow_mfma && mfma_ok && aligned && (use_gemm || g.IC % 32 == 0)) {
        int rc = VPX_RESULT_SUCCESS;
        rc = rebias_weights();
        if (rc) return rc;
        const int corr = in_u8 ? 128 - t.zp_in : -t.zp_in;
        PpeFast pf{};
        pf.zp_out = t.zp_out;
        pf.rowterm = rowterm;
        pf.f16_lo = ppe.f16_lo;
        pf.f16_hi = ppe.f16_hi;
        const int tmin = out_signed ? -128 : 0, tmax = out_signed ? 127 : 255;
        pf.lo = ppe.clamp_lo > tmin ? ppe.clamp_lo : tmin;
        pf.hi = ppe.clamp_hi < tmax ? ppe.clamp_hi : tmax;
        if (pf.lo > tmax) pf.lo = tmax;  // clamp window entirely above / below the storage range
        if (pf.hi < tmin) pf.hi = tmin;
        if (pf.lo > pf.hi) pf.lo = pf.hi;  // inverted window: max-then-min always ends at the upper bound

        if (use_gemm) {
            // 256 x 256 tiles (one workgroup per CU) or 128 x 128 (four times as many, two workgroups per CU): whichever
            // leaves less of the chip idle, counting the padding of edge tiles and the empty part of the last round of
            // workgroups; at equal use the large tile is about an eighth faster from K = 256 on (half the operand traffic per
            // MFMA), about equal at K = 128 and slower at K = 64 (all epilogue).  [25088 x 512 x 128] 14.1 -> 7.8 us,
            // [100352 x 256 x 128] 23.8 -> 14.4 us, [512 x 4096 x 4096] 43 -> 24 us with the small tile; [25088 x 256 x 512]
            // 14.3 -> 11.4 us, [12544 x 1024 x 1024] 26.5 -> 21.1 us with the large one.  VPX_GEMM_TILE=128|256 overrides.
            int cus_gemm = 0;
            rc = device_compute_units(&cus_gemm);
            if (rc) return rc;
            GemmPpe gp{ppe.prelu_mult, ppe.prelu_shift, corr, pf.zp_out, pf.lo, pf.hi, out_signed ? 1 : 0, rowterm, ppe.f16_lo, ppe.f16_hi};
            const GemmRows rows{picks_rows ? 1 : 0, vin.sw, (int)g.OW, (int)(g.OH * g.OW), (unsigned)(g.SX * vin.sw), (unsigned)(g.SY * vin.sh),
                                (unsigned)vin.sn};
            const GemmOut dst{vout.flat == 2 ? 1 : 0, vout.sn, vout.sh, vout.sw, (int)g.OW, (int)(g.OH * g.OW), g.out_bits};
            if (regb_cbw != 0) {
                const GemmLaunch gl{(const int8_t*)t.input, (const int8_t*)wptr, t.weight_table, (uint8_t*)t.output, Mtot, g.OC, g.IC, G,
                                    0, 4, false, in_u8, false, out_signed ? OUT_I8 : OUT_U8, gp, rows, dst};
                rc = launch_gemm_regb(gl, regb_cbw, regb_gw, (int)regb_wgs, s);
                if (rc) return rc;
                *kernel_name = "nce_gemm_regb";
                return VPX_RESULT_SUCCESS;
            }
            const int64_t t256 = gemm_tiles * G, t128 = ((Mtot + 127) / 128) * ((g.OC + 127) / 128) * G;
            const double work = (double)Mtot * (double)g.OC * (double)G;
            const double use256 = work / ((double)((t256 + cus_gemm - 1) / cus_gemm) * cus_gemm * 65536.0);
            const double use128 = work / ((double)((t128 + 2 * cus_gemm - 1) / (2 * cus_gemm)) * 2 * cus_gemm * 16384.0);
            // (fp16 outputs: the large tile's epilogue leaves in two passes and costs more than its main loop saves up to
            // K = 1024 -- [32768 x 512 x 512] 26.6 us small, 30.4 us large; [32768 x 2048 x 512] 58.4 and 54.8)
            const bool large = out_f16 ? (g.IC >= 2048 && use256 * 1.06 > use128)
                               : g.IC >= 256 ? use256 * 1.12 > use128
                                             : (g.IC >= 128 && t256 * 10 >= cus_gemm * 7 && t256 <= cus_gemm && use256 * 1.03 > use128);
            const int tile_knob = knobs.gemm_tile.load();
            const int tile = tile_knob ? tile_knob : (large ? 256 : 128);
            // Eight waves (two per SIMD: one wave's reads and loads issue under the other's MFMAs) win at every K
            // (8192^3: 466 us against 483 us with four waves of 128 x 128).  VPX_GEMM_WAVES=4|8 overrides.
            // (an fp16 output exists in the eight-wave form of the large tile only: the knob does not apply to it)
            const int waves_knob = knobs.gemm_waves.load();
            const int nw = tile == 128 ? 4 : (out_f16 ? 8 : (waves_knob ? waves_knob : 8));
            const int64_t nk = g.IC / 64;
            const bool shortk = tile == 128 && nk <= 3 && !out_f16;
            const GemmLaunch gl{(const int8_t*)t.input, (const int8_t*)wptr, t.weight_table, (uint8_t*)t.output, Mtot, g.OC, g.IC, G,
                                tile, nw, shortk, in_u8, knobs.gemm_pingpong.load() != 0, out_f16 ? OUT_F16 : (out_signed ? OUT_I8 : OUT_U8), gp, rows, dst};
            rc = launch_gemm_mfma(gl, s);
            if (rc) return rc;
            *kernel_name = "nce_gemm_mfma";
            return VPX_RESULT_SUCCESS;
        }

        // Preferred: input patch in LDS, one launch.  R = output rows per workgroup.
        if (allow_lds && g.IC % 64 == 0 && g.OW <= 32 * kPatchMaxMT && g.N * g.OH < (1ll << 30) && Ktot < (1 << 20) &&
            g.IC < (1 << 14) && g.W * g.SX < (1 << 14) && g.N * g.OH * g.OW < (1ll << 31)) {
            // IC of 64 or 128: the one-tile-per-workgroup kernel with padded LDS rows (a tap's fragments of more
            // channels do not fit the registers twice)
            // VPX_CONV_KERNEL=stream starts the choice below the tile kernel (tests compare them)
            const int first = knobs.conv_stream.load();
            int cus_here = 0;
            rc = device_compute_units(&cus_here);
            if (rc) return rc;
            // (with 128 channels and a stride the haloed patch crowds the resident weights out of LDS: the
            // streamed-weights kernel below measures 15.7 us against 20.2 at [32,56,56,128] -> 128, 3x3, stride 2)
            // 3x3 taps of 64 channels: the weights fit the registers of every wave.  Copying them there costs about a
            // microsecond per workgroup, which pays from about 50 000 output positions on ([32,56,56,64] -> 64: 9.1 us
            // against 9.5 us; [4,224,224,64] -> 64: 13.9 against 29.2; [32,28,28,64] -> 64: 7.0 against 6.0; the same input
            // at stride 2: 7.5 against 7.1).
            const size_t out_stride = out_f16 ? kPatchOutStrideF16 : kPatchOutStride;  // staging bytes per position
            // (the weights-in-registers kernel stores bytes straight from its registers: integer outputs only)
            if (!out_f16 && g.IC == 64 && g.KY == 3 && g.KX == 3 && g.H * g.ish < (1ll << 31) &&
                (first < 0 || (first == 0 && g.N * g.OH * g.OW >= 50000))) {
                PatchGeom pg{};
                const int64_t PS = g.IC + 32, WS = Ktot + 32;  // the kernel's LDS strides of a pixel and of a weight row
                auto need = [&](int R) {
                    return 64 * (size_t)WS + (size_t)((R - 1) * g.SY + g.KY) * (size_t)((g.OW - 1) * g.SX + g.KX) * (size_t)PS;
                };
                int cus = 0;
                rc = device_compute_units(&cus);
                if (rc) return rc;
                const int64_t ocb = (g.OC + 63) / 64;
                // Rows per tile: a workgroup costs about 2.9 us whatever its tile (launch, the fetch of its weights and rows,
                // the register copies) and 0.0106 us per output position, and the workgroups run in rounds of one per compute
                // unit -- the plane is cut into the number of tiles for which rounds x (fixed + positions) is smallest
                // ([128,56,56,64]: 512 tiles of 14 rows, two full rounds, 22.5 us; the 384 tiles of 19 rows that one
                // workgroup per compute unit and LDS allowed took 26.4 us, a round and a half; [32,112,112,64]: 7 rows,
                // 23.0 against 26.3 us)
                const int rmin = (int)((128 + g.OW - 1) / g.OW);  // eight waves want eight blocks of 16 positions
                int R = 0;
                double best = 0;
                for (int64_t ty = 1; ty <= g.OH; ty++) {
                    const int64_t r = (g.OH + ty - 1) / ty;
                    if (r < rmin && ty > 1) break;
                    if (need((int)r) > kMaxDynLds) continue;
                    const int64_t rounds = (g.N * ty * ocb + cus - 1) / cus;
                    const double cost = (double)rounds * (2.9 + 0.0106 * (double)(r * g.OW));
                    if (R == 0 || cost < best) {
                        best = cost;
                        R = (int)r;
                    }
                }
                if (R == 0) R = 1;
                if (const int v = knobs.conv_rows.load()) {
                    if (v >= 1 && v <= R) R = v;
                }
                if (need(R) <= kMaxDynLds) {
                    const int tiles_y = (int)((g.OH + R - 1) / R);
                    auto fd = [](int64_t d) { return FastDiv{(uint32_t)d, (uint32_t)(((1ull << 32) + (uint64_t)d - 1) / (uint64_t)d)}; };
                    pg.R = (int)((g.OH + tiles_y - 1) / tiles_y);
                    pg.PH = (pg.R - 1) * g.SY + g.KY;
                    pg.PW = (int)(g.OW - 1) * g.SX + g.KX;
                    pg.MT = (int)((pg.R * g.OW + 31) / 32);
                    pg.nt = 2;
                    pg.ntiles = (int)(g.N * tiles_y);
                    pg.tiles_y = fd(tiles_y);
                    pg.cpr = fd(Ktot / 16);
                    pg.cpp = fd(g.IC / 16);
                    pg.upr = fd((pg.PW * (g.IC / 16) + 63) / 64);
                    pg.ow = fd(g.OW);
                    const size_t lds = need(pg.R);
                    const dim3 grid((unsigned)(g.N * tiles_y), (unsigned)ocb);
                    GemmPpe gp{ppe.prelu_mult, ppe.prelu_shift, corr, pf.zp_out, pf.lo, pf.hi, out_signed ? 1 : 0, rowterm, ppe.f16_lo, ppe.f16_hi, out_f16 ? 1 : 0};
                    const int pad_byte = t.zp_in & 0xff;
                    const bool same_f = ppe.prelu_mult == 1 && ppe.prelu_shift == 0;
                    const PatchLaunch pl{(const int8_t*)t.input, (const int8_t*)wptr, t.weight_table, nullptr, (uint8_t*)t.output, g, pg,
                                         StreamGeom{}, pad_byte, gp, in_u8, same_f, grid, lds};
                    rc = launch_conv_regw(pl, s);
                    if (rc) return rc;
                    *kernel_name = "nce_conv_regw";
                    return VPX_RESULT_SUCCESS;
                }
            }
            if ((g.IC == 64 || (g.IC == 128 && g.SY * g.SX == 1)) && first <= 1) {
                PatchGeom pg{};
                const int64_t PS = g.IC + 16, WS = Ktot + 16;
                auto need = [&](int R) {
                    const size_t patch = (size_t)((R - 1) * g.SY + g.KY) * (size_t)((g.OW - 1) * g.SX + g.KX) * (size_t)PS;
                    const size_t stage = (size_t)((R * g.OW + 31) / 32) * 32 * out_stride;
                    return 64 * (size_t)WS + (patch > stage ? patch : stage);
                };
                int R = (int)(32 * kPatchMaxMT / g.OW);
                if (R > g.OH) R = (int)g.OH;
                while (R > 1 && need(R) > 160 * 1024 - 512) R--;
                if (need(R) <= 160 * 1024 - 512) {
                    const int64_t ocb = (g.OC + 63) / 64;
                    // shorter tiles while they are few: down to 128 positions, or to 64 while there are fewer tiles
                    // than compute units ([32,14,14,256] -> 256, 3x3: 12.1 us with 256 tiles of 7 rows, 15.4 us with 128 of 14)
                    while (R > 1) {
                        const int64_t tiles = g.N * ((g.OH + R - 1) / R) * ocb;
                        if (tiles >= 512 || ((R + 1) / 2) * g.OW < (tiles < cus_here ? 64 : 128)) break;
                        R = (R + 1) / 2;
                    }
                    if (const int v = knobs.conv_rows.load()) {
                        if (v >= 1 && v <= R) R = v;
                    }
                    const int tiles_y = (int)((g.OH + R - 1) / R);
                    auto fd = [](int64_t d) { return FastDiv{(uint32_t)d, (uint32_t)(((1ull << 32) + (uint64_t)d - 1) / (uint64_t)d)}; };
                    pg.R = (int)((g.OH + tiles_y - 1) / tiles_y);
                    pg.PH = (pg.R - 1) * g.SY + g.KY;
                    pg.PW = (int)(g.OW - 1) * g.SX + g.KX;
                    pg.MT = (int)((pg.R * g.OW + 31) / 32);
                    pg.nt = g.OC <= 32 ? 1 : 2;
                    pg.ntiles = (int)(g.N * tiles_y);
                    pg.tiles_y = fd(tiles_y);
                    pg.cpr = fd(Ktot / 16);
                    pg.cpp = fd(g.IC / 16);
                    pg.upr = fd((pg.PW * (g.IC / 16) + 63) / 64);
                    pg.ow = fd(g.OW);
                    const size_t lds = need(pg.R);
                    const dim3 grid((unsigned)(g.N * tiles_y), (unsigned)ocb);
                    GemmPpe gp{ppe.prelu_mult, ppe.prelu_shift, corr, pf.zp_out, pf.lo, pf.hi, out_signed ? 1 : 0, rowterm, ppe.f16_lo, ppe.f16_hi, out_f16 ? 1 : 0};
                    const int pad_byte = t.zp_in & 0xff;
                    const bool same_f = ppe.prelu_mult == 1 && ppe.prelu_shift == 0;
                    const int nw = knobs.conv_waves.load() == 4 ? 4 : 8;
                    const int per_wave = (pg.MT + nw / pg.nt - 1) / (nw / pg.nt);
                    const int ics = (int)(g.IC / 64);
                    const PatchLaunch pl{(const int8_t*)t.input, (const int8_t*)wptr, t.weight_table, nullptr, (uint8_t*)t.output, g, pg,
                                         StreamGeom{}, pad_byte, gp, in_u8, same_f, grid, lds};
                    rc = launch_conv_tile(pl, per_wave, ics, nw, s);
                    if (rc) return rc;
                    *kernel_name = "nce_conv_tile";
                    return VPX_RESULT_SUCCESS;
                }
            }
            // any IC that is a multiple of 64: resident patch, weights streamed a slice at a time
            if (first <= 2) {
                PatchGeom pg{};
                StreamGeom sg{};
                sg.ksl = g.IC % 256 == 0 ? 256 : (g.IC % 128 == 0 ? 128 : 64);
                sg.spt = (int)(g.IC / sg.ksl);
                const int64_t PS = g.IC + 16;
                auto need = [&](int R) {
                    const size_t patch = (size_t)((R - 1) * g.SY + g.KY) * (size_t)((g.OW - 1) * g.SX + g.KX) * (size_t)PS;
                    const size_t stage = (size_t)((R * g.OW + 31) / 32) * 32 * out_stride;
                    return 2 * 64 * (size_t)(sg.ksl + 16) + (patch > stage ? patch : stage);
                };
                int R = (int)(32 * kPatchMaxMT / g.OW);
                if (R > g.OH) R = (int)g.OH;
                while (R > 1 && need(R) > 160 * 1024 - 512) R--;
                if (need(R) <= 160 * 1024 - 512) {
                    const int64_t ocb = (g.OC + 63) / 64;
                    // shorter tiles while they are few: down to 128 positions, or to 64 while there are fewer tiles
                    // than compute units ([32,14,14,256] -> 256, 3x3: 12.1 us with 256 tiles of 7 rows, 15.4 us with 128 of 14)
                    while (R > 1) {
                        const int64_t tiles = g.N * ((g.OH + R - 1) / R) * ocb;
                        if (tiles >= 512 || ((R + 1) / 2) * g.OW < (tiles < cus_here ? 64 : 128)) break;
                        R = (R + 1) / 2;
                    }
                    if (const int v = knobs.conv_rows.load()) {
                        if (v >= 1 && v <= R) R = v;
                    }
                    const int tiles_y = (int)((g.OH + R - 1) / R);
                    auto fd = [](int64_t d) { return FastDiv{(uint32_t)d, (uint32_t)(((1ull << 32) + (uint64_t)d - 1) / (uint64_t)d)}; };
                    pg.R = (int)((g.OH + tiles_y - 1) / tiles_y);
                    pg.PH = (pg.R - 1) * g.SY + g.KY;
                    pg.PW = (int)(g.OW - 1) * g.SX + g.KX;
                    pg.MT = (int)((pg.R * g.OW + 31) / 32);
                    pg.nt = g.OC <= 32 ? 1 : 2;
                    pg.ntiles = (int)(g.N * tiles_y);
                    pg.tiles_y = fd(tiles_y);
                    pg.cpr = fd(Ktot / 16);
                    pg.cpp = fd(g.IC / 16);
                    pg.upr = fd((pg.PW * (g.IC / 16) + 63) / 64);
                    pg.ow = fd(g.OW);
                    // tiles of at most 64 positions per four waves: K split over the waves of a group (slices of four or
                    // eight K steps, both channel tiles in use)
                    // (one tile of 64 positions: eight waves, eight shares of K, where a slice has eight K steps)
                    const int ksplit_waves = knobs.stream_ksplit.load() && pg.nt == 2 && sg.ksl >= 128 ? (pg.MT <= 2 ? (sg.ksl == 256 ? 88 : 4) : (pg.MT <= 4 ? 8 : 0)) : 0;
                    size_t lds = need(pg.R);
                    if (lds < (size_t)(ksplit_waves % 80) * 16384) lds = (size_t)(ksplit_waves % 80) * 16384;  // the partial sums
                    const dim3 grid((unsigned)(g.N * tiles_y), (unsigned)ocb);
                    GemmPpe gp{ppe.prelu_mult, ppe.prelu_shift, corr, pf.zp_out, pf.lo, pf.hi, out_signed ? 1 : 0, rowterm, ppe.f16_lo, ppe.f16_hi, out_f16 ? 1 : 0};
                    const int pad_byte = t.zp_in & 0xff;
                    const bool same_f = ppe.prelu_mult == 1 && ppe.prelu_shift == 0;
                    int32_t* colsum = nullptr;
                    if (corr != 0) {
                        void* ws = nullptr;
                        rc = scratch(sizeof(int32_t) * (size_t)g.OC, &ws);
                        if (rc) return rc;
                        colsum = (int32_t*)ws;
                        rc = launch_colsum((const int8_t*)wptr, colsum, g.OC, Ktot, s);
                        if (rc) return rc;
                    }
                    const int per_wave = (pg.MT + 8 / pg.nt - 1) / (8 / pg.nt);  // eight waves: at most 4 row blocks each
                    const PatchLaunch pl{(const int8_t*)t.input, (const int8_t*)wptr, t.weight_table, colsum, (uint8_t*)t.output, g, pg,
                                         sg, pad_byte, gp, in_u8, same_f, grid, lds};
                    rc = launch_conv_stream(pl, ksplit_waves, per_wave, s);
                    if (rc) return rc;
                    *kernel_name = "nce_conv_stream";
                    return VPX_RESULT_SUCCESS;
                }
            }
        }
        // Fallback: activation fragments gathered from global memory; per-channel parameters come
        // from a small preparation kernel.
        void* ws = nullptr;
        rc = scratch(sizeof(ChanPrep) * (size_t)g.OC, &ws);
        if (rc) return rc;
        ChanPrep* prep = (ChanPrep*)ws;
        rc = launch_fold((const int8_t*)wptr, t.weight_table, prep, g.OC, Ktot, corr, ppe, out_f16 ? 15 : 0, s);
        if (rc) return rc;
        rc = launch_conv_mfma((const int8_t*)t.input, (const int8_t*)wptr, prep, (uint8_t*)t.output, g, t.zp_in & 0xff, pf, in_u8,
                              out_f16 ? OUT_F16 : (out_signed ? OUT_I8 : OUT_U8), s);
        if (rc) return rc;
        *kernel_name = "nce_conv_mfma";
        return VPX_RESULT_SUCCESS;
    }

    if (allow_mfma && mfma_ok && aligned && g.IC % 16 == 0 && g.IC % 32 != 0 && ((Ktot + 31) / 32 * 32 + 16) * 64 <= 64 * 1024) {
        const int corr = in_u8 ? 128 - t.zp_in : -t.zp_in;
        PpeFast pf{};
        pf.zp_out = t.zp_out;
        pf.f16_lo = ppe.f16_lo;
        pf.f16_hi = ppe.f16_hi;
        const int tmin = out_signed ? -128 : 0, tmax = out_signed ? 127 : 255;
        pf.lo = ppe.clamp_lo > tmin ? ppe.clamp_lo : tmin;
        pf.hi = ppe.clamp_hi < tmax ? ppe.clamp_hi : tmax;
        if (pf.lo > tmax) pf.lo = tmax;
        if (pf.hi < tmin) pf.hi = tmin;
        if (pf.lo > pf.hi) pf.lo = pf.hi;
        int rc = rebias_weights();
        if (rc) return rc;
        pf.rowterm = rowterm;
        void* ws = nullptr;
        rc = scratch(sizeof(ChanPrep) * (size_t)g.OC, &ws);
        if (rc) return rc;
        ChanPrep* prep = (ChanPrep*)ws;
        rc = launch_fold((const int8_t*)wptr, t.weight_table, prep, g.OC, Ktot, corr, ppe, out_f16 ? 15 : 0, s);
        if (rc) return rc;
        rc = launch_conv_mfma16((const int8_t*)t.input, (const int8_t*)wptr, prep, (uint8_t*)t.output, g, t.zp_in & 0xff, pf, in_u8,
                                out_f16 ? OUT_F16 : OUT_U8, s);
        if (rc) return rc;
        *kernel_name = "nce_conv_mfma16";
        return VPX_RESULT_SUCCESS;
    }

    const int rc = launch_conv_naive((const uint8_t*)t.input, (const uint8_t*)t.weights, t.weight_table, (uint8_t*)t.output, g, t.zp_in, t.zp_w,
                                     ppe, in_u8, w_u8, out_f16 ? OUT_F16 : (out_signed ? OUT_I8 : OUT_U8), s);
    if (rc) return rc;
    *kernel_name = "nce_conv_naive";
    return VPX_RESULT_SUCCESS;
}

}  // namespace vpx
