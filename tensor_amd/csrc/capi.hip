// extern "C" boundary of the library (include/otter_hip_int8.h): argument checking, handle management,
// weight re-layout at create time and kernel dispatch. No kernels live here.
#include <cmath>
#include <cstring>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "common.hpp"
#include "conv_igemm.hpp"

using namespace ohip;

namespace {

thread_local std::string g_last_error;

int fail(int code, const std::string& msg) {
    g_last_error = msg;
    return code;
}

int hip_fail(hipError_t e, const char* what) {
    (void)hipGetLastError();
    return fail(e == hipErrorOutOfMemory ? OTTER_HIP_ERR_ALLOC : OTTER_HIP_ERR_RUNTIME,
                std::string(what) + ": " + hipGetErrorString(e));
}

#define OHIP_CHECK(expr)                                  \
    do {                                                  \
        hipError_t e__ = (expr);                          \
        if (e__ != hipSuccess) return hip_fail(e__, #expr); \
    } while (0)

bool valid_layout(int l) { return l >= OTTER_HIP_F32 && l <= OTTER_HIP_I32_P8; }

int conv_out_size(int in, int k, int s, int p, int d) { return (in + 2 * p - d * (k - 1) - 1) / s + 1; }

template <typename T>
int upload(T** dev, const T* host, size_t count, size_t padded_count, T pad_value) {
    std::vector<T> tmp(padded_count, pad_value);
    if (host) std::memcpy(tmp.data(), host, count * sizeof(T));
    OHIP_CHECK(hipMalloc((void**)dev, padded_count * sizeof(T)));
    OHIP_CHECK(hipMemcpy(*dev, tmp.data(), padded_count * sizeof(T), hipMemcpyHostToDevice));
    return OTTER_HIP_OK;
}

// ---- the workspace of otter_hip_conv_forward_static ---------------------------------------------------------
// A file-scope device array: every GPU the library runs on holds its own copy, at its own address, until the process
// ends. `scratch` below is only a host-side stand-in for the symbol: the device address comes from
// hipGetSymbolAddress, once per device with that device current, and only that address is handed to kernels.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

}  // namespace

static __device__ __align__(256) unsigned char scratch[OTTER_HIP_STATIC_WORKSPACE_BYTES];

namespace {

// device address of `scratch` on the current device (looked up on first use, then kept); null + error text on failure
void* static_workspace(int* rc) {
    *rc = OTTER_HIP_OK;
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        *rc = hip_fail(e, "hipGetDevice");
        return nullptr;
    }
    if (dev < 0 || dev >= kMaxDevices) {
        *rc = fail(OTTER_HIP_ERR_UNSUPPORTED, "static workspace: device index out of range");
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            *rc = hip_fail(e == hipSuccess ? hipErrorInvalidSymbol : e, "hipGetSymbolAddress(scratch)");
            return nullptr;
        }
        g_scratch_ptr[dev] = p;
    }
    return g_scratch_ptr[dev];
}

}  // namespace

struct otter_hip_conv {
    otter_hip_conv_desc d;
    bool depthwise = false;
    int8_t* w_raw = nullptr;     // [K, C/g, kh, kw]           (direct kernel)
    int8_t* w_igemm = nullptr;   // MFMA lane order            (groups == 1, C % 8 == 0)
    int8_t* w_stem = nullptr;    // MFMA lane order of the few-channel 3x3 kernel (C <= 5, K <= 64)
    int32_t* w_dw = nullptr;     // dot4 weight words          (depthwise, C % 8 == 0)
    int8_t* w_dw_mfma = nullptr; // block-diagonal MFMA operands (depthwise 3x3, C % 8 == 0)
    int8_t* w_xdw = nullptr;     // MFMA operands of a pointwise int8 -> int8 layer for the launch it shares with its depthwise reader
    int32_t* blk_consts = nullptr; // the layer's constants (and depthwise 3x3 weights) as the fused block launch keeps them in LDS
    bool so_positive = true;     // every output scale is finite and > 0
    float* scale_in = nullptr;   // [Kpad]
    float* bias = nullptr;       // [Kpad]; -0.0f everywhere when the layer has no bias
    float* scale_out = nullptr;  // [Kpad] or null
    unsigned* clamp_hi = nullptr; // [Kpad / 2] upper clamps of the rounded int8 results (ReLU / clip, dense layers) or null
    float* in_scale = nullptr;   // [1]
    int c_pad = 0;               // > 0: C is not a multiple of 8; the MFMA path runs on C zero-padded to c_pad
    int force_tm = 0, force_tn = 0;
    int block_rb = 0, block_sl = 0, block_split = 0;  // forced plan of the fused block launch this layer heads (0 = automatic)
};

extern "C" {

const char* otter_hip_last_error(void) { return g_last_error.c_str(); }

int otter_hip_init(int device) {
    int count = 0;
    OHIP_CHECK(hipGetDeviceCount(&count));
    if (device < 0 || device >= count) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_init: no such device");
    OHIP_CHECK(hipSetDevice(device));
    hipDeviceProp_t prop;
    OHIP_CHECK(hipGetDeviceProperties(&prop, device));
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(OTTER_HIP_ERR_UNSUPPORTED,
                    std::string("otter_hip_init: this library is built for gfx950 only, found ") + prop.gcnArchName);
    // this device's copy of the static workspace (otter_hip_conv_forward_static)
    int rc = OTTER_HIP_OK;
    (void)static_workspace(&rc);
    return rc;
}

int otter_hip_shutdown(void) { return OTTER_HIP_OK; }

int otter_hip_device_info(int* compute_units, int* clock_mhz, int* mem_clock_mhz, int* mem_bus_bits) {
    int dev = 0;
    OHIP_CHECK(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    OHIP_CHECK(hipGetDeviceProperties(&prop, dev));
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (clock_mhz) *clock_mhz = prop.clockRate / 1000;
    if (mem_clock_mhz) *mem_clock_mhz = prop.memoryClockRate / 1000;
    if (mem_bus_bits) *mem_bus_bits = prop.memoryBusWidth;
    return OTTER_HIP_OK;
}

int otter_hip_shader_clock_mhz(void* stream_, float* mhz) {
    if (!mhz) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_shader_clock_mhz: null");
    int dev = 0;
    OHIP_CHECK(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    OHIP_CHECK(hipGetDeviceProperties(&prop, dev));
    const int blocks = prop.multiProcessorCount;
    hipStream_t stream = (hipStream_t)stream_;
    unsigned long long* d = nullptr;
    OHIP_CHECK(hipMalloc(&d, sizeof(unsigned long long) * 2 * blocks));
    // about a millisecond of matrix instructions on every SIMD (4 x 20000 of 16 cycles each)
    hipError_t e = run_shader_clock(blocks, 20000, d, stream);
    std::vector<unsigned long long> h(2 * blocks);
    if (e == hipSuccess) e = hipMemcpyAsync(h.data(), d, sizeof(unsigned long long) * 2 * blocks, hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    (void)hipFree(d);
    OHIP_CHECK(e);
    double cyc = 0, ref = 0;
    for (int i = 0; i < blocks; ++i) cyc += (double)h[2 * i], ref += (double)h[2 * i + 1];
    if (ref <= 0) return fail(OTTER_HIP_ERR_RUNTIME, "otter_hip_shader_clock_mhz: the reference counter did not advance");
    *mhz = (float)(cyc / ref * 100.0);  // the reference counter runs at 100 MHz
    return OTTER_HIP_OK;
}

int otter_hip_malloc(void** ptr, size_t bytes) {
    if (!ptr) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_malloc: null");
    OHIP_CHECK(hipMalloc(ptr, bytes ? bytes : 1));
    return OTTER_HIP_OK;
}

int otter_hip_free(void* ptr) {
    if (ptr) OHIP_CHECK(hipFree(ptr));
    return OTTER_HIP_OK;
}

int otter_hip_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream) {
    OHIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, (hipStream_t)stream));
    return OTTER_HIP_OK;
}

int otter_hip_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream) {
    OHIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream));
    return OTTER_HIP_OK;
}

int otter_hip_stream_create(void** stream) {
    hipStream_t s;
    OHIP_CHECK(hipStreamCreate(&s));
    *stream = (void*)s;
    return OTTER_HIP_OK;
}

int otter_hip_stream_destroy(void* stream) {
    OHIP_CHECK(hipStreamDestroy((hipStream_t)stream));
    return OTTER_HIP_OK;
}

int otter_hip_stream_synchronize(void* stream) {
    OHIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
    return OTTER_HIP_OK;
}

// -----------------------------------------------------------------------------------------------------
// convolution
// -----------------------------------------------------------------------------------------------------

int otter_hip_conv_destroy(otter_hip_conv_t* h) {
    if (!h) return OTTER_HIP_OK;
    (void)hipFree(h->w_raw);
    (void)hipFree(h->w_igemm);
    (void)hipFree(h->w_stem);
    (void)hipFree(h->w_dw);
    (void)hipFree(h->w_dw_mfma);
    (void)hipFree(h->w_xdw);
    (void)hipFree(h->blk_consts);
    (void)hipFree(h->scale_in);
    (void)hipFree(h->bias);
    (void)hipFree(h->scale_out);
    (void)hipFree(h->clamp_hi);
    (void)hipFree(h->in_scale);
    delete h;
    return OTTER_HIP_OK;
}

int otter_hip_conv_create(const otter_hip_conv_desc* desc, const int8_t* weight, const float* scale_in,
                          const float* bias, float in_scale, const float* out_scale, int n_out_scale,
                          otter_hip_conv_t** handle) {
    if (!desc || !weight || !scale_in || !handle) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_create: null");
    const otter_hip_conv_desc& d = *desc;
    if (d.in_channels < 1 || d.out_channels < 1 || d.kernel_h < 1 || d.kernel_w < 1 || d.stride_h < 1 ||
        d.stride_w < 1 || d.pad_h < 0 || d.pad_w < 0 || d.dilation_h < 1 || d.dilation_w < 1 || d.groups < 1)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_create: bad geometry");
    if (d.in_channels % d.groups || d.out_channels % d.groups)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_create: channels not divisible by groups");
    if (d.out_kind < OTTER_HIP_OUT_I32 || d.out_kind > OTTER_HIP_OUT_I8)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_create: bad out_kind");
    if (d.activation_type < 0 || d.activation_type > 5)
        return fail(OTTER_HIP_ERR_UNSUPPORTED, "otter_hip_conv_create: activation type not supported");
    if (d.out_kind == OTTER_HIP_OUT_I8 && (!out_scale || (n_out_scale != 1 && n_out_scale != d.out_channels)))
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_create: int8 output needs 1 or K output scales");

    otter_hip_conv* h = new (std::nothrow) otter_hip_conv();
    if (!h) return fail(OTTER_HIP_ERR_ALLOC, "otter_hip_conv_create: host allocation failed");
    h->d = d;
    const int K = d.out_channels, C = d.in_channels, g = d.groups, maxk = d.kernel_h * d.kernel_w;
    h->depthwise = (C == g && g == K);
    // the kernels read the per-channel arrays up to the padded row count (of the last group, for a grouped layer)
    const int kpad = g > 1 ? K + 128 : igemm_padded_rows(K);
    int rc = OTTER_HIP_OK;
    do {
        const size_t wcount = (size_t)K * (C / g) * maxk;
        if ((rc = upload<int8_t>(&h->w_raw, weight, wcount, wcount, 0))) break;
        if ((rc = upload<float>(&h->scale_in, scale_in, K, kpad, 0.f))) break;
        // no bias: -0.0f, so that fma(acc, scale, bias) == acc * scale bit for bit (sign of zero included)
        if ((rc = upload<float>(&h->bias, bias, bias ? K : 0, kpad, -0.0f))) break;
        if (d.out_kind == OTTER_HIP_OUT_I8) {
            std::vector<float> so(K);
            for (int i = 0; i < K; ++i) {
                so[i] = n_out_scale == 1 ? out_scale[0] : out_scale[i];
                if (!(so[i] > 0.f) || std::isinf(so[i])) h->so_positive = false;
            }
            if ((rc = upload<float>(&h->scale_out, so.data(), K, kpad, 1.f))) break;
            if (g == 1 && h->so_positive && (d.activation_type == 1 || d.activation_type == 3)) {
                // the streamed 1x1 kernel reads the clamps of its ReLU / clip epilogue instead of deriving them per wave
                so.resize(kpad, 1.f);
                std::vector<unsigned> qh(kpad / 2);
                conv_pw_stream_clamps(d.activation_type == 3 ? 6.f : __builtin_inff(),
                                      d.out_round_mode == OTTER_HIP_ROUND_SSE ? 0.5f : 0.49999997f, so.data(), kpad, qh.data());
                if ((rc = upload<unsigned>(&h->clamp_hi, qh.data(), qh.size(), qh.size(), 0u))) break;
            }
        }
        if (d.out_kind == OTTER_HIP_OUT_I8 && K % 8 == 0 && C % 8 == 0 &&
            (g == 1 || (h->depthwise && d.kernel_h == 3 && d.kernel_w == 3))) {
            // what the fused block launch (conv_block.hip) copies into LDS: the per-channel arrays as uploaded above
            // (padded the same way), the upper clamps of a ReLU / clip epilogue, a depthwise layer's weights
            const int kp = (K + 31) / 32 * 32;
            std::vector<float> si(kp, 0.f), bi(kp, -0.0f), so(kp, 1.f);
            std::memcpy(si.data(), scale_in, (size_t)K * sizeof(float));
            if (bias) std::memcpy(bi.data(), bias, (size_t)K * sizeof(float));
            for (int i = 0; i < K; ++i) so[i] = n_out_scale == 1 ? out_scale[0] : out_scale[i];
            const bool nonneg = h->so_positive && (d.activation_type == 1 || d.activation_type == 3);
            const float hi = d.activation_type == 3 ? 6.f : __builtin_inff();
            const float half = d.out_round_mode == OTTER_HIP_ROUND_SSE ? 0.5f : 0.49999997f;
            std::vector<int32_t> kc((g == 1 ? block_expand_const_bytes(K) : block_dw_const_bytes(K)) / sizeof(int32_t));
            if (g == 1) block_pack_expand_consts(si.data(), bi.data(), so.data(), K, nonneg, hi, half, kc.data());
            else block_pack_dw_consts(weight, si.data(), bi.data(), so.data(), K, nonneg, hi, half, kc.data());
            if ((rc = upload<int32_t>(&h->blk_consts, kc.data(), kc.size(), kc.size(), 0))) break;
        }
        if ((rc = upload<float>(&h->in_scale, &in_scale, 1, 1, 0.f))) break;
        if (h->depthwise && C % 8) {
            // depthwise on a channel count that is not whole octets: the channels are zero-padded to the next octet on the
            // way in (weights of the padding channels are zero, their results are never stored)
            const int cp = (C + 7) / 8 * 8;
            std::vector<int8_t> wpad((size_t)cp * maxk, 0);
            std::memcpy(wpad.data(), weight, (size_t)C * maxk);
            std::vector<int32_t> wm(dw_packed_weight_bytes(cp, d.kernel_h, d.kernel_w) / sizeof(int32_t));
            dw_pack_weights(wpad.data(), cp, d.kernel_h, d.kernel_w, wm.data());
            if ((rc = upload<int32_t>(&h->w_dw, wm.data(), wm.size(), wm.size(), 0))) break;
            h->c_pad = cp;
        } else if (h->depthwise) {
            std::vector<int32_t> wm(dw_packed_weight_bytes(C, d.kernel_h, d.kernel_w) / sizeof(int32_t));
            dw_pack_weights(weight, C, d.kernel_h, d.kernel_w, wm.data());
            if ((rc = upload<int32_t>(&h->w_dw, wm.data(), wm.size(), wm.size(), 0))) break;
            if (d.kernel_h == d.kernel_w && (d.kernel_h == 3 || d.kernel_h == 5) && d.stride_h == d.stride_w &&
                (d.stride_w == 1 || d.stride_w == 2) && dw_mfma_window_fits(d.kernel_w, d.stride_w, d.pad_w)) {
                std::vector<int8_t> wa(dw_mfma_weight_bytes(C, d.stride_w, d.kernel_w));
                dw_mfma_pack_weights(weight, C, d.stride_w, d.pad_w, d.kernel_w, wa.data());
                if ((rc = upload<int8_t>(&h->w_dw_mfma, wa.data(), wa.size(), wa.size(), 0))) break;
            }

        } else if (g == 1 && C % 8 == 0) {
            std::vector<int8_t> wp(igemm_packed_weight_bytes(K, C, d.kernel_h, d.kernel_w));
            igemm_pack_weights(weight, K, C, d.kernel_h, d.kernel_w, wp.data());
            if ((rc = upload<int8_t>(&h->w_igemm, wp.data(), wp.size(), wp.size(), 0))) break;
            if (maxk == 1 && d.out_kind == OTTER_HIP_OUT_I8 && K % 16 == 0 && C <= 128 && d.stride_h == 1 && d.stride_w == 1 &&
                d.pad_h == 0 && d.pad_w == 0) {
                std::vector<int8_t> wx(xdw_weight_bytes(C, K));
                xdw_pack_weights(weight, C, K, wx.data());
                if ((rc = upload<int8_t>(&h->w_xdw, wx.data(), wx.size(), wx.size(), 0))) break;
            }
        } else if (g > 1 && !h->depthwise && (C / g) % 8 == 0) {
            // grouped: every group's weights packed by itself (one launch, a group per grid.z slice)
            std::vector<int8_t> wp(igemm_grouped_weight_bytes(K, C, g, d.kernel_h, d.kernel_w));
            igemm_pack_weights_grouped(weight, K, C, g, d.kernel_h, d.kernel_w, wp.data());
            if ((rc = upload<int8_t>(&h->w_igemm, wp.data(), wp.size(), wp.size(), 0))) break;
        } else if (g == 1) {
            // C % 8 != 0 (e.g. an RGB stem): zero-pad the input channels to the next octet, weights included
            const int cp = (C + 7) / 8 * 8;
            std::vector<int8_t> wpad((size_t)K * cp * maxk, 0);
            for (int k = 0; k < K; ++k)
                for (int c = 0; c < C; ++c)
                    std::memcpy(&wpad[((size_t)k * cp + c) * maxk], &weight[((size_t)k * C + c) * maxk], maxk);
            std::vector<int8_t> wp(igemm_packed_weight_bytes(K, cp, d.kernel_h, d.kernel_w));
            igemm_pack_weights(wpad.data(), K, cp, d.kernel_h, d.kernel_w, wp.data());
            if ((rc = upload<int8_t>(&h->w_igemm, wp.data(), wp.size(), wp.size(), 0))) break;
            h->c_pad = cp;
            if (C <= 5 && K <= 64 && d.kernel_h == 3 && d.kernel_w == 3) {  // an image stem: see conv_stem.hip
                std::vector<int8_t> wsv(stem_packed_weight_bytes(K));
                stem_pack_weights(weight, K, C, wsv.data());
                if ((rc = upload<int8_t>(&h->w_stem, wsv.data(), wsv.size(), wsv.size(), 0))) break;
            }
        }
    } while (0);
    if (rc != OTTER_HIP_OK) {
        std::string keep = g_last_error;
        otter_hip_conv_destroy(h);
        g_last_error = keep;
        return rc;
    }
    *handle = h;
    return OTTER_HIP_OK;
}

int otter_hip_conv_output_shape(const otter_hip_conv_t* h, int in_h, int in_w, int* out_h, int* out_w) {
    if (!h || !out_h || !out_w) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_output_shape: null");
    *out_h = conv_out_size(in_h, h->d.kernel_h, h->d.stride_h, h->d.pad_h, h->d.dilation_h);
    *out_w = conv_out_size(in_w, h->d.kernel_w, h->d.stride_w, h->d.pad_w, h->d.dilation_w);
    if (*out_h < 1 || *out_w < 1) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_output_shape: empty output");
    return OTTER_HIP_OK;
}

int otter_hip_conv_default_out_layout(const otter_hip_conv_t* h) {
    if (!h) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_default_out_layout: null");
    const int K = h->d.out_channels;
    const bool dw8 = h->depthwise && K % 8 == 0;
    switch (h->d.out_kind) {
    case OTTER_HIP_OUT_I32:
        return dw8 ? OTTER_HIP_I32_P8 : (K % 4 == 0 ? OTTER_HIP_I32_P4 : OTTER_HIP_I32);
    case OTTER_HIP_OUT_F32:
        return dw8 ? OTTER_HIP_F32_P8 : (K % 4 == 0 ? OTTER_HIP_F32_P4 : OTTER_HIP_F32);
    default:
        return K % 8 == 0 ? OTTER_HIP_I8_P8 : OTTER_HIP_I8;
    }
}

size_t otter_hip_conv_workspace_bytes(const otter_hip_conv_t* h, int in_layout, int n, int in_h, int in_w) {
    if (!h || !valid_layout(in_layout)) return 0;
    if (h->c_pad) return (size_t)n * h->c_pad * in_h * in_w;  // the zero-padded Byte8 copy, fp32 or int8 input alike
    if (layout_elem(in_layout) != 0) return 0;
    return (size_t)n * h->d.in_channels * in_h * in_w;
}

// testing / tuning hook: force the MFMA tile shape of a handle (0,0 = automatic)
int otter_hip_conv_set_tile(otter_hip_conv_t* h, int tm, int tn) {
    if (!h) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_set_tile: null");
    h->force_tm = tm;
    h->force_tn = tn;
    return OTTER_HIP_OK;
}

static ConvGeom make_geom(const otter_hip_conv_desc& d, int n, int in_h, int in_w) {
    ConvGeom g;
    g.N = n, g.C = d.in_channels, g.H = in_h, g.W = in_w, g.K = d.out_channels;
    g.kh = d.kernel_h, g.kw = d.kernel_w, g.sh = d.stride_h, g.sw = d.stride_w, g.ph = d.pad_h, g.pw = d.pad_w;
    g.dh = d.dilation_h, g.dw = d.dilation_w, g.groups = d.groups;
    g.OH = conv_out_size(in_h, d.kernel_h, d.stride_h, d.pad_h, d.dilation_h);
    g.OW = conv_out_size(in_w, d.kernel_w, d.stride_w, d.pad_w, d.dilation_w);
    return g;
}

static Epilogue make_epilogue(const otter_hip_conv* h, int out_layout) {
    const otter_hip_conv_desc& d = h->d;
    Epilogue ep;
    ep.scale_in = h->scale_in, ep.bias = h->bias, ep.scale_out = h->scale_out;
    ep.act = d.activation_type, ep.act_p0 = d.activation_param0, ep.round_mode = d.out_round_mode;
    ep.out_kind = d.out_kind, ep.out_layout = out_layout;
    ep.act_lo = (d.activation_type == 1 || d.activation_type == 3) ? 0.f : -__builtin_inff();
    ep.act_hi = d.activation_type == 3 ? 6.f : __builtin_inff();
    ep.round_half = d.out_round_mode == OTTER_HIP_ROUND_SSE ? 0.5f : 0.49999997f;
    ep.so_positive = h->so_positive;
    ep.lrelu = d.activation_type == 2 && d.activation_param0 >= 0.f && d.activation_param0 <= 1.f;
    return ep;
}

// the few-channel 3x3 kernel takes the blob as the caller holds it (unpacked fp32 or int8): no quantize / pad pass
static bool use_stem(const otter_hip_conv* h, int in_layout, const ConvGeom& g_in, const Epilogue& ep) {
    return h->w_stem && h->force_tm == 0 && conv_stem_applicable(g_in, ep, in_layout);
}

// 0 direct, 1 MFMA implicit GEMM, 2 depthwise, 3 MFMA 3x3 with the halo in LDS, 4 few-channel 3x3 (image stem),
// 5 streamed 1x1 over few input channels, 6 pointwise layer straight from an fp32 blob (the blob read once)
// a depthwise 3x3 layer that reads an fp32 Float8 blob and can run quantize + convolution as one launch
static bool use_dw_f32in(const otter_hip_conv* h, int in_layout, const ConvGeom& g, int out_layout) {
    if (in_layout != OTTER_HIP_F32_P8 || !h->w_dw_mfma || h->c_pad || h->force_tm == -3 || h->force_tm == -6) return false;
    if (g.OH < 1 || g.OW < 1 || !dw_f32in_applicable(g, in_layout)) return false;
    const Epilogue ep = make_epilogue(h, out_layout);
    return dw_mfma_applicable(g, ep, dw_mfma_epilogue(ep, g.K), h->so_positive);
}

static int pick_kernel(const otter_hip_conv* h, int int8_layout, const ConvGeom& g, const Epilogue& ep) {
    if (int8_layout == OTTER_HIP_I8_P8) {
        if (h->w_dw) return 2;
        if (h->w_igemm && g.groups > 1) return igemm_grouped_applicable(g, ep) ? 1 : 0;  // else the scalar catch-all
        if (h->w_igemm) {
            if (h->force_tm > 0 || h->force_tm == -4) return 1;  // forced generic kernel (-4: with automatic tiles)
            if (conv_pw_stream_applicable(g, ep)) return 5;
            if (g.OH > 0 && g.OW > 0 && conv3x3_halo_supported(g, ep)) return 3;
            return 1;
        }
    }
    return 0;
}

// A pointwise layer on an fp32 Float8 blob whose quantize_to_int8 runs in the loader of the implicit-GEMM kernel (one
// launch, no int8 copy of the blob). Layers the streamed 1x1 kernel would take from an int8 blob go this way too from 64
// input channels on or up to 65536 pixels. Measured, quantize + streamed kernel against this launch, us with cold
// operands: 256 -> 512 @28x28 b32 20.9 / 20.0, 256 -> 64 @56x56 b16 19.8 / 15.2, 64 -> 384 @28x28 b64 16.4 / 15.7,
// 32 -> 192 @28x28 b64 11.2 / 10.2, 40 -> 240 @28x28 b32 11.0 / 8.3, but 32 -> 192 @56x56 b64 23.0 / 32.9 and
// 16 -> 96 @112x112 b64 35.3 / 72.0 (a 64-deep reduction step is mostly padding there, and the pixels are many).
// set_tile(-6, 0) keeps the two launches; set_tile(-4, 0) takes this launch for every layer it can run.
static bool use_igemm_f32in(const otter_hip_conv* h, int in_layout, const ConvGeom& g, const Epilogue& ep) {
    if (in_layout != OTTER_HIP_F32_P8 || !h->w_igemm || h->c_pad || (h->force_tm != 0 && h->force_tm != -4)) return false;
    if (g.OH < 1 || g.OW < 1 || !igemm_f32in_applicable(g, ep)) return false;
    const int kind = pick_kernel(h, OTTER_HIP_I8_P8, g, ep);
    return kind == 1 || (kind == 5 && (g.C >= 64 || (long)g.N * g.H * g.W <= 65536));
}

// The same layers with 64 .. 256 input channels and 128 output channels or more on the kernel that reads the fp32 blob
// once and walks all output channels per pixel group (conv_pw_f32in_kernel). Measured against the launch above, us with
// cold operands / the same buffers every time: 256 -> 512 @28x28 b32 fp32 out 21.7 / 17.0 against 24.6 / 20.0, int8 out
// 18.4 / 15.1 against 20.8 / 16.5; 64 -> 384 @28x28 b64 14.2 / 11.3 against 17.1 / 13.7; 128 -> 128 @28x28 b64 11.5 / 8.9
// against 12.8 / 9.1; with fewer output channels (256 -> 64 @56x56 b16, 96 -> 24 @56x56 b64) the two are level, and below
// 64 input channels the copy of the weights per workgroup costs more than the pixels it serves (16 -> 96 @112x112 b64:
// 50.7 against 38.4). set_tile(-7, groups | pairs << 3) takes this kernel for every layer it can run.
static bool use_pw_f32in(const otter_hip_conv* h, int in_layout, const ConvGeom& g, const Epilogue& ep) {
    if (in_layout != OTTER_HIP_F32_P8 || !h->w_igemm || h->c_pad || (h->force_tm != 0 && h->force_tm != -7)) return false;
    if (g.OH < 1 || g.OW < 1 || !conv_pw_f32in_applicable(g, ep)) return false;
    if (pick_epilogue(ep, g.K) == EPI_I8_P8_NONNEG && !h->clamp_hi) return false;
    return h->force_tm == -7 || (g.C >= 64 && g.K >= 128);
}

int otter_hip_conv_kernel_kind(const otter_hip_conv_t* h, int in_layout, int n, int in_h, int in_w, int out_layout) {
    if (!h || !valid_layout(in_layout)) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_kernel_kind: bad argument");
    int l = in_layout;
    ConvGeom g = make_geom(h->d, n, in_h, in_w);
    if (use_stem(h, in_layout, g, make_epilogue(h, out_layout))) return 4;
    if (use_pw_f32in(h, in_layout, g, make_epilogue(h, out_layout))) return 6;
    if (use_igemm_f32in(h, in_layout, g, make_epilogue(h, out_layout))) return 1;
    if (layout_elem(l) == 0) l = h->d.in_channels % 8 == 0 ? OTTER_HIP_I8_P8 : OTTER_HIP_I8;
    if (h->c_pad) l = OTTER_HIP_I8_P8, g.C = h->c_pad;
    return pick_kernel(h, l, g, make_epilogue(h, out_layout));
}

int otter_hip_conv3x3_halo_plan(int in_channels, int out_channels, int pad, int n, int in_h, int in_w, int force_fn,
                                int plan[8]) {
    if (!plan || in_channels < 1 || out_channels < 1 || pad < 0 || n < 1 || in_h < 1 || in_w < 1)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv3x3_halo_plan: bad argument");
    otter_hip_conv_desc d{};
    d.in_channels = in_channels, d.out_channels = out_channels, d.kernel_h = d.kernel_w = 3, d.stride_h = d.stride_w = 1;
    d.pad_h = d.pad_w = pad, d.dilation_h = d.dilation_w = 1, d.groups = 1;
    const ConvGeom g = make_geom(d, n, in_h, in_w);
    if (g.OH < 1 || g.OW < 1 || !conv3x3_halo_plan(g, force_fn, plan))
        return fail(OTTER_HIP_ERR_UNSUPPORTED, "otter_hip_conv3x3_halo_plan: the LDS-halo kernel does not take this shape");
    return OTTER_HIP_OK;
}

// the convolution; `twin` (or null) receives the Byte8 quantization of an fp32 result, from the convolution's own
// epilogue where that kernel can write it and from a quantize pass after it otherwise
// `residual` (or null): a blob in the output's layout added to the fp32 result; the twin is then made of the sum
static int conv_forward(const otter_hip_conv_t* h, const void* in, int in_layout, int n, int in_h, int in_w, void* out,
                        int out_layout, void* workspace, size_t workspace_bytes, void* stream_, int8_t* twin,
                        float twin_scale, int twin_round, const float* residual = nullptr) {
    if (!h || !in || !out) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward: null");
    if (!valid_layout(in_layout) || !valid_layout(out_layout))
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward: unknown layout");
    const otter_hip_conv_desc& d = h->d;
    hipStream_t stream = (hipStream_t)stream_;
    if (n < 0 || in_h < 1 || in_w < 1) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward: bad shape");
    if (layout_elem(in_layout) == 2) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward: int32 input");
    if (d.in_channels % layout_pack(in_layout))
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward: input pack does not divide C");
    const int want_elem = d.out_kind == OTTER_HIP_OUT_F32 ? 0 : (d.out_kind == OTTER_HIP_OUT_I8 ? 1 : 2);
    if (layout_elem(out_layout) != want_elem)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward: output layout does not match out_kind");
    if (d.out_channels % layout_pack(out_layout))
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward: output pack does not divide K");

    ConvGeom g = make_geom(d, n, in_h, in_w);
    if (g.OH < 1 || g.OW < 1) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward: empty output");
    if ((size_t)n * g.C * in_h * in_w >= (1ull << 31) || (size_t)n * g.K * g.OH * g.OW >= (1ull << 31))
        return fail(OTTER_HIP_ERR_UNSUPPORTED, "otter_hip_conv_forward: tensor exceeds 2^31 elements; split the batch");
    if (n == 0) return OTTER_HIP_OK;

    // the sum and the twin as a pass of their own, for the kernels that do not write them
    auto quantize_twin = [&]() -> int {
        float* o = (float*)out;
        if (residual && twin && layout_pack(out_layout) != 1)
            OHIP_CHECK(run_eltwise_add_quantize(o, residual, layout_pack(out_layout), o, twin, n, g.K, g.OH * g.OW, twin_scale,
                                                twin_round, stream));
        else {
            if (residual) OHIP_CHECK(run_eltwise_add(o, residual, o, (size_t)n * g.K * g.OH * g.OW, stream));
            if (twin)
                OHIP_CHECK(run_quantize_by(o, layout_pack(out_layout), twin, 8, n, g.K, g.OH * g.OW, twin_scale, twin_round,
                                           stream));
        }
        return OTTER_HIP_OK;
    };

    if (use_stem(h, in_layout, g, make_epilogue(h, out_layout))) {
        OHIP_CHECK(run_conv_stem(in, layout_elem(in_layout) == 0, h->w_stem, out, g, make_epilogue(h, out_layout), h->in_scale,
                                 d.in_round_mode, stream));
        return quantize_twin();
    }

    // A depthwise 3x3 layer on an fp32 Float8 blob: quantize_to_int8 and the convolution in one launch (no int8 copy of
    // the blob is written or read back). set_tile(-3, s) keeps the vector-ALU kernels, set_tile(-6, 0) the two launches.
    if (use_dw_f32in(h, in_layout, g, out_layout)) {
        const Epilogue ep = make_epilogue(h, out_layout);
        OHIP_CHECK(run_conv_dw_f32in((const float*)in, h->w_dw_mfma, out, g, ep, dw_mfma_epilogue(ep, g.K), h->in_scale,
                                     d.in_round_mode, h->force_tm == -2 ? h->force_tn : 0, stream));
        return quantize_twin();
    }

    // A pointwise layer on an fp32 Float8 blob: quantize_to_int8 inside the convolution's launch.
    {
        Epilogue ep = make_epilogue(h, out_layout);
        if (!twin && !residual && use_pw_f32in(h, in_layout, g, ep)) {
            OHIP_CHECK(run_conv_pw_f32in((const float*)in, h->w_igemm, h->clamp_hi, out, g, ep, h->in_scale, d.in_round_mode,
                                         h->force_tm == -7 ? (h->force_tn & 7) : 0, h->force_tm == -7 ? (h->force_tn >> 3) : 0, stream));
            return OTTER_HIP_OK;
        }
        if (use_igemm_f32in(h, in_layout, g, ep)) {
            if ((twin || residual) && (!twin || g.K % 8 == 0) && pick_epilogue(ep, g.K) == EPI_F32_P4) {
                ep.twin = twin, ep.twin_scale = twin_scale;
                ep.twin_half = twin_round == OTTER_HIP_ROUND_SSE ? 0.5f : 0.49999997f;
                ep.residual = residual;
                twin = nullptr, residual = nullptr;  // done by the convolution itself
            }
            OHIP_CHECK(run_conv_igemm_f32in((const float*)in, h->w_igemm, out, g, ep, h->in_scale, d.in_round_mode, stream));
            return quantize_twin();
        }
    }

    // (1) quantize_to_int8 when the blob is not int8 yet (Tensor/ConvolutionLayer.cpp:770-775)
    const int8_t* xq = (const int8_t*)in;
    int q_layout = in_layout;
    if (h->c_pad) {
        // (quantize and) zero-pad the channels into a Byte8 copy; the MFMA kernels then see C = c_pad
        const size_t need = (size_t)n * h->c_pad * in_h * in_w;
        if (!workspace || workspace_bytes < need)
            return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward: this layer needs the workspace reported by "
                                               "otter_hip_conv_workspace_bytes");
        OHIP_CHECK(run_pad_pack8(in, layout_elem(in_layout) == 0, layout_pack(in_layout), (int8_t*)workspace, n, g.C,
                                 h->c_pad, in_h * in_w, h->in_scale, d.in_round_mode, stream));
        xq = (const int8_t*)workspace;
        q_layout = OTTER_HIP_I8_P8;
        g.C = h->c_pad;
    } else if (layout_elem(in_layout) == 0) {
        const size_t need = (size_t)n * g.C * in_h * in_w;
        if (!workspace || workspace_bytes < need)
            return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward: fp32 input needs a workspace of N*C*H*W bytes");
        q_layout = g.C % 8 == 0 ? OTTER_HIP_I8_P8 : OTTER_HIP_I8;
        OHIP_CHECK(run_quantize((const float*)in, layout_pack(in_layout), (int8_t*)workspace, layout_pack(q_layout), n,
                                g.C, in_h * in_w, h->in_scale, 1, d.in_round_mode, stream));
        xq = (const int8_t*)workspace;
    }

    Epilogue ep = make_epilogue(h, out_layout);
    const int kind = pick_kernel(h, q_layout, g, ep);
    if ((twin || residual) && kind == 1 && g.groups == 1 && (!twin || g.K % 8 == 0) && pick_epilogue(ep, g.K) == EPI_F32_P4) {
        ep.twin = twin, ep.twin_scale = twin_scale;
        ep.twin_half = twin_round == OTTER_HIP_ROUND_SSE ? 0.5f : 0.49999997f;
        ep.residual = residual;
        twin = nullptr, residual = nullptr;  // done by the convolution itself
    }

    // (2)+(3)+(4) convolution with the fused epilogue
    switch (kind) {
    case 3:
        OHIP_CHECK(run_conv3x3_halo(xq, h->w_igemm, out, g, ep, h->force_tm < 0 ? h->force_tn : 0, stream));
        break;
    case 2: {
        // set_tile(-2, s): force the strip height; set_tile(-3, s): same, on the vector-ALU kernels
        const int dw_shift = (h->force_tm == -2 || h->force_tm == -3) ? h->force_tn : -1;
        const int epi = dw_mfma_epilogue(ep, g.K);
        const bool mfma = h->w_dw_mfma && h->force_tm != -3 && dw_mfma_applicable(g, ep, epi, h->so_positive);
        // the (image group, channel group) index rides on grid.y: run a very large batch in slices
        const int per = 32768 / (g.C / 8);
        if (per < 1) return fail(OTTER_HIP_ERR_UNSUPPORTED, "otter_hip_conv_forward: too many channels");
        for (int b = 0; b < n; b += per) {
            ConvGeom gs = g;
            gs.N = (n - b < per) ? n - b : per;
            const int8_t* xs = xq + (size_t)b * g.C * in_h * in_w;
            void* os = (char*)out + (size_t)b * g.K * g.OH * g.OW * layout_elem_bytes(out_layout);
            if (mfma) OHIP_CHECK(run_conv_dw_mfma(xs, h->w_dw_mfma, os, gs, ep, epi, dw_shift, stream));
            else OHIP_CHECK(run_conv_dw(xs, h->w_dw, os, gs, ep, dw_shift, stream));
        }
        break;
    }
    case 5:
        // set_tile(-5, groups | slices << 3): force the pixel groups per wave and the slices of the output channels
        OHIP_CHECK(run_conv_pw_stream(xq, h->w_igemm, h->clamp_hi, out, g, ep, h->force_tm == -5 ? (h->force_tn & 7) : 0,
                                      h->force_tm == -5 ? (h->force_tn >> 3) : 0, stream));
        break;
    case 1:
        OHIP_CHECK(run_conv_igemm(xq, h->w_igemm, out, g, ep, h->force_tm > 0 ? h->force_tm : 0,
                                  h->force_tm > 0 ? h->force_tn : 0, stream));
        break;
    default:
        OHIP_CHECK(run_conv_direct(xq, layout_pack(q_layout), h->w_raw, out, g, ep, stream));
        break;
    }
    return quantize_twin();
}

int otter_hip_conv_forward(const otter_hip_conv_t* h, const void* in, int in_layout, int n, int in_h, int in_w,
                           void* out, int out_layout, void* workspace, size_t workspace_bytes, void* stream) {
    return conv_forward(h, in, in_layout, n, in_h, in_w, out, out_layout, workspace, workspace_bytes, stream, nullptr, 0.f,
                        0);
}

int otter_hip_conv_forward_static(const otter_hip_conv_t* h, const void* in, int in_layout, int n, int in_h, int in_w,
                                  void* out, int out_layout, void* stream) {
    if (!h || !valid_layout(in_layout)) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward_static: bad argument");
    const size_t need = otter_hip_conv_workspace_bytes(h, in_layout, n < 0 ? 0 : n, in_h, in_w);
    if (need > (size_t)OTTER_HIP_STATIC_WORKSPACE_BYTES)
        return fail(OTTER_HIP_ERR_UNSUPPORTED,
                    "otter_hip_conv_forward_static: this input needs a workspace of " + std::to_string(need) +
                        " bytes, the static one holds " + std::to_string((size_t)OTTER_HIP_STATIC_WORKSPACE_BYTES) +
                        "; split the batch or use otter_hip_conv_forward with a workspace of your own");
    int rc = OTTER_HIP_OK;
    void* ws = need ? static_workspace(&rc) : nullptr;
    if (rc != OTTER_HIP_OK) return rc;
    return conv_forward(h, in, in_layout, n, in_h, in_w, out, out_layout, ws, need, stream, nullptr, 0.f, 0);
}

// ---- a chain of layers -------------------------------------------------------------------------------------------

static int chain_check(const otter_hip_conv_t* const* hs, int layers, int n, int in_h, int in_w, const char* who) {
    if (!hs || layers < 1) return fail(OTTER_HIP_ERR_INVALID, std::string(who) + ": no layers");
    for (int l = 0; l < layers; ++l) {
        if (!hs[l]) return fail(OTTER_HIP_ERR_INVALID, std::string(who) + ": null layer");
        const otter_hip_conv_desc& d = hs[l]->d;
        if (d.out_kind != OTTER_HIP_OUT_I8 || d.in_channels % 8 || d.out_channels % 8)
            return fail(OTTER_HIP_ERR_INVALID, std::string(who) + ": every layer must map Byte8 to Byte8 (int8 output, channels in octets)");
        if (l && d.in_channels != hs[l - 1]->d.out_channels)
            return fail(OTTER_HIP_ERR_INVALID, std::string(who) + ": channel counts of consecutive layers do not match");
    }
    if (n < 0 || in_h < 1 || in_w < 1) return fail(OTTER_HIP_ERR_INVALID, std::string(who) + ": bad shape");
    return OTTER_HIP_OK;
}

// the blob sizes along the chain: bytes of the output of layer l (Byte8) into out_bytes[l]; returns false on an empty blob
static bool chain_shapes(const otter_hip_conv_t* const* hs, int layers, int n, int h, int w, size_t* out_bytes, int* hh,
                         int* ww) {
    for (int l = 0; l < layers; ++l) {
        hh[l] = h, ww[l] = w;
        const otter_hip_conv_desc& d = hs[l]->d;
        h = conv_out_size(h, d.kernel_h, d.stride_h, d.pad_h, d.dilation_h);
        w = conv_out_size(w, d.kernel_w, d.stride_w, d.pad_w, d.dilation_w);
        if (h < 1 || w < 1) return false;
        out_bytes[l] = (size_t)n * d.out_channels * h * w;
    }
    return true;
}

static int g_chain_min_tiles = 96;  // see chain_single_launch

// true when the chain runs as one persistent launch (conv3x3_chain.hip): every layer the same 3x3 stride-1 pad-1
// geometry, same rounding and epilogue family
static bool chain_single_launch(const otter_hip_conv_t* const* handles, int n_layers, int n, int in_h, int in_w) {
    if (n_layers < 2 || n_layers > 8 || n < 1) return false;
    const otter_hip_conv_desc& d0 = handles[0]->d;
    for (int l = 0; l < n_layers; ++l) {
        const otter_hip_conv_desc& d = handles[l]->d;
        // (a forced fragment count of the LDS-halo kernel on the first layer, force_tm == -1, carries over to the chain)
        const bool tile_ok = handles[l]->force_tm == 0 || (l == 0 && handles[l]->force_tm == -1);
        const bool same = handles[l]->w_igemm && !handles[l]->c_pad && tile_ok && d.in_channels == d0.in_channels &&
                          d.out_channels == d0.out_channels && d.kernel_h == 3 && d.kernel_w == 3 && d.stride_h == 1 &&
                          d.stride_w == 1 && d.pad_h == 1 && d.pad_w == 1 && d.dilation_h == 1 && d.dilation_w == 1 &&
                          d.groups == 1 && d.out_round_mode == d0.out_round_mode && d.out_kind == OTTER_HIP_OUT_I8;
        if (!same) return false;
    }
    const ConvGeom g = make_geom(d0, n, in_h, in_w);
    const Epilogue ep0 = make_epilogue(handles[0], OTTER_HIP_I8_P8);
    for (int l = 1; l < n_layers; ++l)
        if (pick_epilogue(make_epilogue(handles[l], OTTER_HIP_I8_P8), g.K) != pick_epilogue(ep0, g.K)) return false;
    int plan[4];
    if (!(g.OH > 0 && g.OW > 0 && conv3x3_chain_applicable(g, ep0, n_layers, plan, handles[0]->force_tm == -1 ? handles[0]->force_tn : 0))) return false;
    // The single launch pays only where a tile's producers are far enough back in an XCD's list to be finished when
    // it is reached: 64 workgroups per XCD are in flight, and a layer's share of the list must be well above that
    // (measured: 112 tiles per XCD and layer, the 128-channel 56x56 batch-64 stack, gains 8 %; 56 or 32 tiles lose
    // 20-35 % against the layers one by one).
    const long per_xcd_and_layer = (long)((n + 7) / 8) * plan[2];
    return per_xcd_and_layer >= g_chain_min_tiles;
}

int otter_hip_conv_chain_set_min_tiles(int tiles) {
    const int before = g_chain_min_tiles;
    if (tiles >= 0) g_chain_min_tiles = tiles;
    return before;
}

static thread_local int t_chain_last_launches = 0;  // kernels the last otter_hip_conv_chain_forward of this thread enqueued

int otter_hip_conv_chain_launches(const otter_hip_conv_t* const* handles, int n_layers, int n, int in_h, int in_w) {
    int rc = chain_check(handles, n_layers, n, in_h, in_w, "otter_hip_conv_chain_launches");
    if (rc) return rc;
    return chain_single_launch(handles, n_layers, n, in_h, in_w) ? 1 : n_layers;
}

size_t otter_hip_conv_chain_workspace_bytes(const otter_hip_conv_t* const* handles, int n_layers, int n, int in_h, int in_w) {
    if (!handles || n_layers < 1 || n_layers > 64) return 0;
    for (int l = 0; l < n_layers; ++l)
        if (!handles[l]) return 0;
    std::vector<size_t> ob(n_layers);
    std::vector<int> hh(n_layers), ww(n_layers);
    if (!chain_shapes(handles, n_layers, n, in_h, in_w, ob.data(), hh.data(), ww.data())) return 0;
    size_t total = 0;
    for (int l = 0; l + 1 < n_layers; ++l) total += (ob[l] + 255) / 256 * 256;  // one buffer per intermediate blob
    return total;
}

int otter_hip_conv_chain_forward(const otter_hip_conv_t* const* handles, int n_layers, const void* in, int n, int in_h,
                                 int in_w, void* out, void* workspace, size_t workspace_bytes, void* stream_) {
    if (!in || !out) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_chain_forward: null");
    if (n_layers > 64) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_chain_forward: too many layers");
    int rc = chain_check(handles, n_layers, n, in_h, in_w, "otter_hip_conv_chain_forward");
    if (rc) return rc;
    std::vector<size_t> ob(n_layers);
    std::vector<int> hh(n_layers), ww(n_layers);
    if (!chain_shapes(handles, n_layers, n, in_h, in_w, ob.data(), hh.data(), ww.data()))
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_chain_forward: empty output");
    const size_t need = otter_hip_conv_chain_workspace_bytes(handles, n_layers, n, in_h, in_w);
    if (need && (!workspace || workspace_bytes < need))
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_chain_forward: needs the workspace reported by "
                                           "otter_hip_conv_chain_workspace_bytes");
    if (n == 0) return OTTER_HIP_OK;
    // the blobs: in, one workspace buffer per intermediate blob (each written once per call), out
    std::vector<const int8_t*> act(n_layers + 1);
    act[0] = (const int8_t*)in;
    size_t ofs = 0;
    for (int l = 0; l + 1 < n_layers; ++l) {
        act[l + 1] = (const int8_t*)workspace + ofs;
        ofs += (ob[l] + 255) / 256 * 256;
    }
    act[n_layers] = (const int8_t*)out;
    hipStream_t stream = (hipStream_t)stream_;

    // one launch for the whole chain where every layer is the same 3x3 "same" convolution geometry
    if (chain_single_launch(handles, n_layers, n, in_h, in_w)) {
        const ConvGeom g = make_geom(handles[0]->d, n, in_h, in_w);
        std::vector<Epilogue> eps(n_layers);
        std::vector<const int8_t*> wpk(n_layers);
        for (int l = 0; l < n_layers; ++l) {
            eps[l] = make_epilogue(handles[l], OTTER_HIP_I8_P8);
            wpk[l] = handles[l]->w_igemm;
        }
        const hipError_t ce = run_conv3x3_chain(g, eps.data(), wpk.data(), act.data(), n_layers, nullptr, stream,
                                                 handles[0]->force_tm == -1 ? handles[0]->force_tn : 0);
        if (ce == hipSuccess) {
            t_chain_last_launches = 1;
            return OTTER_HIP_OK;
        }
        if (ce != hipErrorNotReady) OHIP_CHECK(ce);
        // (every flag set of this GPU is busy on another stream: this stream takes the layers one by one)
    }
    // anything else: the layers one after the other, the same blobs
    for (int l = 0; l < n_layers; ++l) {
        rc = conv_forward(handles[l], act[l], OTTER_HIP_I8_P8, n, hh[l], ww[l], (void*)act[l + 1], OTTER_HIP_I8_P8, nullptr, 0,
                          stream_, nullptr, 0.f, 0);
        if (rc) return rc;
    }
    t_chain_last_launches = n_layers;
    return OTTER_HIP_OK;
}

int otter_hip_conv_chain_last_launches(void) { return t_chain_last_launches; }

int otter_hip_conv_chain_clock_mhz(float* mhz) {
    if (!mhz) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_chain_clock_mhz: null");
    OHIP_CHECK(conv3x3_chain_clock_mhz(mhz));  // (synchronizes with the device)
    return OTTER_HIP_OK;
}

int otter_hip_conv_chain_status(int* gave_up) {
    if (!gave_up) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_chain_status: null");
    OHIP_CHECK(conv3x3_chain_error(gave_up));  // (synchronizes with the device)
    return OTTER_HIP_OK;
}

int otter_hip_conv_forward_residual(const otter_hip_conv_t* h, const void* in, int in_layout, int n, int in_h, int in_w,
                                    const float* residual, void* out, int out_layout, void* out_q, float q_scale,
                                    int q_round_mode, void* workspace, size_t workspace_bytes, void* stream) {
    if (!h || !residual) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward_residual: null");
    if (h->d.out_kind != OTTER_HIP_OUT_F32)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward_residual: needs an fp32 output");
    if (out_q && h->d.out_channels % 8)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward_residual: the quantized sum needs K % 8 == 0");
    if (out_q && q_round_mode != OTTER_HIP_ROUND_SSE && q_round_mode != OTTER_HIP_ROUND_EXACT)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward_residual: unknown rounding mode");
    if (residual == out) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward_residual: out must not be the residual");
    return conv_forward(h, in, in_layout, n, in_h, in_w, out, out_layout, workspace, workspace_bytes, stream, (int8_t*)out_q,
                        q_scale, q_round_mode, residual);
}

int otter_hip_conv_forward_twin(const otter_hip_conv_t* h, const void* in, int in_layout, int n, int in_h, int in_w,
                                void* out, int out_layout, void* out_q, float q_scale, int q_round_mode, void* workspace,
                                size_t workspace_bytes, void* stream) {
    if (!h || !out_q) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward_twin: null");
    if (h->d.out_kind != OTTER_HIP_OUT_F32 || h->d.out_channels % 8)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward_twin: needs an fp32 output with K % 8 == 0");
    if (q_round_mode != OTTER_HIP_ROUND_SSE && q_round_mode != OTTER_HIP_ROUND_EXACT)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward_twin: unknown rounding mode");
    return conv_forward(h, in, in_layout, n, in_h, in_w, out, out_layout, workspace, workspace_bytes, stream, (int8_t*)out_q,
                        q_scale, q_round_mode);
}

// ---- an inverted-residual block ----------------------------------------------------------------------------------

static int block_check(const otter_hip_conv_t* e, const otter_hip_conv_t* d, const otter_hip_conv_t* p, int n, int in_h,
                       int in_w, const char* who) {
    if (!e || !d || !p) return fail(OTTER_HIP_ERR_INVALID, std::string(who) + ": null layer");
    if (e->d.out_kind != OTTER_HIP_OUT_I8 || d->d.out_kind != OTTER_HIP_OUT_I8 || p->d.out_kind == OTTER_HIP_OUT_I32)
        return fail(OTTER_HIP_ERR_INVALID, std::string(who) + ": the first two layers must write int8, the last int8 or fp32");
    if (e->d.in_channels % 8 || e->d.out_channels % 8 || d->d.out_channels % 8)
        return fail(OTTER_HIP_ERR_INVALID, std::string(who) + ": the blobs inside the block must be Byte8 (channels in octets)");
    if (e->d.out_channels != d->d.in_channels || d->d.out_channels != p->d.in_channels)
        return fail(OTTER_HIP_ERR_INVALID, std::string(who) + ": channel counts of consecutive layers do not match");
    if (n < 0 || in_h < 1 || in_w < 1) return fail(OTTER_HIP_ERR_INVALID, std::string(who) + ": bad shape");
    return OTTER_HIP_OK;
}

// geometry of the three layers on this input; false on an empty blob
static bool block_geoms(const otter_hip_conv_t* e, const otter_hip_conv_t* d, const otter_hip_conv_t* p, int n, int in_h,
                        int in_w, ConvGeom g[3]) {
    g[0] = make_geom(e->d, n, in_h, in_w);
    if (g[0].OH < 1 || g[0].OW < 1) return false;
    g[1] = make_geom(d->d, n, g[0].OH, g[0].OW);
    if (g[1].OH < 1 || g[1].OW < 1) return false;
    g[2] = make_geom(p->d, n, g[1].OH, g[1].OW);
    return g[2].OH >= 1 && g[2].OW >= 1;
}

static int g_block_always = 0;  // see block_single_launch

static bool block_single_launch(const otter_hip_conv_t* e, const otter_hip_conv_t* d, const otter_hip_conv_t* p,
                                const ConvGeom g[3], int out_layout, int plan[6]) {
    if (g_block_always == 2) return false;  // (tuning hook: never)
    if (!e->w_igemm || e->c_pad || e->force_tm || !e->blk_consts || !d->depthwise || !d->blk_consts || d->c_pad || d->force_tm || !p->w_igemm ||
        p->c_pad || p->force_tm)
        return false;
    const Epilogue e1 = make_epilogue(e, OTTER_HIP_I8_P8), e2 = make_epilogue(d, OTTER_HIP_I8_P8), e3 = make_epilogue(p, out_layout);
    if (!conv_block_applicable(g[0], e1, g[1], e2, g[2], e3)) return false;
    if (!conv_block_plan(g[0], g[2], e->block_rb, e->block_sl, e->block_split, plan)) return false;
    if (g_block_always == 1 || e->block_rb || e->block_sl || e->block_split) return true;
    // The single launch pays where the three layers are short, latency-bound launches and its workgroups (a band of
    // rows of one image each, or a share of a band's expanded channels) about fill the 256 compute units once.
    // Measured at batch 64 against the three launches (kernel trace; in brackets the three launches inside a network,
    // where each starts on cold inputs): 14x14 64 -> 384 -> 64 13.2 us against 17.8, 14x14 96 -> 576 -> 96 21.8 against
    // 23.5 (29.8), 28x28 32 -> 192 -> 32 15.2 against 21.8, 7x7 160 -> 960 -> 160 with the slices of an image dealt to
    // four workgroups 18.5 against 20 (23.4), 7x7 160 -> 960 -> 320 as two bands of 20 project tiles, each dealt to two
    // workgroups, 20.8 against 20.3 (24.4). Not taken: 56x56 24 -> 144 -> 24 (896 workgroups of 13 us each on 256
    // compute units) 53 against 45.
    const long wgs = (long)g[0].N * plan[1] * plan[4];
    const int items = ((g[2].K + 31) / 32) * ((plan[0] * g[0].W + 15) / 16);
    return g[0].C <= 192 && g[0].W <= 28 && wgs >= 128 && wgs <= 512 && items <= 24;
}

// The first two layers of a block as one launch (conv_xdw.hip), the last by itself: where the single launch of the
// whole block is not taken. 0: where it was measured faster than the two layers one by one; 1: wherever the kernel
// takes the shapes; -1: never.
static int g_block_pair = 0;

static bool block_pair_launch(const otter_hip_conv_t* e, const otter_hip_conv_t* d, const ConvGeom g[3]) {
    if (g_block_pair < 0 || !e->w_xdw || e->c_pad || e->force_tm || !d->w_dw_mfma || d->c_pad || d->force_tm) return false;
    const Epilogue e1 = make_epilogue(e, OTTER_HIP_I8_P8), e2 = make_epilogue(d, OTTER_HIP_I8_P8);
    if (!xdw_applicable(g[0], e1, pick_epilogue(e1, g[0].K), e->so_positive, g[1], e2, dw_mfma_epilogue(e2, g[1].K), d->so_positive))
        return false;
    if (g[0].C > 32 && g[0].W > 64) return false;  // (those instances of the kernel do not fit the register file)
    if (g_block_pair > 0) return true;
    // Measured at batch 64 against the two layers one by one (kernel trace): with a stride-2 depthwise layer, where the
    // expanded blob is four times what the launch writes, 16 -> 96 @112x112 29.5 us against 46, 24 -> 144 @56x56 17.9
    // against 27, 32 -> 192 @28x28 9.7 against 15, 96 -> 576 @14x14 13.2 against 15; with stride 1 24 -> 144 @56x56 28.6
    // against 31, and the 88 / 176-channel units of the detection model at 52x52 .. 13x13 (batch 16) no gain.
    return g[1].sh == 2 || (size_t)g[0].N * g[0].K * g[0].OH * g[0].OW >= ((size_t)16 << 20);
}

static int block_default_out_layout(const otter_hip_conv_t* p) {
    return p->d.out_kind == OTTER_HIP_OUT_F32 ? OTTER_HIP_F32_P4 : OTTER_HIP_I8_P8;
}

int otter_hip_conv_block_launches(const otter_hip_conv_t* e, const otter_hip_conv_t* d, const otter_hip_conv_t* p, int n,
                                  int in_h, int in_w) {
    int rc = block_check(e, d, p, n, in_h, in_w, "otter_hip_conv_block_launches");
    if (rc) return rc;
    ConvGeom g[3];
    if (!block_geoms(e, d, p, n, in_h, in_w, g)) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_block_launches: empty output");
    int plan[6];
    if (n >= 1 && p->d.out_channels % 8 == 0 && block_single_launch(e, d, p, g, block_default_out_layout(p), plan)) return 1;
    return n >= 1 && block_pair_launch(e, d, g) ? 2 : 3;
}

size_t otter_hip_conv_block_workspace_bytes(const otter_hip_conv_t* e, const otter_hip_conv_t* d, const otter_hip_conv_t* p,
                                            int n, int in_h, int in_w) {
    if (!e || !d || !p || n < 1 || in_h < 1 || in_w < 1) return 0;
    ConvGeom g[3];
    if (!block_geoms(e, d, p, n, in_h, in_w, g)) return 0;
    int plan[6];
    if (p->d.out_channels % 8 == 0 && block_single_launch(e, d, p, g, block_default_out_layout(p), plan))
        return (size_t)plan[5] * sizeof(int);  // the accumulators of a band's workgroups, when there are several
    const size_t b0 = (size_t)n * g[0].K * g[0].OH * g[0].OW, b1 = (size_t)n * g[1].K * g[1].OH * g[1].OW;
    return (b0 + 255) / 256 * 256 + (b1 + 255) / 256 * 256;
}

int otter_hip_conv_block_plan(int in_channels, int expanded_channels, int out_channels, int n, int in_h, int in_w,
                              int rows_per_band, int slice_channels, int split, int plan[6]) {
    if (!plan || in_channels < 8 || in_channels % 8 || expanded_channels < 8 || expanded_channels % 8 || out_channels < 8 ||
        out_channels % 8 || n < 1 || in_h < 1 || in_w < 1 || rows_per_band < 0 || split < 0 ||
        (slice_channels != 0 && slice_channels != 64 && slice_channels != 128))
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_block_plan: bad argument");
    otter_hip_conv_desc d{};
    d.kernel_h = d.kernel_w = 1, d.stride_h = d.stride_w = 1, d.dilation_h = d.dilation_w = 1, d.groups = 1;
    d.in_channels = in_channels, d.out_channels = expanded_channels;
    const ConvGeom ge = make_geom(d, n, in_h, in_w);
    d.in_channels = expanded_channels, d.out_channels = out_channels;
    const ConvGeom gp = make_geom(d, n, in_h, in_w);
    if (!conv_block_plan(ge, gp, rows_per_band, slice_channels, split, plan))
        return fail(OTTER_HIP_ERR_UNSUPPORTED, "otter_hip_conv_block_plan: the single launch does not take this shape");
    return OTTER_HIP_OK;
}

int otter_hip_conv_block_set_always(int on) {
    const int before = g_block_always;
    if (on >= 0) g_block_always = on > 2 ? 1 : on;
    return before;
}

int otter_hip_conv_block_set_pair(int mode) {
    const int before = g_block_pair;
    if (mode >= -1 && mode <= 1) g_block_pair = mode;
    return before;
}

int otter_hip_conv_block_set_plan(otter_hip_conv_t* e, int rows_per_band, int slice_channels, int split) {
    if (!e || rows_per_band < 0 || split < 0 || (slice_channels != 0 && slice_channels != 64 && slice_channels != 128))
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_block_set_plan: bad argument");
    e->block_rb = rows_per_band, e->block_sl = slice_channels, e->block_split = split;
    return OTTER_HIP_OK;
}

int otter_hip_conv_block_forward(const otter_hip_conv_t* e, const otter_hip_conv_t* d, const otter_hip_conv_t* p,
                                 const void* in, int n, int in_h, int in_w, const float* residual, void* out, int out_layout,
                                 void* out_q, float q_scale, int q_round_mode, void* workspace, size_t workspace_bytes,
                                 void* stream_) {
    if (!in || !out) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_block_forward: null");
    int rc = block_check(e, d, p, n, in_h, in_w, "otter_hip_conv_block_forward");
    if (rc) return rc;
    const bool f32 = p->d.out_kind == OTTER_HIP_OUT_F32;
    if (!valid_layout(out_layout) || layout_elem(out_layout) != (f32 ? 0 : 1) || p->d.out_channels % layout_pack(out_layout))
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_block_forward: output layout does not match the last layer");
    if ((residual || out_q) && !f32)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_block_forward: a shortcut sum or a quantized twin needs an fp32 result");
    if (out_q && p->d.out_channels % 8)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_block_forward: the quantized result needs K % 8 == 0");
    if (out_q && q_round_mode != OTTER_HIP_ROUND_SSE && q_round_mode != OTTER_HIP_ROUND_EXACT)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_block_forward: unknown rounding mode");
    if (residual == out) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_block_forward: out must not be the residual");
    ConvGeom g[3];
    if (!block_geoms(e, d, p, n, in_h, in_w, g)) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_block_forward: empty output");
    for (int l = 0; l < 3; ++l)
        if ((size_t)n * g[l].C * g[l].H * g[l].W >= (1ull << 31) || (size_t)n * g[l].K * g[l].OH * g[l].OW >= (1ull << 31))
            return fail(OTTER_HIP_ERR_UNSUPPORTED, "otter_hip_conv_block_forward: tensor exceeds 2^31 elements; split the batch");
    if (n == 0) return OTTER_HIP_OK;
    hipStream_t stream = (hipStream_t)stream_;

    int plan[6];
    if (p->d.out_channels % 8 == 0 && out_layout == block_default_out_layout(p) && block_single_launch(e, d, p, g, out_layout, plan)) {
        const size_t need1 = (size_t)plan[5] * sizeof(int);
        if (need1 && (!workspace || workspace_bytes < need1))
            return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_block_forward: needs the workspace reported by "
                                               "otter_hip_conv_block_workspace_bytes");
        const Epilogue e1 = make_epilogue(e, OTTER_HIP_I8_P8), e2 = make_epilogue(d, OTTER_HIP_I8_P8);
        Epilogue e3 = make_epilogue(p, out_layout);
        e3.residual = residual;
        e3.twin = (int8_t*)out_q, e3.twin_scale = q_scale;
        e3.twin_half = q_round_mode == OTTER_HIP_ROUND_SSE ? 0.5f : 0.49999997f;
        OHIP_CHECK(run_conv_block((const int8_t*)in, e->w_igemm, e->blk_consts, d->blk_consts, p->w_igemm, out, g[0], e1, g[1], e2, g[2], e3,
                                  e->block_rb, e->block_sl, e->block_split, (int*)workspace, stream));
        return OTTER_HIP_OK;
    }
    // the layers one after the other, the intermediate blobs in the workspace
    const size_t b0 = (size_t)n * g[0].K * g[0].OH * g[0].OW, b1 = (size_t)n * g[1].K * g[1].OH * g[1].OW;
    const size_t need = (b0 + 255) / 256 * 256 + (b1 + 255) / 256 * 256;
    if (!workspace || workspace_bytes < need)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_block_forward: needs the workspace reported by "
                                           "otter_hip_conv_block_workspace_bytes");
    void* t0 = workspace;
    void* t1 = (char*)workspace + (b0 + 255) / 256 * 256;
    if (block_pair_launch(e, d, g)) {
        // the pointwise layer and its depthwise reader in one launch: the expanded blob is not made
        const Epilogue e1 = make_epilogue(e, OTTER_HIP_I8_P8), e2 = make_epilogue(d, OTTER_HIP_I8_P8);
        OHIP_CHECK(run_conv_xdw((const int8_t*)in, e->w_xdw, d->w_dw_mfma, t1, g[0], e1, g[1], e2, dw_mfma_epilogue(e2, g[1].K),
                                e->block_rb, stream));
    } else {
        rc = conv_forward(e, in, OTTER_HIP_I8_P8, n, in_h, in_w, t0, OTTER_HIP_I8_P8, nullptr, 0, stream_, nullptr, 0.f, 0);
        if (rc) return rc;
        rc = conv_forward(d, t0, OTTER_HIP_I8_P8, n, g[1].H, g[1].W, t1, OTTER_HIP_I8_P8, nullptr, 0, stream_, nullptr, 0.f, 0);
        if (rc) return rc;
    }
    return conv_forward(p, t1, OTTER_HIP_I8_P8, n, g[2].H, g[2].W, out, out_layout, nullptr, 0, stream_, (int8_t*)out_q, q_scale,
                        q_round_mode, residual);
}

// -----------------------------------------------------------------------------------------------------
// standalone quantize / dequantize / requantize / repack
// -----------------------------------------------------------------------------------------------------

static int check_ew(const char* who, const void* src, const void* dst, int sl, int dl, int se, int de, int n, int c,
                    int h, int w) {
    if (!src || !dst) return fail(OTTER_HIP_ERR_INVALID, std::string(who) + ": null");
    if (!valid_layout(sl) || !valid_layout(dl) || layout_elem(sl) != se || layout_elem(dl) != de)
        return fail(OTTER_HIP_ERR_INVALID, std::string(who) + ": layout / element type mismatch");
    if (n < 0 || c < 1 || h < 1 || w < 1) return fail(OTTER_HIP_ERR_INVALID, std::string(who) + ": bad shape");
    if (c % layout_pack(sl) || c % layout_pack(dl))
        return fail(OTTER_HIP_ERR_INVALID, std::string(who) + ": pack does not divide C");
    if ((size_t)n * c * h * w >= (1ull << 31))
        return fail(OTTER_HIP_ERR_UNSUPPORTED, std::string(who) + ": tensor exceeds 2^31 elements");
    return OTTER_HIP_OK;
}

int otter_hip_quantize(const float* src, int src_layout, int n, int c, int h, int w, const float* scales, int n_scales,
                       int round_mode, int8_t* dst, int dst_layout, void* stream) {
    if (int rc = check_ew("otter_hip_quantize", src, dst, src_layout, dst_layout, 0, 1, n, c, h, w)) return rc;
    if (!scales || (n_scales != 1 && n_scales != c))
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_quantize: need 1 or C scales");
    OHIP_CHECK(run_quantize(src, layout_pack(src_layout), dst, layout_pack(dst_layout), n, c, h * w, scales, n_scales,
                            round_mode, (hipStream_t)stream));
    return OTTER_HIP_OK;
}

int otter_hip_dequantize(const int32_t* src, int src_layout, int n, int c, int h, int w, const float* scale,
                         int n_scale, const float* bias, int n_bias, float* dst, int dst_layout, void* stream) {
    if (int rc = check_ew("otter_hip_dequantize", src, dst, src_layout, dst_layout, 2, 0, n, c, h, w)) return rc;
    if (!scale || (n_scale != 1 && n_scale != c))
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_dequantize: need 1 or C scales");
    if (!bias) n_bias = 0;
    if (n_bias != 0 && n_bias != 1 && n_bias != c)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_dequantize: need 0, 1 or C biases");
    OHIP_CHECK(run_dequantize(src, layout_pack(src_layout), dst, layout_pack(dst_layout), n, c, h * w, scale, n_scale,
                              bias, n_bias, (hipStream_t)stream));
    return OTTER_HIP_OK;
}

int otter_hip_requantize(const int32_t* src, int src_layout, int n, int c, int h, int w, const float* scale_in,
                         int n_scale_in, const float* scale_out, int n_scale_out, const float* bias, int n_bias,
                         int activation_type, float activation_param0, int round_mode, int8_t* dst, int dst_layout,
                         void* stream) {
    if (int rc = check_ew("otter_hip_requantize", src, dst, src_layout, dst_layout, 2, 1, n, c, h, w)) return rc;
    if (!scale_in || (n_scale_in != 1 && n_scale_in != c) || !scale_out || (n_scale_out != 1 && n_scale_out != c))
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_requantize: need 1 or C scales");
    if (!bias) n_bias = 0;
    if (n_bias != 0 && n_bias != 1 && n_bias != c)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_requantize: need 0, 1 or C biases");
    if (activation_type < 0 || activation_type > 5)
        return fail(OTTER_HIP_ERR_UNSUPPORTED, "otter_hip_requantize: activation type not supported");
    OHIP_CHECK(run_requantize(src, layout_pack(src_layout), dst, layout_pack(dst_layout), n, c, h * w, scale_in,
                              n_scale_in, scale_out, n_scale_out, bias, n_bias, activation_type, activation_param0,
                              round_mode, (hipStream_t)stream));
    return OTTER_HIP_OK;
}

int otter_hip_repack(const void* src, int src_layout, int n, int c, int h, int w, void* dst, int dst_layout,
                     void* stream) {
    if (!valid_layout(src_layout)) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_repack: unknown layout");
    const int e = layout_elem(src_layout);
    if (int rc = check_ew("otter_hip_repack", src, dst, src_layout, dst_layout, e, e, n, c, h, w)) return rc;
    OHIP_CHECK(run_repack(src, layout_pack(src_layout), dst, layout_pack(dst_layout), layout_elem_bytes(src_layout), n,
                          c, h * w, (hipStream_t)stream));
    return OTTER_HIP_OK;
}

// -----------------------------------------------------------------------------------------------------
// fp32 glue between the int8 layers of a network
// -----------------------------------------------------------------------------------------------------

int otter_hip_eltwise_add(const float* a, const float* b, float* out, size_t count, void* stream) {
    if (!a || !b || !out) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_eltwise_add: null");
    OHIP_CHECK(run_eltwise_add(a, b, out, count, (hipStream_t)stream));
    return OTTER_HIP_OK;
}

int otter_hip_eltwise_add_quantize(const float* a, const float* b, int layout, int n, int c, int h, int w, float scale,
                                   int round_mode, float* out, int8_t* q, void* stream) {
    if (!a || !b || !out || !q) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_eltwise_add_quantize: null");
    if (layout != OTTER_HIP_F32_P4 && layout != OTTER_HIP_F32_P8)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_eltwise_add_quantize: Float4 or Float8 blobs expected");
    if (n < 0 || c < 8 || c % 8 || h < 1 || w < 1)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_eltwise_add_quantize: the channel count must be a multiple of 8");
    if ((size_t)n * c * h * w >= (1ull << 31))
        return fail(OTTER_HIP_ERR_UNSUPPORTED, "otter_hip_eltwise_add_quantize: tensor exceeds 2^31 elements");
    OHIP_CHECK(run_eltwise_add_quantize(a, b, layout_pack(layout), out, q, n, c, h * w, scale, round_mode, (hipStream_t)stream));
    return OTTER_HIP_OK;
}

int otter_hip_activation(float* x, size_t count, int activation_type, float activation_param0, void* stream) {
    if (!x) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_activation: null");
    if (activation_type < 0 || activation_type > 5)
        return fail(OTTER_HIP_ERR_UNSUPPORTED, "otter_hip_activation: activation type not supported");
    OHIP_CHECK(run_activation(x, count, activation_type, activation_param0, (hipStream_t)stream));
    return OTTER_HIP_OK;
}

int otter_hip_global_avgpool(const float* src, int src_layout, int n, int c, int h, int w, float* dst, void* stream) {
    if (!src || !dst) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_global_avgpool: null");
    if (!valid_layout(src_layout) || layout_elem(src_layout) != 0 || c % layout_pack(src_layout))
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_global_avgpool: bad layout");
    OHIP_CHECK(run_global_avgpool(src, layout_pack(src_layout), n, c, h * w, dst, (hipStream_t)stream));
    return OTTER_HIP_OK;
}

// ---- a convolution with an fp32 result and the global average pooling that is its only reader ----------------------

static bool conv_avgpool_one_launch(const otter_hip_conv_t* h, int in_layout, const ConvGeom& g) {
    if (in_layout != OTTER_HIP_I8_P8 || !h->w_igemm || h->c_pad || h->force_tm || h->d.out_kind != OTTER_HIP_OUT_F32) return false;
    return conv_pw_avgpool_applicable(g, make_epilogue(h, otter_hip_conv_default_out_layout(h)));
}

int otter_hip_conv_avgpool_launches(const otter_hip_conv_t* h, int in_layout, int n, int in_h, int in_w) {
    if (!h || !valid_layout(in_layout) || n < 0 || in_h < 1 || in_w < 1)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_avgpool_launches: bad argument");
    if (h->d.out_kind != OTTER_HIP_OUT_F32) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_avgpool_launches: the layer must have an fp32 result");
    const ConvGeom g = make_geom(h->d, n, in_h, in_w);
    if (g.OH < 1 || g.OW < 1) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_avgpool_launches: empty output");
    return conv_avgpool_one_launch(h, in_layout, g) ? 1 : 2;
}

size_t otter_hip_conv_avgpool_workspace_bytes(const otter_hip_conv_t* h, int in_layout, int n, int in_h, int in_w) {
    if (!h || !valid_layout(in_layout) || n < 1 || in_h < 1 || in_w < 1 || h->d.out_kind != OTTER_HIP_OUT_F32) return 0;
    const ConvGeom g = make_geom(h->d, n, in_h, in_w);
    if (g.OH < 1 || g.OW < 1 || conv_avgpool_one_launch(h, in_layout, g)) return 0;
    const size_t ws = otter_hip_conv_workspace_bytes(h, in_layout, n, in_h, in_w);
    return (ws + 255) / 256 * 256 + (size_t)n * g.K * g.OH * g.OW * sizeof(float);
}

int otter_hip_conv_forward_avgpool(const otter_hip_conv_t* h, const void* in, int in_layout, int n, int in_h, int in_w, float* out,
                                   void* workspace, size_t workspace_bytes, void* stream_) {
    if (!h || !in || !out) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward_avgpool: null");
    if (!valid_layout(in_layout) || n < 0 || in_h < 1 || in_w < 1)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward_avgpool: bad argument");
    if (h->d.out_kind != OTTER_HIP_OUT_F32)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward_avgpool: the layer must have an fp32 result");
    const ConvGeom g = make_geom(h->d, n, in_h, in_w);
    if (g.OH < 1 || g.OW < 1) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward_avgpool: empty output");
    if (n == 0) return OTTER_HIP_OK;
    if (conv_avgpool_one_launch(h, in_layout, g)) {
        const Epilogue ep = make_epilogue(h, otter_hip_conv_default_out_layout(h));
        OHIP_CHECK(run_conv_pw_avgpool((const int8_t*)in, h->w_igemm, out, g, ep, (hipStream_t)stream_));
        return OTTER_HIP_OK;
    }
    // the layer into the workspace, then the mean of that blob
    const size_t ws = (otter_hip_conv_workspace_bytes(h, in_layout, n, in_h, in_w) + 255) / 256 * 256;
    const size_t need = ws + (size_t)n * g.K * g.OH * g.OW * sizeof(float);
    if (!workspace || workspace_bytes < need)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_conv_forward_avgpool: needs the workspace reported by "
                                           "otter_hip_conv_avgpool_workspace_bytes");
    const int out_layout = otter_hip_conv_default_out_layout(h);
    float* blob = (float*)((char*)workspace + ws);
    int rc = conv_forward(h, in, in_layout, n, in_h, in_w, blob, out_layout, ws ? workspace : nullptr, ws, stream_, nullptr, 0.f, 0);
    if (rc) return rc;
    return otter_hip_global_avgpool(blob, out_layout, n, g.K, g.OH, g.OW, out, stream_);
}

int otter_hip_inner_product(const float* x, int n, int in_features, const float* weight, const float* bias,
                            int out_features, float* y, void* stream) {
    if (!x || !weight || !y) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_inner_product: null");
    OHIP_CHECK(run_inner_product(x, weight, bias, y, n, in_features, out_features, (hipStream_t)stream));
    return OTTER_HIP_OK;
}

// -----------------------------------------------------------------------------------------------------
// fp32 layout glue of the reference's int8 model files
// -----------------------------------------------------------------------------------------------------

static int check_f32_pair(const char* who, const void* src, const void* dst, int sl, int dl, int sc, int dc) {
    if (!src || !dst) return fail(OTTER_HIP_ERR_INVALID, std::string(who) + ": null");
    if (!valid_layout(sl) || !valid_layout(dl) || layout_elem(sl) != 0 || layout_elem(dl) != 0)
        return fail(OTTER_HIP_ERR_INVALID, std::string(who) + ": fp32 layouts expected");
    if (sc < 1 || dc < 1 || sc % layout_pack(sl) || dc % layout_pack(dl))
        return fail(OTTER_HIP_ERR_INVALID, std::string(who) + ": pack does not divide C");
    return OTTER_HIP_OK;
}

int otter_hip_copy_channels(const float* src, int src_layout, int src_c, int src_c0, float* dst, int dst_layout,
                            int dst_c, int dst_c0, int count, int n, int h, int w, void* stream) {
    if (int rc = check_f32_pair("otter_hip_copy_channels", src, dst, src_layout, dst_layout, src_c, dst_c)) return rc;
    if (n < 0 || h < 1 || w < 1 || count < 0 || src_c0 < 0 || dst_c0 < 0 || src_c0 + count > src_c || dst_c0 + count > dst_c)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_copy_channels: channel range outside the blob");
    if ((size_t)n * src_c * h * w >= (1ull << 31) || (size_t)n * dst_c * h * w >= (1ull << 31))
        return fail(OTTER_HIP_ERR_UNSUPPORTED, "otter_hip_copy_channels: tensor exceeds 2^31 elements");
    OHIP_CHECK(run_copy_channels(src, src_c, layout_pack(src_layout), src_c0, dst, dst_c, layout_pack(dst_layout), dst_c0,
                                 count, n, h, w, (hipStream_t)stream));
    return OTTER_HIP_OK;
}

int otter_hip_copy_channels_quantize(const float* src, int src_layout, int src_c, int src_c0, float* dst, int dst_layout,
                                     int dst_c, int dst_c0, int count, int n, int h, int w, int8_t* dst_q, float scale,
                                     int round_mode, void* stream) {
    if (int rc = check_f32_pair("otter_hip_copy_channels_quantize", src, dst, src_layout, dst_layout, src_c, dst_c)) return rc;
    if (!dst_q) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_copy_channels_quantize: null");
    if (n < 0 || h < 1 || w < 1 || count < 0 || src_c0 < 0 || dst_c0 < 0 || src_c0 + count > src_c || dst_c0 + count > dst_c)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_copy_channels_quantize: channel range outside the blob");
    if (round_mode != OTTER_HIP_ROUND_SSE && round_mode != OTTER_HIP_ROUND_EXACT)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_copy_channels_quantize: unknown rounding mode");
    if (dst_c % 8 || !copy_channels_moves_quads(layout_pack(src_layout), src_c0, layout_pack(dst_layout), dst_c0, count))
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_copy_channels_quantize: needs packed layouts on both sides, dst_c % 8 == 0, "
                                           "src_c0 % 4 == 0 and a destination range of whole packs");
    if ((size_t)n * src_c * h * w >= (1ull << 31) || (size_t)n * dst_c * h * w >= (1ull << 31))
        return fail(OTTER_HIP_ERR_UNSUPPORTED, "otter_hip_copy_channels_quantize: tensor exceeds 2^31 elements");
    OHIP_CHECK(run_copy_channels(src, src_c, layout_pack(src_layout), src_c0, dst, dst_c, layout_pack(dst_layout), dst_c0,
                                 count, n, h, w, (hipStream_t)stream, dst_q, scale, round_mode));
    return OTTER_HIP_OK;
}

int otter_hip_channel_shuffle(const float* src, int src_layout, float* dst, int dst_layout, int n, int c, int h, int w,
                              int groups, void* stream) {
    if (int rc = check_f32_pair("otter_hip_channel_shuffle", src, dst, src_layout, dst_layout, c, c)) return rc;
    if (n < 0 || h < 1 || w < 1 || groups < 1 || c % groups)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_channel_shuffle: groups must divide C");
    if ((size_t)n * c * h * w >= (1ull << 31))
        return fail(OTTER_HIP_ERR_UNSUPPORTED, "otter_hip_channel_shuffle: tensor exceeds 2^31 elements");
    OHIP_CHECK(run_channel_shuffle(src, layout_pack(src_layout), dst, layout_pack(dst_layout), n, c, h, w, groups,
                                   (hipStream_t)stream));
    return OTTER_HIP_OK;
}

int otter_hip_concat_channels(const float* const* srcs, const int* src_layouts, const int* src_channels, int count,
                              float* dst, int dst_layout, int n, int h, int w, int8_t* dst_q, float scale, int round_mode,
                              void* stream) {
    if (!srcs || !src_layouts || !src_channels || !dst) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_concat_channels: null");
    if (count < 1 || count > CONCAT_MAX)
        return fail(OTTER_HIP_ERR_UNSUPPORTED, "otter_hip_concat_channels: 1 to 8 sources (use otter_hip_copy_channels for more)");
    if (n < 0 || h < 1 || w < 1) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_concat_channels: bad shape");
    if (!valid_layout(dst_layout) || layout_elem(dst_layout) != 0 || layout_pack(dst_layout) % 4)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_concat_channels: F32_P4 or F32_P8 destination expected");
    ConcatSources cs;
    int total = 0;
    for (int i = 0; i < count; ++i) {
        if (!srcs[i] || !valid_layout(src_layouts[i]) || layout_elem(src_layouts[i]) != 0 || layout_pack(src_layouts[i]) % 4 ||
            src_channels[i] < 1 || src_channels[i] % layout_pack(src_layouts[i]))
            return fail(OTTER_HIP_ERR_INVALID, "otter_hip_concat_channels: packed fp32 sources with whole packs expected");
        cs.ptr[i] = srcs[i], cs.channels[i] = src_channels[i], cs.pack[i] = layout_pack(src_layouts[i]), cs.first[i] = total;
        total += src_channels[i];
    }
    for (int i = count; i < CONCAT_MAX; ++i) cs.ptr[i] = nullptr, cs.channels[i] = 0, cs.pack[i] = 4, cs.first[i] = 0x7fffffff;
    cs.count = count;
    if (total % layout_pack(dst_layout))
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_concat_channels: the destination pack does not divide the channel sum");
    if (dst_q && total % 8) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_concat_channels: the quantized blob needs C % 8 == 0");
    if (dst_q && round_mode != OTTER_HIP_ROUND_SSE && round_mode != OTTER_HIP_ROUND_EXACT)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_concat_channels: unknown rounding mode");
    if ((size_t)n * total * h * w >= (1ull << 31))
        return fail(OTTER_HIP_ERR_UNSUPPORTED, "otter_hip_concat_channels: tensor exceeds 2^31 elements");
    OHIP_CHECK(run_concat_channels(cs, dst, total, layout_pack(dst_layout), n, h, w, dst_q, scale, round_mode,
                                   (hipStream_t)stream));
    return OTTER_HIP_OK;
}

int otter_hip_channel_shuffle_quantize(const float* src, int src_layout, float* dst, int dst_layout, int n, int c, int h,
                                       int w, int groups, int8_t* dst_q, float scale, int round_mode, void* stream) {
    if (int rc = check_f32_pair("otter_hip_channel_shuffle_quantize", src, dst, src_layout, dst_layout, c, c)) return rc;
    if (!dst_q) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_channel_shuffle_quantize: null");
    if (n < 0 || h < 1 || w < 1) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_channel_shuffle_quantize: bad shape");
    if (round_mode != OTTER_HIP_ROUND_SSE && round_mode != OTTER_HIP_ROUND_EXACT)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_channel_shuffle_quantize: unknown rounding mode");
    if (!channel_shuffle_can_quantize(layout_pack(src_layout), layout_pack(dst_layout), c, groups))
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_channel_shuffle_quantize: needs 2 groups, F32_P8 on both sides, C % 16 == 0");
    if ((size_t)n * c * h * w >= (1ull << 31))
        return fail(OTTER_HIP_ERR_UNSUPPORTED, "otter_hip_channel_shuffle_quantize: tensor exceeds 2^31 elements");
    OHIP_CHECK(run_channel_shuffle(src, 8, dst, 8, n, c, h, w, groups, (hipStream_t)stream, dst_q, scale, round_mode));
    return OTTER_HIP_OK;
}

int otter_hip_shuffle2_split(const float* a, int a_layout, const float* b, int b_layout, int n, int channels_each, int h,
                             int w, float* first_half, float* second_half, int8_t* second_half_q, float scale,
                             int round_mode, void* stream) {
    if (!a || !b || !first_half || !second_half) return fail(OTTER_HIP_ERR_INVALID, "otter_hip_shuffle2_split: null");
    if ((a_layout != OTTER_HIP_F32_P4 && a_layout != OTTER_HIP_F32_P8) || (b_layout != OTTER_HIP_F32_P4 && b_layout != OTTER_HIP_F32_P8))
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_shuffle2_split: Float4 or Float8 inputs expected");
    if (n < 0 || channels_each < 8 || channels_each % 8 || h < 1 || w < 1)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_shuffle2_split: each input needs a multiple of 8 channels");
    if ((size_t)n * channels_each * 2 * h * w >= (1ull << 31))
        return fail(OTTER_HIP_ERR_UNSUPPORTED, "otter_hip_shuffle2_split: tensor exceeds 2^31 elements");
    OHIP_CHECK(run_shuffle2_split(a, layout_pack(a_layout), b, layout_pack(b_layout), first_half, second_half, second_half_q,
                                  scale, round_mode, n, channels_each, h * w, (hipStream_t)stream));
    return OTTER_HIP_OK;
}

int otter_hip_maxpool2d(const float* src, int src_layout, int n, int c, int h, int w, int kernel_h, int kernel_w,
                        int stride_h, int stride_w, int pad_h, int pad_w, int dilation_h, int dilation_w, int out_h,
                        int out_w, float pad_value, float* dst, int dst_layout, void* stream) {
    if (int rc = check_f32_pair("otter_hip_maxpool2d", src, dst, src_layout, dst_layout, c, c)) return rc;
    if (n < 0 || h < 1 || w < 1 || kernel_h < 1 || kernel_w < 1 || stride_h < 1 || stride_w < 1 || pad_h < 0 || pad_w < 0 ||
        dilation_h < 1 || dilation_w < 1 || out_h < 1 || out_w < 1)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_maxpool2d: bad geometry");
    // every window must start inside the padded input (what the reference's shape rule guarantees)
    if ((out_h - 1) * stride_h >= h + pad_h || (out_w - 1) * stride_w >= w + pad_w)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_maxpool2d: output larger than the pooling geometry allows");
    if ((size_t)n * c * h * w >= (1ull << 31) || (size_t)n * c * out_h * out_w >= (1ull << 31))
        return fail(OTTER_HIP_ERR_UNSUPPORTED, "otter_hip_maxpool2d: tensor exceeds 2^31 elements");
    OHIP_CHECK(run_maxpool(src, layout_pack(src_layout), dst, layout_pack(dst_layout), n, c, h, w, out_h, out_w, kernel_h,
                           kernel_w, stride_h, stride_w, pad_h, pad_w, dilation_h, dilation_w, pad_value, (hipStream_t)stream));
    return OTTER_HIP_OK;
}

int otter_hip_upsample2d(const float* src, int src_layout, int n, int c, int h, int w, int out_h, int out_w, int mode,
                         int align_corner, float* dst, int dst_layout, void* stream) {
    if (int rc = check_f32_pair("otter_hip_upsample2d", src, dst, src_layout, dst_layout, c, c)) return rc;
    if (n < 0 || h < 1 || w < 1 || out_h < 1 || out_w < 1)
        return fail(OTTER_HIP_ERR_INVALID, "otter_hip_upsample2d: bad shape");
    if (mode != 1 && mode != 2) return fail(OTTER_HIP_ERR_UNSUPPORTED, "otter_hip_upsample2d: mode must be 1 or 2");
    if (mode == 2 && (h < 2 || w < 2))
        return fail(OTTER_HIP_ERR_UNSUPPORTED, "otter_hip_upsample2d: bilinear needs at least 2x2 input");
    if ((size_t)n * c * h * w >= (1ull << 31) || (size_t)n * c * out_h * out_w >= (1ull << 31))
        return fail(OTTER_HIP_ERR_UNSUPPORTED, "otter_hip_upsample2d: tensor exceeds 2^31 elements");
    OHIP_CHECK(run_upsample(src, layout_pack(src_layout), dst, layout_pack(dst_layout), n, c, h, w, out_h, out_w, mode,
                            align_corner ? 1 : 0, (hipStream_t)stream));
    return OTTER_HIP_OK;
}

}  // extern "C"
