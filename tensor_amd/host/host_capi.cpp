// extern "C" facade over the C++ host layer, for hosts that cannot include otter_hip.hpp (the python tests and the
// benchmark drive the Net through it). Options are "key=value;key=value" strings with the reference's own keys.
#include <chrono>
#include <cstring>
#include <string>

#include "../../include/otter_hip_int8.h"
#include "otter_file.hpp"
#include "otter_hip.hpp"

using namespace otter;

namespace {
thread_local std::string g_err;
int fail(const std::string& s) {
    g_err = s;
    return -1;
}
LayerOption parse_options(const char* opts) {
    LayerOption lo;
    std::string s(opts ? opts : "");
    size_t pos = 0;
    while (pos < s.size()) {
        size_t e = s.find(';', pos);
        if (e == std::string::npos) e = s.size();
        const std::string kv = s.substr(pos, e - pos);
        const size_t eq = kv.find('=');
        if (eq != std::string::npos) lo[kv.substr(0, eq)] = kv.substr(eq + 1);
        pos = e + 1;
    }
    return lo;
}
Tensor f32_vec(const float* p, int n) { return Tensor::from_blob(p, {n}, ScalarType::Float); }
}  // namespace

extern "C" {

const char* otter_host_last_error(void) { return g_err.c_str(); }

void* otter_host_net_create(int use_packing_layout, int lightmode) {
    try {
        if (otter_hip_init(0)) {
            g_err = otter_hip_last_error();
            return nullptr;
        }
        Net* n = new Net();
        n->option.use_packing_layout = use_packing_layout != 0;
        n->option.lightmode = lightmode != 0;
        return n;
    } catch (const std::exception& e) {
        g_err = e.what();
        return nullptr;
    }
}

void otter_host_net_destroy(void* net) { delete static_cast<Net*>(net); }

int otter_host_net_add_layer(void* net, const char* options) {
    try {
        static_cast<Net*>(net)->addLayer(parse_options(options));
        return 0;
    } catch (const std::exception& e) {
        return fail(e.what());
    }
}

// initial != 0: CompileMode::Initial (random model + pipelines); else the weights are injected afterwards
int otter_host_net_compile(void* net, int initial) {
    try {
        static_cast<Net*>(net)->compile(initial ? CompileMode::Initial : CompileMode::Inference);
        return 0;
    } catch (const std::exception& e) {
        return fail(e.what());
    }
}

// fills the public members of a ConvolutionLayer exactly as load_model would (Tensor/ConvolutionLayer.cpp:245-296:
// depthwise layers get their blob scales replicated per group) and builds its pipeline
int otter_host_net_set_conv(void* net, const char* layer_name, const int8_t* weight, const float* bias,
                            const float* weight_scales, int n_weight_scales, float in_scale, float top_scale) {
    try {
        Net* n = static_cast<Net*>(net);
        auto* L = dynamic_cast<ConvolutionLayer*>(n->layer_by_name(layer_name));
        if (!L) return fail(std::string("no Convolution layer named ") + layer_name);
        const int K = L->out_channels, C = L->in_channels, g = L->groups;
        L->weight_data = Tensor::from_blob(weight, {K, C / g, L->kernel_height, L->kernel_width}, ScalarType::Byte);
        if (L->bias_term && bias) L->bias_data = f32_vec(bias, K);
        std::vector<float> ws(K);
        for (int i = 0; i < K; ++i) ws[i] = n_weight_scales == 1 ? weight_scales[0] : weight_scales[i];
        L->weight_data_int8_scales = f32_vec(ws.data(), K);
        const bool dw = C == g && g == K;
        std::vector<float> bs(dw ? g : 1, in_scale), ts(dw ? g : 1, top_scale);
        L->bottom_blob_int8_scales = f32_vec(bs.data(), (int)bs.size());
        if (L->int8_scale_term > 100) L->top_blob_int8_scales = f32_vec(ts.data(), (int)ts.size());
        const int rc = L->create_pipeline(n->option);
        if (rc) return fail(std::string("create_pipeline: ") + otter_hip_last_error());
        n->invalidate_plan();
        return 0;
    } catch (const std::exception& e) {
        return fail(e.what());
    }
}

// Calibration aid: while `on`, an int8-output convolution (int8_scale_term > 100) runs as its fp32-output twin
// (int8_scale_term - 100: same weights and input scale, dequantize + activation instead of requantize), so that a
// calibrator can look at the values its output scale has to cover. `on` = 0 restores the layer.
int otter_host_net_conv_fp32_probe(void* net, const char* layer_name, int on) {
    try {
        Net* n = static_cast<Net*>(net);
        auto* L = dynamic_cast<ConvolutionLayer*>(n->layer_by_name(layer_name));
        if (!L) return fail(std::string("no Convolution layer named ") + layer_name);
        if (on && L->int8_scale_term > 100) L->int8_scale_term -= 100;
        else if (!on && L->int8_scale_term > 0 && L->int8_scale_term < 100 && L->top_blob_int8_scales.defined()) L->int8_scale_term += 100;
        else return 0;
        const int rc = L->create_pipeline(n->option);
        if (rc) return fail(std::string("create_pipeline: ") + otter_hip_last_error());
        return 0;
    } catch (const std::exception& e) {
        return fail(e.what());
    }
}

int otter_host_net_get_scale_in(void* net, const char* layer_name, float* out) {
    auto* L = dynamic_cast<ConvolutionLayer*>(static_cast<Net*>(net)->layer_by_name(layer_name));
    if (!L || !L->scale_in_data.defined()) return fail("no such layer / pipeline not built");
    std::memcpy(out, L->scale_in_data.data_ptr<float>(), sizeof(float) * L->out_channels);
    return 0;
}

int otter_host_net_set_inner_product(void* net, const char* layer_name, const float* weight, const float* bias) {
    try {
        auto* L = dynamic_cast<InnerProductLayer*>(static_cast<Net*>(net)->layer_by_name(layer_name));
        if (!L) return fail(std::string("no InnerProduct layer named ") + layer_name);
        L->weight_data = Tensor::from_blob(weight, {L->out_features, L->in_features}, ScalarType::Float);
        if (L->bias_term && bias) L->bias_data = f32_vec(bias, L->out_features);
        return 0;
    } catch (const std::exception& e) {
        return fail(e.what());
    }
}

// One pass: input NCHW (fp32 or int8) on the host -> extract(out_name, type 0) -> unpacked host result.
// out_dtype: 0 fp32, 1 int8, 2 int32. repeat > 1 re-runs the pass with the input resident on the device and returns
// the mean seconds per pass in *seconds (device-synchronised around the timed region).
int otter_host_net_run(void* net, const char* in_name, const void* x, int x_is_int8, int n, int c, int h, int w,
                       const char* out_name, void* out, size_t out_capacity_bytes, int* out_dtype, int64_t* out_shape4,
                       int repeat, double* seconds) {
    try {
        Net* N = static_cast<Net*>(net);
        Tensor in = Tensor::from_blob(x, {n, c, h, w}, x_is_int8 ? ScalarType::Byte : ScalarType::Float);
        in.device_ptr();  // resident before the timed region
        Tensor feat;
        auto pass = [&]() -> int {
            Extractor ex = N->create_extractor();
            if (ex.input(in_name, in)) return -1;
            return ex.extract(out_name, feat, 1);
        };
        int rc = pass();
        if (rc) return fail("forward failed with code " + std::to_string(rc) + ": " + otter_hip_last_error());
        if (repeat > 1) {
            otter_hip_stream_synchronize(nullptr);
            const auto t0 = std::chrono::steady_clock::now();
            for (int i = 0; i < repeat; ++i)
                if ((rc = pass())) return fail("forward failed with code " + std::to_string(rc));
            otter_hip_stream_synchronize(nullptr);
            if (seconds) *seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() / repeat;
        }
        if (feat.dim() == 4 && feat.elempack() != 1) feat = feat.packing(1);
        const ScalarType b = base_of(feat.scalar_type());
        if (out_dtype) *out_dtype = b == ScalarType::Float ? 0 : (b == ScalarType::Byte ? 1 : 2);
        if (out_shape4)
            for (int i = 0; i < 4; ++i) out_shape4[i] = i < feat.dim() ? feat.size(i) : 1;
        if (out) {
            if (feat.nbytes() > out_capacity_bytes) return fail("output buffer too small");
            std::memcpy(out, feat.data_ptr(), feat.nbytes());
        }
        return 0;
    } catch (const std::exception& e) {
        return fail(e.what());
    }
}

// A session keeps the input resident on the device and runs passes without synchronising, so that a caller can time
// a stream of passes with its own events. out_name may list several blobs separated by commas (the heads of a
// detection network): a pass extracts every one of them from the same Extractor, the fetch returns the last.
struct otter_host_session {
    Net* net;
    std::string in_name, out_name;
    Tensor in, out;
};

void* otter_host_session_create(void* net, const char* in_name, const void* x, int x_is_int8, int n, int c, int h, int w,
                                const char* out_name) {
    try {
        auto* s = new otter_host_session();
        s->net = static_cast<Net*>(net);
        s->in_name = in_name;
        s->out_name = out_name;
        s->in = Tensor::from_blob(x, {n, c, h, w}, x_is_int8 ? ScalarType::Byte : ScalarType::Float);
        s->in.device_ptr();
        return s;
    } catch (const std::exception& e) {
        g_err = e.what();
        return nullptr;
    }
}

int otter_host_session_pass(void* session) {
    try {
        auto* s = static_cast<otter_host_session*>(session);
        Extractor ex = s->net->create_extractor();
        if (ex.input(s->in_name, s->in)) return fail("no such input blob");
        size_t pos = 0;
        while (pos <= s->out_name.size()) {
            size_t e = s->out_name.find(',', pos);
            if (e == std::string::npos) e = s->out_name.size();
            const int rc = ex.extract(s->out_name.substr(pos, e - pos), s->out, 1);
            if (rc) return fail("forward failed with code " + std::to_string(rc) + ": " + otter_hip_last_error());
            pos = e + 1;
        }
        return 0;
    } catch (const std::exception& e) {
        return fail(e.what());
    }
}

// copies the last pass's result (unpacked) to the host; returns the number of bytes, or -1
long otter_host_session_fetch(void* session, void* out, size_t capacity) {
    try {
        auto* s = static_cast<otter_host_session*>(session);
        if (!s->out.defined()) return fail("no pass has run");
        Tensor f = (s->out.dim() == 4 && s->out.elempack() != 1) ? s->out.packing(1) : s->out;
        if (f.nbytes() > capacity) return fail("output buffer too small");
        std::memcpy(out, f.data_ptr(), f.nbytes());
        return (long)f.nbytes();
    } catch (const std::exception& e) {
        return fail(e.what());
    }
}

void otter_host_session_destroy(void* session) { delete static_cast<otter_host_session*>(session); }

// function-level mirror checks: quantize_to_int8 -> convolution -> requantize / dequantize on packed host tensors
int otter_host_functional_chain(const float* x, int n, int c, int h, int w, float in_scale, const int8_t* weight, int k,
                                int kh, int kw, int stride, int pad, int groups, const float* scale_in, const float* bias,
                                int int8_out, float top_scale, int act, int32_t* acc_out, void* out) {
    try {
        if (otter_hip_init(0)) return fail(otter_hip_last_error());
        Tensor xin = Tensor::from_blob(x, {n, c, h, w}, ScalarType::Float);
        if (c % 8 == 0) xin = xin.packing(8);
        else if (c % 4 == 0) xin = xin.packing(4);
        Tensor xq = quantize_to_int8(xin, f32_vec(&in_scale, 1), true);
        Tensor wt = Tensor::from_blob(weight, {k, c / groups, kh, kw}, ScalarType::Byte);
        Tensor acc = convolution(xq, wt, Tensor(), Tensor(), {stride, stride}, {pad, pad}, {1, 1}, false, {0, 0}, groups, true);
        Tensor si = f32_vec(scale_in, k), bi = bias ? f32_vec(bias, k) : Tensor();
        Tensor y = int8_out ? requantize_from_int32_to_int8(acc, si, f32_vec(&top_scale, 1), bi, act, Tensor(), true)
                            : dequantize_from_int32(acc, si, bi, true);
        Tensor a1 = acc.elempack() != 1 ? acc.packing(1) : acc;
        if (acc_out) std::memcpy(acc_out, a1.data_ptr(), a1.nbytes());
        Tensor y1 = y.elempack() != 1 ? y.packing(1) : y;
        std::memcpy(out, y1.data_ptr(), y1.nbytes());
        return 0;
    } catch (const std::exception& e) {
        return fail(e.what());
    }
}

// ---------------------------------------------------------------------------------------------------
// model files
// ---------------------------------------------------------------------------------------------------

// Net::load_otter (Tensor/Net.cpp:518-536)
int otter_host_net_load_otter(void* net, const char* path, int initial) {
    try {
        if (static_cast<Net*>(net)->load_otter(path, initial ? CompileMode::Initial : CompileMode::Inference))
            return fail(std::string("cannot read ") + path);
        return 0;
    } catch (const std::exception& e) {
        return fail(e.what());
    }
}

// Net::load_weight (Tensor/Net.cpp:538-586); ncnn != 0: ncnn `.bin`, else Otter's fp32 stream
int otter_host_net_load_weight(void* net, const char* path, int ncnn) {
    try {
        const int rc = static_cast<Net*>(net)->load_weight(path, ncnn ? Net::WeightType::Ncnn : Net::WeightType::Otter);
        return rc ? fail("load_weight returned " + std::to_string(rc) + ": " + otter_hip_last_error()) : 0;
    } catch (const std::exception& e) {
        return fail(e.what());
    }
}

// One line per layer, "type name bottoms tops N C H W" (the logical shape of its first top blob) and for a convolution
// its weights as load_model will ask for them: "... K C groups kh kw bias_term int8_scale_term".
// how many runs of convolution layers went through the chain entry point as one launch, in this process
long otter_host_chain_forward_count(void) { return ConvolutionLayer::chain_forward_count(); }
long otter_host_block_forward_count(void) { return ConvolutionLayer::block_forward_count(); }

long otter_host_net_describe(void* net, char* buf, size_t capacity) {
    try {
        const std::string out = static_cast<Net*>(net)->describe();
        if (out.size() + 1 > capacity) return fail("description larger than the buffer");
        std::memcpy(buf, out.c_str(), out.size() + 1);
        return (long)out.size();
    } catch (const std::exception& e) {
        return fail(e.what());
    }
}

// One pass with any number of blobs set beforehand (Extractor::input on each), e.g. a layer's bottoms when a test
// drives a single layer: inputs are NCHW fp32 / int8 on the host, shapes4 holds 4 entries per input.
int otter_host_net_eval(void* net, int n_inputs, const char* const* in_names, const void* const* in_ptrs,
                        const int* in_is_int8, const int64_t* shapes4, const char* out_name, void* out,
                        size_t out_capacity_bytes, int* out_dtype, int64_t* out_shape4) {
    try {
        Net* N = static_cast<Net*>(net);
        Extractor ex = N->create_extractor();
        ex.set_lightmode(false);
        for (int i = 0; i < n_inputs; ++i) {
            const int64_t* s = shapes4 + 4 * i;
            Tensor in = Tensor::from_blob(in_ptrs[i], {s[0], s[1], s[2], s[3]}, in_is_int8[i] ? ScalarType::Byte : ScalarType::Float);
            if (ex.input(in_names[i], in)) return fail(std::string("unknown blob ") + in_names[i]);
        }
        Tensor feat;
        const int rc = ex.extract(out_name, feat, 0);
        if (rc) return fail("forward failed with code " + std::to_string(rc) + ": " + otter_hip_last_error());
        if (feat.dim() == 4 && feat.elempack() != 1) feat = feat.packing(1);
        const ScalarType b = base_of(feat.scalar_type());
        if (out_dtype) *out_dtype = b == ScalarType::Float ? 0 : (b == ScalarType::Byte ? 1 : 2);
        if (out_shape4)
            for (int i = 0; i < 4; ++i) out_shape4[i] = i < feat.dim() ? feat.size(i) : 1;
        if (out) {
            if (feat.nbytes() > out_capacity_bytes) return fail("output buffer too small");
            std::memcpy(out, feat.data_ptr(), feat.nbytes());
        }
        return 0;
    } catch (const std::exception& e) {
        return fail(e.what());
    }
}

// What OtterLeader::readProject makes of a file, as text: "N <project name>", "G key=value" per file-level
// parameter, then per block "T <name>" and "P key=value" for every option Net::load_otter passes to the layer.
long otter_host_otter_dump(const char* path, char* buf, size_t capacity) {
    try {
        core::OtterLeader leader;
        if (!leader.readProject(path)) return fail("readProject failed");
        std::string out = "N " + leader.getProjectName() + "\n";
        for (const core::Param& p : leader.getParams()) out += "G " + p.type + "=" + p.info + "\n";
        for (size_t i = 0; i < leader.teams_size(); ++i) {
            out += "T " + leader.getTeamName((int)i) + "\n";
            for (const core::Param& p : leader.getTeamParams((int)i)) out += "P " + p.type + "=" + p.info + "\n";
        }
        if (out.size() + 1 > capacity) return fail("dump larger than the buffer");
        std::memcpy(buf, out.c_str(), out.size() + 1);
        return (long)out.size();
    } catch (const std::exception& e) {
        return fail(e.what());
    }
}

// InitializerNcnnFromDataReader over a file: reads `n` tensors of the given shapes (4 entries each, unused trailing
// entries 0) and kinds (0 weight with tag, 1 plain fp32), appends their bytes to `out`, records 0 (fp32) / 1 (int8) /
// -1 (undefined) per tensor in `dtypes`, and reports the bytes left in the file.
long otter_host_ncnn_read(const char* path, int n, const long long* shapes, const int* kinds, int* dtypes,
                          unsigned char* out, size_t capacity, long long* remain) {
    FILE* f = std::fopen(path, "rb");
    if (!f) return fail("cannot open file");
    size_t used = 0;
    try {
        DataReaderFromStdio dr(f);
        InitializerNcnnFromDataReader init(dr);
        for (int i = 0; i < n; ++i) {
            std::vector<int64_t> shape;
            for (int d = 0; d < 4 && shapes[i * 4 + d] > 0; ++d) shape.push_back(shapes[i * 4 + d]);
            Tensor t = init.load(shape, kinds[i]);
            if (!t.defined()) {
                dtypes[i] = -1;
                continue;
            }
            dtypes[i] = t.scalar_type() == ScalarType::Byte ? 1 : 0;
            if (used + t.nbytes() > capacity) {
                std::fclose(f);
                return fail("tensors larger than the buffer");
            }
            std::memcpy(out + used, t.data_ptr(), t.nbytes());
            used += t.nbytes();
        }
        *remain = (long long)dr.remain();
    } catch (const std::exception& e) {
        std::fclose(f);
        return fail(e.what());
    }
    std::fclose(f);
    return (long)used;
}

}  // extern "C"
