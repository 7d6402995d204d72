// TEST INFRASTRUCTURE -- not part of the shipped library.
//
// Thin extern "C" facade over the *real* reference (chenjunhao0315/Tensor, "Otter"), compiled from the
// sources where they lie under /root/reference by oracle/Makefile into oracle/_ref/libotter_ref.so.
// It exists so that the python tests can (a) pin the C restatement in oracle/otter_int8_oracle.c
// against the reference's own arithmetic and (b) time the reference's OpenMP/AVX2 int8 path on the
// host cores next to the GPU numbers. Nothing here re-implements reference code: every function
// just marshals plain NCHW buffers into otter::Tensor objects and calls the reference entry points
//
//   otter::quantize_to_int8                 Tensor/Quantize.hpp:15
//   otter::convolution                      Tensor/Convolution.hpp:17
//   otter::dequantize_from_int32            Tensor/Quantize.hpp:17
//   otter::requantize_from_int32_to_int8    Tensor/Quantize.hpp:19
//   otter::ConvolutionLayer                 Tensor/ConvolutionLayer.hpp:15  (parse_param .. forward)
//
// The reference int8 conv kernels are batch-1 only (Tensor/Padding.cpp:26-29), so every entry point
// loops over the batch and issues one reference call per image.
//
// Layout handling mirrors what Net::convert_layout (Tensor/Net.cpp:380-411) does before a layer that
// supports packing: fp32 -> elempack 8 if C%8==0 else 4 if C%4==0 else 1; int8 -> 8 if C%8==0 else 1.

#include "OTensor.hpp"
#include "Quantize.hpp"
#include "Convolution.hpp"
#include "ConvolutionLayer.hpp"
#include "LayerRegistry.hpp"
#include "NetOption.hpp"
#include "Net.hpp"
#include "ParamDict.hpp"
#include "Otter.hpp"
#include "Initializer.hpp"
#include "DataReader.hpp"

#include <chrono>
#include <cstring>
#include <cstdio>
#include <string>
#include <vector>
#include <omp.h>

using otter::Tensor;
using otter::ScalarType;

namespace {

thread_local std::string g_err;

int fail(const std::string& s) {
    g_err = s;
    return -1;
}

Tensor make_f32(const float* p, std::vector<int64_t> sizes) {
    if (!p) return Tensor();
    Tensor t = otter::empty(sizes, ScalarType::Float);
    std::memcpy(t.data_ptr(), p, sizeof(float) * t.numel());
    return t;
}

Tensor make_i8(const signed char* p, std::vector<int64_t> sizes) {
    if (!p) return Tensor();
    Tensor t = otter::empty(sizes, ScalarType::Byte);
    std::memcpy(t.data_ptr(), p, t.numel());
    return t;
}

Tensor make_i32(const int* p, std::vector<int64_t> sizes) {
    if (!p) return Tensor();
    Tensor t = otter::empty(sizes, ScalarType::Int);
    std::memcpy(t.data_ptr(), p, sizeof(int) * t.numel());
    return t;
}

// what Net::convert_layout would hand to a packing-aware layer
Tensor convert_layout(const Tensor& t, bool use_packing) {
    if (!use_packing) return t;
    int64_t c = t.size(1) * t.elempack();
    auto dt = t.scalar_type();
    int dst = 1;
    if (dt == ScalarType::Float || dt == ScalarType::Float4 || dt == ScalarType::Float8) {
        if (c % 8 == 0) dst = 8;
        else if (c % 4 == 0) dst = 4;
    } else if (dt == ScalarType::Byte || dt == ScalarType::Byte4 || dt == ScalarType::Byte8) {
        if (c % 8 == 0) dst = 8;
    } else if (dt == ScalarType::Int || dt == ScalarType::Int4 || dt == ScalarType::Int8) {
        if (c % 4 == 0) dst = 4;
    }
    if (t.elempack() != dst) return t.packing(dst);
    return t;
}

void copy_out(const Tensor& t_, void* dst, size_t elem_bytes) {
    Tensor t = (t_.elempack() != 1) ? t_.packing(1) : t_;
    t = t.contiguous();
    std::memcpy(dst, t.data_ptr(), elem_bytes * t.numel());
}

}  // namespace

extern "C" {

__attribute__((visibility("default"))) const char* otter_ref_last_error() { return g_err.c_str(); }

__attribute__((visibility("default"))) int otter_ref_num_threads() { return omp_get_max_threads(); }

__attribute__((visibility("default"))) void otter_ref_set_num_threads(int n) { omp_set_num_threads(n); }

// quantize_to_int8 on one NCHW fp32 tensor. `packing`: 0 = keep unpacked, else convert_layout first.
__attribute__((visibility("default"))) int otter_ref_quantize(const float* x, int n, int c, int h, int w,
                                                               const float* scales, int n_scales, int packing,
                                                               signed char* out) {
    try {
        Tensor s = make_f32(scales, {n_scales});
        for (int b = 0; b < n; ++b) {
            Tensor xi = make_f32(x + (size_t)b * c * h * w, {1, c, h, w});
            xi = convert_layout(xi, packing != 0);
            Tensor q = otter::quantize_to_int8(xi, s, packing != 0);
            copy_out(q, out + (size_t)b * c * h * w, 1);
        }
    } catch (const std::exception& e) {
        return fail(e.what());
    }
    return 0;
}

// otter::convolution on int8 input -> int32 accumulators, both NCHW. Weight [K, C/g, kh, kw] int8.
__attribute__((visibility("default"))) int otter_ref_conv_int32(const signed char* xq, int n, int c, int h, int w,
                                                                 const signed char* wq, int k, int kh, int kw,
                                                                 int stride_h, int stride_w, int pad_h, int pad_w,
                                                                 int dil_h, int dil_w, int groups, int packing,
                                                                 int* out, int oh, int ow) {
    try {
        Tensor wt = make_i8(wq, {k, c / groups, kh, kw});
        float one = 1.f;
        Tensor in_s = make_f32(&one, {1});
        std::vector<float> ws(k, 1.f);
        Tensor w_s = make_f32(ws.data(), {k});
        for (int b = 0; b < n; ++b) {
            Tensor xi = make_i8(xq + (size_t)b * c * h * w, {1, c, h, w});
            xi = convert_layout(xi, packing != 0);
            Tensor acc = otter::convolution(xi, wt, Tensor(), Tensor(), {stride_h, stride_w}, {pad_h, pad_w},
                                            {dil_h, dil_w}, false, {0, 0}, groups, packing != 0, in_s, w_s);
            Tensor a1 = (acc.elempack() != 1) ? acc.packing(1) : acc;
            if (a1.size(1) != k || a1.size(2) != oh || a1.size(3) != ow)
                return fail("otter_ref_conv_int32: unexpected output shape");
            copy_out(a1, out + (size_t)b * k * oh * ow, sizeof(int));
        }
    } catch (const std::exception& e) {
        return fail(e.what());
    }
    return 0;
}

// dequantize_from_int32 on NCHW int32. `packing`: convert_layout to Int4 first when C%4==0.
__attribute__((visibility("default"))) int otter_ref_dequantize(const int* acc, int n, int c, int h, int w,
                                                                 const float* scale, int n_scale, const float* bias,
                                                                 int n_bias, int packing, float* out) {
    try {
        Tensor s = make_f32(scale, {n_scale});
        Tensor bi = (bias && n_bias > 0) ? make_f32(bias, {n_bias}) : otter::empty({0}, ScalarType::Float);
        for (int b = 0; b < n; ++b) {
            Tensor a = make_i32(acc + (size_t)b * c * h * w, {1, c, h, w});
            a = convert_layout(a, packing != 0);
            Tensor y = otter::dequantize_from_int32(a, s, bi, packing != 0);
            copy_out(y, out + (size_t)b * c * h * w, sizeof(float));
        }
    } catch (const std::exception& e) {
        return fail(e.what());
    }
    return 0;
}

// requantize_from_int32_to_int8 on NCHW int32.
__attribute__((visibility("default"))) int otter_ref_requantize(const int* acc, int n, int c, int h, int w,
                                                                 const float* scale_in, int n_scale_in,
                                                                 const float* scale_out, int n_scale_out,
                                                                 const float* bias, int n_bias, int act_type,
                                                                 const float* act_params, int n_act_params,
                                                                 int packing, signed char* out) {
    try {
        Tensor si = make_f32(scale_in, {n_scale_in});
        Tensor so = make_f32(scale_out, {n_scale_out});
        Tensor bi = (bias && n_bias > 0) ? make_f32(bias, {n_bias}) : Tensor();
        Tensor ap = (act_params && n_act_params > 0) ? make_f32(act_params, {n_act_params}) : Tensor();
        for (int b = 0; b < n; ++b) {
            Tensor a = make_i32(acc + (size_t)b * c * h * w, {1, c, h, w});
            a = convert_layout(a, packing != 0);
            Tensor q = otter::requantize_from_int32_to_int8(a, si, so, bi, act_type, ap, packing != 0);
            copy_out(q, out + (size_t)b * c * h * w, 1);
        }
    } catch (const std::exception& e) {
        return fail(e.what());
    }
    return 0;
}

// ---------------------------------------------------------------------------------------------
// Layer level: a real otter::ConvolutionLayer driven through parse_param -> compute_output_shape ->
// load_param -> (weights injected into the public members) -> create_pipeline -> forward.
// ---------------------------------------------------------------------------------------------

struct otter_ref_conv_layer {
    otter::ConvolutionLayer* layer;
    otter::NetOption opt;
    int c, k;
};

// options: "key=value;key=value" pairs using the reference's own option keys
// (Tensor/ConvolutionLayer.cpp:58-156). weight_scales: [n_wscales]; in_scale: bottom_blob_int8_scales[0];
// top_scale: used when int8_scale_term > 100.
__attribute__((visibility("default"))) otter_ref_conv_layer* otter_ref_conv_layer_create(
    const char* options, int in_n, int in_c, int in_h, int in_w, const signed char* weight, const float* bias,
    const float* weight_scales, int n_wscales, float in_scale, float top_scale, int use_packing) {
    try {
        static otter::Net* keep_registry_linked = new otter::Net();  // pulls in the layer registrations
        (void)keep_registry_linked;
        otter::LayerOption lo;
        std::string s(options ? options : "");
        size_t pos = 0;
        while (pos < s.size()) {
            size_t e = s.find(';', pos);
            if (e == std::string::npos) e = s.size();
            std::string kv = s.substr(pos, e - pos);
            size_t eq = kv.find('=');
            if (eq != std::string::npos) lo[kv.substr(0, eq)] = kv.substr(eq + 1);
            pos = e + 1;
        }
        // through the registry, as Net::compile does (Tensor/Net.cpp:196): whatever creator is registered under
        // "Convolution" makes the layer -- the stock one, or the GPU layer of ref_hip_layer.cpp while that is switched on
        auto* L = static_cast<otter::ConvolutionLayer*>(otter::LayerRegistry::CreateLayer("Convolution"));
        L->bottom_shapes.push_back(otter::tensor({in_n, in_c, in_h, in_w}, ScalarType::Int).view({1, -1}));
        otter::ParamDict pd;
        L->parse_param(lo, pd);
        L->compute_output_shape(pd);
        L->load_param(pd);
        const int K = L->out_channels, C = L->in_channels, g = L->groups;
        L->weight_data = make_i8(weight, {K, C / g, L->kernel_height, L->kernel_width});
        if (L->bias_term && bias) L->bias_data = make_f32(bias, {K});
        const bool dw = (C == g && g == K);
        // same replication rules as ConvolutionLayer::load_model (Tensor/ConvolutionLayer.cpp:254-293)
        if (dw) {
            std::vector<float> ws(g), bs(g, in_scale), ts(g, top_scale);
            for (int i = 0; i < g; ++i) ws[i] = (n_wscales == 1) ? weight_scales[0] : weight_scales[i];
            L->weight_data_int8_scales = make_f32(ws.data(), {g});
            L->bottom_blob_int8_scales = make_f32(bs.data(), {g});
            if (L->int8_scale_term > 100) L->top_blob_int8_scales = make_f32(ts.data(), {g});
        } else {
            std::vector<float> ws(K);
            for (int i = 0; i < K; ++i) ws[i] = (n_wscales == 1) ? weight_scales[0] : weight_scales[i];
            L->weight_data_int8_scales = make_f32(ws.data(), {K});
            L->bottom_blob_int8_scales = make_f32(&in_scale, {1});
            if (L->int8_scale_term > 100) L->top_blob_int8_scales = make_f32(&top_scale, {1});
        }
        auto* h = new otter_ref_conv_layer();
        h->layer = L;
        h->opt.use_packing_layout = use_packing != 0;
        h->c = C;
        h->k = K;
        if (L->create_pipeline(h->opt) != 0) {
            fail("create_pipeline failed");
            delete L;
            delete h;
            return nullptr;
        }
        return h;
    } catch (const std::exception& e) {
        fail(e.what());
        return nullptr;
    }
}

__attribute__((visibility("default"))) void otter_ref_conv_layer_destroy(otter_ref_conv_layer* h) {
    if (!h) return;
    delete h->layer;
    delete h;
}

__attribute__((visibility("default"))) int otter_ref_conv_layer_int8_out(const otter_ref_conv_layer* h) {
    return h->layer->int8_scale_term > 100;
}

__attribute__((visibility("default"))) void otter_ref_conv_layer_scale_in(const otter_ref_conv_layer* h, float* out) {
    std::memcpy(out, h->layer->scale_in_data.data_ptr(), sizeof(float) * h->k);
}

// forward over a batch (looped); input fp32 (in_is_int8 = 0) or int8 NCHW; output NCHW fp32 or int8 depending
// on int8_scale_term. Returns seconds spent inside Layer::forward (+ the convert_layout that precedes it
// in the reference's Net), or a negative value on error. `repeat` > 1 re-runs the whole batch and reports
// the minimum.
__attribute__((visibility("default"))) double otter_ref_conv_layer_forward(const otter_ref_conv_layer* h,
                                                                            const void* x, int in_is_int8, int n,
                                                                            int hh, int ww, void* out, int repeat) {
    try {
        const int C = h->c, K = h->k;
        const bool int8_out = h->layer->int8_scale_term > 100;
        double best = 1e30;
        std::vector<Tensor> inputs;
        for (int b = 0; b < n; ++b) {
            if (in_is_int8)
                inputs.push_back(make_i8((const signed char*)x + (size_t)b * C * hh * ww, {1, C, hh, ww}));
            else
                inputs.push_back(make_f32((const float*)x + (size_t)b * C * hh * ww, {1, C, hh, ww}));
        }
        for (int r = 0; r < (repeat < 1 ? 1 : repeat); ++r) {
            double t_acc = 0;
            for (int b = 0; b < n; ++b) {
                Tensor top;
                auto t0 = std::chrono::steady_clock::now();
                Tensor xi = convert_layout(inputs[b], h->opt.use_packing_layout);
                int rc = h->layer->forward(xi, top, h->opt);
                auto t1 = std::chrono::steady_clock::now();
                if (rc != 0) {
                    fail("forward returned " + std::to_string(rc));
                    return -1.0;
                }
                t_acc += std::chrono::duration<double>(t1 - t0).count();
                if (out) {
                    Tensor t1p = (top.elempack() != 1) ? top.packing(1) : top;
                    size_t per = (size_t)K * t1p.size(2) * t1p.size(3);
                    if (int8_out)
                        copy_out(t1p, (signed char*)out + (size_t)b * per, 1);
                    else
                        copy_out(t1p, (float*)out + (size_t)b * per, sizeof(float));
                }
            }
            if (t_acc < best) best = t_acc;
        }
        return best;
    } catch (const std::exception& e) {
        fail(e.what());
        return -1.0;
    }
}

// ---------------------------------------------------------------------------------------------
// Net level: the reference's own Net reading a `.otter` description (Tensor/Net.cpp:518-536) and an ncnn `.bin`
// (Tensor/Net.cpp:538-586), run on one image with every intermediate blob kept.
// ---------------------------------------------------------------------------------------------
struct RefNet {
    otter::Net net;
    std::vector<Tensor> blobs;       // unpacked copies of every blob of the last run
    std::vector<std::string> names;  // blob names in index order
};

__attribute__((visibility("default"))) void* otter_ref_net_open(const char* otter_path, const char* bin_path,
                                                                int use_packing_layout) {
    try {
        RefNet* h = new RefNet();
        h->net.option.use_packing_layout = use_packing_layout != 0;
        h->net.option.lightmode = false;
        if (h->net.load_otter(otter_path, otter::CompileMode::Inference) != 0) {
            delete h;
            fail("load_otter failed");
            return nullptr;
        }
        if (bin_path && h->net.load_weight(bin_path, otter::Net::WeightType::Ncnn) != 0) {
            delete h;
            fail("load_weight failed");
            return nullptr;
        }
        return h;
    } catch (const std::exception& e) {
        fail(e.what());
        return nullptr;
    }
}

__attribute__((visibility("default"))) void otter_ref_net_close(void* h) { delete static_cast<RefNet*>(h); }

// Runs the net on one fp32 image [1, c, hh, w] fed to `input_blob` and extracts `n_names` blobs (each unpacked to
// elempack 1 by Extractor::extract(..., 0), Tensor/Net.cpp:729-731). Returns seconds spent in the extraction of
// the LAST name (the whole forward pass when the earlier names are upstream of it is then already done, so pass
// the final outputs first to time the network), or a negative value on error.
__attribute__((visibility("default"))) double otter_ref_net_run(void* hv, const char* input_blob, const float* x, int c,
                                                                int hh, int w, const char* const* names, int n_names) {
    RefNet* h = static_cast<RefNet*>(hv);
    try {
        auto ex = h->net.create_extractor();
        ex.set_lightmode(false);
        if (ex.input(std::string(input_blob), make_f32(x, {1, c, hh, w})) != 0) return fail("unknown input blob");
        h->blobs.clear();
        h->names.clear();
        double first = -1.0;
        for (int i = 0; i < n_names; ++i) {
            Tensor t;
            auto t0 = std::chrono::steady_clock::now();
            int rc = ex.extract(std::string(names[i]), t, 0);
            auto t1 = std::chrono::steady_clock::now();
            if (rc != 0) return fail(std::string("extract failed for ") + names[i]);
            if (i == 0) first = std::chrono::duration<double>(t1 - t0).count();
            h->blobs.push_back(t.contiguous());
            h->names.push_back(names[i]);
        }
        return first;
    } catch (const std::exception& e) {
        fail(e.what());
        return -1.0;
    }
}

// Shape and element type of an extracted blob: dims[0..3] (missing leading dims = 1), *is_int8.
__attribute__((visibility("default"))) int otter_ref_net_blob_info(void* hv, int index, long long* dims, int* is_int8) {
    RefNet* h = static_cast<RefNet*>(hv);
    if (index < 0 || index >= (int)h->blobs.size()) return fail("blob index");
    const Tensor& t = h->blobs[index];
    for (int i = 0; i < 4; ++i) dims[i] = 1;
    const int nd = (int)t.dim();
    for (int i = 0; i < nd && i < 4; ++i) dims[4 - nd + i] = t.size(i);
    *is_int8 = t.scalar_type() == ScalarType::Byte;
    return t.scalar_type() == ScalarType::Byte || t.scalar_type() == ScalarType::Float ? 0 : fail("blob dtype");
}

__attribute__((visibility("default"))) int otter_ref_net_blob_copy(void* hv, int index, void* dst, size_t capacity) {
    RefNet* h = static_cast<RefNet*>(hv);
    if (index < 0 || index >= (int)h->blobs.size()) return fail("blob index");
    const Tensor& t = h->blobs[index];
    const size_t bytes = (size_t)t.numel() * (t.scalar_type() == ScalarType::Byte ? 1 : 4);
    if (bytes > capacity) return fail("blob larger than the buffer");
    std::memcpy(dst, t.data_ptr(), bytes);
    return 0;
}

// The reference's reading of a `.otter` file as text: "T <block name>" per layer block followed by "P <key>=<value>"
// per option that Net::load_otter would see (OtterLeader::getTeamParams), "N <project name>" first.
__attribute__((visibility("default"))) long otter_ref_otter_dump(const char* path, char* buf, size_t capacity) {
    try {
        otter::core::OtterLeader leader;
        if (!leader.readProject(path)) return fail("readProject failed");
        std::string out = "N " + leader.getProjectName() + "\n";
        for (size_t i = 0; i < leader.params_size(); ++i) out += "G " + leader.getParam((int)i).type + "=" + leader.getParam((int)i).info + "\n";
        for (size_t i = 0; i < leader.teams_size(); ++i) {
            out += "T " + leader.getTeamName((int)i) + "\n";
            for (const auto& p : leader.getTeamParams((int)i)) out += "P " + p.type + "=" + p.info + "\n";
        }
        if (out.size() + 1 > capacity) return fail("dump larger than the buffer");
        std::memcpy(buf, out.c_str(), out.size() + 1);
        return (long)out.size();
    } catch (const std::exception& e) {
        return fail(e.what());
    }
}

// InitializerNcnnFromDataReader over a file (Tensor/Initializer.cpp:56-190): reads `n` tensors of the given shapes
// (4 entries each, unused trailing entries 0) and kinds (0 weight with tag, 1 plain fp32), appends their bytes to
// `out`, records 0 (fp32) / 1 (int8) / -1 (undefined) per tensor in `dtypes`, and reports the bytes left in the file.
__attribute__((visibility("default"))) long otter_ref_ncnn_read(const char* path, int n, const long long* shapes,
                                                                const int* kinds, int* dtypes, unsigned char* out,
                                                                size_t capacity, long long* remain) {
    FILE* f = std::fopen(path, "rb");
    if (!f) return fail("cannot open file");
    size_t used = 0;
    try {
        otter::DataReaderFromStdio dr(f);
        otter::InitializerNcnnFromDataReader init(dr);
        for (int i = 0; i < n; ++i) {
            std::vector<int64_t> shape;
            for (int d = 0; d < 4 && shapes[i * 4 + d] > 0; ++d) shape.push_back(shapes[i * 4 + d]);
            Tensor t = init.load(shape, kinds[i]);
            if (!t.defined()) {
                dtypes[i] = -1;
                continue;
            }
            dtypes[i] = t.scalar_type() == ScalarType::Byte ? 1 : 0;
            const size_t bytes = (size_t)t.numel() * (dtypes[i] ? 1 : 4);
            if (used + bytes > capacity) {
                std::fclose(f);
                return fail("tensors larger than the buffer");
            }
            std::memcpy(out + used, t.data_ptr(), bytes);
            used += bytes;
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
