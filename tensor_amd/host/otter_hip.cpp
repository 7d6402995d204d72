// Implementation of the host-side mirror of Otter's Layer / ConvolutionLayer / Net interface over the C ABI.
#include "otter_hip.hpp"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <atomic>
#include <mutex>
#include <random>
#include <sstream>

#include "../../include/otter_hip_int8.h"
#include "otter_file.hpp"

namespace otter {

// set by ConvolutionLayer::forward_chain, cleared by the download that asks otter_hip_conv_chain_status
static std::atomic<bool> g_chain_unchecked{false};

namespace {

void hip_check(int rc, const char* what) {
    if (rc != 0) throw Error(std::string(what) + ": " + otter_hip_last_error());
}

std::string trim(std::string s) {
    s.erase(std::remove_if(s.begin(), s.end(), [](unsigned char c) { return c == ' '; }), s.end());
    return s;
}

std::vector<std::string> split_list(const std::string& s) {
    std::vector<std::string> out;
    std::stringstream ss(s);
    std::string item;
    while (std::getline(ss, item, ',')) {
        item = trim(item);
        if (!item.empty()) out.push_back(item);
    }
    return out;
}

}  // namespace

// ---------------------------------------------------------------------------------------------------
// dtypes
// ---------------------------------------------------------------------------------------------------
int elempack_of(ScalarType t) {
    switch (t) {
    case ScalarType::Float4:
    case ScalarType::Int4:
        return 4;
    case ScalarType::Float8:
    case ScalarType::Byte8:
    case ScalarType::Int8:
        return 8;
    default:
        return 1;
    }
}

ScalarType base_of(ScalarType t) {
    switch (t) {
    case ScalarType::Float:
    case ScalarType::Float4:
    case ScalarType::Float8:
        return ScalarType::Float;
    case ScalarType::Byte:
    case ScalarType::Byte8:
        return ScalarType::Byte;
    case ScalarType::Int:
    case ScalarType::Int4:
    case ScalarType::Int8:
        return ScalarType::Int;
    default:
        return ScalarType::Undefined;
    }
}

size_t elemsize_of(ScalarType t) { return (base_of(t) == ScalarType::Byte ? 1 : 4) * (size_t)elempack_of(t); }

ScalarType scalar_type_of(ScalarType base, int p) {
    base = base_of(base);
    if (base == ScalarType::Float) return p == 8 ? ScalarType::Float8 : (p == 4 ? ScalarType::Float4 : ScalarType::Float);
    if (base == ScalarType::Byte) return p == 8 ? ScalarType::Byte8 : ScalarType::Byte;
    if (base == ScalarType::Int) return p == 8 ? ScalarType::Int8 : (p == 4 ? ScalarType::Int4 : ScalarType::Int);
    return ScalarType::Undefined;
}

int hip_layout_of(ScalarType t) {
    switch (t) {
    case ScalarType::Float: return OTTER_HIP_F32;
    case ScalarType::Float4: return OTTER_HIP_F32_P4;
    case ScalarType::Float8: return OTTER_HIP_F32_P8;
    case ScalarType::Byte: return OTTER_HIP_I8;
    case ScalarType::Byte8: return OTTER_HIP_I8_P8;
    case ScalarType::Int: return OTTER_HIP_I32;
    case ScalarType::Int4: return OTTER_HIP_I32_P4;
    case ScalarType::Int8: return OTTER_HIP_I32_P8;
    default: return -1;
    }
}

static ScalarType scalar_type_of_layout(int layout) {
    static const ScalarType map[] = {ScalarType::Float, ScalarType::Float4, ScalarType::Float8, ScalarType::Byte,
                                     ScalarType::Byte8, ScalarType::Int,    ScalarType::Int4,   ScalarType::Int8};
    return map[layout];
}

// ---------------------------------------------------------------------------------------------------
// Tensor
// ---------------------------------------------------------------------------------------------------
// Device blobs are recycled through a size-keyed free list (the role CPUCachingAllocator plays in the reference,
// Tensor/CPUCachingAllocator.hpp): a network asks for the same sizes on every pass, and hipFree would synchronise
// the device each time. All work of this layer is issued on one stream, so a recycled buffer is never still in use.
namespace {
struct DevicePool {
    std::mutex mu;
    std::multimap<size_t, void*> free_list;
    void* get(size_t bytes) {
        {
            std::lock_guard<std::mutex> g(mu);
            auto it = free_list.find(bytes);
            if (it != free_list.end()) {
                void* p = it->second;
                free_list.erase(it);
                return p;
            }
        }
        void* p = nullptr;
        if (otter_hip_malloc(&p, bytes) != 0) {
            release_all();
            hip_check(otter_hip_malloc(&p, bytes), "device allocation");
        }
        return p;
    }
    void put(size_t bytes, void* p) {
        std::lock_guard<std::mutex> g(mu);
        free_list.emplace(bytes, p);
    }
    void release_all() {
        std::lock_guard<std::mutex> g(mu);
        for (auto& kv : free_list) otter_hip_free(kv.second);
        free_list.clear();
    }
};
DevicePool& pool() {
    static DevicePool* p = new DevicePool();
    return *p;
}
}  // namespace

void device_cache_clear() { pool().release_all(); }

struct Tensor::Storage {
    void* host = nullptr;
    void* dev = nullptr;
    size_t bytes = 0;
    bool host_valid = false, dev_valid = false;
    std::shared_ptr<Storage> q8;  // the blob's own int8 quantization, if its producer made one
    std::vector<int64_t> q8_sizes;
    float q8_scale = 0.f;
    int q8_round = 0;
    ~Storage() {
        std::free(host);
        if (dev) pool().put(bytes, dev);
    }
};

int64_t Tensor::numel() const {
    int64_t n = 1;
    for (auto s : sizes_) n *= s;
    return sizes_.empty() ? 0 : n;
}

Tensor Tensor::empty(const std::vector<int64_t>& sizes, ScalarType dtype) {
    Tensor t;
    t.sizes_ = sizes;
    t.dtype_ = dtype;
    t.st_ = std::make_shared<Storage>();
    t.st_->bytes = t.nbytes();
    t.st_->host = std::malloc(t.st_->bytes ? t.st_->bytes : 1);
    if (!t.st_->host) throw Error("Tensor::empty: host allocation failed");
    t.st_->host_valid = true;
    return t;
}

Tensor Tensor::empty_device(const std::vector<int64_t>& sizes, ScalarType dtype) {
    Tensor t;
    t.sizes_ = sizes;
    t.dtype_ = dtype;
    t.st_ = std::make_shared<Storage>();
    t.st_->bytes = t.nbytes();
    t.st_->dev = pool().get(t.st_->bytes);
    t.st_->dev_valid = true;
    return t;
}

Tensor Tensor::from_blob(const void* data, const std::vector<int64_t>& sizes, ScalarType dtype) {
    Tensor t = empty(sizes, dtype);
    std::memcpy(t.st_->host, data, t.st_->bytes);
    return t;
}

const void* Tensor::data_ptr() const {
    OTTER_CHECK(defined(), "data_ptr of an undefined tensor");
    Storage& s = *st_;
    if (!s.host) {
        s.host = std::malloc(s.bytes ? s.bytes : 1);
        if (!s.host) throw Error("Tensor: host allocation failed");
    }
    if (!s.host_valid) {
        OTTER_CHECK(s.dev_valid, "tensor has no valid copy");
        hip_check(otter_hip_memcpy_d2h(s.host, s.dev, s.bytes, nullptr), "download");
        hip_check(otter_hip_stream_synchronize(nullptr), "download");
        // Blobs computed behind a chain launch are only good if none of its bounded waits gave up: asked once per
        // download that follows such a launch (the device is idle here anyway).
        if (g_chain_unchecked.exchange(false)) {
            int gave_up = 0;
            hip_check(otter_hip_conv_chain_status(&gave_up), "chain status");
            if (gave_up) throw Error("a chain launch gave up waiting for a producer tile: the blobs computed since are not valid");
        }
        s.host_valid = true;
    }
    return s.host;
}

void* Tensor::data_ptr() {
    void* p = const_cast<void*>(static_cast<const Tensor*>(this)->data_ptr());
    st_->dev_valid = false;  // the caller may write through the pointer
    return p;
}

void* Tensor::device_ptr() const {
    OTTER_CHECK(defined(), "device_ptr of an undefined tensor");
    Storage& s = *st_;
    if (!s.dev) s.dev = pool().get(s.bytes);
    if (!s.dev_valid) {
        OTTER_CHECK(s.host_valid, "tensor has no valid copy");
        hip_check(otter_hip_memcpy_h2d(s.dev, s.host, s.bytes, nullptr), "upload");
        s.dev_valid = true;
    }
    return s.dev;
}

bool Tensor::on_device() const { return st_ && st_->dev_valid; }

void Tensor::mark_device_written() {
    st_->dev_valid = true;
    st_->host_valid = false;
}

Tensor Tensor::view(const std::vector<int64_t>& sizes) const {
    Tensor t = *this;
    int64_t n = 1, neg = -1;
    std::vector<int64_t> s = sizes;
    for (size_t i = 0; i < s.size(); ++i) {
        if (s[i] < 0) neg = (int64_t)i;
        else n *= s[i];
    }
    if (neg >= 0) s[neg] = numel() / n;
    t.sizes_ = s;
    OTTER_CHECK(t.numel() == numel(), "view: size mismatch");
    return t;
}

void Tensor::attach_quantized(const Tensor& q, float scale, int round_mode) {
    OTTER_CHECK(defined() && q.defined() && q.scalar_type() == ScalarType::Byte8, "attach_quantized: a Byte8 blob expected");
    st_->q8 = q.st_;
    st_->q8_sizes = q.sizes_;
    st_->q8_scale = scale;
    st_->q8_round = round_mode;
}

bool Tensor::quantized_twin(float scale, int round_mode, Tensor& q) const {
    if (!defined() || !st_->q8 || st_->q8_scale != scale || st_->q8_round != round_mode) return false;
    q.st_ = st_->q8;
    q.sizes_ = st_->q8_sizes;
    q.dtype_ = ScalarType::Byte8;
    return true;
}

Tensor Tensor::packing(int p) const {
    OTTER_CHECK(defined() && dim() == 4, "packing: 4-d tensor expected");
    const int p0 = elempack();
    if (p == p0) return *this;
    const int64_t N = sizes_[0], C = sizes_[1] * p0, H = sizes_[2], W = sizes_[3];
    OTTER_CHECK(C % p == 0, "packing: elempack does not divide the channel count");
    const ScalarType dt = scalar_type_of(dtype_, p);
    OTTER_CHECK(dt != ScalarType::Undefined && elempack_of(dt) == p, "packing: no such packed dtype");
    if (on_device()) {  // keep it on the device
        Tensor out = empty_device({N, C / p, H, W}, dt);
        hip_check(otter_hip_repack(device_ptr(), hip_layout_of(dtype_), (int)N, (int)C, (int)H, (int)W, out.device_ptr(),
                                   hip_layout_of(dt), nullptr),
                  "packing");
        return out;
    }
    Tensor out = empty({N, C / p, H, W}, dt);
    const size_t eb = base_of(dtype_) == ScalarType::Byte ? 1 : 4;
    const char* s = static_cast<const char*>(data_ptr());
    char* d = static_cast<char*>(out.st_->host);
    const int64_t HW = H * W;
    for (int64_t n = 0; n < N; ++n)
        for (int64_t c = 0; c < C; ++c)
            for (int64_t i = 0; i < HW; ++i)
                std::memcpy(d + ((((n * (C / p) + c / p) * HW + i) * p) + c % p) * eb,
                            s + ((((n * (C / p0) + c / p0) * HW + i) * p0) + c % p0) * eb, eb);
    return out;
}

// ---------------------------------------------------------------------------------------------------
// ParamDict / options
// ---------------------------------------------------------------------------------------------------
int ParamDict::get(int id, int def) const {
    auto it = params_.find(id);
    return it == params_.end() || it->second.type != 1 ? def : it->second.i;
}
float ParamDict::get(int id, float def) const {
    auto it = params_.find(id);
    return it == params_.end() || it->second.type != 2 ? def : it->second.f;
}
Tensor ParamDict::get(int id, const Tensor& def) const {
    auto it = params_.find(id);
    return it == params_.end() || it->second.type != 3 ? def : it->second.t;
}
void ParamDict::set(int id, int i) {
    params_[id].type = 1;
    params_[id].i = i;
}
void ParamDict::set(int id, float f) {
    params_[id].type = 2;
    params_[id].f = f;
}
void ParamDict::set(int id, const Tensor& t) {
    params_[id].type = 3;
    params_[id].t = t;
}
void ParamDict::clear() { params_.clear(); }

bool opt_find(const LayerOption& o, const std::string& k) { return o.find(k) != o.end(); }
int opt_find_int(const LayerOption& o, const std::string& k, int def) {
    auto it = o.find(k);
    return it == o.end() ? def : std::atoi(it->second.c_str());
}
float opt_find_float(const LayerOption& o, const std::string& k, float def) {
    auto it = o.find(k);
    return it == o.end() ? def : (float)std::atof(it->second.c_str());
}
std::string opt_find_string(const LayerOption& o, const std::string& k, const std::string& def) {
    auto it = o.find(k);
    return it == o.end() ? def : it->second;
}

// ---------------------------------------------------------------------------------------------------
// Layer base + registry
// ---------------------------------------------------------------------------------------------------
int Layer::parse_param(LayerOption&, ParamDict&) { return 0; }
int Layer::compute_output_shape(ParamDict&) {
    top_shapes = bottom_shapes;
    return 0;
}
int Layer::load_param(const ParamDict&) { return 0; }
int Layer::init_model() { return 0; }
int Layer::load_model(const Initializer&) { return 0; }
int Layer::create_pipeline(const NetOption&) { return 0; }
int Layer::forward(const Tensor& bottom, Tensor& top, const NetOption& opt) const {
    if (!support_inplace) return -1;
    top = bottom;
    return forward_inplace(top, opt);
}
int Layer::forward(const std::vector<Tensor>& bottoms, std::vector<Tensor>& tops, const NetOption& opt) const {
    if (!support_inplace) return -1;
    tops = bottoms;
    for (auto& t : tops) {
        int rc = forward_inplace(t, opt);
        if (rc) return rc;
    }
    return 0;
}
int Layer::forward_inplace(Tensor&, const NetOption&) const { return -1; }

static std::map<std::string, LayerRegistry::Creator>& registry() {
    static auto* r = new std::map<std::string, LayerRegistry::Creator>();
    return *r;
}
void LayerRegistry::AddCreator(const std::string& type, Creator creator) { registry()[type] = creator; }
Layer* LayerRegistry::CreateLayer(const std::string& type) {
    auto it = registry().find(type);
    return it == registry().end() ? nullptr : it->second();
}
std::vector<std::string> LayerRegistry::TypeList() {
    std::vector<std::string> v;
    for (auto& kv : registry()) v.push_back(kv.first);
    return v;
}

// ---------------------------------------------------------------------------------------------------
// ConvolutionLayer
// ---------------------------------------------------------------------------------------------------
ConvolutionLayer::ConvolutionLayer() {
    one_blob_only = true;
    support_inplace = false;
    support_packing = true;
}

ConvolutionLayer::~ConvolutionLayer() {
    if (handle_) otter_hip_conv_destroy(handle_);
}

// option keys and defaults of Tensor/ConvolutionLayer.cpp:58-156
int ConvolutionLayer::parse_param(LayerOption& option, ParamDict& pd) {
    pd.clear();
    auto pair = [&](const char* hk, const char* wk, const char* k, int def, int lo, int& h, int& w) {
        h = opt_find_int(option, hk, -1);
        w = opt_find_int(option, wk, -1);
        const int both = opt_find_int(option, k, def);
        if (h < lo) h = both;
        if (w < lo) w = both;
    };
    int kh, kw, sh, sw, ph, pw, dh, dw, oph, opw;
    pair("kernel_h", "kernel_w", "kernel", 3, 1, kh, kw);
    pair("stride_h", "stride_w", "stride", 1, 1, sh, sw);
    pair("padding_h", "padding_w", "padding", 0, 0, ph, pw);
    pair("dilation_h", "dilation_w", "dilation", 1, 1, dh, dw);
    pair("output_padding_h", "output_padding_w", "output_padding", 0, 0, oph, opw);
    int bias = opt_find(option, "batchnorm") ? 0 : 1;
    if (opt_find(option, "bias_term")) bias = option["bias_term"] == "false" ? 0 : 1;
    const std::string act = opt_find_string(option, "activation", "");
    int act_type = act == "Relu" ? 1 : act == "LRelu" ? 2 : act == "Relu6" ? 3 : act == "Sigmoid" ? 4 : 0;
    Tensor act_params;
    if (opt_find(option, "activation_params")) {
        auto items = split_list(option["activation_params"]);
        act_params = Tensor::empty({(int64_t)items.size()}, ScalarType::Float);
        for (size_t i = 0; i < items.size(); ++i) act_params.data_ptr<float>()[i] = (float)std::atof(items[i].c_str());
    }
    if (opt_find(option, "batchnorm")) act_type = 0;
    pd.set((int)ConvParam::In_channels, opt_find_int(option, "in_channels", 1));
    pd.set((int)ConvParam::Out_channels, opt_find_int(option, "out_channels", 1));
    pd.set((int)ConvParam::Kernel_height, kh);
    pd.set((int)ConvParam::Kernel_width, kw);
    pd.set((int)ConvParam::Stride_height, sh);
    pd.set((int)ConvParam::Stride_width, sw);
    pd.set((int)ConvParam::Padding_height, ph);
    pd.set((int)ConvParam::Padding_width, pw);
    pd.set((int)ConvParam::Dilation_height, dh);
    pd.set((int)ConvParam::Dilation_width, dw);
    pd.set((int)ConvParam::Output_padding_height, oph);
    pd.set((int)ConvParam::Output_padding_width, opw);
    pd.set((int)ConvParam::Group, opt_find_int(option, "groups", 1));
    pd.set((int)ConvParam::Bias_term, bias);
    pd.set((int)ConvParam::Int8_scale_term, opt_find_int(option, "int8_scale_term", 0));
    pd.set((int)ConvParam::Activation_type, act_type);
    pd.set((int)ConvParam::Activation_params, act_params);
    return 0;
}

// Tensor/ConvolutionLayer.cpp:158-183
int ConvolutionLayer::compute_output_shape(ParamDict& pd) {
    OTTER_CHECK(!bottom_shapes.empty() && bottom_shapes[0].size() == 4, "Convolution: 4-d bottom shape expected");
    const auto& in = bottom_shapes[0];
    const int K = pd.get((int)ConvParam::Out_channels, 1);
    const int kh = pd.get((int)ConvParam::Kernel_height, 3), kw = pd.get((int)ConvParam::Kernel_width, 3);
    const int sh = pd.get((int)ConvParam::Stride_height, 1), sw = pd.get((int)ConvParam::Stride_width, 1);
    const int ph = pd.get((int)ConvParam::Padding_height, 0), pw = pd.get((int)ConvParam::Padding_width, 0);
    const int dh = pd.get((int)ConvParam::Dilation_height, 1), dw = pd.get((int)ConvParam::Dilation_width, 1);
    const int g = pd.get((int)ConvParam::Group, 1);
    const int64_t ow = (in[3] + 2 * pw - dw * (kw - 1) - 1) / sw + 1;
    const int64_t oh = (in[2] + 2 * ph - dh * (kh - 1) - 1) / sh + 1;
    pd.set((int)ConvParam::In_channels, (int)in[1]);
    pd.set((int)ConvParam::Weight_data_size, (int)(in[1] / g * kh * kw * K));
    top_shapes = {{in[0], K, oh, ow}};
    return 0;
}

int ConvolutionLayer::load_param(const ParamDict& pd) {
    in_channels = pd.get((int)ConvParam::In_channels, 1);
    out_channels = pd.get((int)ConvParam::Out_channels, 1);
    kernel_height = pd.get((int)ConvParam::Kernel_height, 3);
    kernel_width = pd.get((int)ConvParam::Kernel_width, 3);
    stride_height = pd.get((int)ConvParam::Stride_height, 1);
    stride_width = pd.get((int)ConvParam::Stride_width, 1);
    padding_height = pd.get((int)ConvParam::Padding_height, 0);
    padding_width = pd.get((int)ConvParam::Padding_width, 0);
    dilation_height = pd.get((int)ConvParam::Dilation_height, 1);
    dilation_width = pd.get((int)ConvParam::Dilation_width, 1);
    output_padding_height = pd.get((int)ConvParam::Output_padding_height, 0);
    output_padding_width = pd.get((int)ConvParam::Output_padding_width, 0);
    groups = pd.get((int)ConvParam::Group, 1);
    bias_term = pd.get((int)ConvParam::Bias_term, 0);
    weight_data_size = pd.get((int)ConvParam::Weight_data_size, 0);
    int8_scale_term = pd.get((int)ConvParam::Int8_scale_term, 0);
    activation_type = pd.get((int)ConvParam::Activation_type, 0);
    activation_params = pd.get((int)ConvParam::Activation_params, Tensor());
    return 0;
}

// random int8 model (the "no weight file" mode of Tensor/ConvolutionLayer.cpp:208-243; signed weights here)
int ConvolutionLayer::init_model() {
    if (!int8_scale_term) return -1;  // fp32 convolutions are not part of this path
    std::mt19937 rng(1234u + (unsigned)out_channels * 31u + (unsigned)in_channels);
    const int64_t per = (int64_t)(in_channels / groups) * kernel_height * kernel_width;
    weight_data = Tensor::empty({out_channels, in_channels / groups, kernel_height, kernel_width}, ScalarType::Byte);
    int8_t* w = weight_data.data_ptr<int8_t>();
    std::uniform_int_distribution<int> wd(-127, 127);
    for (int64_t i = 0; i < per * out_channels; ++i) w[i] = (int8_t)wd(rng);
    std::uniform_real_distribution<float> ud(0.f, 1.f);
    if (bias_term) {
        bias_data = Tensor::empty({out_channels}, ScalarType::Float);
        for (int i = 0; i < out_channels; ++i) bias_data.data_ptr<float>()[i] = ud(rng);
    }
    const bool dw = in_channels == groups && groups == out_channels;
    weight_data_int8_scales = Tensor::empty({out_channels}, ScalarType::Float);
    for (int i = 0; i < out_channels; ++i) weight_data_int8_scales.data_ptr<float>()[i] = 50.f + 200.f * ud(rng);
    const int nb = dw ? groups : 1;
    bottom_blob_int8_scales = Tensor::empty({nb}, ScalarType::Float);
    const float bs = 10.f + 50.f * ud(rng);
    for (int i = 0; i < nb; ++i) bottom_blob_int8_scales.data_ptr<float>()[i] = bs;
    if (int8_scale_term > 100) {
        top_blob_int8_scales = Tensor::empty({nb}, ScalarType::Float);
        const float ts = 5.f + 20.f * ud(rng);
        for (int i = 0; i < nb; ++i) top_blob_int8_scales.data_ptr<float>()[i] = ts;
    }
    return 0;
}

// order of the ncnn weight stream: Tensor/ConvolutionLayer.cpp:245-296
// Tensor/ConvolutionLayer.cpp:245-293: Otter's own stream holds the bias before the weight and no scales; ncnn's
// holds weight, bias, then the int8 scales
int ConvolutionLayer::load_model(const Initializer& in) {
    if (in.type != InitializerType::Ncnn) {
        if (bias_term) bias_data = in.load({out_channels}, 1);
        weight_data = in.load({out_channels, in_channels / groups, kernel_height, kernel_width}, 0);
        return weight_data.defined() && (!bias_term || bias_data.defined()) ? 0 : -1;
    }
    weight_data = in.load({out_channels, in_channels / groups, kernel_height, kernel_width}, 0);
    if (!weight_data.defined()) return -1;
    if (bias_term) bias_data = in.load({out_channels}, 1);
    const bool dw = in_channels == groups && groups == out_channels;
    auto replicate = [&](const Tensor& one, int n) {
        Tensor t = Tensor::empty({n}, ScalarType::Float);
        for (int i = 0; i < n; ++i) t.data_ptr<float>()[i] = one.data_ptr<float>()[0];
        return t;
    };
    if (dw) {
        if (int8_scale_term == 1 || int8_scale_term == 101) {
            weight_data_int8_scales = in.load({groups}, 1);
            bottom_blob_int8_scales = replicate(in.load({1}, 1), groups);
        } else if (int8_scale_term == 2 || int8_scale_term == 102) {
            weight_data_int8_scales = replicate(in.load({1}, 1), groups);
            bottom_blob_int8_scales = replicate(in.load({1}, 1), groups);
        }
        if (int8_scale_term > 100) top_blob_int8_scales = replicate(in.load({1}, 1), groups);
    } else {
        if (int8_scale_term) {
            weight_data_int8_scales = in.load({out_channels}, 1);
            bottom_blob_int8_scales = in.load({1}, 1);
        }
        if (int8_scale_term > 100) top_blob_int8_scales = in.load({1}, 1);
    }
    return 0;
}

int ConvolutionLayer::create_pipeline(const NetOption& opt) {
    if (weight_data.defined() && weight_data.scalar_type() == ScalarType::Byte) return create_pipeline_int8(opt);
    return -1;  // fp32 convolution: outside the accelerated path
}

// which rounding primitive the reference's quantize of this layer's input ends in (Tensor/QuantizeX86.cpp:402)
int ConvolutionLayer::input_round_mode(const NetOption& opt) const {
    return (opt.use_packing_layout && in_channels % 8 == 0) ? OTTER_HIP_ROUND_SSE : OTTER_HIP_ROUND_EXACT;
}

// Tensor/ConvolutionLayer.cpp:666-752: scale_in on the host (true division), weights re-laid-out once
int ConvolutionLayer::create_pipeline_int8(const NetOption& opt) {
    OTTER_CHECK(weight_data_int8_scales.defined() && bottom_blob_int8_scales.defined(),
                "Convolution: int8 scales missing");
    scale_in_data = Tensor::empty({out_channels}, ScalarType::Float);
    const float* ws = weight_data_int8_scales.data_ptr<float>();
    const float in_scale = bottom_blob_int8_scales.data_ptr<float>()[0];
    for (int p = 0; p < out_channels; ++p)
        scale_in_data.data_ptr<float>()[p] = ws[p] == 0 ? 0.f : 1.f / (in_scale * ws[p]);

    otter_hip_conv_desc d;
    d.in_channels = in_channels, d.out_channels = out_channels;
    d.kernel_h = kernel_height, d.kernel_w = kernel_width, d.stride_h = stride_height, d.stride_w = stride_width;
    d.pad_h = padding_height, d.pad_w = padding_width, d.dilation_h = dilation_height, d.dilation_w = dilation_width;
    d.groups = groups, d.activation_type = activation_type;
    d.activation_param0 = activation_params.defined() ? activation_params.data_ptr<float>()[0] : 0.1f;
    d.out_kind = int8_scale_term > 100 ? OTTER_HIP_OUT_I8 : OTTER_HIP_OUT_F32;
    // which rounding primitive the reference's routing ends in (Tensor/QuantizeX86.cpp:402,1177-1179,1729)
    const bool pk = opt.use_packing_layout;
    const bool dw8 = in_channels == groups && groups == out_channels && in_channels % 8 == 0;
    d.in_round_mode = input_round_mode(opt);
    d.out_round_mode = (pk && (dw8 || out_channels % 4 == 0)) ? OTTER_HIP_ROUND_SSE : OTTER_HIP_ROUND_EXACT;
    if (handle_) {
        otter_hip_conv_destroy(handle_);
        handle_ = nullptr;
    }
    const float* top = top_blob_int8_scales.defined() ? top_blob_int8_scales.data_ptr<float>() : nullptr;
    if (d.out_kind == OTTER_HIP_OUT_I8 && !top) return -1;
    return otter_hip_conv_create(&d, weight_data.data_ptr<int8_t>(), scale_in_data.data_ptr<float>(),
                                 bias_term && bias_data.defined() ? bias_data.data_ptr<float>() : nullptr, in_scale, top,
                                 top ? 1 : 0, &handle_);
}

int ConvolutionLayer::forward(const Tensor& bottom, Tensor& top, const NetOption& opt) const {
    if (int8_scale_term) return forward_int8(bottom, nullptr, fuse_scale, fuse_round, top, opt);
    return -1;
}

int ConvolutionLayer::forward_residual(const Tensor& bottom, const Tensor& shortcut, float q_scale, int q_round, Tensor& sum,
                                       const NetOption& opt) const {
    if (!int8_scale_term || int8_scale_term > 100 || !shortcut.defined()) return 1;
    return forward_int8(bottom, &shortcut, q_scale, q_round, sum, opt);
}

int ConvolutionLayer::forward_avgpool(const Tensor& bottom_in, Tensor& mean, const NetOption& opt) const {
    if (!handle_ || !int8_scale_term || int8_scale_term > 100 || force_out_layout >= 0 || !opt.use_packing_layout) return 1;
    if (!bottom_in.defined() || bottom_in.dim() != 4) return 1;
    Tensor bottom = bottom_in, twin;
    if (base_of(bottom_in.scalar_type()) == ScalarType::Float && in_channels % 8 == 0 &&
        bottom_in.quantized_twin(bottom_blob_int8_scales.data_ptr<float>()[0], input_round_mode(opt), twin))
        bottom = twin;
    if (bottom.scalar_type() != ScalarType::Byte8 || bottom.channels() != in_channels) return 1;
    const int N = (int)bottom.size(0), H = (int)bottom.size(2), W = (int)bottom.size(3);
    if (otter_hip_conv_avgpool_launches(handle_, OTTER_HIP_I8_P8, N, H, W) != 1) return 1;
    try {
        mean = Tensor::empty_device({N, out_channels, 1, 1}, ScalarType::Float);
        const int rc = otter_hip_conv_forward_avgpool(handle_, bottom.device_ptr(), OTTER_HIP_I8_P8, N, H, W,
                                                      (float*)mean.device_ptr(), nullptr, 0, nullptr);
        if (rc) return rc;
        mean.mark_device_written();
    } catch (const Error&) {
        return -100;
    }
    return 0;
}

// Tensor/ConvolutionLayer.cpp:754-847, whole batch in one launch; with `shortcut` the Eltwise sum behind it as well
int ConvolutionLayer::forward_int8(const Tensor& bottom_in, const Tensor* shortcut, float q_scale, int q_round, Tensor& top,
                                   const NetOption& opt) const {
    if (!handle_ || !bottom_in.defined() || bottom_in.dim() != 4) return -1;
    // the producer may already have quantized this blob with this layer's scale (see Net::plan_fused_quantize)
    Tensor bottom = bottom_in, twin;
    if (base_of(bottom_in.scalar_type()) == ScalarType::Float && in_channels % 8 == 0 &&
        bottom_in.quantized_twin(bottom_blob_int8_scales.data_ptr<float>()[0], input_round_mode(opt), twin))
        bottom = twin;
    const int in_layout = hip_layout_of(bottom.scalar_type());
    if (in_layout < 0 || base_of(bottom.scalar_type()) == ScalarType::Int) return -1;
    const int N = (int)bottom.size(0), H = (int)bottom.size(2), W = (int)bottom.size(3);
    if (bottom.channels() != in_channels) return -1;
    int oh = 0, ow = 0;
    if (otter_hip_conv_output_shape(handle_, H, W, &oh, &ow)) return -1;
    int out_layout = otter_hip_conv_default_out_layout(handle_);
    if (!opt.use_packing_layout)
        out_layout = int8_scale_term > 100 ? OTTER_HIP_I8 : OTTER_HIP_F32;
    if (force_out_layout >= 0) out_layout = force_out_layout;
    const ScalarType odt = scalar_type_of_layout(out_layout);
    if (shortcut) {  // the sum is taken in the layout this layer writes: the shortcut must already have it
        if (shortcut->scalar_type() != odt || elempack_of(odt) != 4 || shortcut->dim() != 4 || shortcut->size(0) != N ||
            shortcut->channels() != out_channels || shortcut->size(2) != oh || shortcut->size(3) != ow)
            return 1;
    }
    try {
        top = Tensor::empty_device({N, out_channels / elempack_of(odt), oh, ow}, odt);
        Tensor ws;
        const size_t ws_bytes = otter_hip_conv_workspace_bytes(handle_, in_layout, N, H, W);
        if (ws_bytes) ws = Tensor::empty_device({(int64_t)ws_bytes}, ScalarType::Byte);
        int rc;
        const bool with_q = q_scale > 0.f && out_layout == OTTER_HIP_F32_P4 && out_channels % 8 == 0;
        if (shortcut) {
            Tensor q;
            if (with_q) q = Tensor::empty_device({N, out_channels / 8, oh, ow}, ScalarType::Byte8);
            rc = otter_hip_conv_forward_residual(handle_, bottom.device_ptr(), in_layout, N, H, W,
                                                 (const float*)shortcut->device_ptr(), top.device_ptr(), out_layout,
                                                 with_q ? q.device_ptr() : nullptr, q_scale, q_round,
                                                 ws_bytes ? ws.device_ptr() : nullptr, ws_bytes, nullptr);
            if (rc) return rc;
            if (with_q) {
                q.mark_device_written();
                top.attach_quantized(q, q_scale, q_round);
            }
        } else if (with_q) {
            Tensor q = Tensor::empty_device({N, out_channels / 8, oh, ow}, ScalarType::Byte8);
            rc = otter_hip_conv_forward_twin(handle_, bottom.device_ptr(), in_layout, N, H, W, top.device_ptr(), out_layout,
                                             q.device_ptr(), q_scale, q_round, ws_bytes ? ws.device_ptr() : nullptr,
                                             ws_bytes, nullptr);
            if (rc) return rc;
            q.mark_device_written();
            top.attach_quantized(q, q_scale, q_round);
        } else {
            rc = otter_hip_conv_forward(handle_, bottom.device_ptr(), in_layout, N, H, W, top.device_ptr(), out_layout,
                                        ws_bytes ? ws.device_ptr() : nullptr, ws_bytes, nullptr);
            if (rc) return rc;
        }
        top.mark_device_written();
    } catch (const Error&) {
        return -100;
    }
    return 0;
}

static std::atomic<long> g_chain_forwards{0};
long ConvolutionLayer::chain_forward_count() { return g_chain_forwards.load(); }

int ConvolutionLayer::forward_chain(const std::vector<const ConvolutionLayer*>& run, const Tensor& bottom, Tensor& top,
                                    const NetOption& opt) {
    if (run.size() < 2 || !opt.use_packing_layout || !bottom.defined() || bottom.dim() != 4 ||
        bottom.scalar_type() != ScalarType::Byte8)
        return 1;
    std::vector<const otter_hip_conv*> handles;
    for (const ConvolutionLayer* c : run) {
        if (!c->handle_ || c->int8_scale_term <= 100 || c->force_out_layout >= 0) return 1;
        handles.push_back(c->handle_);
    }
    const int N = (int)bottom.size(0), H = (int)bottom.size(2), W = (int)bottom.size(3);
    if (bottom.channels() != run.front()->in_channels) return 1;
    if (otter_hip_conv_chain_launches(handles.data(), (int)handles.size(), N, H, W) != 1) return 1;
    int h = H, w = W;
    for (const otter_hip_conv* hd : handles) {
        int oh = 0, ow = 0;
        if (otter_hip_conv_output_shape(hd, h, w, &oh, &ow)) return 1;
        h = oh, w = ow;
    }
    try {
        top = Tensor::empty_device({N, run.back()->out_channels / 8, h, w}, ScalarType::Byte8);
        const size_t ws_bytes = otter_hip_conv_chain_workspace_bytes(handles.data(), (int)handles.size(), N, H, W);
        Tensor ws;
        if (ws_bytes) ws = Tensor::empty_device({(int64_t)ws_bytes}, ScalarType::Byte);
        const int rc = otter_hip_conv_chain_forward(handles.data(), (int)handles.size(), bottom.device_ptr(), N, H, W,
                                                    top.device_ptr(), ws_bytes ? ws.device_ptr() : nullptr, ws_bytes, nullptr);
        if (rc) return rc;
        top.mark_device_written();
        ++g_chain_forwards;
        g_chain_unchecked.store(true);
    } catch (const Error&) {
        return -100;
    }
    return 0;
}

static std::atomic<long> g_block_forwards{0};
long ConvolutionLayer::block_forward_count() { return g_block_forwards.load(); }

int ConvolutionLayer::forward_block(const ConvolutionLayer* e, const ConvolutionLayer* d, const ConvolutionLayer* p,
                                    const Tensor& bottom, const Tensor* shortcut, float q_scale, int q_round, Tensor& top,
                                    const NetOption& opt) {
    if (!opt.use_packing_layout || !bottom.defined() || bottom.dim() != 4 || bottom.scalar_type() != ScalarType::Byte8) return 1;
    if (!e->handle_ || !d->handle_ || !p->handle_ || e->int8_scale_term <= 100 || d->int8_scale_term <= 100 || !p->int8_scale_term)
        return 1;
    if (e->force_out_layout >= 0 || d->force_out_layout >= 0 || p->force_out_layout >= 0) return 1;
    const int N = (int)bottom.size(0), H = (int)bottom.size(2), W = (int)bottom.size(3);
    if (bottom.channels() != e->in_channels || p->out_channels % 8) return 1;
    {  // one launch for the block, or one for its first two layers and one for the last; three are the layers one by one
        const int launches = otter_hip_conv_block_launches(e->handle_, d->handle_, p->handle_, N, H, W);
        if (launches != 1 && launches != 2) return 1;
    }
    int oh = H, ow = W;
    for (const ConvolutionLayer* c : {e, d, p}) {
        int h2 = 0, w2 = 0;
        if (otter_hip_conv_output_shape(c->handle_, oh, ow, &h2, &w2)) return 1;
        oh = h2, ow = w2;
    }
    const bool f32 = p->int8_scale_term <= 100;
    const ScalarType odt = f32 ? ScalarType::Float4 : ScalarType::Byte8;
    if (shortcut) {
        if (!f32 || shortcut->scalar_type() != odt || shortcut->dim() != 4 || shortcut->size(0) != N ||
            shortcut->channels() != p->out_channels || shortcut->size(2) != oh || shortcut->size(3) != ow)
            return 1;
    }
    try {
        top = Tensor::empty_device({N, p->out_channels / elempack_of(odt), oh, ow}, odt);
        const bool with_q = f32 && q_scale > 0.f;
        Tensor q;
        if (with_q) q = Tensor::empty_device({N, p->out_channels / 8, oh, ow}, ScalarType::Byte8);
        const size_t ws_bytes = otter_hip_conv_block_workspace_bytes(e->handle_, d->handle_, p->handle_, N, H, W);
        Tensor ws;
        if (ws_bytes) ws = Tensor::empty_device({(int64_t)ws_bytes}, ScalarType::Byte);
        const int rc = otter_hip_conv_block_forward(e->handle_, d->handle_, p->handle_, bottom.device_ptr(), N, H, W,
                                                    shortcut ? (const float*)shortcut->device_ptr() : nullptr, top.device_ptr(),
                                                    f32 ? OTTER_HIP_F32_P4 : OTTER_HIP_I8_P8, with_q ? q.device_ptr() : nullptr,
                                                    q_scale, q_round, ws_bytes ? ws.device_ptr() : nullptr, ws_bytes, nullptr);
        if (rc) return rc;
        top.mark_device_written();
        if (with_q) {
            q.mark_device_written();
            top.attach_quantized(q, q_scale, q_round);
        }
        ++g_block_forwards;
    } catch (const Error&) {
        return -100;
    }
    return 0;
}

// ---------------------------------------------------------------------------------------------------
// functional API
// ---------------------------------------------------------------------------------------------------
static Tensor to_device_f32(const Tensor& t) { return t; }

Tensor quantize_to_int8(const Tensor& src, const Tensor& scale_data, bool pack) {
    OTTER_CHECK(src.defined() && src.dim() == 4 && base_of(src.scalar_type()) == ScalarType::Float,
                "quantize_to_int8: 4-d fp32 tensor expected");
    const int64_t N = src.size(0), C = src.channels(), H = src.size(2), W = src.size(3);
    // Tensor/QuantizeX86.cpp:47-58,402,554: only a packed source becomes Byte8
    const bool to8 = pack && src.elempack() > 1 && C % 8 == 0;
    const ScalarType odt = to8 ? ScalarType::Byte8 : ScalarType::Byte;
    Tensor out = Tensor::empty_device({N, C / elempack_of(odt), H, W}, odt);
    Tensor scales = to_device_f32(scale_data);
    hip_check(otter_hip_quantize((const float*)src.device_ptr(), hip_layout_of(src.scalar_type()), (int)N, (int)C, (int)H,
                                 (int)W, (const float*)scales.device_ptr(), (int)scales.numel(),
                                 to8 ? OTTER_HIP_ROUND_SSE : OTTER_HIP_ROUND_EXACT, (int8_t*)out.device_ptr(),
                                 hip_layout_of(odt), nullptr),
              "quantize_to_int8");
    out.mark_device_written();
    return out;
}

Tensor dequantize_from_int32(const Tensor& src, const Tensor& scale_data, const Tensor& bias_data, bool) {
    OTTER_CHECK(src.defined() && src.dim() == 4 && base_of(src.scalar_type()) == ScalarType::Int,
                "dequantize_from_int32: 4-d int32 tensor expected");
    const int64_t N = src.size(0), C = src.channels(), H = src.size(2), W = src.size(3);
    const ScalarType odt = scalar_type_of(ScalarType::Float, src.elempack());  // Int4 -> Float4, Int8 -> Float8
    Tensor out = Tensor::empty_device({N, C / elempack_of(odt), H, W}, odt);
    const bool has_bias = bias_data.defined() && bias_data.numel() > 0;
    hip_check(otter_hip_dequantize((const int32_t*)src.device_ptr(), hip_layout_of(src.scalar_type()), (int)N, (int)C,
                                   (int)H, (int)W, (const float*)scale_data.device_ptr(), (int)scale_data.numel(),
                                   has_bias ? (const float*)bias_data.device_ptr() : nullptr,
                                   has_bias ? (int)bias_data.numel() : 0, (float*)out.device_ptr(), hip_layout_of(odt),
                                   nullptr),
              "dequantize_from_int32");
    out.mark_device_written();
    return out;
}

Tensor requantize_from_int32_to_int8(const Tensor& src, const Tensor& scale_in, const Tensor& scale_out,
                                     const Tensor& bias, int act, const Tensor& act_params, bool pack) {
    OTTER_CHECK(src.defined() && src.dim() == 4 && base_of(src.scalar_type()) == ScalarType::Int,
                "requantize_from_int32_to_int8: 4-d int32 tensor expected");
    const int64_t N = src.size(0), C = src.channels(), H = src.size(2), W = src.size(3);
    // Tensor/QuantizeX86.cpp:1177-1179,1729: elempack 4/8 source -> SIMD rounding, Byte8 when C % 8 == 0
    const bool packed_src = src.elempack() > 1;
    const ScalarType odt = (pack && packed_src && C % 8 == 0) ? ScalarType::Byte8 : ScalarType::Byte;
    Tensor out = Tensor::empty_device({N, C / elempack_of(odt), H, W}, odt);
    const bool has_bias = bias.defined() && bias.numel() > 0;
    hip_check(otter_hip_requantize((const int32_t*)src.device_ptr(), hip_layout_of(src.scalar_type()), (int)N, (int)C,
                                   (int)H, (int)W, (const float*)scale_in.device_ptr(), (int)scale_in.numel(),
                                   (const float*)scale_out.device_ptr(), (int)scale_out.numel(),
                                   has_bias ? (const float*)bias.device_ptr() : nullptr, has_bias ? (int)bias.numel() : 0,
                                   act, act_params.defined() ? act_params.data_ptr<float>()[0] : 0.1f,
                                   packed_src ? OTTER_HIP_ROUND_SSE : OTTER_HIP_ROUND_EXACT, (int8_t*)out.device_ptr(),
                                   hip_layout_of(odt), nullptr),
              "requantize_from_int32_to_int8");
    out.mark_device_written();
    return out;
}

Tensor convolution(const Tensor& input, const Tensor& weight, const Tensor&, const Tensor&, const std::vector<int>& stride,
                   const std::vector<int>& padding, const std::vector<int>& dilation, bool transposed,
                   const std::vector<int>&, int64_t groups, bool packed, const Tensor&, const Tensor&) {
    OTTER_CHECK(!transposed, "convolution: transposed convolution is not part of the int8 path");
    OTTER_CHECK(input.defined() && input.dim() == 4 && base_of(input.scalar_type()) == ScalarType::Byte,
                "convolution: int8 input expected");
    OTTER_CHECK(weight.defined() && weight.dim() == 4 && weight.scalar_type() == ScalarType::Byte,
                "convolution: int8 weight [K, C/g, kh, kw] expected");
    const int K = (int)weight.size(0), C = (int)input.channels();
    OTTER_CHECK(weight.size(1) * groups == C, "convolution: expected input channels == weight channels * groups");
    otter_hip_conv_desc d;
    d.in_channels = C, d.out_channels = K, d.kernel_h = (int)weight.size(2), d.kernel_w = (int)weight.size(3);
    d.stride_h = stride[0], d.stride_w = stride[stride.size() > 1 ? 1 : 0];
    d.pad_h = padding[0], d.pad_w = padding[padding.size() > 1 ? 1 : 0];
    d.dilation_h = dilation[0], d.dilation_w = dilation[dilation.size() > 1 ? 1 : 0];
    d.groups = (int)groups, d.activation_type = 0, d.activation_param0 = 0.f, d.out_kind = OTTER_HIP_OUT_I32;
    d.out_round_mode = d.in_round_mode = OTTER_HIP_ROUND_SSE;
    std::vector<float> ones((size_t)K, 1.f);
    otter_hip_conv* h = nullptr;
    hip_check(otter_hip_conv_create(&d, weight.data_ptr<int8_t>(), ones.data(), nullptr, 1.f, nullptr, 0, &h), "convolution");
    int layout = packed ? otter_hip_conv_default_out_layout(h) : OTTER_HIP_I32;
    int oh = 0, ow = 0;
    const int N = (int)input.size(0), H = (int)input.size(2), W = (int)input.size(3);
    int rc = otter_hip_conv_output_shape(h, H, W, &oh, &ow);
    Tensor out;
    if (!rc) {
        const ScalarType odt = scalar_type_of_layout(layout);
        out = Tensor::empty_device({N, K / elempack_of(odt), oh, ow}, odt);
        rc = otter_hip_conv_forward(h, input.device_ptr(), hip_layout_of(input.scalar_type()), N, H, W, out.device_ptr(),
                                    layout, nullptr, 0, nullptr);
        if (!rc) out.mark_device_written();
    }
    otter_hip_conv_destroy(h);
    hip_check(rc, "convolution");
    return out;
}

// ---------------------------------------------------------------------------------------------------
// glue layers
// ---------------------------------------------------------------------------------------------------
namespace {

class InputLayer : public Layer {
public:
    InputLayer() { one_blob_only = true; }
    int parse_param(LayerOption& o, ParamDict& pd) override {  // Tensor/InputLayer.cpp:21-25
        pd.set(0, opt_find_int(o, "batchsize", 1));
        pd.set(1, opt_find_int(o, "channel", 1));
        pd.set(2, opt_find_int(o, "height", 1));
        pd.set(3, opt_find_int(o, "width", 1));
        return 0;
    }
    int compute_output_shape(ParamDict& pd) override {
        top_shapes = {{pd.get(0, 1), pd.get(1, 1), pd.get(2, 1), pd.get(3, 1)}};
        return 0;
    }
    std::string type() const override { return "Input"; }
};

class ActivationLayer : public Layer {
public:
    explicit ActivationLayer(int act, const char* name) : act_(act), name_(name) {
        one_blob_only = true;
        support_inplace = true;
        support_packing = true;
    }
    int parse_param(LayerOption& o, ParamDict& pd) override {
        pd.set(0, opt_find_float(o, "alpha", 0.1f));
        return 0;
    }
    int load_param(const ParamDict& pd) override {
        slope_ = pd.get(0, 0.1f);
        return 0;
    }
    // writes a fresh blob: the input may be shared with another consumer through a Split layer
    int forward_inplace(Tensor& t, const NetOption&) const override {
        if (!t.defined() || base_of(t.scalar_type()) != ScalarType::Float || t.dim() != 4) return -1;
        Tensor out = Tensor::empty_device(t.sizes(), t.scalar_type());
        const int l = hip_layout_of(t.scalar_type());
        if (otter_hip_repack(t.device_ptr(), l, (int)t.size(0), (int)t.channels(), (int)t.size(2), (int)t.size(3),
                             out.device_ptr(), l, nullptr))
            return -1;
        if (otter_hip_activation((float*)out.device_ptr(), (size_t)out.numel() * out.elempack(), act_, slope_, nullptr))
            return -1;
        out.mark_device_written();
        t = out;
        return 0;
    }
    std::string type() const override { return name_; }

private:
    int act_;
    float slope_ = 0.1f;
    const char* name_;
};

// Element-wise sum of fp32 blobs of one shape (Tensor/EltwiseLayer.cpp:48-80, Tensor/ShortCutLayer.cpp), in the first
// blob's layout. With fuse_scale > 0 the last addition also writes the int8 blob the readers would make of the sum.
static int sum_blobs(const std::vector<Tensor>& b, float fuse_scale, int fuse_round, std::vector<Tensor>& tops) {
    if (b.size() < 2) return -1;
    Tensor acc = b[0];
    for (size_t i = 1; i < b.size(); ++i) {
        if (base_of(b[i].scalar_type()) != ScalarType::Float || b[i].channels() != acc.channels()) return -1;
        Tensor rhs = b[i].elempack() == acc.elempack() ? b[i] : b[i].packing(acc.elempack());
        Tensor out = Tensor::empty_device(acc.sizes(), acc.scalar_type());
        const bool last = i + 1 == b.size();
        if (last && fuse_scale > 0.f && acc.dim() == 4 && acc.channels() % 8 == 0 && (acc.elempack() == 4 || acc.elempack() == 8)) {
            // the readers are int8 convolutions: hand them the quantized blob along with the sum
            Tensor q = Tensor::empty_device({acc.size(0), acc.channels() / 8, acc.size(2), acc.size(3)}, ScalarType::Byte8);
            if (otter_hip_eltwise_add_quantize((const float*)acc.device_ptr(), (const float*)rhs.device_ptr(),
                                               hip_layout_of(acc.scalar_type()), (int)acc.size(0), (int)acc.channels(),
                                               (int)acc.size(2), (int)acc.size(3), fuse_scale, fuse_round,
                                               (float*)out.device_ptr(), (int8_t*)q.device_ptr(), nullptr))
                return -1;
            out.mark_device_written();
            q.mark_device_written();
            out.attach_quantized(q, fuse_scale, fuse_round);
            acc = out;
            continue;
        }
        if (otter_hip_eltwise_add((const float*)acc.device_ptr(), (const float*)rhs.device_ptr(), (float*)out.device_ptr(),
                                  (size_t)acc.numel() * acc.elempack(), nullptr))
            return -1;
        out.mark_device_written();
        acc = out;
    }
    tops.assign(1, acc);
    return 0;
}

class EltwiseLayer : public Layer {  // Tensor/EltwiseLayer.cpp: operation "Sum"
public:
    EltwiseLayer() { support_packing = true; }
    int parse_param(LayerOption& o, ParamDict&) override {
        return opt_find_string(o, "eltwise_type", "Sum") == "Sum" ? 0 : -1;
    }
    int compute_output_shape(ParamDict&) override {
        top_shapes = {bottom_shapes[0]};
        return 0;
    }
    int forward(const std::vector<Tensor>& b, std::vector<Tensor>& tops, const NetOption&) const override {
        return sum_blobs(b, fuse_scale, fuse_round, tops);
    }
    std::string type() const override { return "Eltwise"; }
};

class SplitLayer : public Layer {  // Tensor/SplitLayer.cpp: every top shares the bottom blob
public:
    int compute_output_shape(ParamDict&) override {
        top_shapes.assign(tops.size(), bottom_shapes[0]);
        return 0;
    }
    int forward(const std::vector<Tensor>& b, std::vector<Tensor>& t, const NetOption&) const override {
        t.assign(tops.size(), b[0]);
        return 0;
    }
    std::string type() const override { return "Split"; }
};

class GlobalAvgPoolLayer : public Layer {
public:
    GlobalAvgPoolLayer() {
        one_blob_only = true;
        support_packing = true;
    }
    int compute_output_shape(ParamDict&) override {
        top_shapes = {{bottom_shapes[0][0], bottom_shapes[0][1], 1, 1}};
        return 0;
    }
    int forward(const Tensor& b, Tensor& top, const NetOption&) const override {
        if (base_of(b.scalar_type()) != ScalarType::Float || b.dim() != 4) return -1;
        top = Tensor::empty_device({b.size(0), b.channels(), 1, 1}, ScalarType::Float);
        if (otter_hip_global_avgpool((const float*)b.device_ptr(), hip_layout_of(b.scalar_type()), (int)b.size(0),
                                     (int)b.channels(), (int)b.size(2), (int)b.size(3), (float*)top.device_ptr(), nullptr))
            return -1;
        top.mark_device_written();
        return 0;
    }
    std::string type() const override { return "GlobalAvgPool"; }
};

// the fp32 layers that the reference's int8 model files put between their convolutions; every one takes a 4-D fp32
// blob in any elempack on the device and leaves its result there
static bool f32_4d(const Tensor& t) { return t.defined() && t.dim() == 4 && base_of(t.scalar_type()) == ScalarType::Float; }
static int best_pack(int64_t channels) { return channels % 8 == 0 ? 8 : (channels % 4 == 0 ? 4 : 1); }
static Tensor empty_f32_device(int64_t n, int64_t c, int64_t h, int64_t w) {
    const int p = best_pack(c);  // what Net::convert_layout would hand to the next packing-aware layer
    return Tensor::empty_device({n, c / p, h, w}, scalar_type_of(ScalarType::Float, p));
}

class MaxPoolLayer : public Layer {  // Tensor/MaxPoolLayer.cpp
public:
    MaxPoolLayer() {
        one_blob_only = true;
        support_packing = true;
    }
    int parse_param(LayerOption& o, ParamDict& pd) override {  // Tensor/MaxPoolLayer.cpp:26-72
        auto pair = [&](const char* kh, const char* kw, const char* k, int def, int min_ok, int& h, int& w) {
            h = opt_find_int(o, kh, -1), w = opt_find_int(o, kw, -1);
            const int both = opt_find_int(o, k, def);
            if (h < min_ok || w < min_ok) {
                if (h < 0) h = both;
                if (w < 0) w = both;
            }
        };
        int sh, sw, kh, kw, ph, pw, dh, dw;
        pair("stride_h", "stride_w", "stride", 1, 1, sh, sw);
        kh = opt_find_int(o, "kernel_h", -1), kw = opt_find_int(o, "kernel_w", -1);
        const int k = opt_find_int(o, "kernel", opt_find_int(o, "stride", 1));
        if (kh < 1 || kw < 1) {
            if (kh < 0) kh = k;
            if (kw < 0) kw = k;
        }
        pair("padding_h", "padding_w", "padding", 0, 0, ph, pw);
        pair("dilation_h", "dilation_w", "dilation", 1, 1, dh, dw);
        pd.set(0, kh), pd.set(1, kw), pd.set(2, sh), pd.set(3, sw), pd.set(4, ph), pd.set(5, pw), pd.set(6, dh), pd.set(7, dw);
        pd.set(8, opt_find(o, "ceil_mode") ? 1 : 0);
        if (opt_find(o, "darknet_mode")) return -1;  // darknet's asymmetric padding: not on this path
        return 0;
    }
    // Tensor/Pool.hpp:33-50
    static int out_size(int in, int k, int p, int s, int d, bool ceil_mode) {
        const int num = in + 2 * p - d * (k - 1) - 1 + (ceil_mode ? s - 1 : 0);
        int out = (num >= 0 ? num / s : -((-num + s - 1) / s)) + 1;
        if (ceil_mode && (out - 1) * s >= in + p) --out;
        return out;
    }
    int compute_output_shape(ParamDict& pd) override {
        const auto& in = bottom_shapes[0];
        const bool cm = pd.get(8, 0) != 0;
        top_shapes = {{in[0], in[1], out_size((int)in[2], pd.get(0, 3), pd.get(4, 0), pd.get(2, 1), pd.get(6, 1), cm),
                       out_size((int)in[3], pd.get(1, 3), pd.get(5, 0), pd.get(3, 1), pd.get(7, 1), cm)}};
        return 0;
    }
    int load_param(const ParamDict& pd) override {
        kh_ = pd.get(0, 1), kw_ = pd.get(1, 1), sh_ = pd.get(2, 1), sw_ = pd.get(3, 1), ph_ = pd.get(4, 0), pw_ = pd.get(5, 0);
        dh_ = pd.get(6, 1), dw_ = pd.get(7, 1), ceil_ = pd.get(8, 0) != 0;
        return 0;
    }
    // Tensor/Pool.cpp:1185-1199: on x86 a packed blob (what Net::convert_layout makes of a channel count that is a
    // multiple of 4) takes dedicated stride-2 kernels -- 3x3 for elempack 8 and 4, 2x2 for elempack 4 only (the
    // elempack-8 branch repeats the 3x3 test) -- and those pad with zeros; everything else pads with -inf.
    float pad_value(int64_t channels, const NetOption& opt) const {
        const bool plain = !ceil_ && dh_ == 1 && dw_ == 1 && sh_ == 2 && sw_ == 2;
        const int pack = !opt.use_packing_layout ? 1 : (channels % 8 == 0 ? 8 : (channels % 4 == 0 ? 4 : 1));
        const bool k3 = kh_ == 3 && kw_ == 3, k2 = kh_ == 2 && kw_ == 2;
        if (plain && ((k3 && pack != 1) || (k2 && pack == 4))) return 0.f;
        return -__builtin_inff();
    }
    int forward(const Tensor& b, Tensor& top, const NetOption& opt) const override {
        if (!f32_4d(b)) return -1;
        const int H = (int)b.size(2), W = (int)b.size(3);
        const int OH = out_size(H, kh_, ph_, sh_, dh_, ceil_), OW = out_size(W, kw_, pw_, sw_, dw_, ceil_);
        if (OH < 1 || OW < 1) return -1;
        top = empty_f32_device(b.size(0), b.channels(), OH, OW);
        if (otter_hip_maxpool2d((const float*)b.device_ptr(), hip_layout_of(b.scalar_type()), (int)b.size(0), (int)b.channels(),
                                H, W, kh_, kw_, sh_, sw_, ph_, pw_, dh_, dw_, OH, OW, pad_value(b.channels(), opt),
                                (float*)top.device_ptr(), hip_layout_of(top.scalar_type()), nullptr))
            return -1;
        top.mark_device_written();
        return 0;
    }
    std::string type() const override { return "MaxPool"; }

private:
    int kh_ = 1, kw_ = 1, sh_ = 1, sw_ = 1, ph_ = 0, pw_ = 0, dh_ = 1, dw_ = 1;
    bool ceil_ = false;
};

class ConcatLayer : public Layer {  // Tensor/ConcatLayer.cpp, channel axis
public:
    ConcatLayer() { support_packing = true; }
    int parse_param(LayerOption& o, ParamDict& pd) override {
        pd.set(0, opt_find_int(o, "axis", 1));
        return pd.get(0, 1) == 1 ? 0 : -1;  // the reference's model files concatenate channels only
    }
    int compute_output_shape(ParamDict&) override {
        auto s = bottom_shapes[0];
        for (size_t i = 1; i < bottom_shapes.size(); ++i) s[1] += bottom_shapes[i][1];
        top_shapes = {s};
        return 0;
    }
    int forward(const std::vector<Tensor>& b, std::vector<Tensor>& tops, const NetOption&) const override {
        if (b.empty()) return -1;
        int64_t C = 0;
        for (const Tensor& t : b) {
            if (!f32_4d(t) || t.size(0) != b[0].size(0) || t.size(2) != b[0].size(2) || t.size(3) != b[0].size(3)) return -1;
            C += t.channels();
        }
        Tensor out = empty_f32_device(b[0].size(0), C, b[0].size(2), b[0].size(3));
        // the readers are int8 convolutions: every copy also writes its channels of the quantized blob, when all of
        // them move whole quads of channels
        bool with_q = fuse_scale > 0.f && C % 8 == 0 && out.elempack() % 4 == 0;
        for (const Tensor& t : b) with_q = with_q && t.channels() % 4 == 0 && t.elempack() % 4 == 0;
        Tensor q;
        if (with_q) q = Tensor::empty_device({b[0].size(0), C / 8, b[0].size(2), b[0].size(3)}, ScalarType::Byte8);
        bool quads = b.size() <= 8 && out.elempack() % 4 == 0;
        for (const Tensor& t : b) quads = quads && t.elempack() % 4 == 0;
        if (quads) {  // every blob packed: the whole layer is one launch
            const float* ptrs[8];
            int layouts[8], channels[8];
            for (size_t i = 0; i < b.size(); ++i)
                ptrs[i] = (const float*)b[i].device_ptr(), layouts[i] = hip_layout_of(b[i].scalar_type()), channels[i] = (int)b[i].channels();
            if (otter_hip_concat_channels(ptrs, layouts, channels, (int)b.size(), (float*)out.device_ptr(),
                                          hip_layout_of(out.scalar_type()), (int)b[0].size(0), (int)b[0].size(2),
                                          (int)b[0].size(3), with_q ? (int8_t*)q.device_ptr() : nullptr, fuse_scale, fuse_round,
                                          nullptr))
                return -1;
            out.mark_device_written();
            if (with_q) {
                q.mark_device_written();
                out.attach_quantized(q, fuse_scale, fuse_round);
            }
            tops.assign(1, out);
            return 0;
        }
        // one copy per input; it can quantize on the way only if every input fills whole packs of the result
        for (const Tensor& t : b) with_q = with_q && t.channels() % out.elempack() == 0;
        int at = 0;
        for (const Tensor& t : b) {
            const int c = (int)t.channels();
            const int rc = with_q ? otter_hip_copy_channels_quantize(
                                        (const float*)t.device_ptr(), hip_layout_of(t.scalar_type()), c, 0,
                                        (float*)out.device_ptr(), hip_layout_of(out.scalar_type()), (int)C, at, c,
                                        (int)t.size(0), (int)t.size(2), (int)t.size(3), (int8_t*)q.device_ptr(), fuse_scale,
                                        fuse_round, nullptr)
                                  : otter_hip_copy_channels((const float*)t.device_ptr(), hip_layout_of(t.scalar_type()), c, 0,
                                                            (float*)out.device_ptr(), hip_layout_of(out.scalar_type()), (int)C,
                                                            at, c, (int)t.size(0), (int)t.size(2), (int)t.size(3), nullptr);
            if (rc) return -1;
            at += c;
        }
        out.mark_device_written();
        if (with_q) {
            q.mark_device_written();
            out.attach_quantized(q, fuse_scale, fuse_round);
        }
        tops.assign(1, out);
        return 0;
    }
    std::string type() const override { return "Concat"; }
};

class CropLayer : public Layer {  // Tensor/CropLayer.cpp, channel axis
public:
    CropLayer() {
        one_blob_only = true;
        support_packing = true;
    }
    int parse_param(LayerOption& o, ParamDict& pd) override {
        pd.set(0, opt_find_int(o, "axis", 1)), pd.set(1, opt_find_int(o, "start", -1)), pd.set(2, opt_find_int(o, "end", -1));
        return pd.get(0, 1) == 1 ? 0 : -1;
    }
    int compute_output_shape(ParamDict& pd) override {
        auto s = bottom_shapes[0];
        s[1] = pd.get(2, -1) - pd.get(1, -1);
        top_shapes = {s};
        return 0;
    }
    int load_param(const ParamDict& pd) override {
        start_ = pd.get(1, -1), end_ = pd.get(2, -1);
        return 0;
    }
    // native::slice on the logical channel index (Tensor/TensorShape.cpp:264-294): negative bounds count from the
    // end, both are clamped to [0, C]
    int forward(const Tensor& b, Tensor& top, const NetOption&) const override {
        if (!f32_4d(b)) return -1;
        const int C = (int)b.channels();
        int lo = start_, hi = end_ == -1 ? C : end_;
        if (lo < 0) lo += C;
        if (hi < 0) hi += C;
        lo = std::min(std::max(lo, 0), C);
        hi = std::min(std::max(hi, lo), C);
        if (hi == lo) return -1;
        top = empty_f32_device(b.size(0), hi - lo, b.size(2), b.size(3));
        if (otter_hip_copy_channels((const float*)b.device_ptr(), hip_layout_of(b.scalar_type()), C, lo, (float*)top.device_ptr(),
                                    hip_layout_of(top.scalar_type()), hi - lo, 0, hi - lo, (int)b.size(0), (int)b.size(2),
                                    (int)b.size(3), nullptr))
            return -1;
        top.mark_device_written();
        return 0;
    }
    std::string type() const override { return "Crop"; }
    int start() const { return start_; }
    int end() const { return end_; }

private:
    int start_ = -1, end_ = -1;
};

class ChannelShuffleLayer : public Layer {  // Tensor/ChannelShuffleLayer.cpp
public:
    ChannelShuffleLayer() {
        one_blob_only = true;
        support_packing = true;  // the kernel reads and writes any elempack, so no unpacking round trip is needed
    }
    int parse_param(LayerOption& o, ParamDict& pd) override {
        pd.set(0, opt_find_int(o, "groups", 1));
        return 0;
    }
    int load_param(const ParamDict& pd) override {
        groups_ = pd.get(0, 1);
        return 0;
    }
    int forward(const Tensor& b, Tensor& top, const NetOption&) const override {
        if (!f32_4d(b) || groups_ < 1 || b.channels() % groups_) return -1;
        top = Tensor::empty_device(b.sizes(), b.scalar_type());
        const int l = hip_layout_of(b.scalar_type());
        if (fuse_scale > 0.f && groups_ == 2 && b.elempack() == 8 && b.channels() % 16 == 0) {
            // the readers are int8 convolutions: hand them the quantized blob along with the shuffled one
            Tensor q = Tensor::empty_device(b.sizes(), ScalarType::Byte8);
            if (otter_hip_channel_shuffle_quantize((const float*)b.device_ptr(), l, (float*)top.device_ptr(), l, (int)b.size(0),
                                                   (int)b.channels(), (int)b.size(2), (int)b.size(3), groups_,
                                                   (int8_t*)q.device_ptr(), fuse_scale, fuse_round, nullptr))
                return -1;
            top.mark_device_written();
            q.mark_device_written();
            top.attach_quantized(q, fuse_scale, fuse_round);
            return 0;
        }
        if (otter_hip_channel_shuffle((const float*)b.device_ptr(), l, (float*)top.device_ptr(), l, (int)b.size(0),
                                      (int)b.channels(), (int)b.size(2), (int)b.size(3), groups_, nullptr))
            return -1;
        top.mark_device_written();
        return 0;
    }
    std::string type() const override { return "ChannelShuffle"; }
    int groups() const { return groups_; }

private:
    int groups_ = 1;
};

class ShortCutLayer : public Layer {  // Tensor/ShortCutLayer.cpp: element-wise sum of blobs of equal channel count
public:
    ShortCutLayer() { support_packing = true; }
    int compute_output_shape(ParamDict&) override {
        top_shapes = {bottom_shapes[0]};
        return 0;
    }
    int forward(const std::vector<Tensor>& b, std::vector<Tensor>& tops, const NetOption&) const override {
        if (b.size() < 2 || !f32_4d(b[0])) return -1;
        for (size_t i = 1; i < b.size(); ++i)
            // different channel counts select darknet's partial shortcut, which the reference leaves unimplemented
            if (!f32_4d(b[i]) || b[i].channels() != b[0].channels() || b[i].size(2) != b[0].size(2) || b[i].size(3) != b[0].size(3))
                return -1;
        return sum_blobs(b, fuse_scale, fuse_round, tops);
    }
    std::string type() const override { return "ShortCut"; }
};

// Post-processing heads of the reference's model files (box decoding, NMS): host code outside the convolution path.
// The layer type is known so that such a file compiles; asking for its output fails with -1 ("not supported",
// Tensor/Layer.cpp:50-59) while every blob that feeds it can be extracted.
class OffPathLayer : public Layer {
public:
    explicit OffPathLayer(const char* name) : name_(name) {}
    int compute_output_shape(ParamDict&) override {
        top_shapes.assign(tops.size(), bottom_shapes.empty() ? std::vector<int64_t>{1, 1, 1, 1} : bottom_shapes[0]);
        return 0;
    }
    int forward(const std::vector<Tensor>&, std::vector<Tensor>&, const NetOption&) const override { return -1; }
    std::string type() const override { return name_; }

private:
    const char* name_;
};

class UpsampleLayer : public Layer {  // Tensor/UpsampleLayer.cpp
public:
    UpsampleLayer() {
        one_blob_only = true;
        support_packing = true;
    }
    int parse_param(LayerOption& o, ParamDict& pd) override {  // Tensor/UpsampleLayer.cpp:25-60
        const std::string m = opt_find_string(o, "upsample_mode", "nearest");
        const int mode = m == "nearest" ? 1 : (m == "bilinear" ? 2 : (m == "bicubic" ? 3 : -1));
        OTTER_CHECK(mode <= 2, "Unsupport upsample type");
        pd.set(0, mode);
        pd.set(1, opt_find_int(o, "output_height", 0)), pd.set(2, opt_find_int(o, "output_width", 0));
        pd.set(3, opt_find_float(o, "scale_height", 1.f)), pd.set(4, opt_find_float(o, "scale_width", 1.f));
        pd.set(5, opt_find_float(o, "stride", 1.f));
        pd.set(6, opt_find(o, "align_corner") && o["align_corner"] != "false" ? 1 : 0);
        return mode < 1 ? -1 : 0;
    }
    int compute_output_shape(ParamDict& pd) override {  // Tensor/UpsampleLayer.cpp:62-96
        const auto& in = bottom_shapes[0];
        int oh = pd.get(1, 0), ow = pd.get(2, 0);
        float shf = pd.get(3, 0.f), swf = pd.get(4, 0.f);
        const float stride = pd.get(5, 1.f);
        if (oh && ow) shf = (float)(oh / in[2]), swf = (float)(ow / in[3]);
        if (stride != 0) shf = swf = stride;
        if (shf && swf) oh = (int)(in[2] * shf), ow = (int)(in[3] * swf);
        pd.set(3, shf), pd.set(4, swf), pd.set(1, oh), pd.set(2, ow);
        top_shapes = {{in[0], in[1], oh, ow}};
        return 0;
    }
    int load_param(const ParamDict& pd) override {
        mode_ = pd.get(0, 0), scale_h_ = pd.get(3, 0.f), scale_w_ = pd.get(4, 0.f), align_corner_ = pd.get(6, 0);
        return 0;
    }
    // Tensor/UpsampleLayer.cpp:108-124: the output size from the scales; packed blobs go through otter::Interpolate,
    // whose align_corners argument the layer leaves at its default (false). Blobs whose channel count is not a multiple
    // of 4 take the reference's unpacked kernels, which interpolate differently: they are not on this path.
    int forward(const Tensor& b, Tensor& top, const NetOption&) const override {
        if (!f32_4d(b) || b.channels() % 4) return -1;
        const int H = (int)b.size(2), W = (int)b.size(3);
        const int OH = (int)(H * scale_h_), OW = (int)(W * scale_w_);
        if (OH < 1 || OW < 1) return -1;
        top = empty_f32_device(b.size(0), b.channels(), OH, OW);
        if (otter_hip_upsample2d((const float*)b.device_ptr(), hip_layout_of(b.scalar_type()), (int)b.size(0), (int)b.channels(),
                                 H, W, OH, OW, mode_, 0, (float*)top.device_ptr(), hip_layout_of(top.scalar_type()), nullptr))
            return -1;
        top.mark_device_written();
        return 0;
    }
    std::string type() const override { return "Upsample"; }

private:
    int mode_ = 1, align_corner_ = 0;
    float scale_h_ = 1.f, scale_w_ = 1.f;
};

}  // namespace

// Tensor/InnerProductLayer.cpp (fp32 only in the reference as well)
InnerProductLayer::InnerProductLayer() { one_blob_only = true; }
int InnerProductLayer::parse_param(LayerOption& o, ParamDict& pd) {
    pd.set(0, opt_find_int(o, "out_features", 0));
    int bias = 1;
    if (opt_find(o, "bias_term")) bias = o["bias_term"] == "false" ? 0 : 1;
    pd.set(1, bias);
    return 0;
}
int InnerProductLayer::compute_output_shape(ParamDict& pd) {
    const auto& in = bottom_shapes[0];
    in_features = (int)(in[1] * in[2] * in[3]);
    pd.set(2, in_features);
    top_shapes = {{in[0], pd.get(0, 0), 1, 1}};
    return 0;
}
int InnerProductLayer::load_param(const ParamDict& pd) {
    out_features = pd.get(0, 0);
    bias_term = pd.get(1, 1);
    in_features = pd.get(2, in_features);
    return 0;
}
int InnerProductLayer::init_model() {
    std::mt19937 rng(99u + (unsigned)out_features);
    std::normal_distribution<float> nd(0.f, std::sqrt(2.f / (float)in_features));
    weight_data = Tensor::empty({out_features, in_features}, ScalarType::Float);
    for (int64_t i = 0; i < weight_data.numel(); ++i) weight_data.data_ptr<float>()[i] = nd(rng);
    if (bias_term) {
        bias_data = Tensor::empty({out_features}, ScalarType::Float);
        for (int i = 0; i < out_features; ++i) bias_data.data_ptr<float>()[i] = 0.01f * nd(rng);
    }
    return 0;
}
int InnerProductLayer::load_model(const Initializer& in) {
    weight_data = in.load({out_features, in_features}, 0);
    if (bias_term) bias_data = in.load({out_features}, 1);
    return 0;
}
int InnerProductLayer::forward(const Tensor& b, Tensor& top, const NetOption&) const {
    if (!weight_data.defined() || b.scalar_type() != ScalarType::Float) return -1;
    const int N = (int)b.size(0);
    if (b.numel() != (int64_t)N * in_features) return -1;
    top = Tensor::empty_device({N, out_features, 1, 1}, ScalarType::Float);
    if (otter_hip_inner_product((const float*)b.device_ptr(), N, in_features, (const float*)weight_data.device_ptr(),
                                bias_term ? (const float*)bias_data.device_ptr() : nullptr, out_features,
                                (float*)top.device_ptr(), nullptr))
        return -1;
    top.mark_device_written();
    return 0;
}

void register_hip_layers() {
    LayerRegistry::AddCreator("Input", []() -> Layer* { return new InputLayer(); });
    LayerRegistry::AddCreator("Convolution", []() -> Layer* { return new ConvolutionLayer(); });
    LayerRegistry::AddCreator("Relu", []() -> Layer* { return new ActivationLayer(1, "Relu"); });
    LayerRegistry::AddCreator("LRelu", []() -> Layer* { return new ActivationLayer(2, "LRelu"); });
    LayerRegistry::AddCreator("Relu6", []() -> Layer* { return new ActivationLayer(3, "Relu6"); });
    LayerRegistry::AddCreator("Eltwise", []() -> Layer* { return new EltwiseLayer(); });
    LayerRegistry::AddCreator("Split", []() -> Layer* { return new SplitLayer(); });
    LayerRegistry::AddCreator("InnerProduct", []() -> Layer* { return new InnerProductLayer(); });
    LayerRegistry::AddCreator("GlobalAvgPool", []() -> Layer* { return new GlobalAvgPoolLayer(); });
    LayerRegistry::AddCreator("MaxPool", []() -> Layer* { return new MaxPoolLayer(); });
    LayerRegistry::AddCreator("Concat", []() -> Layer* { return new ConcatLayer(); });
    LayerRegistry::AddCreator("Crop", []() -> Layer* { return new CropLayer(); });
    LayerRegistry::AddCreator("ChannelShuffle", []() -> Layer* { return new ChannelShuffleLayer(); });
    LayerRegistry::AddCreator("ShortCut", []() -> Layer* { return new ShortCutLayer(); });
    LayerRegistry::AddCreator("Upsample", []() -> Layer* { return new UpsampleLayer(); });
    LayerRegistry::AddCreator("NanodetPlusDetectionOutput",
                              []() -> Layer* { return new OffPathLayer("NanodetPlusDetectionOutput"); });
}

// ---------------------------------------------------------------------------------------------------
// Net / Extractor
// ---------------------------------------------------------------------------------------------------
Net::Net() {
    static bool once = (register_hip_layers(), true);
    (void)once;
}

Net::~Net() {
    for (Layer* l : layers_) delete l;
}

// Tensor/Net.cpp:40-80 (the automatic batch-norm / activation companions do not apply to int8 layers)
void Net::addLayer(LayerOption option) {
    if (!opt_find(option, "name")) option["name"] = std::to_string(layer_options_.size());
    if (!opt_find(option, "output")) option["output"] = option["name"];
    layer_options_.push_back(option);
}

// Tensor/Net.cpp:82-172: default input = previous layer's first output; a blob with several consumers gets an
// automatic Split layer
void Net::graph_construct() {
    for (size_t i = 0; i < layer_options_.size(); ++i) {
        LayerOption& l = layer_options_[i];
        if (i > 0 && !opt_find(l, "input") && l["type"] != "Input")
            l["input"] = split_list(layer_options_[i - 1]["output"])[0];
    }
    // consumers per blob name
    for (size_t i = 0; i < layer_options_.size(); ++i) {
        std::map<std::string, std::vector<size_t>> users;
        const auto outs = split_list(layer_options_[i]["output"]);
        for (size_t j = 0; j < layer_options_.size(); ++j) {
            if (layer_options_[j]["type"] == "Input") continue;
            for (const auto& in : split_list(layer_options_[j]["input"]))
                for (const auto& o : outs)
                    if (in == o) users[o].push_back(j);
        }
        size_t inserted = 0;
        for (auto& kv : users) {
            if (kv.second.size() < 2) continue;
            LayerOption sp;
            sp["type"] = "Split";
            sp["name"] = "auto_sp_" + std::to_string(i) + "_" + kv.first;
            sp["input"] = kv.first;
            std::string outs_s;
            for (size_t k = 0; k < kv.second.size(); ++k) {
                const std::string nn = "asp_" + kv.first + "_" + std::to_string(k);
                outs_s += (k ? "," : "") + nn;
                // rewrite that consumer's input list (a consumer using the blob twice gets two split outputs)
                size_t idx = kv.second[k] + (kv.second[k] > i ? inserted : 0);
                auto ins = split_list(layer_options_[idx]["input"]);
                for (auto& s : ins)
                    if (s == kv.first) {
                        s = nn;
                        break;
                    }
                std::string joined;
                for (size_t q = 0; q < ins.size(); ++q) joined += (q ? "," : "") + ins[q];
                layer_options_[idx]["input"] = joined;
            }
            sp["output"] = outs_s;
            layer_options_.insert(layer_options_.begin() + i + 1 + inserted, sp);
            ++inserted;
        }
        i += inserted;
    }
}

void Net::compile(CompileMode mode) {
    graph_construct();
    std::map<std::string, int> blob_index;
    for (auto& lo : layer_options_) {
        Layer* layer = LayerRegistry::CreateLayer(lo["type"]);
        OTTER_CHECK(layer != nullptr, "Unknown layer type: " + lo["type"]);
        layer->name = lo["name"];
        const int li = (int)layers_.size();
        if (lo["type"] != "Input")
            for (const auto& in : split_list(lo["input"])) {
                auto it = blob_index.find(in);
                OTTER_CHECK(it != blob_index.end(), "layer " + layer->name + ": unknown input blob " + in);
                layer->bottoms.push_back(it->second);
                blobs_[it->second].consumers.push_back(li);
                const Layer* prod = layers_[blobs_[it->second].producer];
                size_t k = 0;
                while (prod->tops[k] != it->second) ++k;
                layer->bottom_shapes.push_back(prod->top_shapes[k]);
            }
        for (const auto& out : split_list(lo["output"])) {
            Blob b;
            b.name = out;
            b.producer = li;
            blob_index[out] = (int)blobs_.size();
            layer->tops.push_back((int)blobs_.size());
            blobs_.push_back(b);
        }
        ParamDict pd;
        OTTER_CHECK(layer->parse_param(lo, pd) == 0, "layer " + layer->name + ": parse_param failed");
        OTTER_CHECK(layer->compute_output_shape(pd) == 0, "layer " + layer->name + ": compute_output_shape failed");
        OTTER_CHECK(layer->load_param(pd) == 0, "layer " + layer->name + ": load_param failed");
        // The description already says which convolutions are fp32 (int8_scale_term 0, e.g. conv_1 of the reference's
        // benchmark/nanodet-plus-m-1.5x_416_int8_mixed.otter): refuse the graph here, by name, rather than return a bare
        // -1 from that layer's forward later.
        if (const auto* conv = dynamic_cast<const ConvolutionLayer*>(layer))
            OTTER_CHECK(conv->int8_scale_term != 0,
                        "layer " + layer->name + ": an fp32 convolution (int8_scale_term 0) is outside the int8 path this "
                        "library accelerates; keep such a graph on the reference's Net with the GPU layer registered for "
                        "its int8 convolutions, which leaves this layer to the stock ConvolutionLayer");
        if (mode == CompileMode::Initial) {
            layer->init_model();
            layer->create_pipeline(option);
        }
        layers_.push_back(layer);
    }
}

// Tensor/Net.cpp:518-536: one layer per block of the file, the block's name as its type, its parameters (those of
// the nested `Param` block included) as its options
int Net::load_otter(const char* model_structure, CompileMode compile_mode) {
    core::OtterLeader leader;
    if (!leader.readProject(model_structure)) return -1;
    for (size_t i = 0; i < leader.teams_size(); ++i) {
        LayerOption opt;
        opt["type"] = leader.getTeamName((int)i);
        for (const core::Param& p : leader.getTeamParams((int)i)) opt[p.type] = p.info;
        addLayer(opt);
    }
    compile(compile_mode);
    return 0;
}

// Tensor/Net.cpp:538-586
int Net::load_weight(const char* weight_path, WeightType type) {
    FILE* fp = std::fopen(weight_path, "rb");
    if (!fp) {
        std::fprintf(stderr, "Open weight file fail!\n");
        return -1;
    }
    const int status = load_weight(fp, type);
    std::fclose(fp);
    return status;
}

int Net::load_weight(FILE* f, WeightType type) {
    if (layers_.empty()) {
        std::fprintf(stderr, "[Net] Empty graph!\n");
        return -1;
    }
    DataReaderFromStdio dr(f);
    if (type == WeightType::Ncnn) {
        InitializerNcnnFromDataReader initializer(dr);
        const int ret = load_weight(initializer);
        const size_t remain = dr.remain();
        if (remain) std::printf("Network may initialize fail, remain weight %zd\n", remain);
        return remain || ret;
    }
    int version[2];  // Tensor/Net.cpp:507-516: Otter's stream starts with major / minor
    if (dr.read(version, sizeof(version)) != sizeof(version)) return -1;
    InitializerFromDataReader initializer(dr);
    return load_weight(initializer);
}

const std::vector<std::string> Net::blob_names() const {
    std::vector<std::string> v;
    for (const Blob& b : blobs_) v.push_back(b.name);
    return v;
}

std::string Net::describe() const {
    std::ostringstream o;
    for (const Layer* l : layers_) {
        auto join = [&](const std::vector<int>& v) {
            std::string s;
            for (size_t i = 0; i < v.size(); ++i) s += (i ? "," : "") + blobs_[v[i]].name;
            return s.empty() ? std::string("-") : s;
        };
        o << l->type() << ' ' << l->name << ' ' << join(l->bottoms) << ' ' << join(l->tops);
        for (int d = 0; d < 4; ++d) o << ' ' << (l->top_shapes.empty() ? 0 : l->top_shapes[0][d]);
        if (const auto* c = dynamic_cast<const ConvolutionLayer*>(l))
            o << ' ' << c->out_channels << ' ' << c->in_channels << ' ' << c->groups << ' ' << c->kernel_height << ' '
              << c->kernel_width << ' ' << c->bias_term << ' ' << c->int8_scale_term;
        o << '\n';
    }
    return o.str();
}

// Tensor/Net.cpp:588-611: every layer reads its tensors from the stream in order, then builds its pipeline
int Net::load_weight(const Initializer& initializer) {
    planned_ = false;
    for (Layer* l : layers_) {
        int rc = l->load_model(initializer);
        if (rc) return rc;
        rc = l->create_pipeline(option);
        if (rc && l->type() == "Convolution") return rc;
    }
    return 0;
}

int Net::find_blob_index_by_name(const std::string& name) const {
    for (size_t i = 0; i < blobs_.size(); ++i)
        if (blobs_[i].name == name) return (int)i;
    return -1;
}

Layer* Net::layer_by_name(const std::string& name) const {
    for (Layer* l : layers_)
        if (l->name == name) return l;
    return nullptr;
}

// Tensor/Net.cpp:350-505: lazy, recursive, memoised in the extractor's blob table
int Net::forward_layer(int li, std::vector<Tensor>& blobs, const NetOption& opt) const {
    const Layer* layer = layers_[li];
    {
        const auto unit = shuffle_units_.find(li);
        if (unit != shuffle_units_.end()) {
            const ShuffleUnit& u = unit->second;
            // only when nothing inside the unit has been computed (or set by the caller) yet
            if (!blobs[layers_[u.concat]->tops[0]].defined() && !blobs[layers_[u.shuffle]->tops[0]].defined() &&
                !blobs[layer->bottoms[0]].defined()) {
                const int rc = forward_shuffle_unit(u, blobs, opt);
                if (rc <= 0) return rc;
            }
        }
    }
    {
        const auto unit = residual_units_.find(li);
        // only when the convolution's own result has not been computed (or set by the caller)
        if (unit != residual_units_.end() && !blobs[layers_[unit->second.conv]->tops[0]].defined()) {
            const int rc = forward_residual_unit(unit->second, blobs, opt);
            if (rc <= 0) return rc;
        }
    }
    {
        const auto unit = pool_units_.find(li);
        // only when the convolution's own result has not been computed (or set by the caller)
        if (unit != pool_units_.end() && !blobs[layers_[unit->second]->tops[0]].defined()) {
            const auto* conv = static_cast<const ConvolutionLayer*>(layers_[unit->second]);
            const int b = conv->bottoms[0];
            if (!blobs[b].defined()) {
                const int rc = forward_layer(blobs_[b].producer, blobs, opt);
                if (rc) return rc;
            }
            Tensor mean;
            const int rc = conv->forward_avgpool(blobs[b], mean, opt);
            if (rc < 0) return rc;
            if (rc == 0) {
                blobs[layer->tops[0]] = mean;
                if (opt.lightmode && blobs_[b].consumers.size() == 1) blobs[b] = Tensor();
                return 0;
            }
        }
    }
    {
        const auto unit = block_units_.find(li);
        // only when neither blob inside the block has been computed (or set by the caller) yet
        if (unit != block_units_.end() && !blobs[layers_[unit->second.expand]->tops[0]].defined() &&
            !blobs[layers_[unit->second.depthwise]->tops[0]].defined()) {
            const int rc = forward_block_unit(unit->second, li, -1, blobs, opt);
            if (rc <= 0) return rc;
        }
    }
    {
        const auto unit = chain_units_.find(li);
        if (unit != chain_units_.end()) {
            // only when nothing inside the run has been computed (or set by the caller) yet
            bool fresh = true;
            for (size_t k = 0; k + 1 < unit->second.size(); ++k)
                fresh = fresh && !blobs[layers_[unit->second[k]]->tops[0]].defined();
            if (fresh) {
                const int rc = forward_chain_unit(unit->second, blobs, opt);
                if (rc <= 0) return rc;
            }
        }
    }
    for (int b : layer->bottoms)
        if (!blobs[b].defined()) {
            int rc = forward_layer(blobs_[b].producer, blobs, opt);
            if (rc) return rc;
        }
    if (layer->type() == "Input") return blobs[layer->tops[0]].defined() ? 0 : -1;
    if (layer->one_blob_only) {
        Tensor bottom = blobs[layer->bottoms[0]];
        Tensor top;
        int rc;
        if (layer->support_inplace) {
            // an in-place layer may only overwrite its input when nobody else reads that blob
            top = bottom;
            rc = layer->forward_inplace(top, opt);
        } else {
            rc = layer->forward(bottom, top, opt);
        }
        if (rc) return rc;
        blobs[layer->tops[0]] = top;
    } else {
        std::vector<Tensor> bottoms, tops;
        for (int b : layer->bottoms) bottoms.push_back(blobs[b]);
        int rc = layer->forward(bottoms, tops, opt);
        if (rc) return rc;
        for (size_t k = 0; k < layer->tops.size(); ++k) blobs[layer->tops[k]] = tops[k];
    }
    if (opt.lightmode)  // Tensor/Net.cpp:449-451: the inputs are not needed any more
        for (int b : layer->bottoms)
            if (blobs_[b].consumers.size() == 1) blobs[b] = Tensor();
    return 0;
}

// An fp32 blob that feeds int8 convolutions is quantized by each of them before anything else happens; when they agree
// on the scale and the rounding primitive, its producer is told so (Layer::fuse_scale) and, if it is a layer that can
// -- an element-wise sum, a channel concatenation, an int8 convolution with an fp32 result -- does it on the way (one
// pass over the blob instead of two, one launch less per reader). Readers behind the automatic Split layers count.
void Net::plan_fused_quantize() const {
    for (Layer* l : layers_) {
        l->fuse_scale = 0.f;
        if (l->tops.size() != 1 || l->type() == "Split" || l->type() == "Input") continue;
        if (const auto* pc = dynamic_cast<const ConvolutionLayer*>(l))
            if (!pc->int8_scale_term || pc->int8_scale_term > 100) continue;  // fp32 results only
        std::vector<int> pending(l->tops.begin(), l->tops.end());
        float scale = 0.f;
        int round = 0;
        bool agree = true;
        while (!pending.empty()) {
            const int b = pending.back();
            pending.pop_back();
            for (int ci : blobs_[b].consumers) {
                const Layer* c = layers_[ci];
                if (c->type() == "Split") {
                    pending.insert(pending.end(), c->tops.begin(), c->tops.end());
                } else if (const auto* conv = dynamic_cast<const ConvolutionLayer*>(c)) {
                    if (!conv->int8_scale_term || !conv->bottom_blob_int8_scales.defined() || conv->in_channels % 8) continue;
                    const float s = conv->bottom_blob_int8_scales.data_ptr<float>()[0];
                    const int r = conv->input_round_mode(option);
                    if (scale != 0.f && (s != scale || r != round)) agree = false;
                    scale = s, round = r;
                }
            }
        }
        if (agree && scale > 0.f) l->fuse_scale = scale, l->fuse_round = round;
    }
    // Residual block tails: Eltwise / ShortCut sum of two blobs, one the fp32 result of an int8 convolution read by
    // nothing else
    residual_units_.clear();
    for (size_t ei = 0; ei < layers_.size(); ++ei) {
        const Layer* e = layers_[ei];
        if ((e->type() != "Eltwise" && e->type() != "ShortCut") || e->bottoms.size() != 2) continue;
        int best = -1;
        for (int k = 0; k < 2; ++k) {
            const int b = e->bottoms[k], pi = blobs_[b].producer;
            const auto* pc = pi < 0 ? nullptr : dynamic_cast<const ConvolutionLayer*>(layers_[pi]);
            if (!pc || !pc->int8_scale_term || pc->int8_scale_term > 100 || pc->force_out_layout >= 0) continue;
            if (blobs_[b].consumers.size() != 1 || pc->out_channels % 4) continue;
            if (e->bottoms[0] == e->bottoms[1]) continue;
            if (best < 0 || pi > blobs_[e->bottoms[best]].producer) best = k;  // the later one: the other is ready by then
        }
        if (best >= 0) residual_units_[(int)ei] = ResidualUnit{blobs_[e->bottoms[best]].producer, (int)ei, e->bottoms[1 - best]};
    }
    // Classifier tails: a GlobalAvgPool layer on the fp32 result of an int8 convolution read by nothing else
    pool_units_.clear();
    for (size_t pi = 0; pi < layers_.size(); ++pi) {
        const Layer* p = layers_[pi];
        if (p->type() != "GlobalAvgPool" || p->bottoms.size() != 1) continue;
        const int b = p->bottoms[0], ci = blobs_[b].producer;
        const auto* pc = ci < 0 ? nullptr : dynamic_cast<const ConvolutionLayer*>(layers_[ci]);
        if (!pc || !pc->int8_scale_term || pc->int8_scale_term > 100 || pc->force_out_layout >= 0 || pc->bottoms.size() != 1) continue;
        if (blobs_[b].consumers.size() != 1) continue;
        pool_units_[(int)pi] = ci;
    }
    // ShuffleNetV2 unit tails: Concat of two equal blobs -> ChannelShuffle(2) -> exactly the two half Crops
    shuffle_units_.clear();
    auto sole_reader = [&](int blob) { return blobs_[blob].consumers.size() == 1 ? blobs_[blob].consumers[0] : -1; };
    for (size_t ci = 0; ci < layers_.size(); ++ci) {
        const Layer* cat = layers_[ci];
        if (cat->type() != "Concat" || cat->bottoms.size() != 2 || cat->bottom_shapes[0] != cat->bottom_shapes[1]) continue;
        const int64_t ch = cat->bottom_shapes[0][1];
        if (ch % 8) continue;
        const int si = sole_reader(cat->tops[0]);
        const auto* sh = si < 0 ? nullptr : dynamic_cast<const ChannelShuffleLayer*>(layers_[si]);
        if (!sh || sh->groups() != 2) continue;
        int sp = sole_reader(sh->tops[0]);
        if (sp < 0 || layers_[sp]->type() != "Split" || layers_[sp]->tops.size() != 2) continue;
        int lo = -1, hi = -1;
        for (int t : layers_[sp]->tops) {
            const int r = sole_reader(t);
            const auto* crop = r < 0 ? nullptr : dynamic_cast<const CropLayer*>(layers_[r]);
            if (!crop) continue;
            if (crop->start() == 0 && crop->end() == ch) lo = r;
            if (crop->start() == ch && (crop->end() == 2 * ch || crop->end() == -1)) hi = r;
        }
        if (lo < 0 || hi < 0) continue;
        // int8 convolutions reading the second half (the unit's next branch) and agreeing on the scale
        float hs = 0.f;
        int hr = 0;
        bool agree = true;
        for (int rc : blobs_[layers_[hi]->tops[0]].consumers) {
            const auto* conv = dynamic_cast<const ConvolutionLayer*>(layers_[rc]);
            if (!conv || !conv->int8_scale_term || !conv->bottom_blob_int8_scales.defined() || conv->in_channels % 8) {
                agree = false;
                continue;
            }
            const float sc = conv->bottom_blob_int8_scales.data_ptr<float>()[0];
            const int r = conv->input_round_mode(option);
            if (hs != 0.f && (sc != hs || r != hr)) agree = false;
            hs = sc, hr = r;
        }
        const ShuffleUnit u{(int)ci, si, lo, hi, agree && hs > 0.f ? hs : 0.f, hr};
        shuffle_units_[lo] = u;
        shuffle_units_[hi] = u;
    }
    // Inverted-residual blocks: 1x1 (int8 result) -> depthwise (int8 result) -> 1x1, each blob with one reader
    block_units_.clear();
    for (size_t li = 0; li < layers_.size(); ++li) {
        const auto* pc = dynamic_cast<const ConvolutionLayer*>(layers_[li]);
        auto pointwise = [](const ConvolutionLayer* c) {
            return c->groups == 1 && c->kernel_height == 1 && c->kernel_width == 1 && c->stride_height == 1 &&
                   c->stride_width == 1 && c->padding_height == 0 && c->padding_width == 0 && c->bottoms.size() == 1 &&
                   c->tops.size() == 1 && c->force_out_layout < 0;
        };
        if (!pc || !pc->int8_scale_term || !pointwise(pc) || pc->out_channels % 8) continue;
        const int di = blobs_[pc->bottoms[0]].producer;
        const auto* dc = di < 0 ? nullptr : dynamic_cast<const ConvolutionLayer*>(layers_[di]);
        if (!dc || dc->int8_scale_term <= 100 || dc->groups != dc->in_channels || dc->groups != dc->out_channels ||
            dc->bottoms.size() != 1 || dc->force_out_layout >= 0 || sole_reader(dc->tops[0]) != (int)li)
            continue;
        const int ei = blobs_[dc->bottoms[0]].producer;
        const auto* ec = ei < 0 ? nullptr : dynamic_cast<const ConvolutionLayer*>(layers_[ei]);
        if (!ec || ec->int8_scale_term <= 100 || !pointwise(ec) || ec->in_channels % 8 || sole_reader(ec->tops[0]) != di) continue;
        block_units_[(int)li] = BlockUnit{ei, di, (int)li};
    }
    // Runs of int8 -> int8 convolutions, each blob read by the next convolution only (no Split: one reader), at most 8 long
    chain_units_.clear();
    auto chainable = [&](int li) {
        const auto* c = dynamic_cast<const ConvolutionLayer*>(layers_[li]);
        // (what the chain entry point runs as one launch, as far as the layer alone tells: the same 3x3 "same"
        // convolution over one channel count; the rest is decided per input by otter_hip_conv_chain_launches)
        return c && c->int8_scale_term > 100 && c->force_out_layout < 0 && c->bottoms.size() == 1 && c->tops.size() == 1 &&
               c->in_channels % 8 == 0 && c->in_channels == c->out_channels && c->groups == 1 && c->kernel_height == 3 &&
               c->kernel_width == 3 && c->stride_height == 1 && c->stride_width == 1 && c->padding_height == 1 &&
               c->padding_width == 1 && c->dilation_height == 1 && c->dilation_width == 1;
    };
    for (size_t li = 0; li < layers_.size(); ++li) {
        if (!chainable((int)li)) continue;
        const int pi = blobs_[layers_[li]->bottoms[0]].producer;
        if (pi >= 0 && chainable(pi) && sole_reader(layers_[pi]->tops[0]) == (int)li) continue;  // not the head of a run
        std::vector<int> run = {(int)li};
        for (;;) {
            const int next = sole_reader(layers_[run.back()]->tops[0]);
            if (next < 0 || !chainable(next)) break;
            if (static_cast<const ConvolutionLayer*>(layers_[next])->in_channels !=
                static_cast<const ConvolutionLayer*>(layers_[run.back()])->out_channels)
                break;
            run.push_back(next);
        }
        for (size_t k = 0; k + 1 < run.size(); k += 8) {  // pieces of at most 8 layers, at least 2
            const size_t end = std::min(run.size(), k + 8);
            if (end - k >= 2) chain_units_[run[end - 1]] = std::vector<int>(run.begin() + k, run.begin() + end);
        }
    }
    planned_ = true;
}

// A run of convolutions in one launch (ConvolutionLayer::forward_chain). Returns 1 when the run or the blob at hand does
// not allow it; the caller then runs the layers one by one.
int Net::forward_chain_unit(const std::vector<int>& run, std::vector<Tensor>& blobs, const NetOption& opt) const {
    const Layer* head = layers_[run.front()];
    const int in_blob = head->bottoms[0];
    if (!blobs[in_blob].defined()) {
        const int rc = forward_layer(blobs_[in_blob].producer, blobs, opt);
        if (rc) return rc;
    }
    std::vector<const ConvolutionLayer*> convs;
    for (int li : run) convs.push_back(static_cast<const ConvolutionLayer*>(layers_[li]));
    Tensor top;
    const int rc = ConvolutionLayer::forward_chain(convs, blobs[in_blob], top, opt);
    if (rc) return rc;
    blobs[layers_[run.back()]->tops[0]] = top;
    if (opt.lightmode && blobs_[in_blob].consumers.size() == 1) blobs[in_blob] = Tensor();
    return 0;
}

// An inverted-residual block (and the sum with its shortcut) in one launch (ConvolutionLayer::forward_block). Returns 1
// when the layers or the blobs at hand do not allow it; the caller then runs the layers one by one.
int Net::forward_block_unit(const BlockUnit& u, int out_layer, int shortcut, std::vector<Tensor>& blobs,
                            const NetOption& opt) const {
    const auto* ec = static_cast<const ConvolutionLayer*>(layers_[u.expand]);
    const auto* dc = static_cast<const ConvolutionLayer*>(layers_[u.depthwise]);
    const auto* pc = static_cast<const ConvolutionLayer*>(layers_[u.project]);
    const int in_blob = ec->bottoms[0];
    for (int b : {shortcut, in_blob})
        if (b >= 0 && !blobs[b].defined()) {
            const int rc = forward_layer(blobs_[b].producer, blobs, opt);
            if (rc) return rc;
        }
    // the block reads Byte8: the blob itself, or the int8 twin its producer made with the first layer's scale
    Tensor bottom = blobs[in_blob], twin;
    if (bottom.defined() && base_of(bottom.scalar_type()) == ScalarType::Float &&
        bottom.quantized_twin(ec->bottom_blob_int8_scales.data_ptr<float>()[0], ec->input_round_mode(opt), twin))
        bottom = twin;
    const Layer* out = layers_[out_layer];
    Tensor top;
    const int rc = ConvolutionLayer::forward_block(ec, dc, pc, bottom, shortcut >= 0 ? &blobs[shortcut] : nullptr, out->fuse_scale,
                                                   out->fuse_round, top, opt);
    if (rc) return rc;
    blobs[out->tops[0]] = top;
    if (opt.lightmode)
        for (int b : {shortcut, in_blob})
            if (b >= 0 && blobs_[b].consumers.size() == 1) blobs[b] = Tensor();
    return 0;
}

// Convolution and Eltwise sum in one launch (otter_hip_conv_forward_residual). Returns 1 when the blobs at hand do not
// allow it; the caller then runs the layers one by one.
int Net::forward_residual_unit(const ResidualUnit& u, std::vector<Tensor>& blobs, const NetOption& opt) const {
    const auto* conv = static_cast<const ConvolutionLayer*>(layers_[u.conv]);
    const Layer* e = layers_[u.eltwise];
    {
        // the convolution may be the last layer of an inverted-residual block: then the whole block and the sum in one launch
        const auto bu = block_units_.find(u.conv);
        if (bu != block_units_.end() && !blobs[layers_[bu->second.expand]->tops[0]].defined() &&
            !blobs[layers_[bu->second.depthwise]->tops[0]].defined()) {
            const int rc = forward_block_unit(bu->second, u.eltwise, u.shortcut, blobs, opt);
            if (rc <= 0) return rc;
        }
    }
    for (int b : {u.shortcut, conv->bottoms[0]})
        if (!blobs[b].defined()) {
            const int rc = forward_layer(blobs_[b].producer, blobs, opt);
            if (rc) return rc;
        }
    Tensor sum;
    const int rc = conv->forward_residual(blobs[conv->bottoms[0]], blobs[u.shortcut], e->fuse_scale, e->fuse_round, sum, opt);
    if (rc) return rc;
    blobs[e->tops[0]] = sum;
    if (opt.lightmode)
        for (int b : {u.shortcut, conv->bottoms[0]})
            if (blobs_[b].consumers.size() == 1) blobs[b] = Tensor();
    return 0;
}

// One kernel for a whole unit (otter_hip_shuffle2_split) when the blobs between its ends are not wanted by anybody else.
int Net::forward_shuffle_unit(const ShuffleUnit& u, std::vector<Tensor>& blobs, const NetOption& opt) const {
    const Layer* cat = layers_[u.concat];
    for (int b : cat->bottoms)
        if (!blobs[b].defined()) {
            const int rc = forward_layer(blobs_[b].producer, blobs, opt);
            if (rc) return rc;
        }
    Tensor a = blobs[cat->bottoms[0]], b = blobs[cat->bottoms[1]];
    if (!f32_4d(a) || !f32_4d(b) || a.channels() != b.channels() || a.channels() % 8 || a.size(0) != b.size(0) ||
        a.size(2) != b.size(2) || a.size(3) != b.size(3))
        return 1;  // not the shapes the plan assumed: the caller falls back to the layers one by one
    if (a.elempack() == 1) a = a.packing(8);
    if (b.elempack() == 1) b = b.packing(8);
    const std::vector<int64_t> out_sizes = {a.size(0), a.channels() / 8, a.size(2), a.size(3)};
    Tensor lo = Tensor::empty_device(out_sizes, ScalarType::Float8), hi = Tensor::empty_device(out_sizes, ScalarType::Float8);
    Tensor hq;
    if (u.hi_scale > 0.f) hq = Tensor::empty_device(out_sizes, ScalarType::Byte8);
    if (otter_hip_shuffle2_split((const float*)a.device_ptr(), hip_layout_of(a.scalar_type()), (const float*)b.device_ptr(),
                                 hip_layout_of(b.scalar_type()), (int)a.size(0), (int)a.channels(),
                                 (int)a.size(2), (int)a.size(3), (float*)lo.device_ptr(), (float*)hi.device_ptr(),
                                 hq.defined() ? (int8_t*)hq.device_ptr() : nullptr, u.hi_scale, u.hi_round, nullptr))
        return -1;
    lo.mark_device_written();
    hi.mark_device_written();
    if (hq.defined()) {
        hq.mark_device_written();
        hi.attach_quantized(hq, u.hi_scale, u.hi_round);
    }
    blobs[layers_[u.crop_lo]->tops[0]] = lo;
    blobs[layers_[u.crop_hi]->tops[0]] = hi;
    if (opt.lightmode)
        for (int bb : cat->bottoms)
            if (blobs_[bb].consumers.size() == 1) blobs[bb] = Tensor();
    return 0;
}

Extractor Net::create_extractor() const {
    {
        // extractors may be created from several threads over one const Net: plan once, under a lock
        static std::mutex plan_mutex;
        std::lock_guard<std::mutex> lock(plan_mutex);
        if (!planned_) plan_fused_quantize();
    }
    return Extractor(this, blobs_.size());
}

Extractor::Extractor(const Net* net, size_t blob_count) : option(net->option), net_(net), blob_tensors_(blob_count) {}

void Extractor::clear() { blob_tensors_.assign(blob_tensors_.size(), Tensor()); }

int Extractor::input(const std::string& name, const Tensor& in) {
    const int i = net_->find_blob_index_by_name(name);
    if (i < 0) return -1;
    blob_tensors_[i] = in;
    return 0;
}

int Extractor::extract(const std::string& name, Tensor& feat, int type) {
    const int i = net_->find_blob_index_by_name(name);
    if (i < 0) return -1;
    int ret = 0;
    if (!blob_tensors_[i].defined()) ret = net_->forward_layer(net_->blobs_[i].producer, blob_tensors_, option);
    if (ret) return ret;
    feat = blob_tensors_[i];
    if (option.use_packing_layout && type == 0 && feat.dim() == 4 && feat.elempack() != 1) feat = feat.packing(1);
    return 0;
}

}  // namespace otter
