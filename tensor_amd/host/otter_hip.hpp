// Host side of the MI355X int8 convolution path: the part of Otter's C++ interface that the path lives behind
// (Tensor handle with the packed dtypes, NetOption, ParamDict, Layer, LayerRegistry, ConvolutionLayer, the
// functional quantize / convolution entry points, Net / Extractor), re-implemented over the C ABI in
// include/otter_hip_int8.h. Names, option keys, argument meaning and int return codes are the reference's, so that
// code written against Otter's Layer / Net API drives the GPU path unchanged; everything outside the int8
// convolution path (fp32 convolutions, detection heads, image I/O ...) is not here.
//
// Activations may live on the host, on the device, or both: a Tensor produced by a GPU layer stays on the device
// until somebody asks for its host pointer, so consecutive layers of a Net chain without host round trips.
#pragma once

#include <cstdint>
#include <cstdio>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

struct otter_hip_conv;

namespace otter {

// Tensor/Exception.hpp:88-91
struct Error : std::runtime_error {
    using std::runtime_error::runtime_error;
};
#define OTTER_CHECK(cond, msg)                     \
    do {                                           \
        if (!(cond)) throw ::otter::Error(msg);    \
    } while (0)

// the dtypes of the int8 path (Tensor/ScalarType.hpp:45-74): element type x elempack
enum class ScalarType { Undefined, Float, Float4, Float8, Byte, Byte8, Int, Int4, Int8 };

int elempack_of(ScalarType t);
size_t elemsize_of(ScalarType t);          // bytes of one packed element
ScalarType scalar_type_of(ScalarType base, int elempack);  // get_update_scalarType
ScalarType base_of(ScalarType t);          // Float / Byte / Int
int hip_layout_of(ScalarType t);           // otter_hip_layout

class Tensor {
public:
    Tensor() = default;
    static Tensor empty(const std::vector<int64_t>& sizes, ScalarType dtype);        // host storage
    static Tensor empty_device(const std::vector<int64_t>& sizes, ScalarType dtype); // device storage only
    static Tensor from_blob(const void* data, const std::vector<int64_t>& sizes, ScalarType dtype);  // copies

    bool defined() const { return (bool)st_; }
    int64_t dim() const { return (int64_t)sizes_.size(); }
    int64_t size(int i) const { return sizes_[i]; }
    const std::vector<int64_t>& sizes() const { return sizes_; }
    ScalarType scalar_type() const { return dtype_; }
    int elempack() const { return elempack_of(dtype_); }
    int64_t numel() const;          // packed elements
    size_t nbytes() const { return (size_t)numel() * elemsize_of(dtype_); }
    int64_t channels() const { return dim() == 4 ? sizes_[1] * elempack() : 0; }  // logical C

    // Tensor::packing (Tensor/Tensor.cpp:29-35): [N,C/p,H,W] with elempack p -> elempack `p`
    Tensor packing(int p) const;
    Tensor view(const std::vector<int64_t>& sizes) const;

    void* data_ptr();               // host pointer; downloads first if the fresh copy is on the device
    const void* data_ptr() const;
    template <typename T>
    T* data_ptr() { return static_cast<T*>(data_ptr()); }
    template <typename T>
    const T* data_ptr() const { return static_cast<const T*>(data_ptr()); }

    void* device_ptr() const;       // device pointer; uploads first if the fresh copy is on the host
    bool on_device() const;         // a valid device copy exists
    void mark_device_written();     // the device copy is now the fresh one

    // An fp32 blob may carry its own int8 quantization (Byte8, made by the layer that produced the blob in the same
    // pass): a convolution whose input scale and rounding primitive match reads that instead of quantizing again.
    void attach_quantized(const Tensor& q, float scale, int round_mode);
    bool quantized_twin(float scale, int round_mode, Tensor& q) const;

private:
    struct Storage;
    std::shared_ptr<Storage> st_;
    std::vector<int64_t> sizes_;
    ScalarType dtype_ = ScalarType::Undefined;
};

// Tensor/NetOption.hpp
class NetOption {
public:
    bool lightmode = true;
    bool train = false;
    bool use_non_lib_optimize = true;
    bool use_packing_layout = true;
    bool use_fp16_storage = true;
    int openmp_blocktime = 20;
};
enum class CompileMode { Inference, Initial };

// Tensor/ParamDict.hpp
class ParamDict {
public:
    int get(int id, int def) const;
    float get(int id, float def) const;
    Tensor get(int id, const Tensor& def) const;
    void set(int id, int i);
    void set(int id, float f);
    void set(int id, const Tensor& t);
    void clear();

private:
    struct Entry {
        int type = 0;
        int i = 0;
        float f = 0;
        Tensor t;
    };
    std::map<int, Entry> params_;
};

using LayerOption = std::unordered_map<std::string, std::string>;
#define OUTPUT_SHAPE_HINT 30
bool opt_find(const LayerOption& o, const std::string& k);
int opt_find_int(const LayerOption& o, const std::string& k, int def);
float opt_find_float(const LayerOption& o, const std::string& k, float def);
std::string opt_find_string(const LayerOption& o, const std::string& k, const std::string& def);

// Weight source of load_model (Tensor/Initializer.hpp): hands out consecutive tensors of a weight stream.
// type 0 = weight (may be int8), 1 = fp32 vector.
enum class InitializerType { Otter, Ncnn };
class Initializer {
public:
    virtual ~Initializer() = default;
    virtual Tensor load(const std::vector<int64_t>& shape, int type) const = 0;
    InitializerType type = InitializerType::Ncnn;  // decides the order in which a layer asks for its tensors
};

// Tensor/Layer.hpp:23-62
class Layer {
public:
    Layer() = default;
    virtual ~Layer() = default;
    virtual int parse_param(LayerOption& option, ParamDict& pd);
    virtual int compute_output_shape(ParamDict& pd);
    virtual int load_param(const ParamDict& pd);
    virtual int init_model();
    virtual int load_model(const Initializer& initializer);
    virtual int create_pipeline(const NetOption& opt);
    virtual std::string type() const { return "Undefined"; }

    // 0 success; -1 not supported; -100 allocation failure (Tensor/Layer.cpp:50-59)
    virtual int forward(const Tensor& bottom_blob, Tensor& top_blob, const NetOption& opt) const;
    virtual int forward(const std::vector<Tensor>& bottom_blobs, std::vector<Tensor>& top_blobs,
                        const NetOption& opt) const;
    virtual int forward_inplace(Tensor& bottom_blob, const NetOption& opt) const;

    bool support_inplace = false;
    bool one_blob_only = false;
    bool support_packing = false;
    std::vector<int> bottoms, tops;
    std::vector<std::vector<int64_t>> bottom_shapes, top_shapes;  // logical [N,C,H,W]
    std::string name;
    // Set by Net::plan_fused_quantize for a layer with one fp32 top blob that int8 convolutions read: fuse_scale > 0 is
    // their common input scale, fuse_round their rounding primitive. A layer that can quantize on the way attaches the
    // int8 blob to its top blob (Tensor::attach_quantized); one that cannot ignores the two.
    float fuse_scale = 0.f;
    int fuse_round = 0;
};

// Tensor/LayerRegistry.hpp:17-85: string-keyed factory; a later AddCreator overrides an earlier one
class LayerRegistry {
public:
    typedef Layer* (*Creator)();
    static void AddCreator(const std::string& type, Creator creator);
    static Layer* CreateLayer(const std::string& type);   // nullptr for an unknown type
    static std::vector<std::string> TypeList();
};
// registers the GPU layers of this library under the reference's type strings
// ("Input", "Convolution", "Relu", "Relu6", "LRelu", "Eltwise", "Split", "InnerProduct", "GlobalAvgPool")
void register_hip_layers();

// Tensor/ConvolutionLayer.hpp:15-99 -- same public members, same option keys; int8 path on the GPU
enum class ConvParam : int {
    In_channels, Out_channels, Kernel_height, Kernel_width, Stride_height, Stride_width, Padding_height, Padding_width,
    Dilation_height, Dilation_width, Output_padding_height, Output_padding_width, Group, Bias_term, Weight_data_size,
    Int8_scale_term, Activation_type, Activation_params
};

class ConvolutionLayer : public Layer {
public:
    ConvolutionLayer();
    ~ConvolutionLayer() override;
    int parse_param(LayerOption& option, ParamDict& pd) override;
    int compute_output_shape(ParamDict& pd) override;
    int load_param(const ParamDict& pd) override;
    int init_model() override;
    int load_model(const Initializer& initializer) override;
    int create_pipeline(const NetOption& opt) override;
    int forward(const Tensor& bottom_blob, Tensor& top_blob, const NetOption& opt) const override;
    std::string type() const override { return "Convolution"; }

    int in_channels = 1, out_channels = 1, kernel_height = 3, kernel_width = 3, stride_height = 1, stride_width = 1;
    int padding_height = 0, padding_width = 0, dilation_height = 1, dilation_width = 1;
    int output_padding_height = 0, output_padding_width = 0, groups = 1, bias_term = 0, int8_scale_term = 0;
    int weight_data_size = 0, activation_type = 0;
    Tensor activation_params;
    Tensor weight_data, bias_data;
    Tensor weight_data_int8_scales, bottom_blob_int8_scales, top_blob_int8_scales, scale_in_data;
    // when set, forward() produces fp32 even if int8_scale_term > 100 is absent etc.; -1 = the reference's rule
    int force_out_layout = -1;
    int input_round_mode(const NetOption& opt) const;
    // This layer followed by the Eltwise sum with `shortcut` in one launch (otter_hip_conv_forward_residual), for a layer
    // with an fp32 result whose only reader is that sum: sum = activation(convolution) + shortcut, quantized on the way
    // with q_scale (> 0) for the int8 convolutions that read the sum. Returns 1, and does nothing, when the blobs do not
    // have the layouts that takes (the caller then runs the two layers one after the other).
    int forward_residual(const Tensor& bottom_blob, const Tensor& shortcut, float q_scale, int q_round, Tensor& sum,
                         const NetOption& opt) const;
    // This layer (fp32 result) and the global average pooling that is its only reader through
    // otter_hip_conv_forward_avgpool, when that is one launch for this input; `mean` is [N, K, 1, 1]. Returns 1, and does
    // nothing, otherwise (the caller then runs the two layers one after the other).
    int forward_avgpool(const Tensor& bottom_blob, Tensor& mean, const NetOption& opt) const;
    // A run of int8 -> int8 convolution layers, each reading the one before, as one call of the C ABI's chain entry point
    // when that takes the run as a single launch (otter_hip_conv_chain_launches == 1); `top` is the last layer's blob,
    // the blobs in between are not made. Returns 1, and does nothing, for any other run or input.
    static int forward_chain(const std::vector<const ConvolutionLayer*>& run, const Tensor& bottom_blob, Tensor& top,
                             const NetOption& opt);
    static long chain_forward_count();  // runs executed that way so far in this process (for tests)
    // expand (1x1, int8 result) -> depthwise (int8 result) -> project (1x1) [+ shortcut] as one launch
    // (otter_hip_conv_block_forward). Returns 1 when the layers or the blobs at hand do not allow the single launch.
    static int forward_block(const ConvolutionLayer* expand, const ConvolutionLayer* depthwise, const ConvolutionLayer* project,
                             const Tensor& bottom_blob, const Tensor* shortcut, float q_scale, int q_round, Tensor& top,
                             const NetOption& opt);
    static long block_forward_count();  // blocks executed that way so far in this process (for tests)

private:
    int create_pipeline_int8(const NetOption& opt);
    int forward_int8(const Tensor& bottom_blob, const Tensor* shortcut, float q_scale, int q_round, Tensor& top_blob,
                     const NetOption& opt) const;
    otter_hip_conv* handle_ = nullptr;
};

// Tensor/InnerProductLayer.hpp (fp32; the reference has no int8 inner product either)
class InnerProductLayer : public Layer {
public:
    InnerProductLayer();
    int parse_param(LayerOption& option, ParamDict& pd) override;
    int compute_output_shape(ParamDict& pd) override;
    int load_param(const ParamDict& pd) override;
    int init_model() override;
    int load_model(const Initializer& initializer) override;
    int forward(const Tensor& bottom_blob, Tensor& top_blob, const NetOption& opt) const override;
    std::string type() const override { return "InnerProduct"; }
    int in_features = 0, out_features = 0, bias_term = 1;
    Tensor weight_data, bias_data;
};

// returns every cached device blob to the driver
void device_cache_clear();

// Functional entry points (Tensor/Quantize.hpp:15-19, Tensor/Convolution.hpp:17-30), int8 path only.
Tensor quantize_to_int8(const Tensor& src, const Tensor& scale_data, bool pack = false);
Tensor dequantize_from_int32(const Tensor& src, const Tensor& scale_data, const Tensor& bias_data, bool pack = false);
Tensor requantize_from_int32_to_int8(const Tensor& src, const Tensor& scale_in_data, const Tensor& scale_out_data,
                                     const Tensor& bias_data, int activation_type, const Tensor& activation_params,
                                     bool pack = false);
// int8 input + int8 weight [K, C/g, kh, kw] -> int32 accumulators (Int4 when packed and K % 4 == 0, Int8-packed for
// depthwise with C % 8 == 0, else Int)
Tensor convolution(const Tensor& input, const Tensor& weight, const Tensor& weight_o, const Tensor& bias,
                   const std::vector<int>& stride, const std::vector<int>& padding, const std::vector<int>& dilation,
                   bool transposed, const std::vector<int>& output_padding, int64_t groups, bool packed = true,
                   const Tensor& input_int8_scales = Tensor(), const Tensor& weight_int8_scales = Tensor());

// Tensor/Net.hpp:22-114 (subset: graph build, lazy forward, extractor)
class Extractor;
class Net {
    friend class Extractor;

public:
    Net();
    ~Net();
    void addLayer(LayerOption option);
    void compile(CompileMode mode = CompileMode::Initial);
    // Tensor/Net.hpp:38-48: a `.otter` description, then a weight stream (Otter's fp32 stream or ncnn's `.bin`)
    enum class WeightType { Otter, Ncnn };
    int load_otter(const char* model_structure, CompileMode compile_mode);
    int load_weight(const char* weight_path, WeightType type = WeightType::Otter);
    int load_weight(FILE* f, WeightType type = WeightType::Otter);
    int load_weight(const Initializer& initializer);
    Extractor create_extractor() const;
    // Tells every Eltwise layer whose sum is read by int8 convolutions which scale to quantize it with on the way
    // (runs by itself before the first pass after the convolutions' scales changed).
    void plan_fused_quantize() const;
    void invalidate_plan() { planned_ = false; }
    const std::vector<std::string> blob_names() const;
    std::string describe() const;  // one line per layer: type, name, bottoms, tops, top shape, convolution weights
    int find_blob_index_by_name(const std::string& name) const;
    Layer* layer_by_name(const std::string& name) const;
    size_t layer_count() const { return layers_.size(); }
    NetOption option;

private:
    void graph_construct();
    int forward_layer(int layer_index, std::vector<Tensor>& blobs, const NetOption& opt) const;
    struct Blob {
        std::string name;
        int producer = -1;
        std::vector<int> consumers;
    };
    std::vector<Layer*> layers_;
    std::vector<Blob> blobs_;
    std::vector<LayerOption> layer_options_;
    mutable bool planned_ = false;
    // Concat(a, b) -> ChannelShuffle(2) -> Crop(first half) + Crop(second half), found by the plan: either Crop layer's
    // index -> the unit; forward_layer runs the whole unit in one kernel when none of its inner blobs exists yet
    struct ShuffleUnit {
        int concat, shuffle, crop_lo, crop_hi;
        float hi_scale;  // > 0: the second half is read by int8 convolutions with this input scale ...
        int hi_round;    // ... and this rounding primitive: quantize it on the way
    };
    mutable std::map<int, ShuffleUnit> shuffle_units_;
    int forward_shuffle_unit(const ShuffleUnit& u, std::vector<Tensor>& blobs, const NetOption& opt) const;
    // The tail of a residual block, found by the plan: an Eltwise sum of two blobs, one of them the fp32 result of an
    // int8 convolution that nothing else reads. Eltwise layer's index -> the unit; forward_layer runs convolution and
    // sum in one launch when the convolution's result does not exist yet.
    struct ResidualUnit {
        int conv, eltwise;
        int shortcut;  // blob index of the other operand
    };
    mutable std::map<int, ResidualUnit> residual_units_;
    int forward_residual_unit(const ResidualUnit& u, std::vector<Tensor>& blobs, const NetOption& opt) const;
    // The tail of a classifier, found by the plan: a GlobalAvgPool layer whose input is the fp32 result of an int8
    // convolution that nothing else reads. Pooling layer's index -> the convolution's; forward_layer hands both to
    // ConvolutionLayer::forward_avgpool when the convolution's result does not exist yet.
    mutable std::map<int, int> pool_units_;
    // Runs of 2..8 int8 -> int8 convolution layers, each read only by the next, found by the plan: last layer's index ->
    // the run; forward_layer hands the run to ConvolutionLayer::forward_chain when none of its blobs exists yet.
    // Inverted-residual blocks, found by the plan: a 1x1 convolution whose only input is the int8 result of a depthwise
    // convolution read by nothing else, which in turn reads the int8 result of a 1x1 convolution read by nothing else.
    // Last layer's index -> the three; forward_layer (and the residual unit the last layer may be part of) hands them to
    // ConvolutionLayer::forward_block when neither inner blob exists yet.
    struct BlockUnit {
        int expand, depthwise, project;
    };
    mutable std::map<int, BlockUnit> block_units_;
    // out_layer: the layer whose top blob receives the result (the project layer, or the Eltwise sum behind it when
    // shortcut >= 0)
    int forward_block_unit(const BlockUnit& u, int out_layer, int shortcut, std::vector<Tensor>& blobs,
                           const NetOption& opt) const;
    mutable std::map<int, std::vector<int>> chain_units_;
    int forward_chain_unit(const std::vector<int>& run, std::vector<Tensor>& blobs, const NetOption& opt) const;
};

class Extractor {
    friend class Net;

public:
    void clear();
    void set_lightmode(bool lightmode) { option.lightmode = lightmode; }
    int input(const std::string& blob_name, const Tensor& in);
    // type 0: unpacked (elempack 1) host-visible result, as the reference; type 1: whatever layout the layer left
    int extract(const std::string& blob_name, Tensor& feat, int type);
    NetOption option;

private:
    Extractor(const Net* net, size_t blob_count);
    const Net* net_;
    std::vector<Tensor> blob_tensors_;
};

}  // namespace otter
