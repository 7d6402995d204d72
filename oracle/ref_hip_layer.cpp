// TEST INFRASTRUCTURE -- not part of the shipped library; nothing under tensor_amd/ links or loads it.
//
// The reference-side binding of the C ABI (include/otter_hip_int8.h), compiled against the REFERENCE's own headers:
// the file a maintainer of chenjunhao0315/Tensor would add to route the int8 convolution layers of a stock
// otter::Net to the GPU. It is built by oracle/Makefile (target refhip) into oracle/_ref/libotter_ref_hip.so together
// with the compiled reference and the facade of ref_shim.cpp, and exists so that a test can run the reference's own
// Net - load_otter, load_weight, Extractor - with this layer registered under "Convolution" and compare the blobs with
// the stock reference's.
//
//   LayerRegistry::AddCreator overwrites an entry       Tensor/LayerRegistry.hpp:27-33
//   Net::compile creates layers by option["type"]       Tensor/Net.cpp:196
//   ConvolutionLayer (members, create_pipeline, forward) Tensor/ConvolutionLayer.hpp:15-85, .cpp:605-847
//
// The layer keeps the reference's contract: it takes the host blob Net::convert_layout hands it (Float / Float4 /
// Float8 / Byte / Byte8), and returns a host blob of the dtype the stock layer would return (Byte8 / Byte after
// requantize, Float4 / Float8 / Float after dequantize), so every other layer of the net is unaffected. Blobs cross
// the bus per layer: the reference's Tensor has no device pointer (Tensor/Device.hpp:15-18).
#include "ConvolutionLayer.hpp"
#include "LayerRegistry.hpp"
#include "NetOption.hpp"
#include "OTensor.hpp"
#include "TensorFactory.hpp"

#include <cstring>
#include <string>

extern "C" {
#include "otter_hip_int8.h"
}

namespace otter {

namespace {

int hip_layout_of(ScalarType t) {
    switch (t) {
    case ScalarType::Float: return OTTER_HIP_F32;
    case ScalarType::Float4: return OTTER_HIP_F32_P4;
    case ScalarType::Float8: return OTTER_HIP_F32_P8;
    case ScalarType::Byte: return OTTER_HIP_I8;
    case ScalarType::Byte8: return OTTER_HIP_I8_P8;
    default: return -1;
    }
}

ScalarType dtype_of_layout(int layout) {
    switch (layout) {
    case OTTER_HIP_F32_P4: return ScalarType::Float4;
    case OTTER_HIP_F32_P8: return ScalarType::Float8;
    case OTTER_HIP_I8: return ScalarType::Byte;
    case OTTER_HIP_I8_P8: return ScalarType::Byte8;
    default: return ScalarType::Float;
    }
}

int pack_of_layout(int layout) {
    return (layout == OTTER_HIP_F32_P8 || layout == OTTER_HIP_I8_P8) ? 8 : (layout == OTTER_HIP_F32_P4 ? 4 : 1);
}

struct DeviceBuffer {  // freed on every return path
    void* p = nullptr;
    ~DeviceBuffer() { otter_hip_free(p); }
};

long g_gpu_forwards = 0;  // how many forward() calls went to the GPU (the test checks that the layer was really used)

}  // namespace

class HipConvolutionLayer : public ConvolutionLayer {  // inherits parse_param / load_param / load_model
public:
    ~HipConvolutionLayer() override { otter_hip_conv_destroy(h_); }

    int create_pipeline(const NetOption& opt) override {
        int rc = ConvolutionLayer::create_pipeline(opt);  // int8: computes scale_in_data (ConvolutionLayer.cpp:667-679)
        if (rc) return rc;
        if (!int8_scale_term || weight_data.scalar_type() != ScalarType::Byte) return 0;  // fp32 layers: stock CPU path
        const bool pk = opt.use_packing_layout;
        const bool dw8 = in_channels == groups && groups == out_channels && in_channels % 8 == 0;
        otter_hip_conv_desc d;
        d.in_channels = in_channels, d.out_channels = out_channels;
        d.kernel_h = kernel_height, d.kernel_w = kernel_width, d.stride_h = stride_height, d.stride_w = stride_width;
        d.pad_h = padding_height, d.pad_w = padding_width, d.dilation_h = dilation_height, d.dilation_w = dilation_width;
        d.groups = groups, d.activation_type = activation_type;
        d.activation_param0 = activation_params.defined() ? activation_params.data_ptr<float>()[0] : 0.1f;
        d.out_kind = int8_scale_term > 100 ? OTTER_HIP_OUT_I8 : OTTER_HIP_OUT_F32;
        // which rounding primitive the reference's routing ends in (Tensor/QuantizeX86.cpp:402,1177-1179,1729)
        d.in_round_mode = (pk && in_channels % 8 == 0) ? OTTER_HIP_ROUND_SSE : OTTER_HIP_ROUND_EXACT;
        d.out_round_mode = (pk && (dw8 || out_channels % 4 == 0)) ? OTTER_HIP_ROUND_SSE : OTTER_HIP_ROUND_EXACT;
        const float* top = int8_scale_term > 100 ? top_blob_int8_scales.data_ptr<float>() : nullptr;
        return otter_hip_conv_create(&d, (const int8_t*)weight_data.data_ptr(), scale_in_data.data_ptr<float>(),
                                     bias_term ? bias_data.data_ptr<float>() : nullptr,
                                     bottom_blob_int8_scales.data_ptr<float>()[0], top, top ? 1 : 0, &h_);
    }

    int forward(const Tensor& bottom_blob, Tensor& top_blob, const NetOption& opt) const override {
        if (!h_) return ConvolutionLayer::forward(bottom_blob, top_blob, opt);
        const Tensor bottom = bottom_blob.contiguous();
        const int in_layout = hip_layout_of(bottom.scalar_type());
        if (in_layout < 0 || bottom.dim() != 4) return -1;
        const int n = (int)bottom.size(0), h = (int)bottom.size(2), w = (int)bottom.size(3);
        if (bottom.size(1) * bottom.elempack() != in_channels) return -1;
        int oh = 0, ow = 0;
        if (otter_hip_conv_output_shape(h_, h, w, &oh, &ow)) return -1;
        int out_layout = otter_hip_conv_default_out_layout(h_);
        if (!opt.use_packing_layout) out_layout = int8_scale_term > 100 ? OTTER_HIP_I8 : OTTER_HIP_F32;
        const size_t in_bytes = (size_t)n * in_channels * h * w * (in_layout <= OTTER_HIP_F32_P8 ? 4 : 1);
        const size_t out_bytes = (size_t)n * out_channels * oh * ow * (int8_scale_term > 100 ? 1 : 4);
        const size_t ws_bytes = otter_hip_conv_workspace_bytes(h_, in_layout, n, h, w);
        DeviceBuffer in, out, ws;
        if (otter_hip_malloc(&in.p, in_bytes) || otter_hip_malloc(&out.p, out_bytes)) return -100;
        if (ws_bytes && otter_hip_malloc(&ws.p, ws_bytes)) return -100;
        if (otter_hip_memcpy_h2d(in.p, bottom.data_ptr(), in_bytes, nullptr)) return -1;
        int rc = otter_hip_conv_forward(h_, in.p, in_layout, n, h, w, out.p, out_layout, ws.p, ws_bytes, nullptr);
        if (rc) return rc;
        top_blob = otter::empty({n, out_channels / pack_of_layout(out_layout), oh, ow}, dtype_of_layout(out_layout));
        if (otter_hip_memcpy_d2h(top_blob.data_ptr(), out.p, out_bytes, nullptr)) return -1;
        if (otter_hip_stream_synchronize(nullptr)) return -1;
        ++g_gpu_forwards;
        return 0;
    }

private:
    otter_hip_conv_t* h_ = nullptr;
};

static Layer* Creator_HipConvolutionLayer() { return new HipConvolutionLayer(); }

}  // namespace otter

extern "C" {

// Registers (on != 0) the GPU layer under "Convolution", or puts the creator that was registered before it back.
// Nets compiled afterwards use it; nets that already exist keep their layers. Returns 0, or the C ABI's status if
// the GPU cannot be initialised.
__attribute__((visibility("default"))) int otter_ref_use_hip_convolution(int on) {
    static otter::LayerRegistry::Creator stock = nullptr;
    auto& reg = otter::LayerRegistry::Registry();
    if (on) {
        const int rc = otter_hip_init(0);
        if (rc) return rc;
        if (!stock) stock = reg["Convolution"];
        otter::LayerRegistry::AddCreator("Convolution", otter::Creator_HipConvolutionLayer);
    } else if (stock) {
        otter::LayerRegistry::AddCreator("Convolution", stock);
    }
    return 0;
}

__attribute__((visibility("default"))) long otter_ref_hip_forward_count(void) { return otter::g_gpu_forwards; }

__attribute__((visibility("default"))) const char* otter_ref_hip_last_error(void) { return otter_hip_last_error(); }

}  // extern "C"
