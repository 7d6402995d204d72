/* TEST INFRASTRUCTURE -- CPU restatement of the reference's int8 convolution arithmetic.
 *
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load this library, and only
 * as the checker. The shipped GPU library never links, loads or falls back to anything in oracle/.
 *
 * All tensors are plain NCHW arrays (elempack 1). "Byte" tensors hold signed int8, as in the reference
 * (Tensor/ConvolutionMM2D.cpp:611-633 casts to signed char).
 */
#ifndef OTTER_INT8_ORACLE_H
#define OTTER_INT8_ORACLE_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* rounding primitive selected by the reference's routing */
enum {
    OTTER_ORACLE_ROUND_SSE = 0,   /* float2int8_sse: trunc(v + copysign(0.5f, v)), Tensor/VecIntrinsic.hpp:71-95 */
    OTTER_ORACLE_ROUND_EXACT = 1  /* float2int8: (int)round(v), Tensor/QuantizeX86.cpp:18-23 */
};

int8_t otter_oracle_float2int8(float v, int round_mode);
float otter_oracle_activation(float v, int act_type, const float* act_params);

/* which rounding primitive the reference ends up in */
int otter_oracle_quantize_round_mode(int channels, int use_packing);
int otter_oracle_requantize_round_mode(int in_channels, int out_channels, int groups, int use_packing);

void otter_oracle_scale_in(const float* weight_scales, int out_channels, float in_scale, float* scale_in);

void otter_oracle_quantize(const float* x, int n, int c, int h, int w, const float* scales, int n_scales,
                           int round_mode, int8_t* out);

int otter_oracle_conv_out_size(int in, int kernel, int stride, int pad, int dilation);

int otter_oracle_conv_int32(const int8_t* x, int n, int c, int h, int w, const int8_t* wt, int k, int kh, int kw,
                            int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, int groups,
                            int32_t* out);

void otter_oracle_dequantize(const int32_t* acc, int n, int c, int hw, const float* scale, int n_scale,
                             const float* bias, int n_bias, float* out);

void otter_oracle_requantize(const int32_t* acc, int n, int c, int hw, const float* scale_in, int n_scale_in,
                             const float* scale_out, int n_scale_out, const float* bias, int n_bias, int act_type,
                             const float* act_params, int round_mode, int8_t* out);

void otter_oracle_activation_f32(float* x, size_t count, int act_type, const float* act_params);

/* whole ConvolutionLayer::forward_int8 on a batch. in_is_int8: x is int8 (quantize skipped) else fp32.
 * int8_out: int8_scale_term > 100. acc_out may be NULL. Returns 0, or -1 for a shape the reference rejects. */
int otter_oracle_conv_layer_forward(const void* x, int in_is_int8, int n, int c, int h, int w, const int8_t* wt,
                                    int k, int kh, int kw, int stride_h, int stride_w, int pad_h, int pad_w,
                                    int dil_h, int dil_w, int groups, const float* bias,
                                    const float* weight_scales, int n_wscales, float in_scale, float top_scale,
                                    int int8_out, int act_type, const float* act_params, int use_packing,
                                    int32_t* acc_out, void* out);

/* reference channel packing [N,C,H,W] <-> [N,C/p,H,W,p] (Tensor/TensorPacking.cpp:1397-1552) */
void otter_oracle_pack(const void* src, size_t elem_bytes, int n, int c, int hw, int p, void* dst);
void otter_oracle_unpack(const void* src, size_t elem_bytes, int n, int c, int hw, int p, void* dst);

/* glue ops used by the network-level checks */
void otter_oracle_eltwise_add(const float* a, const float* b, size_t count, float* out);
void otter_oracle_global_avgpool(const float* x, int n, int c, int hw, float* out);
void otter_oracle_inner_product(const float* x, int n, int in_f, const float* wt, const float* bias, int out_f,
                                float* out);

void otter_oracle_set_num_threads(int n);
int otter_oracle_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif
