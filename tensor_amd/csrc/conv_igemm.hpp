// Host interface of the MFMA implicit-GEMM convolution (conv_igemm.hip) and the other kernel families.
#pragma once
#include "common.hpp"

namespace ohip {

// conv_igemm.hip
int igemm_padded_rows(int K);
int igemm_channel_groups(int C);
int igemm_row_channel(int row);
// tap_pack > 1 (igemm_tap_pack): that many kernel taps of at most 64 / tap_pack channels share a reduction step
size_t igemm_packed_weight_bytes(int K, int C, int kh, int kw, int tap_pack = 1);
void igemm_pack_weights(const int8_t* w, int K, int C, int kh, int kw, int8_t* dst, int tap_pack = 1);
int igemm_tap_pack(int C, int kh, int kw);
void igemm_choose_tiles(const ConvGeom& g, int* tm, int* tn);
bool igemm_grouped_applicable(const ConvGeom& g, const Epilogue& ep);
size_t igemm_grouped_weight_bytes(int K, int C, int groups, int kh, int kw);
void igemm_pack_weights_grouped(const int8_t* w, int K, int C, int groups, int kh, int kw, int8_t* dst);
hipError_t run_conv_igemm(const int8_t* x, const int8_t* wpk, void* out, const ConvGeom& g, const Epilogue& ep, int tm,
                          int tn, hipStream_t stream);

// conv_pw.hip: 1x1 stride-1 int8 -> int8 over at most 64 input channels, streamed (reads the implicit-GEMM weight packing)
bool conv_pw_stream_applicable(const ConvGeom& g, const Epilogue& ep);
void conv_pw_stream_plan(const ConvGeom& g, int* groups, int* slices);
void conv_pw_stream_clamps(float act_hi, float round_half, const float* scale_out, int n, unsigned* dst);
hipError_t run_conv_pw_stream(const int8_t* x, const int8_t* wpk, const unsigned* qh, void* out, const ConvGeom& g,
                              const Epilogue& ep, int force_groups, int force_slices, hipStream_t stream);

// conv_block.hip: 1x1 expand -> depthwise 3x3 -> 1x1 project (+ shortcut sum, + int8 twin) as one launch
bool conv_block_applicable(const ConvGeom& ge, const Epilogue& e1, const ConvGeom& gd, const Epilogue& e2, const ConvGeom& gp,
                           const Epilogue& e3);
struct BlockArgs;
bool conv_block_plan(const ConvGeom& ge, const ConvGeom& gp, int force_rb, int force_sl, int force_split, int plan[6],
                     BlockArgs* out = nullptr);
size_t block_expand_const_bytes(int K);
void block_pack_expand_consts(const float* si, const float* bi, const float* so, int K, bool nonneg, float act_hi,
                              float round_half, int32_t* dst);
size_t block_dw_const_bytes(int C);
void block_pack_dw_consts(const int8_t* w, const float* si, const float* bi, const float* so, int C, bool nonneg, float act_hi,
                          float round_half, int32_t* dst);
hipError_t run_conv_block(const int8_t* x, const int8_t* w_exp, const int32_t* k1, const int32_t* k2, const int8_t* w_prj, void* out,
                          const ConvGeom& ge, const Epilogue& e1, const ConvGeom& gd, const Epilogue& e2, const ConvGeom& gp,
                          const Epilogue& e3, int force_rb, int force_sl, int force_split, int* workspace, hipStream_t stream);

// conv3x3.hip
bool conv3x3_halo_supported(const ConvGeom& g, const Epilogue& ep);
bool conv3x3_halo_plan(const ConvGeom& g, int force_fn, int plan[8]);
hipError_t run_conv3x3_halo(const int8_t* x, const int8_t* wpk, void* out, const ConvGeom& g, const Epilogue& ep,
                            int force_fn, hipStream_t stream);

// conv3x3_chain.hip: a chain of same-shape 3x3 int8 -> int8 layers as one persistent launch
bool conv3x3_chain_applicable(const ConvGeom& g, const Epilogue& ep, int layers, int plan[4], int force_fn = 0);
hipError_t run_conv3x3_chain(const ConvGeom& g, const Epilogue* eps, const int8_t* const* wpk, const int8_t* const* act,
                             int layers, int* error_word_out, hipStream_t stream, int force_fn = 0);
hipError_t conv3x3_chain_error(int* error_word);
hipError_t conv3x3_chain_clock_mhz(float* mhz);

// conv_direct.hip
hipError_t run_conv_direct(const int8_t* x, int in_pack, const int8_t* wt, void* out, const ConvGeom& g,
                           const Epilogue& ep, hipStream_t stream);

// conv_dw.hip
size_t dw_mfma_weight_bytes(int C, int stride, int ks);
bool dw_mfma_window_fits(int ks, int stride, int pad_w);
void dw_mfma_pack_weights(const int8_t* w, int C, int stride, int pad_w, int ks, int8_t* dst);
int dw_mfma_epilogue(const Epilogue& ep, int K);
bool dw_mfma_applicable(const ConvGeom& g, const Epilogue& ep, int epi, bool scale_out_positive);
// the same layer straight from an fp32 Float8 blob (quantize + depthwise convolution in one launch)
// a pointwise layer of at most 256 input channels straight from an fp32 Float8 blob, the blob read once (conv_pw.hip)
bool conv_pw_f32in_applicable(const ConvGeom& g, const Epilogue& ep);
hipError_t run_conv_pw_f32in(const float* x, const int8_t* wpk, const unsigned* qh, void* out, const ConvGeom& g, const Epilogue& ep,
                             const float* in_scale, int in_round_mode, int force_groups, int force_pairs, hipStream_t stream);
// a pointwise layer straight from an fp32 Float8 blob: quantize_to_int8 in the loader of the implicit-GEMM kernel
bool igemm_f32in_applicable(const ConvGeom& g, const Epilogue& ep);
hipError_t run_conv_igemm_f32in(const float* x, const int8_t* wpk, void* out, const ConvGeom& g, const Epilogue& ep,
                                const float* in_scale, int in_round_mode, hipStream_t stream);
// pointwise int8 convolution with an fp32 result + the mean over the image, one launch (conv_pw.hip)
bool conv_pw_avgpool_applicable(const ConvGeom& g, const Epilogue& ep);
hipError_t run_conv_pw_avgpool(const int8_t* x, const int8_t* wpk, float* out, const ConvGeom& g, const Epilogue& ep,
                               hipStream_t stream);
// pointwise int8 -> int8 convolution + depthwise 3x3 int8 -> int8 convolution as one launch (conv_xdw.hip)
size_t xdw_weight_bytes(int Cin, int K);
void xdw_pack_weights(const int8_t* w, int Cin, int K, int8_t* dst);
bool xdw_applicable(const ConvGeom& gx, const Epilogue& epx, int epi_x, bool sox_positive, const ConvGeom& gd, const Epilogue& ep,
                    int epi_d, bool so_positive);
hipError_t run_conv_xdw(const int8_t* x, const int8_t* wx, const int8_t* wa, void* out, const ConvGeom& gx, const Epilogue& epx,
                        const ConvGeom& g, const Epilogue& ep, int epi_d, int strip_rows, hipStream_t stream);
bool dw_f32in_applicable(const ConvGeom& g, int in_layout);
hipError_t run_conv_dw_f32in(const float* x, const int8_t* wa, void* out, const ConvGeom& g, const Epilogue& ep, int epi,
                             const float* in_scale, int in_round_mode, int strip_rows, hipStream_t stream);
hipError_t run_conv_dw_mfma(const int8_t* x, const int8_t* wa, void* out, const ConvGeom& g, const Epilogue& ep, int epi,
                            int strip_shift, hipStream_t stream);
size_t dw_packed_weight_bytes(int C, int kh, int kw);
void dw_pack_weights(const int8_t* w, int C, int kh, int kw, int32_t* dst);
hipError_t run_conv_dw(const int8_t* x, const int32_t* wmask, void* out, const ConvGeom& g, const Epilogue& ep,
                       int strip_shift, hipStream_t stream);

// elementwise.hip
hipError_t run_quantize(const float* src, int sp, int8_t* dst, int dp, int N, int C, int HW, const float* scales,
                        int n_scales, int round_mode, hipStream_t stream);
// one scale for every channel, passed by value
hipError_t run_quantize_by(const float* src, int sp, int8_t* dst, int dp, int N, int C, int HW, float scale, int round_mode,
                           hipStream_t stream);
hipError_t run_pad_pack8(const void* src, bool src_is_float, int sp, int8_t* dst, int N, int C, int Cp, int HW,
                         const float* scale, int round_mode, hipStream_t stream);
hipError_t run_dequantize(const int32_t* src, int sp, float* dst, int dp, int N, int C, int HW, const float* scale,
                          int n_scale, const float* bias, int n_bias, hipStream_t stream);
hipError_t run_requantize(const int32_t* src, int sp, int8_t* dst, int dp, int N, int C, int HW, const float* scale_in,
                          int n_scale_in, const float* scale_out, int n_scale_out, const float* bias, int n_bias,
                          int act, float act_p0, int round_mode, hipStream_t stream);
hipError_t run_repack(const void* src, int sp, void* dst, int dp, int elem_bytes, int N, int C, int HW,
                      hipStream_t stream);


// glue.hip
hipError_t run_eltwise_add(const float* a, const float* b, float* out, size_t n, hipStream_t stream);
hipError_t run_activation(float* x, size_t n, int act, float p0, hipStream_t stream);
hipError_t run_eltwise_add_quantize(const float* a, const float* b, int pack, float* out, int8_t* q, int N, int C, int HW,
                                    float scale, int round_mode, hipStream_t stream);
hipError_t run_global_avgpool(const float* x, int pack, int N, int C, int HW, float* out, hipStream_t stream);
hipError_t run_shader_clock(int blocks, int iters, unsigned long long* out, hipStream_t stream);
hipError_t run_inner_product(const float* x, const float* w, const float* b, float* y, int N, int IN, int OUT,
                             hipStream_t stream);

// conv_stem.hip: 3x3 convolution of a blob with at most 5 channels, straight from the unpacked fp32 / int8 blob
size_t stem_packed_weight_bytes(int K);
void stem_pack_weights(const int8_t* w, int K, int C, int8_t* dst);
bool conv_stem_applicable(const ConvGeom& g, const Epilogue& ep, int in_layout);
hipError_t run_conv_stem(const void* x, bool in_f32, const int8_t* wpk, void* out, const ConvGeom& g, const Epilogue& ep,
                         const float* in_scale, int in_round, hipStream_t stream);

// reshape.hip: fp32 layout glue (pack = elempack of the layout on that side)
// q (or null): also the Byte8 quantization of the copied channels, in a blob of Cd channels; needs
// copy_channels_moves_quads(...) and Cd % 8 == 0
hipError_t run_copy_channels(const float* src, int Cs, int ps, int cs0, float* dst, int Cd, int pd, int cd0, int cnt, int N,
                             int H, int W, hipStream_t stream, int8_t* q = nullptr, float scale = 0.f, int round_mode = 0);
bool copy_channels_moves_quads(int ps, int cs0, int pd, int cd0, int cnt);
// a Concat over channels in one launch (packed layouts, channel counts in multiples of 4)
constexpr int CONCAT_MAX = 8;
struct ConcatSources {
    const float* ptr[CONCAT_MAX];
    int channels[CONCAT_MAX], pack[CONCAT_MAX], first[CONCAT_MAX];  // first: destination channel of the source's channel 0
    int count;
};
hipError_t run_concat_channels(const ConcatSources& srcs, float* dst, int Cd, int pd, int N, int H, int W, int8_t* q,
                               float scale, int round_mode, hipStream_t stream);
// q (or null): also the Byte8 quantization of the shuffled blob; needs channel_shuffle_can_quantize(...)
hipError_t run_channel_shuffle(const float* src, int ps, float* dst, int pd, int N, int C, int H, int W, int groups,
                               hipStream_t stream, int8_t* q = nullptr, float scale = 0.f, int round_mode = 0);
bool channel_shuffle_can_quantize(int ps, int pd, int C, int groups);
hipError_t run_shuffle2_split(const float* a, int pa, const float* b, int pb, float* c1, float* c2, int8_t* q2, float scale,
                              int round_mode, int N, int Ch, int HW, hipStream_t stream);
hipError_t run_maxpool(const float* src, int ps, float* dst, int pd, int N, int C, int H, int W, int OH, int OW, int kh,
                       int kw, int sh, int sw, int ph, int pw, int dh, int dw, float pad_value, hipStream_t stream);
hipError_t run_upsample(const float* src, int ps, float* dst, int pd, int N, int C, int H, int W, int OH, int OW, int mode,
                        int align_corner, hipStream_t stream);

}  // namespace ohip
