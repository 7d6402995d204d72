/*
 * otter_hip_int8.h -- C ABI of the MI355X (gfx950) implementation of Otter's int8 convolution path.
 *
 * This is the only boundary that touches HIP. Plain pointers and sizes, int status codes, no C++ types.
 * Every tensor pointer is a DEVICE pointer unless a parameter says "host". Every call that launches work
 * takes the hipStream_t to launch on (as void*, NULL = the default stream) and returns without waiting
 * for the GPU. Handles are immutable after creation and may be used from several host threads.
 *
 * Each entry point names the reference interface it stands in for (paths relative to the reference
 * repository root).
 *
 * Status codes follow the reference's Layer convention (Tensor/Layer.cpp:50-59): 0 ok, -1 not supported,
 * -100 allocation failure; -2 invalid argument and -3 HIP runtime error are added. Nothing throws across
 * this boundary; otter_hip_last_error() returns the text for the calling thread's last failure.
 */
#ifndef OTTER_HIP_INT8_H
#define OTTER_HIP_INT8_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define OTTER_HIP_OK 0
#define OTTER_HIP_ERR_UNSUPPORTED (-1)
#define OTTER_HIP_ERR_INVALID (-2)
#define OTTER_HIP_ERR_RUNTIME (-3)
#define OTTER_HIP_ERR_ALLOC (-100)

/* Tensor layouts = the reference's dtype x elempack (Tensor/ScalarType.hpp:45-74). A packed tensor with
 * logical shape [N,C,H,W] is stored [N, C/p, H, W, p] (Tensor/TensorPacking.cpp:1397-1552). "I8" holds
 * signed int8 in the reference's Byte dtype. */
typedef enum {
    OTTER_HIP_F32 = 0,    /* Float   [N,C,H,W]     */
    OTTER_HIP_F32_P4 = 1, /* Float4  [N,C/4,H,W,4] */
    OTTER_HIP_F32_P8 = 2, /* Float8  [N,C/8,H,W,8] */
    OTTER_HIP_I8 = 3,     /* Byte    [N,C,H,W]     */
    OTTER_HIP_I8_P8 = 4,  /* Byte8   [N,C/8,H,W,8] */
    OTTER_HIP_I32 = 5,    /* Int     [N,C,H,W]     */
    OTTER_HIP_I32_P4 = 6, /* Int4    [N,C/4,H,W,4] */
    OTTER_HIP_I32_P8 = 7  /* Int8    [N,C/8,H,W,8] (eight int32 lanes, the depthwise accumulator type) */
} otter_hip_layout;

/* what a convolution handle produces */
typedef enum {
    OTTER_HIP_OUT_I32 = 0, /* raw accumulators: what otter::convolution returns on int8 input */
    OTTER_HIP_OUT_F32 = 1, /* dequantize_from_int32 (+ the activation layer), int8_scale_term <= 100 */
    OTTER_HIP_OUT_I8 = 2   /* requantize_from_int32_to_int8, int8_scale_term > 100 */
} otter_hip_out_kind;

/* rounding primitive of fp32 -> int8 (both saturate to [-127, 127]) */
typedef enum {
    OTTER_HIP_ROUND_SSE = 0,  /* trunc(v + copysign(0.5f, v)): float2int8_sse, Tensor/VecIntrinsic.hpp:71-95;
                                 what every packed (elempack 4/8) quantize / requantize loop uses */
    OTTER_HIP_ROUND_EXACT = 1 /* round half away from zero: float2int8, Tensor/QuantizeX86.cpp:18-23;
                                 what the unpacked loops use */
} otter_hip_round_mode;

/* ------------------------------------------------------------------------------------------------ */
/* library                                                                                          */
/* ------------------------------------------------------------------------------------------------ */

/* Selects the GPU and checks that it is a gfx950. No counterpart in the reference (Device has the single
 * value CPU, Tensor/Device.hpp:15-18). */
int otter_hip_init(int device);
int otter_hip_shutdown(void);
const char* otter_hip_last_error(void);

/* compute units, engine clock in MHz, memory clock in MHz, memory bus width in bits: inputs of the roofline */
int otter_hip_device_info(int* compute_units, int* clock_mhz, int* mem_clock_mhz, int* mem_bus_bits);
/* The shader clock the GPU holds under int8 matrix load, measured now: about a millisecond of matrix instructions on
 * every SIMD, timed with the shader-cycle counter against the constant 100 MHz counter. The published matrix peak
 * assumes the maximum engine clock of otter_hip_device_info; compute units x 4 SIMDs x 2048 int8 operations per cycle x
 * this clock is what the matrix cores can do on the box at hand. Allocates a few KB and synchronizes `stream`. No
 * counterpart in the reference (a CPU library). */
int otter_hip_shader_clock_mhz(void* stream, float* mhz);

/* Device memory + copies for hosts that do not link HIP themselves. Stand in for otter::empty() /
 * Tensor::data_ptr() ownership of blobs (Tensor/TensorFactory.hpp, Tensor/Net.cpp:413-505). */
int otter_hip_malloc(void** ptr, size_t bytes);
int otter_hip_free(void* ptr);
int otter_hip_memcpy_h2d(void* dst_dev, const void* src_host, size_t bytes, void* stream);
int otter_hip_memcpy_d2h(void* dst_host, const void* src_dev, size_t bytes, void* stream);
int otter_hip_stream_create(void** stream);
int otter_hip_stream_destroy(void* stream);
int otter_hip_stream_synchronize(void* stream);

/* ------------------------------------------------------------------------------------------------ */
/* convolution layer                                                                                */
/* ------------------------------------------------------------------------------------------------ */

typedef struct otter_hip_conv otter_hip_conv_t;

/* Mirrors the state of otter::ConvolutionLayer after load_param (Tensor/ConvolutionLayer.hpp:40-77,
 * Tensor/ConvolutionLayer.cpp:185-206). */
typedef struct {
    int in_channels, out_channels;
    int kernel_h, kernel_w;
    int stride_h, stride_w;
    int pad_h, pad_w;
    int dilation_h, dilation_w;
    int groups;
    int activation_type;     /* 0 none, 1 ReLU, 2 LeakyReLU, 3 clip [0,6], 4 sigmoid, 5 mish
                                (Tensor/ConvolutionLayer.cpp:113-122, Tensor/QuantizeX86.hpp:72-106; the layer's
                                option strings select 1-4, mish exists in the requantize function only). 4 and 5
                                are evaluated with the device's exp / log / tanh: the reference's values come
                                from polynomial approximations and an approximate-reciprocal instruction, so an
                                int8 result may differ from it by one step where the scaled value is at a
                                rounding tie. */
    float activation_param0; /* LeakyReLU slope */
    int out_kind;            /* otter_hip_out_kind */
    int out_round_mode;      /* otter_hip_round_mode used when out_kind is I8 */
    int in_round_mode;       /* otter_hip_round_mode used when forward() is handed fp32 input */
} otter_hip_conv_desc;

/* ConvolutionLayer::create_pipeline_int8 (Tensor/ConvolutionLayer.cpp:666-752): uploads and re-lays-out the
 * int8 weights once. All array arguments are HOST pointers:
 *   weight    [K, C/groups, kh, kw] int8  (ConvolutionLayer::weight_data)
 *   scale_in  [K]  = 1/(in_scale*weight_scale[k]), computed by the caller exactly as :667-679 does; it is
 *                    never recomputed on the device
 *   bias      [K] or NULL                  (ConvolutionLayer::bias_data)
 *   in_scale  bottom_blob_int8_scales[0], used only when forward() receives fp32 input
 *   out_scale [n_out_scale] (1 or K), top_blob_int8_scales, used only for OTTER_HIP_OUT_I8 */
int otter_hip_conv_create(const otter_hip_conv_desc* desc, const int8_t* weight, const float* scale_in,
                          const float* bias, float in_scale, const float* out_scale, int n_out_scale,
                          otter_hip_conv_t** handle);
int otter_hip_conv_destroy(otter_hip_conv_t* handle);

/* Output geometry (Tensor/ConvolutionUtils.hpp:173-191) and the layout the reference would produce for
 * this layer in packing mode (Tensor/ConvolutionLayer.cpp:777-787, Tensor/QuantizeX86.cpp:650-653,1729). */
int otter_hip_conv_output_shape(const otter_hip_conv_t* handle, int in_h, int in_w, int* out_h, int* out_w);
int otter_hip_conv_default_out_layout(const otter_hip_conv_t* handle);

/* Bytes of device scratch forward() needs for this input (0 unless the input is fp32: the quantized copy). */
size_t otter_hip_conv_workspace_bytes(const otter_hip_conv_t* handle, int in_layout, int n, int in_h, int in_w);

/* ConvolutionLayer::forward_int8 (Tensor/ConvolutionLayer.cpp:754-847) for a whole batch:
 * [quantize_to_int8 ->] convolution -> dequantize_from_int32 (+activation) | requantize_from_int32_to_int8.
 *   in_layout : I8_P8 or I8 (already quantized blob, :770-775) or F32 / F32_P4 / F32_P8 (quantized first
 *               with in_scale; needs `workspace`)
 *   out_layout: any layout whose element type matches out_kind and whose pack divides K
 * Batch images are independent (the reference runs them one by one, Tensor/Padding.cpp:26-29). */
int otter_hip_conv_forward(const otter_hip_conv_t* handle, const void* in, int in_layout, int n, int in_h, int in_w,
                           void* out, int out_layout, void* workspace, size_t workspace_bytes, void* stream);

/* No counterpart in the reference. For callers that cannot allocate device memory -- code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc: otter_hip_conv_forward with the workspace (the quantized copy
 * of an fp32 input, or the channel-padded copy of a blob with C % 8 != 0) taken from a static device array of
 * OTTER_HIP_STATIC_WORKSPACE_BYTES that the library holds on every GPU it runs on for the life of the process. Makes
 * no hipMalloc / hipFree call. An input whose otter_hip_conv_workspace_bytes exceeds the array is refused with
 * OTTER_HIP_ERR_UNSUPPORTED. Every call on one GPU shares that GPU's array: calls that overlap on one GPU (different
 * streams or host threads) race; calls on one stream are ordered. Same results as otter_hip_conv_forward. */
#define OTTER_HIP_STATIC_WORKSPACE_BYTES (32u << 20)
int otter_hip_conv_forward_static(const otter_hip_conv_t* handle, const void* in, int in_layout, int n, int in_h,
                                  int in_w, void* out, int out_layout, void* stream);

/* The same forward for a layer with an fp32 result (out_kind F32, K % 8 == 0) whose top blob is read by int8
 * convolutions next: besides `out`, writes what each of those readers would compute first, its quantize_to_int8 of the
 * blob (Tensor/ConvolutionLayer.cpp:770-775), out_q = float2int8(out * q_scale) as Byte8 [N][K/8][OH*OW][8].
 * q_scale = the readers' bottom_blob_int8_scales[0], q_round_mode = their input rounding primitive. The implicit-GEMM
 * kernel writes out_q from its own epilogue (Float4 output, clamp-type activation); every other case runs the
 * quantize pass after the convolution, with the same result. */
int otter_hip_conv_forward_twin(const otter_hip_conv_t* handle, const void* in, int in_layout, int n, int in_h,
                                int in_w, void* out, int out_layout, void* out_q, float q_scale, int q_round_mode,
                                void* workspace, size_t workspace_bytes, void* stream);

/* The tail of a residual block in one call: an int8 convolution with an fp32 result followed by the Eltwise sum with
 * the block's shortcut (Tensor/ConvolutionLayer.cpp:754-847, then Tensor/EltwiseLayer.cpp:48-80), out =
 * activation(convolution) + residual, both in out_layout, same shape. With out_q (or null; needs K % 8 == 0) also the
 * quantize_to_int8 of the sum for the int8 convolutions that read it, as in otter_hip_conv_forward_twin. The
 * convolution's own result is not stored anywhere: use this only when the Eltwise layer is its sole reader. The
 * implicit-GEMM kernel adds (and quantizes) in its epilogue (Float4 output, clamp-type activation); every other case
 * runs the separate passes behind the convolution, with the same result. */
int otter_hip_conv_forward_residual(const otter_hip_conv_t* handle, const void* in, int in_layout, int n, int in_h,
                                    int in_w, const float* residual, void* out, int out_layout, void* out_q,
                                    float q_scale, int q_round_mode, void* workspace, size_t workspace_bytes,
                                    void* stream);

/* A chain of layers that each map an int8 Byte8 blob to an int8 Byte8 blob (consecutive Convolution layers of a
 * Net, Tensor/Net.cpp:413-505 runs them one after the other): out = layer[n-1](... layer[0](in)). The result is what
 * n calls of otter_hip_conv_forward give. The intermediate blobs live in `workspace`
 * (otter_hip_conv_chain_workspace_bytes, one buffer per intermediate blob). Where all layers are the same 3x3
 * stride-1 pad-1 geometry with 33..128 channels, the chain runs as ONE persistent launch in which a tile of a layer
 * starts as soon as the tiles of the previous layer it reads are done; otherwise as n launches. The single launch
 * waits on flags between workgroups; every wait is bounded, and otter_hip_conv_chain_status reports (after
 * synchronizing the device) whether one ever gave up, in which case the outputs of the chain calls since the last
 * status call are not valid. The flags live in static device memory, four sets per GPU. A set belongs to the stream
 * that launched on it last (calls on different streams may overlap); a stream without one takes a free set or the
 * least recently used set whose last launch has completed, and only when all four are busy does a call run its chain
 * as n launches (otter_hip_conv_chain_last_launches tells). Like every entry point here it allocates nothing, and
 * after one eager call on a stream it may be captured into a HIP graph on that stream and replayed (a launch takes
 * its sequence number from device memory, not from the kernel arguments); the set a captured call was given stays
 * with the capturing stream for the life of the process, so do not replay such a graph on another stream while that
 * stream runs chains of its own. */
size_t otter_hip_conv_chain_workspace_bytes(const otter_hip_conv_t* const* handles, int n_layers, int n, int in_h, int in_w);
int otter_hip_conv_chain_forward(const otter_hip_conv_t* const* handles, int n_layers, const void* in, int n, int in_h,
                                 int in_w, void* out, void* workspace, size_t workspace_bytes, void* stream);
int otter_hip_conv_chain_status(int* gave_up);
/* The number of convolution launches the last otter_hip_conv_chain_forward on the calling host thread actually made
 * (1: the single persistent launch; n_layers: layer by layer, also when every flag set was busy; 0: none yet). The
 * reference has no counterpart (its Net runs a layer per call, Tensor/Net.cpp:413-505). */
int otter_hip_conv_chain_last_launches(void);
/* The shader clock the most recent single-launch chain on this GPU ran at, in MHz (0: there has been none): its last
 * workgroup reads the shader-cycle counter and the constant 100 MHz counter over its life. For the roofline: the
 * published matrix peak assumes the maximum engine clock, a kernel that keeps matrix cores, vector ALU and LDS busy
 * holds less. Synchronizes the device. No counterpart in the reference. */
int otter_hip_conv_chain_clock_mhz(float* mhz);
/* For tests and profiling: the number of convolution launches otter_hip_conv_chain_forward makes for this chain and
 * input (1: the single persistent launch; n_layers: layer by layer), or a negative status. */
int otter_hip_conv_chain_launches(const otter_hip_conv_t* const* handles, int n_layers, int n, int in_h, int in_w);
/* Tuning / test hook with no counterpart in the reference: the single launch is only used where one layer's share
 * of an XCD's tile list (images / 8 x tiles per image) is at least `tiles` (default 96: below that the tiles' producers
 * are still running when they are reached, and the layers one by one are faster). 0 makes every chain that qualifies
 * by shape a single launch (the tests do that on small shapes). Process-wide; returns the previous value; a negative
 * argument only queries. */
int otter_hip_conv_chain_set_min_tiles(int tiles);

/* An inverted-residual block as networks spell it -- a 1x1 Convolution (int8 result), a depthwise 3x3 Convolution
 * (int8 result) and a 1x1 Convolution, each read only by the next (Tensor/Net.cpp:413-505 runs them one after the other,
 * ConvolutionLayer::forward_int8, Tensor/ConvolutionLayer.cpp:754-847, three times), optionally followed by the Eltwise
 * sum with the block's shortcut (Tensor/EltwiseLayer.cpp:48-80). `in` is the Byte8 input of the first layer; out is the
 * last layer's result: fp32 in OTTER_HIP_F32_P4 (then `residual`, or NULL, is a blob of that layout added to it, and
 * out_q, or NULL, receives the Byte8 quantization float2int8(out * q_scale) with q_round_mode, as in
 * otter_hip_conv_forward_residual / _twin) or int8 Byte8 (residual and out_q NULL). The result is what the three (four)
 * calls give, bit for bit. Where the depthwise layer is stride 1 pad 1 on an image at most 64 pixels wide, the first
 * layer reads at most 192 channels and the activations are none / ReLU / clip, the block can run as ONE launch that
 * keeps the expanded tensor in LDS; it does (otter_hip_conv_block_launches says 1) for the
 * shapes where that was measured faster than the three launches (images up to 28 pixels wide, 128..512 workgroups
 * over the batch, at most 24 tiles of 32 channels x 16 pixels of the last layer per band), or for every shape that qualifies after
 * otter_hip_conv_block_set_always(1) / a forced plan. Where a batch has fewer bands than half the compute units, the
 * expanded channels of a band are dealt to several workgroups whose accumulators meet in `workspace` (the last to
 * arrive adds them up: integer sums, the same result). Otherwise, where the first layer reads at most 128 channels and
 * writes a multiple of 16, the depthwise layer is 3x3 stride 1 / 2 on an image at most 128 pixels wide (64 when the first
 * layer reads more than 32 channels) and both clamp at zero or neither clamps, the first two layers can run as ONE
 * launch that keeps the expanded rows in LDS, the last layer by itself; they do (otter_hip_conv_block_launches says 2)
 * where that was measured faster, or wherever they can after otter_hip_conv_block_set_pair(1); any other block makes
 * three launches. The blobs between the launches live in `workspace`;
 * otter_hip_conv_block_workspace_bytes gives the size either way (0 for a single launch with one workgroup per band). */
int otter_hip_conv_block_launches(const otter_hip_conv_t* expand, const otter_hip_conv_t* depthwise,
                                  const otter_hip_conv_t* project, int n, int in_h, int in_w);
size_t otter_hip_conv_block_workspace_bytes(const otter_hip_conv_t* expand, const otter_hip_conv_t* depthwise,
                                            const otter_hip_conv_t* project, int n, int in_h, int in_w);
int otter_hip_conv_block_forward(const otter_hip_conv_t* expand, const otter_hip_conv_t* depthwise,
                                 const otter_hip_conv_t* project, const void* in, int n, int in_h, int in_w,
                                 const float* residual, void* out, int out_layout, void* out_q, float q_scale,
                                 int q_round_mode, void* workspace, size_t workspace_bytes, void* stream);
/* Test hook with no counterpart in the reference, host arithmetic only (no GPU needed): the launch plan of the single
 * launch for a block in_channels -> expanded_channels -> out_channels on n images of in_h x in_w (stride-1 depthwise
 * layer), with rows_per_band / slice_channels / split forced (0 = automatic). plan = { output rows per band, bands per
 * image, expanded channels per slice, LDS bytes per workgroup, workgroups per band (each takes a share of the slices),
 * 32-bit words of workspace for their accumulators }. -1 when the single launch cannot take the shape. */
int otter_hip_conv_block_plan(int in_channels, int expanded_channels, int out_channels, int n, int in_h, int in_w,
                              int rows_per_band, int slice_channels, int split, int plan[6]);
/* Tuning / test hook with no counterpart in the reference: 1 = every block that qualifies by shape runs as the single
 * launch, 0 = only the shapes measured faster that way (default), 2 = none does. Process-wide; returns the previous
 * value; a negative argument only queries. */
int otter_hip_conv_block_set_always(int on);
/* Tuning / test hook with no counterpart in the reference: how a block that does not run as the single launch runs its
 * first two layers: 0 = as one launch where that was measured faster (a stride-2 depthwise layer, or an expanded blob
 * of 16 MiB or more; default), 1 = wherever the kernel takes the shapes, -1 = always one by one. Process-wide; returns
 * the previous value; any other argument only queries. */
int otter_hip_conv_block_set_pair(int mode);
/* Tuning / test hook with no counterpart in the reference: force the single launch's output rows per band, the
 * expanded channels per LDS slice (64 or 128) and the workgroups a band's slices are dealt to, for blocks whose first
 * layer is `expand`; 0 = automatic. */
int otter_hip_conv_block_set_plan(otter_hip_conv_t* expand, int rows_per_band, int slice_channels, int split);

/* Which kernel family forward() would launch for this input: 0 direct (scalar fallback), 1 MFMA implicit
 * GEMM, 2 depthwise, 3 MFMA 3x3 halo kernel, 4 few-channel 3x3 kernel (an image stem read straight from the unpacked
 * blob), 5 streamed 1x1 kernel (int8 -> int8 over at most 64 input channels), 6 pointwise layer on an fp32 Float8 blob
 * of 64..256 channels, quantize and convolution in one launch that reads the blob once. (Other pointwise and depthwise 3x3
 * layers on an fp32 Float8 blob also quantize inside the convolution's launch; they report 1 and 2.) For tests and
 * profiling. */
int otter_hip_conv_kernel_kind(const otter_hip_conv_t* handle, int in_layout, int n, int in_h, int in_w,
                               int out_layout);

/* Tuning / test hook with no counterpart in the reference. (0, 0): automatic choice. tm > 0: force the generic
 * MFMA implicit-GEMM kernel with a tile of tm output channels x tn pixels (tm in {32,64,128}, tn in
 * {64,128,256}; tn + 1 forces the kernel variant that stages one 64-deep slice of the reduction at a time, tn + 2 the
 * variant that stages several, tn alone leaves that choice automatic). tm < 0: keep the 3x3 halo kernel where it applies and force its pixel-fragment count to tn
 * (4..7, 0 = automatic; set on the first layer of a chain it also applies to otter_hip_conv_chain_forward's single
 * launch). tm == -2 on a depthwise 3x3 layer: force the matrix-core kernel's strip height to tn
 * steps of 8 / stride output rows (0 = automatic). tm == -3: use the vector-ALU depthwise kernels instead, with a
 * strip height of (8 >> tn) output rows for stride 1 and (4 >> tn) for stride 2, tn in 0..2. tm == -4: the generic
 * implicit-GEMM kernel with its automatic tile choice, where the LDS-halo or the streamed 1x1 kernel would be picked.
 * tm == -5 on a layer the streamed 1x1 kernel takes: tn = groups | slices << 3 forces the 16-pixel groups a wave owns
 * (2 or 4) and the slices the output channels are cut into (0 = automatic for either). tm == -6: quantize an fp32 blob
 * in a launch of its own (the two launches of the reference's order) where the convolution's launch would do it.
 * tm == -7 on a pointwise layer: kernel 6 above wherever it can run, tn = groups | pairs << 3 forcing the 16-pixel
 * groups a wave owns (1 or 2) and the pairs of 16 output channels per LDS round (0 = automatic for either). */
int otter_hip_conv_set_tile(otter_hip_conv_t* handle, int tm, int tn);

/* Test hook with no counterpart in the reference, host arithmetic only (no GPU needed): the launch plan of the 3x3
 * stride-1 LDS-halo kernel for a dense layer of this shape. plan = { pixel fragments per wave, pixels per tile, tiles
 * per image, persistent workgroups (grid.x), row blocks (grid.y), 1 if a workgroup reuses the per-lane LDS offsets of
 * its first tile for its later tiles, LDS rows per tile, input channels per LDS stage }. Workgroup b walks tiles
 * b, b + grid.x, ...; tile t (after the XCD swizzle t' = (t % 8) * (T / 8) + t / 8 for t < 8 * (T / 8), T = all tiles)
 * is pixels [ (t' % tiles_per_image) * pixels_per_tile, ... ) of image t' / tiles_per_image. */
int otter_hip_conv3x3_halo_plan(int in_channels, int out_channels, int pad, int n, int in_h, int in_w, int force_fn,
                                int plan[8]);

/* ------------------------------------------------------------------------------------------------ */
/* standalone quantize / dequantize / requantize                                                    */
/* ------------------------------------------------------------------------------------------------ */

/* otter::quantize_to_int8 (Tensor/Quantize.hpp:15, Tensor/QuantizeX86.cpp:47-644):
 * q = sat127(round(x * scale[n_scales == 1 ? 0 : c])). scales is a DEVICE array. */
int otter_hip_quantize(const float* src, int src_layout, int n, int c, int h, int w, const float* scales,
                       int n_scales, int round_mode, int8_t* dst, int dst_layout, void* stream);

/* otter::dequantize_from_int32 (Tensor/Quantize.hpp:17, Tensor/QuantizeX86.cpp:646-1161):
 * y = fma(float(acc), scale[c], bias[c]) (bias may be NULL). scale / bias are DEVICE arrays. */
int otter_hip_dequantize(const int32_t* src, int src_layout, int n, int c, int h, int w, const float* scale,
                         int n_scale, const float* bias, int n_bias, float* dst, int dst_layout, void* stream);

/* otter::requantize_from_int32_to_int8 (Tensor/Quantize.hpp:19, Tensor/QuantizeX86.cpp:1163-2129):
 * v = fma(float(acc), scale_in[c], bias[c]); v = act(v); q = sat127(round(v * scale_out[c])). */
int otter_hip_requantize(const int32_t* src, int src_layout, int n, int c, int h, int w, const float* scale_in,
                         int n_scale_in, const float* scale_out, int n_scale_out, const float* bias, int n_bias,
                         int activation_type, float activation_param0, int round_mode, int8_t* dst,
                         int dst_layout, void* stream);

/* Tensor::packing (Tensor/Tensor.cpp:29-35, Tensor/TensorPacking.cpp:141-158): re-pack between layouts of
 * the same element type on the device (what Net::convert_layout does on the host, Tensor/Net.cpp:380-411). */
int otter_hip_repack(const void* src, int src_layout, int n, int c, int h, int w, void* dst, int dst_layout,
                     void* stream);

/* ------------------------------------------------------------------------------------------------ */
/* fp32 glue between the int8 layers of a network (all pointers are device pointers)                */
/* ------------------------------------------------------------------------------------------------ */

/* EltwiseLayer::forward, operation sum (Tensor/EltwiseLayer.cpp:48-80): out = a + b over `count` floats of two
 * blobs in the same layout. */
int otter_hip_eltwise_add(const float* a, const float* b, float* out, size_t count, void* stream);

/* The same sum and, in the same pass, what the int8 convolution that reads it would compute first: its
 * quantize_to_int8 of the fp32 bottom blob (ConvolutionLayer::forward_int8, Tensor/ConvolutionLayer.cpp:770-775),
 * q = float2int8(out * scale) written as Byte8. a, b, out in `layout` (OTTER_HIP_F32_P4 or _P8), c % 8 == 0;
 * scale = the consumer's bottom_blob_int8_scales[0], round_mode = its input rounding primitive. */
int otter_hip_eltwise_add_quantize(const float* a, const float* b, int layout, int n, int c, int h, int w, float scale,
                                   int round_mode, float* out, int8_t* q, void* stream);

/* ReluLayer / LReluLayer / Relu6Layer / SigmoidLayer::forward_inplace (Tensor/ReluLayer.cpp, LReluLayer.cpp:45-,
 * Relu6Layer.cpp:29-100) on a device blob; activation_type as in otter_hip_conv_desc. */
int otter_hip_activation(float* x, size_t count, int activation_type, float activation_param0, void* stream);

/* Global average pooling to [N, C] (unpacked). The reference registry has no average-pooling layer
 * (Tensor/LayerDeclaration.hpp:42-68); this is the fp32 mean over H*W that the MobileNetV2-style network needs. */
int otter_hip_global_avgpool(const float* src, int src_layout, int n, int c, int h, int w, float* dst, void* stream);

/* ConvolutionLayer::forward_int8 (Tensor/ConvolutionLayer.cpp:754-847) of a layer with an fp32 result, followed by the
 * mean over H*W of that result to out[N, K] (what otter_hip_global_avgpool computes; the tail of a classifier). For a
 * pointwise layer on a Byte8 input and an image of at most 64 pixels it is ONE launch and the layer's own blob is
 * never made (otter_hip_conv_avgpool_launches says 1, the workspace is 0 bytes); otherwise the layer runs into
 * `workspace` and the mean is taken from there. The convolution's values are those of otter_hip_conv_forward bit for
 * bit; their sum is taken in another order than otter_hip_global_avgpool takes it (fp32, same tolerance). */
int otter_hip_conv_avgpool_launches(const otter_hip_conv_t* conv, int in_layout, int n, int in_h, int in_w);
size_t otter_hip_conv_avgpool_workspace_bytes(const otter_hip_conv_t* conv, int in_layout, int n, int in_h, int in_w);
int otter_hip_conv_forward_avgpool(const otter_hip_conv_t* conv, const void* in, int in_layout, int n, int in_h, int in_w,
                                   float* out, void* workspace, size_t workspace_bytes, void* stream);

/* InnerProductLayer::forward, fp32 (Tensor/InnerProductLayer.cpp:176-): y[n][o] = sum_i x[n][i]*weight[o][i] + bias[o].
 * bias may be NULL. */
int otter_hip_inner_product(const float* x, int n, int in_features, const float* weight, const float* bias,
                            int out_features, float* y, void* stream);

/* ------------------------------------------------------------------------------------------------ */
/* fp32 layout glue of the reference's int8 model files (benchmark/nanodet-plus-m-1.5x_416_int8_*.otter):  */
/* every blob between their convolutions is fp32; src and dst may be in any fp32 layout each          */
/* ------------------------------------------------------------------------------------------------ */

/* dst[:, dst_c0 : dst_c0+count] = src[:, src_c0 : src_c0+count] over channels. One call per input is
 * ConcatLayer::forward with axis 1 (Tensor/ConcatLayer.cpp:54-67); with dst_c = count, dst_c0 = 0 it is
 * CropLayer::forward with axis 1 (Tensor/CropLayer.cpp:69-75, native::slice on the logical channel index). */
int otter_hip_copy_channels(const float* src, int src_layout, int src_c, int src_c0, float* dst, int dst_layout,
                            int dst_c, int dst_c0, int count, int n, int h, int w, void* stream);

/* The same copy and, in the same pass, the copied channels of what an int8 convolution reading dst would compute
 * first: its quantize_to_int8 of the blob (Tensor/ConvolutionLayer.cpp:770-775), dst_q = float2int8(dst * scale) as
 * Byte8 [N][dst_c/8][H*W][8]. One call per input of a Concat layer fills the whole of dst_q. Both layouts packed
 * (F32_P4 / F32_P8), dst_c % 8 == 0, src_c0 % 4 == 0, and the destination range made of whole packs of dst_layout. */
int otter_hip_copy_channels_quantize(const float* src, int src_layout, int src_c, int src_c0, float* dst,
                                     int dst_layout, int dst_c, int dst_c0, int count, int n, int h, int w,
                                     int8_t* dst_q, float scale, int round_mode, void* stream);

/* ConcatLayer::forward with axis 1 (Tensor/ConcatLayer.cpp:54-67) in one launch: `count` (1 to 8) blobs of one batch
 * size and image size, src_channels[i] channels each in layout src_layouts[i], one after the other along the channel
 * axis of dst. Packed layouts only (F32_P4 / F32_P8 on every side; otter_hip_copy_channels covers the rest). With dst_q
 * (or NULL; needs a channel sum divisible by 8) also the quantize_to_int8 of dst that an int8 convolution reading it
 * would compute first (Tensor/ConvolutionLayer.cpp:770-775): dst_q = float2int8(dst * scale) as Byte8. */
int otter_hip_concat_channels(const float* const* srcs, const int* src_layouts, const int* src_channels, int count,
                              float* dst, int dst_layout, int n, int h, int w, int8_t* dst_q, float scale,
                              int round_mode, void* stream);

/* ChannelShuffleLayer::forward (Tensor/ChannelShuffleLayer.cpp:37-41, Tensor/ChannelShuffleKernel.cpp:19-55):
 * out[:, j*groups + i] = in[:, i*(C/groups) + j]. */
int otter_hip_channel_shuffle(const float* src, int src_layout, float* dst, int dst_layout, int n, int c, int h, int w,
                              int groups, void* stream);

/* The same shuffle and, in the same pass, what an int8 convolution reading dst would compute first: its
 * quantize_to_int8 of the blob (Tensor/ConvolutionLayer.cpp:770-775), dst_q = float2int8(dst * scale) as Byte8. For the
 * ShuffleNetV2 case only: 2 groups, F32_P8 on both sides, C % 16 == 0. */
int otter_hip_channel_shuffle_quantize(const float* src, int src_layout, float* dst, int dst_layout, int n, int c,
                                       int h, int w, int groups, int8_t* dst_q, float scale, int round_mode,
                                       void* stream);

/* The tail of a ShuffleNetV2 unit as the reference's model files spell it -- ConcatLayer(a, b) -> ChannelShuffleLayer with
 * 2 groups -> two CropLayers taking the first and the second half of the channels (Tensor/ConcatLayer.cpp:54-67,
 * Tensor/ChannelShuffleKernel.cpp:19-55, Tensor/CropLayer.cpp:69-75) -- in one pass: first_half[2j+i] = (i ? b : a)[j],
 * second_half[2j+i] = (i ? b : a)[channels_each/2 + j]. The outputs are Float8 (OTTER_HIP_F32_P8), a and b each Float4 or
 * Float8; channels_each % 8 == 0.
 * second_half_q (may be NULL): the Byte8 quantization of second_half, float2int8(v * scale) with round_mode, for the int8
 * convolution that reads that half next (its quantize_to_int8, Tensor/ConvolutionLayer.cpp:770-775). */
int otter_hip_shuffle2_split(const float* a, int a_layout, const float* b, int b_layout, int n, int channels_each, int h,
                             int w, float* first_half, float* second_half, int8_t* second_half_q, float scale,
                             int round_mode, void* stream);

/* MaxPoolLayer::forward (Tensor/MaxPoolLayer.cpp:123-134): max over a kernel window of the padded input; out_h /
 * out_w as MaxPoolLayer::compute_output_shape gives them (Tensor/Pool.hpp:33-50). pad_value is what a tap outside
 * the image counts as: -INFINITY in the reference's generic kernel, 0 in its packed 3x3 and 2x2 stride-2 kernels,
 * which pad the blob with zeros first (Tensor/Pool.cpp:752-1160; selection rule at :1185-1199). */
int otter_hip_maxpool2d(const float* src, int src_layout, int n, int c, int h, int w, int kernel_h, int kernel_w,
                        int stride_h, int stride_w, int pad_h, int pad_w, int dilation_h, int dilation_w, int out_h,
                        int out_w, float pad_value, float* dst, int dst_layout, void* stream);

/* UpsampleLayer::forward (Tensor/UpsampleLayer.cpp:108-124) through otter::Interpolate's packed path
 * (Tensor/TensorInterpolation.cpp:16-45 coefficients, :161-272 bilinear, :670-690 nearest), which is what the
 * reference's Net runs for channel counts that are multiples of 4. mode 1 nearest, 2 bilinear. */
int otter_hip_upsample2d(const float* src, int src_layout, int n, int c, int h, int w, int out_h, int out_w, int mode,
                         int align_corner, float* dst, int dst_layout, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* OTTER_HIP_INT8_H */