"""Case table shared by the golden-vector generator and the tests that replay the vectors.

Every case stays inside what the reference itself executes correctly in packed mode (groups == 1 or
depthwise with C % 8 == 0, batch looped, no C % 8 != 0 with K % 4 != 0); the shapes it crashes or hangs on
(packed C=3 K=4 1x1, grouped non-depthwise, depthwise with C % 8 != 0, unpacked depthwise) are never sent to the
compiled reference.
"""

# name, C, K, kernel, stride, pad, dilation, groups, H, W, N, in_is_int8, int8_out, bias, activation, act_params
LAYER_CASES = [
    ("c0_like_3x3_f32_f32",          8,  8, 3, 1, 1, 1,  1, 10,  9, 2, False, False, False, "",      None),
    ("c2_like_1x1_bias_relu_f32",   16, 16, 1, 1, 0, 1,  1,  7,  6, 2, False, False, True,  "Relu",  None),
    ("c3_like_3x3_i8_i8_relu",      16, 16, 3, 1, 1, 1,  1,  9,  8, 2, True,  True,  True,  "Relu",  None),
    ("stem_3x3s2_c3_relu6_i8",       3,  8, 3, 2, 1, 1,  1, 13, 11, 2, False, True,  True,  "Relu6", None),
    ("stem_3x3s1_c3_f32",            3,  8, 3, 1, 1, 1,  1,  8,  8, 1, False, False, True,  "",      None),
    ("pack8to1_3x3_k6_f32",          8,  6, 3, 1, 1, 1,  1,  8,  6, 1, False, False, True,  "Relu",  None),
    ("pack8to1_3x3_k6_i8",           8,  6, 3, 1, 1, 1,  1,  7,  5, 2, True,  True,  True,  "Relu",  None),
    ("k12_1x1s2_i8_byte1",          16, 12, 1, 2, 0, 1,  1,  9,  9, 1, True,  True,  False, "",      None),
    ("dilated_3x3d2_i8",             8,  8, 3, 1, 2, 2,  1,  9,  9, 1, True,  True,  True,  "Relu",  None),
    ("lrelu_3x3_i8",                 8, 16, 3, 1, 1, 1,  1,  6,  7, 1, False, True,  True,  "LRelu", [0.2]),
    ("relu6_1x1_f32",               24, 16, 1, 1, 0, 1,  1,  6,  6, 1, True,  False, True,  "Relu6", None),
    ("c64k32_3x3s2_i8",             64, 32, 3, 2, 1, 1,  1, 12, 12, 1, True,  True,  True,  "Relu",  None),
    ("c128k128_3x3_i8",            128,128, 3, 1, 1, 1,  1,  6,  6, 1, True,  True,  True,  "Relu",  None),
    ("k5x5_c8_i8",                   8,  8, 5, 1, 2, 1,  1,  9,  7, 1, True,  True,  True,  "",      None),
    ("dw_c1_like_3x3s1_relu6",      16, 16, 3, 1, 1, 1, 16, 12, 10, 2, False, True,  True,  "Relu6", None),
    ("dw_c1_like_3x3s2_relu6",      16, 16, 3, 2, 1, 1, 16, 12, 11, 2, False, True,  True,  "Relu6", None),
    ("dw_5x5_i8_f32",               24, 24, 5, 1, 2, 1, 24,  9,  9, 1, True,  False, True,  "",      None),
    ("dw_3x3_i8_i8_nobias_relu",     8,  8, 3, 1, 1, 1,  8,  7,  9, 2, True,  True,  False, "Relu",  None),
    ("dw_3x3s2_nopad_i8_f32_relu",  32, 32, 3, 2, 0, 1, 32,  9,  9, 1, True,  False, True,  "Relu",  None),
]

# The same layer with `use_packing_layout = false` (Tensor/NetOption.hpp; the unpacked sgemm_conv2d_int8_x86 route,
# Tensor/ConvolutionMM2DInt8X86.cpp:1182-1262, scalar float2int8 in quantize / requantize). Same columns. fp32 outputs
# keep OH*OW % 4 == 0: the reference's unpacked dequantize leaves a ragged tail unwritten
# (Tensor/QuantizeX86.cpp:1115-1125). Depthwise is left out: the reference throws there in unpacked mode.
UNPACKED_LAYER_CASES = [
    ("unpacked_3x3_c8k8_i8_relu",     8,  8, 3, 1, 1, 1,  1,  8,  6, 2, True,  True,  True,  "Relu",  None),
    ("unpacked_3x3_c16k16_f32_f32",  16, 16, 3, 1, 1, 1,  1,  8,  8, 1, False, False, True,  "",      None),
    ("unpacked_1x1_c12k6_i8",        12,  6, 1, 1, 0, 1,  1,  7,  5, 2, True,  True,  False, "",      None),
    ("unpacked_3x3s2_c3k8_relu6_i8",  3,  8, 3, 2, 1, 1,  1, 13, 11, 2, False, True,  True,  "Relu6", None),
    ("unpacked_3x3_c8k20_f32_lrelu",  8, 20, 3, 1, 1, 1,  1,  6,  6, 1, False, False, True,  "LRelu", [0.1]),
]


def layer_options(case):
    """The reference's own option keys (Tensor/ConvolutionLayer.cpp:58-156)."""
    name, C, K, k, s, p, d, g, H, W, N, in_i8, i8_out, bias, act, act_params = case
    dw = (C == g == K)
    term = (1 if dw else 2) + (100 if i8_out else 0)
    o = {"type": "Convolution", "in_channels": C, "out_channels": K, "kernel": k, "stride": s, "padding": p,
         "dilation": d, "groups": g, "bias_term": "true" if bias else "false", "int8_scale_term": term}
    if act:
        o["activation"] = act
    if act_params:
        o["activation_params"] = ",".join(str(v) for v in act_params)
    return o


def make_inputs(case, seed):
    """Seeded synthetic tensors in the style of the benchmark configurations."""
    import numpy as np
    name, C, K, k, s, p, d, g, H, W, N, in_i8, i8_out, bias, act, act_params = case
    rng = np.random.default_rng(seed)
    wf = rng.normal(0, 0.05, (K, C // g, k, k)).astype(np.float32)
    wmax = np.abs(wf).reshape(K, -1).max(axis=1)
    w_scales = (np.float32(127) / wmax).astype(np.float32)
    wq = np.clip(np.round(wf * w_scales[:, None, None, None]), -127, 127).astype(np.int8)
    if in_i8:
        x = rng.integers(-127, 128, size=(N, C, H, W)).astype(np.int8)
        in_scale = np.float32(127.0 / 4.0)
    else:
        x = rng.uniform(-1, 1, (N, C, H, W)).astype(np.float32)
        in_scale = np.float32(127) / np.abs(x).max()
    b = rng.normal(0, 0.5, K).astype(np.float32) if bias else None
    top_scale = np.float32(127.0 / 6.0) if act == "Relu6" else np.float32(rng.uniform(8.0, 30.0))
    return dict(x=x, wq=wq, w_scales=w_scales, in_scale=np.float32(in_scale), bias=b, top_scale=top_scale)
