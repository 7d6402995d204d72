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


# Layers whose results sit on the ONE value where the reference's two rounding primitives part ways:
# float2int8_sse (Tensor/VecIntrinsic.hpp:71-95, the packed SIMD loops) rounds 0.49999997f (the largest float below one
# half) to 1 because fl(0.49999997f + 0.5f) = 1.0f, float2int8 = (int)round(v) (the scalar loops) rounds it to 0; for
# every other float the two agree. Which primitive a LAYER ends in is decided by the reference's routing over
# (C, K, groups, packing) -- Tensor/QuantizeX86.cpp:402,492-545,617-641 (quantize), :1177-1179,1723-1870,2075-2120
# (requantize) -- and random tensors never meet that value, so these cases are the only vectors that pin the routing.
# Same columns as LAYER_CASES plus use_packing_layout. int8-input cases put the tie into the requantize step, fp32-input
# cases into the quantize step (make_tie_inputs).
TIE_ROUTE_CASES = [
    ("tie_requant_k8_packed_1x1",      8,  8, 1, 1, 0, 1,  1, 6, 6, 2, True,  True, True, "",     None, True),
    ("tie_requant_k8_packed_3x3_relu", 8,  8, 3, 1, 1, 1,  1, 6, 6, 1, True,  True, True, "Relu", None, True),
    ("tie_requant_k12_packed_byte",   16, 12, 1, 1, 0, 1,  1, 6, 6, 1, True,  True, True, "",     None, True),
    ("tie_requant_k6_packed_8to1",     8,  6, 3, 1, 1, 1,  1, 6, 6, 1, True,  True, True, "",     None, True),
    ("tie_requant_dw16_packed",       16, 16, 3, 1, 1, 1, 16, 6, 6, 1, True,  True, True, "",     None, True),
    ("tie_requant_dw16s2_packed",     16, 16, 3, 2, 1, 1, 16, 7, 7, 1, True,  True, True, "",     None, True),
    ("tie_requant_k8_unpacked",        8,  8, 3, 1, 1, 1,  1, 6, 6, 1, True,  True, True, "",     None, False),
    ("tie_requant_k12_unpacked",      16, 12, 1, 1, 0, 1,  1, 6, 6, 1, True,  True, True, "",     None, False),
    ("tie_quant_c8_packed",            8,  8, 1, 1, 0, 1,  1, 6, 6, 1, False, True, True, "",     None, True),
    ("tie_quant_c16_packed_dw",       16, 16, 3, 1, 1, 1, 16, 6, 6, 1, False, True, True, "",     None, True),
    ("tie_quant_c4_packed",            4,  8, 3, 1, 1, 1,  1, 6, 6, 1, False, True, True, "",     None, True),
    ("tie_quant_c3_packed_stem",       3,  8, 3, 2, 1, 1,  1, 9, 9, 1, False, True, True, "",     None, True),
    ("tie_quant_c8_unpacked",          8,  8, 1, 1, 0, 1,  1, 6, 6, 1, False, True, True, "",     None, False),
]


def make_tie_inputs(case):
    """Inputs that put layer results exactly on +-0.49999997f (and on neighbours where both primitives agree).

    Weights: the centre tap of input channel 0 (depthwise: of the channel itself) is +1 for even and -1 for odd output
    channels, every other weight is 0, so an accumulator is +-x[channel 0].
    int8 input (requantize side): in_scale = w_scale = 16, hence scale_in = 1/256 exactly; x takes values in
    {64, -64, 32, 96, 0, 17}; bias = +-(0.25f - 2^-25); top_scale = 1. acc = 64 with the positive bias gives
    fma(64, 2^-8, 0.25 - 2^-25) = 0.49999997f with no rounding on the way, acc = -64 with the negative bias its negative.
    fp32 input (quantize side): in_scale = 1, x takes values in {+-0.49999997f, 0.5, 0.25, 1.4999999f, -2.5, 0};
    w_scale = 0.125 (scale_in = 8), bias = 0.25, top_scale = 1, so the int8 result is 8 x the quantized input and never
    itself near a tie."""
    import numpy as np
    name, C, K, k, s, p, d, g, H, W, N, in_i8, i8_out, bias, act, act_params, packing = case
    rng = np.random.default_rng(sum(map(ord, name)))
    wq = np.zeros((K, C // g, k, k), np.int8)
    for o in range(K):
        wq[o, 0, k // 2, k // 2] = 1 if o % 2 == 0 else -1
    just_below_half = np.nextafter(np.float32(0.5), np.float32(0))
    if in_i8:
        x = np.zeros((N, C, H, W), np.int8)
        vals = np.array([64, -64, 32, 96, 0, 17, -96], np.int8)
        chans = range(C) if g == C else [0]
        for c in chans:
            x[:, c] = rng.choice(vals, size=(N, H, W), p=[0.3, 0.3, 0.1, 0.1, 0.1, 0.05, 0.05])
        in_scale, w_scale = np.float32(16), np.float32(16)
        t = np.float32(0.25) - np.float32(2.0 ** -25)
        b = np.array([t if (o % 4) < 2 else -t for o in range(K)], np.float32)
    else:
        x = np.zeros((N, C, H, W), np.float32)
        vals = np.array([just_below_half, -just_below_half, 0.5, 0.25, np.nextafter(np.float32(1.5), np.float32(0)), -2.5, 0.0],
                        np.float32)
        chans = range(C) if g == C else [0]
        for c in chans:
            x[:, c] = rng.choice(vals, size=(N, H, W), p=[0.3, 0.3, 0.1, 0.1, 0.1, 0.05, 0.05])
        in_scale, w_scale = np.float32(1), np.float32(0.125)
        b = np.full(K, 0.25, np.float32)
    return dict(x=x, wq=wq, w_scales=np.full(K, w_scale, np.float32), in_scale=in_scale, bias=b, top_scale=np.float32(1.0))
