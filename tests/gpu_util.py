"""Helpers shared by the GPU parity tests: run one ConvolutionLayer-shaped problem through the C ABI."""
import numpy as np

from tensor_amd import capi

ACT = {"": 0, "Relu": 1, "LRelu": 2, "Relu6": 3}


def in_layout_for(x, C, use_packing=True):
    """The layout Net::convert_layout hands to the layer (Tensor/Net.cpp:388-405)."""
    if not use_packing:
        return capi.I8 if x.dtype == np.int8 else capi.F32
    if x.dtype == np.int8:
        return capi.I8_P8 if C % 8 == 0 else capi.I8
    if C % 8 == 0:
        return capi.F32_P8
    if C % 4 == 0:
        return capi.F32_P4
    return capi.F32


def host_scale_in(w_scales, in_scale):
    """ConvolutionLayer::create_pipeline_int8 (Tensor/ConvolutionLayer.cpp:667-679) as the host does it."""
    ws = np.asarray(w_scales, np.float32)
    with np.errstate(divide="ignore"):
        si = (np.float32(1.0) / (np.float32(in_scale) * ws)).astype(np.float32)
    si[ws == 0] = 0
    return si


def run_conv(hip, oracle, x, wq, w_scales, in_scale, *, stride=1, pad=0, dil=1, groups=1, bias=None, top_scale=1.0,
             out_kind=capi.OUT_I32, act=0, act_p0=0.0, out_layout=None, in_layout=None, tile=None, use_packing=True):
    """x: NCHW numpy (fp32 or int8). Returns the NCHW numpy result of the GPU layer."""
    n, C, H, W = x.shape
    K = wq.shape[0]
    conv = hip.conv(wq=wq, scale_in=host_scale_in(np.broadcast_to(w_scales, (K,)), in_scale), bias=bias,
                    in_scale=float(in_scale), out_scale=[top_scale] if out_kind == capi.OUT_I8 else None,
                    stride=(stride, stride), pad=(pad, pad), dil=(dil, dil), groups=groups, act=act, act_p0=act_p0,
                    out_kind=out_kind, out_round=oracle.requantize_round_mode(C, K, groups, use_packing),
                    in_round=oracle.quantize_round_mode(C, use_packing))
    if tile is not None:
        conv.set_tile(*tile)
    in_layout = in_layout_for(x, C, use_packing) if in_layout is None else in_layout
    if out_layout is None:
        # unpacked mode: every blob is elempack 1 (Tensor/Net.cpp:388-405 with use_packing_layout = false)
        out_layout = conv.default_out_layout() if use_packing else \
            {capi.OUT_I32: capi.I32, capi.OUT_F32: capi.F32, capi.OUT_I8: capi.I8}[out_kind]
    xd = hip.to_device(capi.pack_np(x, capi.layout_pack(in_layout)))
    out = conv.forward(xd, in_layout, n, H, W, out_layout)
    hip.torch.cuda.synchronize()
    oh, ow = conv.out_hw(H, W)
    kind = conv.kernel_kind(in_layout, n, H, W, out_layout)
    res = capi.unpack_np(out.cpu().numpy(), capi.layout_pack(out_layout), (n, K, oh, ow))
    conv.close()
    return res, kind


def mobilenet_oracle_forward(oracle, layers, params, x, upto=None):
    """The MobileNetV2-style network of tensor_amd.mobilenet on the CPU oracle, layer by layer
    (ConvolutionLayer::forward_int8 semantics, Tensor/ConvolutionLayer.cpp:754-847). Returns every blob by name."""
    from tensor_amd.mobilenet import _act_id
    blobs = {"data": x}
    for l in layers:
        if l["kind"] == "conv":
            p = params[l["name"]]
            blobs[l["name"]] = oracle.conv_layer_forward(
                blobs[l["input"]], p["wq"], p["ws"], p["in_scale"], stride=(l["stride"],) * 2, pad=(l["k"] // 2,) * 2,
                groups=l["groups"], bias=p["bias"], top_scale=p["top_scale"], int8_out=l["int8_out"],
                act_type=_act_id(l["act"]))
        elif l["kind"] == "add":
            blobs[l["name"]] = blobs[l["a"]] + blobs[l["b"]]
        elif l["kind"] == "pool":
            blobs[l["name"]] = oracle.global_avgpool(blobs[l["input"]])
        elif l["kind"] == "fc":
            p = params[l["name"]]
            blobs[l["name"]] = oracle.inner_product(blobs[l["input"]].reshape(x.shape[0], -1), p["w"], p["bias"])
        if upto == l["name"]:
            break
    return blobs
