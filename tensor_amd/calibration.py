"""Post-training calibration for the int8 convolution path.

The reference has no calibration tool: its int8 models come out of ncnn's `ncnn2int8` with the scales already in the
`.bin`. This utility produces the same kind of model from fp32 weights and a batch of calibration inputs, with the
scale convention of the reference (`q = round(x * scale)`, symmetric, zero point 0, Tensor/ConvolutionLayer.cpp:666-679):

* weights: one scale per output channel, `127 / max|w_k|` (one scale for the whole tensor where the layer's
  `int8_scale_term` is 2 / 102 and it is depthwise, as Tensor/ConvolutionLayer.cpp:262-275 expects);
* activations: `127 / max|x|` of the blob over the calibration batch; an int8 blob's scale is fixed by its producer
  (`top_blob_int8_scales`) and reused as the consumer's `bottom_blob_int8_scales`, as ncnn does.

The network runs on the GPU while it is calibrated: layers are visited in order, each is fed the blobs computed so far,
and an int8-output convolution is first run as its fp32-output twin so that the range its output scale must cover is
seen exactly. The result can be written as an ncnn `.bin` (tensor_amd.modelfile) and read back by Net::load_weight."""
import numpy as np

from . import modelfile


def quantize_weights(wf, per_channel=True):
    """fp32 [K, C/g, kh, kw] -> (int8 weights, fp32 scales [K] or [1]); round half away from zero, saturate at 127."""
    wf = np.asarray(wf, np.float32)
    K = wf.shape[0]
    if per_channel:
        amax = np.abs(wf).reshape(K, -1).max(axis=1)
    else:
        amax = np.abs(wf).max(keepdims=True).reshape(1)
    amax = np.where(amax > 0, amax, np.float32(1)).astype(np.float32)
    ws = (np.float32(127) / amax).astype(np.float32)
    t = wf * (ws[:, None, None, None] if per_channel else ws[0])
    wq = np.clip(np.trunc(t + np.copysign(np.float32(0.5), t)), -127, 127).astype(np.int8)
    return wq, ws


def activation_scale(x):
    amax = np.float32(np.abs(x).max())
    return float(np.float32(127) / amax) if amax > 0 else 1.0


def calibrate_net(net, weights, inputs):
    """net: a compiled hostnet.Net (e.g. after load_otter); weights: {convolution name: (fp32 weight, fp32 bias or
    None)}; inputs: {input blob name: calibration batch [N, C, H, W] fp32}. Sets every convolution of the net up with
    its quantized weights and scales and returns ({name: record for modelfile.conv_record}, {blob name: host array})."""
    layers = net.describe()
    alias = {t: l[2][0] for l in layers if l[0] == "Split" for t in l[3]}
    blobs = {k: np.ascontiguousarray(v, np.float32) for k, v in inputs.items()}
    blob_scale = {}  # int8 blobs: the scale they were written with
    records = {}
    for typ, name, bottoms, tops, c, _shape in layers:
        if typ in ("Input", "Split"):
            continue
        ins = {b: blobs[alias.get(b, b)] for b in bottoms}
        if typ != "Convolution":
            try:
                blobs[tops[0]] = net.eval(ins, tops[0])
            except Exception:
                if all(alias.get(b, b) in blobs for b in bottoms) and typ.endswith("DetectionOutput"):
                    continue  # post-processing heads are not on the GPU path
                raise
            continue
        src = alias.get(bottoms[0], bottoms[0])
        x = blobs[src]
        bottom_scale = blob_scale[src] if x.dtype == np.int8 else activation_scale(x)
        w, b = weights[name]
        depthwise = c["C"] == c["groups"] == c["K"]
        wq, ws = quantize_weights(w, per_channel=not (depthwise and c["int8_scale_term"] in (2, 102)))
        top_scale = 1.0
        if c["int8_scale_term"] > 100:
            net.set_conv(name, wq, b, ws, bottom_scale, 1.0)
            net.conv_fp32_probe(name, True)
            top_scale = activation_scale(net.eval(ins, tops[0]))
            net.conv_fp32_probe(name, False)
        net.set_conv(name, wq, b, ws, bottom_scale, top_scale)
        y = net.eval(ins, tops[0])
        blobs[tops[0]] = y
        if y.dtype == np.int8:
            blob_scale[tops[0]] = top_scale
        records[name] = dict(wq=wq, bias=None if b is None else np.asarray(b, np.float32), weight_scales=ws,
                             bottom_scale=np.float32(bottom_scale), top_scale=np.float32(top_scale),
                             int8_scale_term=c["int8_scale_term"])
    return records, blobs


def to_bin(net, records):
    """The ncnn `.bin` of a calibrated network: every convolution's record in layer order."""
    return b"".join(modelfile.conv_record(**records[name]) for typ, name, *_ in net.describe() if typ == "Convolution")
