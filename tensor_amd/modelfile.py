"""Writers for the weight streams that go with a `.otter` network description: the ncnn `.bin` layout that
`Net::load_weight(path, WeightType::Ncnn)` reads (Tensor/Initializer.cpp:56-190, Tensor/ConvolutionLayer.cpp:245-293).
The reference ships descriptions of its int8 models (benchmark/*.otter) but no weights; the tests and the benchmark
fill such a description with synthetic int8 weights through these helpers and read it back through the loader."""
import numpy as np

TAG_FP16 = 0x01306B47
TAG_INT8 = 0x000D4B38
TAG_FP32 = 0x0002C056


def _pad4(b):
    return b + b"\0" * (-len(b) % 4)


def weight_int8(wq):
    """A tagged int8 weight tensor: tag, bytes, padded to a multiple of 4."""
    return np.uint32(TAG_INT8).tobytes() + _pad4(np.ascontiguousarray(wq, np.int8).tobytes())


def weight_fp16(w):
    return np.uint32(TAG_FP16).tobytes() + _pad4(np.ascontiguousarray(w, np.float16).tobytes())


def weight_fp32(w, tagged=False):
    return np.uint32(TAG_FP32 if tagged else 0).tobytes() + np.ascontiguousarray(w, np.float32).tobytes()


def weight_table(table256, index):
    """The 256-entry table form: any tag whose bytes do not sum to zero and that is none of the three above."""
    return np.uint32(0x00000001).tobytes() + np.ascontiguousarray(table256, np.float32).tobytes() + \
        _pad4(np.ascontiguousarray(index, np.uint8).tobytes())


def vector(v):
    return np.ascontiguousarray(v, np.float32).tobytes()


def conv_record(wq, bias, weight_scales, bottom_scale, top_scale, int8_scale_term):
    """The tensors one int8 Convolution reads, in order: weight, bias, weight scales ([K] for 1/101, [1] for a depthwise
    2/102), bottom scale [1], top scale [1] when int8_scale_term > 100."""
    out = weight_int8(wq)
    if bias is not None:
        out += vector(bias)
    out += vector(weight_scales) + vector([bottom_scale])
    if int8_scale_term > 100:
        out += vector([top_scale])
    return out


def synthetic_int8_weights(layers, rng, bottom_scale=24.0):
    """A `.bin` for every Convolution of `layers` (hostnet.Net.describe()): for the int8 ones, int8 weights uniform in [-127, 127] whose
    per-channel scale makes the dequantised weights He-like (so that activations stay O(1) through the network), a
    small bias, and one activation scale for every blob. Returns (bytes, {layer name: dict of what was written})."""
    blob = b""
    written = {}
    for typ, name, _bottoms, _tops, c, _shape in layers:
        if typ != "Convolution":
            continue
        K, cin, g = c["K"], c["C"], c["groups"]
        fan_in = cin // g * c["kh"] * c["kw"]
        if not c["int8_scale_term"]:
            # an fp32 convolution inside an int8 model (conv_1 of the reference's ..._int8_mixed.otter): untagged fp32
            # weights, He-like so that its result is O(1) like every other blob, then the bias
            w = rng.normal(0, np.sqrt(2.0 / fan_in), (K, cin // g, c["kh"], c["kw"])).astype(np.float32)
            bias = rng.normal(0, 0.05, K).astype(np.float32) if c["bias_term"] else None
            blob += weight_fp32(w) + (vector(bias) if bias is not None else b"")
            written[name] = dict(w=w, bias=bias, int8_scale_term=0)
            continue
        wq = rng.integers(-127, 128, size=(K, cin // g, c["kh"], c["kw"])).astype(np.int8)
        dw = cin == g and g == K
        n_ws = 1 if (dw and c["int8_scale_term"] in (2, 102)) else K
        ws = (73.3 / np.sqrt(2.0 / fan_in) * rng.uniform(0.8, 1.25, n_ws)).astype(np.float32)
        bias = rng.normal(0, 0.05, K).astype(np.float32) if c["bias_term"] else None
        rec = dict(wq=wq, bias=bias, weight_scales=ws, bottom_scale=np.float32(bottom_scale),
                   top_scale=np.float32(bottom_scale), int8_scale_term=c["int8_scale_term"])
        blob += conv_record(**rec)
        written[name] = rec
    return blob, written
