"""MobileNetV2-style int8 network (width 1.0) for the benchmark configuration "net images/sec at batch 64":
3x3 stride-2 stem to 32 channels, 17 inverted-residual blocks (expand 6, depthwise 3x3, linear 1x1 project, fp32
element-wise add when stride 1 and channels match), 1x1 conv to 1280, global average pool, 1280->1000 inner product.

Quantization follows the ncnn convention the reference's int8 models use (benchmark/*_int8_*.otter): a convolution
writes int8 (int8_scale_term 101/102, requantize) when every consumer is an int8 convolution, and fp32 (1/2,
dequantize) when an Eltwise / pooling layer consumes it; activation scales are 127/max|activation| on a seeded
calibration batch; weights are He-normal, quantized per output channel.

The network itself runs through the C++ host layer (otter::Net); this module only describes it, calibrates it with
the GPU convolution layers, and provides the CPU-oracle forward used by the parity test.
"""
import numpy as np

BLOCKS = [(1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2), (6, 320, 1, 1)]


def describe(num_classes=1000):
    """Layer list in execution order. Convolution entries: name, cin, cout, k, stride, groups, act, input blob,
    int8_out; other entries: ("add", name, a, b), ("pool", name, input), ("fc", name, input, in_f, out_f)."""
    blocks = []
    cin = 32
    for t, c, n, s in BLOCKS:
        for i in range(n):
            blocks.append((t, cin, c, s if i == 0 else 1))
            cin = c
    residual = [s == 1 and ci == co for (t, ci, co, s) in blocks]
    layers = [dict(kind="conv", name="stem", cin=3, cout=32, k=3, stride=2, groups=1, act="Relu6", input="data",
                   int8_out=True)]
    cur = "stem"
    for b, (t, ci, co, s) in enumerate(blocks):
        block_in = cur
        hidden = ci * t
        if t != 1:
            layers.append(dict(kind="conv", name="b%d_expand" % b, cin=ci, cout=hidden, k=1, stride=1, groups=1,
                               act="Relu6", input=cur, int8_out=True))
            cur = "b%d_expand" % b
        layers.append(dict(kind="conv", name="b%d_dw" % b, cin=hidden, cout=hidden, k=3, stride=s, groups=hidden,
                           act="Relu6", input=cur, int8_out=True))
        nxt_res = residual[b + 1] if b + 1 < len(blocks) else False
        layers.append(dict(kind="conv", name="b%d_project" % b, cin=hidden, cout=co, k=1, stride=1, groups=1, act="",
                           input="b%d_dw" % b, int8_out=not (residual[b] or nxt_res)))
        cur = "b%d_project" % b
        if residual[b]:
            layers.append(dict(kind="add", name="b%d_add" % b, a=block_in, b=cur))
            cur = "b%d_add" % b
    layers.append(dict(kind="conv", name="head", cin=320, cout=1280, k=1, stride=1, groups=1, act="Relu6", input=cur,
                       int8_out=False))
    layers.append(dict(kind="pool", name="pool", input="head"))
    layers.append(dict(kind="fc", name="fc", input="pool", in_f=1280, out_f=num_classes))
    return layers


def conv_macs_per_image(layers, hw):
    total, h = 0, hw
    size = {"data": hw}
    for l in layers:
        if l["kind"] == "conv":
            hin = size[l["input"]]
            hout = (hin + 2 * (l["k"] // 2) - l["k"]) // l["stride"] + 1
            size[l["name"]] = hout
            total += l["cout"] * (l["cin"] // l["groups"]) * l["k"] ** 2 * hout * hout
        elif l["kind"] == "add":
            size[l["name"]] = size[l["a"]]
        elif l["kind"] == "fc":
            total += l["in_f"] * l["out_f"]
    return total


def activation_bytes_per_image(layers, hw):
    """Compulsory traffic of the convolution layers: each reads its input and writes its output once."""
    total = 0
    size, chan, kind = {"data": hw}, {"data": 3}, {"data": 4}
    for l in layers:
        if l["kind"] == "conv":
            hin = size[l["input"]]
            hout = (hin + 2 * (l["k"] // 2) - l["k"]) // l["stride"] + 1
            size[l["name"]], chan[l["name"]] = hout, l["cout"]
            kind[l["name"]] = 1 if l["int8_out"] else 4
            total += l["cin"] * hin * hin * kind[l["input"]] + l["cout"] * hout * hout * kind[l["name"]]
            total += l["cout"] * (l["cin"] // l["groups"]) * l["k"] ** 2
        elif l["kind"] == "add":
            size[l["name"]], chan[l["name"]], kind[l["name"]] = size[l["a"]], chan[l["a"]], 4
            total += 3 * 4 * chan[l["a"]] * size[l["a"]] ** 2
    return total


def init_weights(layers, rng):
    """He-normal fp32 weights, quantized per output channel (scale 127/max|w_k|); bias ~N(0, 0.01)."""
    params = {}
    for l in layers:
        if l["kind"] == "conv":
            cg = l["cin"] // l["groups"]
            wf = rng.normal(0, np.sqrt(2.0 / (cg * l["k"] ** 2)), (l["cout"], cg, l["k"], l["k"])).astype(np.float32)
            ws = (np.float32(127) / np.abs(wf).reshape(l["cout"], -1).max(axis=1)).astype(np.float32)
            wq = np.clip(np.round(wf * ws[:, None, None, None]), -127, 127).astype(np.int8)
            params[l["name"]] = dict(wq=wq, ws=ws, bias=rng.normal(0, 0.01, l["cout"]).astype(np.float32))
        elif l["kind"] == "fc":
            params[l["name"]] = dict(w=rng.normal(0, np.sqrt(2.0 / l["in_f"]), (l["out_f"], l["in_f"])).astype(np.float32),
                                     bias=rng.normal(0, 0.01, l["out_f"]).astype(np.float32))
    return params


def _act_id(name):
    return {"": 0, "Relu": 1, "Relu6": 3}[name]


def calibrate(hip, capi, layers, params, x_cal):
    """Walks the network on the calibration batch with the GPU layers and fixes every convolution's input scale and
    (for int8 outputs) output scale: 127/max|activation|. Blobs are kept as (device tensor, layout, scale or None)."""
    torch = hip.torch
    n, _, h, w = x_cal.shape
    blobs = {"data": (hip.to_device(x_cal), capi.F32, 3, h, None)}
    for l in layers:
        if l["kind"] == "conv":
            t, layout, c, hin, scale = blobs[l["input"]]
            p = params[l["name"]]
            if scale is None:
                scale = float(np.float32(127) / np.float32(t.abs().max().item()))
            p["in_scale"] = scale
            si = (np.float32(1.0) / (np.float32(scale) * p["ws"])).astype(np.float32)
            common = dict(wq=p["wq"], scale_in=si, bias=p["bias"], in_scale=scale, stride=(l["stride"],) * 2,
                          pad=(l["k"] // 2,) * 2, groups=l["groups"], act=_act_id(l["act"]),
                          in_round=capi.ROUND_SSE if c % 8 == 0 else capi.ROUND_EXACT)
            probe = hip.conv(out_kind=capi.OUT_F32, **common)
            y = probe.forward(t, layout, n, hin, hin)
            hout = probe.out_hw(hin, hin)[0]
            ylayout = probe.default_out_layout()
            probe.close()
            if l["int8_out"]:
                amax = float(y.abs().max().item())
                p["top_scale"] = float(np.float32(127) / np.float32(amax))
                conv = hip.conv(out_kind=capi.OUT_I8, out_scale=[p["top_scale"]], **common)
                y = conv.forward(t, layout, n, hin, hin)
                ylayout = conv.default_out_layout()
                conv.close()
                blobs[l["name"]] = (y, ylayout, l["cout"], hout, p["top_scale"])
            else:
                p["top_scale"] = 1.0
                blobs[l["name"]] = (y, ylayout, l["cout"], hout, None)
        elif l["kind"] == "add":
            a, b = blobs[l["a"]], blobs[l["b"]]
            assert a[1] == b[1] and a[4] is None and b[4] is None, "Eltwise operands must be fp32 in one layout"
            blobs[l["name"]] = (a[0] + b[0], a[1], a[2], a[3], None)
    torch.cuda.synchronize()
    return params


def build_net(hostnet, layers, params, batch, hw, num_classes=1000):
    """The otter::Net (C++ host layer) for this description, with the calibrated weights injected."""
    net = hostnet.Net()
    net.add_layer(type="Input", name="data", batchsize=batch, channel=3, height=hw, width=hw)
    for l in layers:
        if l["kind"] == "conv":
            dw = l["groups"] == l["cin"] == l["cout"]
            opts = dict(type="Convolution", name=l["name"], input=l["input"], out_channels=l["cout"], kernel=l["k"],
                        stride=l["stride"], padding=l["k"] // 2, groups=l["groups"],
                        int8_scale_term=(1 if dw else 2) + (100 if l["int8_out"] else 0))
            if l["act"]:
                opts["activation"] = l["act"]
            net.add_layer(**opts)
        elif l["kind"] == "add":
            net.add_layer(type="Eltwise", name=l["name"], input="%s,%s" % (l["a"], l["b"]))
        elif l["kind"] == "pool":
            net.add_layer(type="GlobalAvgPool", name=l["name"], input=l["input"])
        elif l["kind"] == "fc":
            net.add_layer(type="InnerProduct", name=l["name"], input=l["input"], out_features=l["out_f"])
    net.compile()
    for l in layers:
        p = params.get(l["name"])
        if l["kind"] == "conv":
            net.set_conv(l["name"], p["wq"], p["bias"], p["ws"], p["in_scale"], p["top_scale"])
        elif l["kind"] == "fc":
            net.set_inner_product(l["name"], p["w"], p["bias"])
    return net


def build_bench(hip, capi, rng, batch=64, hw=224, calib=32):
    from . import hostnet
    layers = describe()
    params = init_weights(layers, rng)
    calibrate(hip, capi, layers, params, rng.uniform(0, 1, (calib, 3, hw, hw)).astype(np.float32))
    net = build_net(hostnet, layers, params, batch, hw)
    x = rng.uniform(0, 1, (batch, 3, hw, hw)).astype(np.float32)
    sess = net.session("data", x, "fc")
    macs = conv_macs_per_image(layers, hw)
    return dict(name="c4", step=sess.run, ops=2.0 * macs * batch, launches=len(layers), images=batch,
                dom_ops=2.0 * macs * batch, dom_bytes=activation_bytes_per_image(layers, hw) * batch, bound="hbm",
                workload="MobileNetV2-style int8 net, width 1.0, 64x3x224x224 fp32 in, through otter::Net (C++ host "
                         "layer): %d convolutions + 10 adds + avgpool + inner product" % sum(l["kind"] == "conv" for l in layers),
                dom_kernel="whole network (all kernels of one forward pass)", dom_fn=None, x=x, params=[],
                shape=(batch, 3, hw, hw), _keep=(net, sess))


KERNEL_NAMES = {0: "direct", 1: "implicit GEMM (MFMA)", 2: "depthwise", 3: "3x3 LDS-halo (MFMA)", 4: "few-channel 3x3",
                5: "streamed 1x1 (MFMA)"}


def per_layer(hip, capi, rng, time_fn, batch=64, hw=224, calib=32):
    """Every convolution layer of the network by itself, through the C ABI, on a device-resident input of the layer's
    own shape (the image for the stem, Byte8 elsewhere: inside the network the producers write their readers' int8
    input). time_fn(closure) -> milliseconds per call. Returns one dict per layer: shape, kernel family, time,
    algorithmic bytes (input + output + weights) and operations with the rates they amount to. The time is that of a
    host loop of forward() calls, which cannot go below the host's cost of one call (about 8 us from Python); the
    kernels' own durations are in a kernel trace of the same run, where a small fill kernel marks each layer's end."""
    layers = describe()
    params = init_weights(layers, rng)
    calibrate(hip, capi, layers, params, rng.uniform(0, 1, (calib, 3, hw, hw)).astype(np.float32))
    size = {"data": hw}
    rows = []
    hip.torch.full((3,), -1.0, device="cuda")  # (end of the calibration's launches in a kernel trace)
    for l in layers:
        if l["kind"] != "conv":
            if l["kind"] == "add":
                size[l["name"]] = size[l["a"]]
            continue
        p = params[l["name"]]
        hin = size[l["input"]]
        cin, cout, k, s = l["cin"], l["cout"], l["k"], l["stride"]
        si = (np.float32(1.0) / (np.float32(p["in_scale"]) * p["ws"])).astype(np.float32)
        conv = hip.conv(wq=p["wq"], scale_in=si, bias=p["bias"], in_scale=p["in_scale"], stride=(s, s), pad=(k // 2,) * 2,
                        groups=l["groups"], act=_act_id(l["act"]),
                        in_round=capi.ROUND_SSE if cin % 8 == 0 else capi.ROUND_EXACT,
                        out_kind=capi.OUT_I8 if l["int8_out"] else capi.OUT_F32,
                        out_scale=[p["top_scale"]] if l["int8_out"] else None)
        hout = conv.out_hw(hin, hin)[0]
        size[l["name"]] = hout
        if l["name"] == "stem":
            x = hip.to_device(rng.uniform(0, 1, (batch, 3, hin, hin)).astype(np.float32))
            in_layout, in_bytes = capi.F32, 4 * batch * 3 * hin * hin
        else:
            x = hip.to_device(rng.integers(-127, 128, size=batch * cin * hin * hin, dtype=np.int8))
            in_layout, in_bytes = capi.I8_P8, batch * cin * hin * hin
        out_layout = conv.default_out_layout()
        out = hip.empty(batch * cout * hout * hout, capi.layout_dtype(out_layout))
        ms = time_fn(lambda: conv.forward(x, in_layout, batch, hin, hin, out_layout, out=out))
        out_bytes = batch * cout * hout * hout * (1 if l["int8_out"] else 4)
        nbytes = in_bytes + out_bytes + p["wq"].size
        ops = 2.0 * batch * cout * hout * hout * (cin // l["groups"]) * k * k
        rows.append(dict(layer=l["name"], cin=cin, cout=cout, k=k, stride=s, groups=l["groups"], h_in=hin, h_out=hout,
                         out="int8" if l["int8_out"] else "fp32",
                         kernel=KERNEL_NAMES.get(conv.kernel_kind(in_layout, batch, hin, hin, out_layout), "?"),
                         us=ms * 1e3, mbytes=nbytes / 1e6, gbs=nbytes / (ms * 1e-3) / 1e9, gops=ops / 1e9,
                         tops=ops / (ms * 1e-3) / 1e12))
        conv.close()
        del x, out
        # a fill kernel between two layers: in a kernel trace of this run it separates one layer's launches from the next's
        hip.torch.full((3,), float(len(rows)), device="cuda")
    return rows

