"""The C++ host layer (tensor_amd/host): Otter's ConvolutionLayer / Net interface driving the GPU path.
CPU: the library loads and exports its facade. GPU: networks built with the reference's option keys reproduce the
oracle's layer-by-layer result bit for bit (int8) / within 1e-5 (fp32)."""
import numpy as np
import pytest

from tensor_amd import hostnet


def test_host_library_exports():
    lib = hostnet.load_cdll()
    for name in hostnet.EXPORTS:
        assert hasattr(lib, name), name


def _qweights(rng, K, Cg, k):
    wf = rng.normal(0, 0.05, (K, Cg, k, k)).astype(np.float32)
    ws = (np.float32(127) / np.abs(wf).reshape(K, -1).max(axis=1)).astype(np.float32)
    return np.clip(np.round(wf * ws[:, None, None, None]), -127, 127).astype(np.int8), ws


@pytest.mark.gpu
def test_net_chain_int8_activations_flow_between_layers(oracle):
    """Input -> 3x3 conv (102, Relu) -> depthwise 3x3 s2 (101, Relu6) -> 1x1 conv (2): the chain the reference runs
    as Byte8 -> Byte8 -> Float4."""
    rng = np.random.default_rng(5)
    x = rng.uniform(-1, 1, (2, 16, 20, 20)).astype(np.float32)
    w1, s1 = _qweights(rng, 16, 16, 3)
    w2, s2 = _qweights(rng, 16, 1, 3)
    w3, s3 = _qweights(rng, 8, 16, 1)
    b1, b2, b3 = (rng.normal(0, 0.1, n).astype(np.float32) for n in (16, 16, 8))
    in1 = np.float32(127) / np.abs(x).max()
    t1, t2 = np.float32(21.0), np.float32(127.0 / 6.0)
    net = hostnet.Net()
    net.add_layer(type="Input", name="data", batchsize=2, channel=16, height=20, width=20)
    net.add_layer(type="Convolution", name="c1", out_channels=16, kernel=3, padding=1, int8_scale_term=102,
                  activation="Relu")
    net.add_layer(type="Convolution", name="c2", out_channels=16, kernel=3, stride=2, padding=1, groups=16,
                  int8_scale_term=101, activation="Relu6")
    net.add_layer(type="Convolution", name="c3", out_channels=8, kernel=1, int8_scale_term=2)
    net.compile()
    net.set_conv("c1", w1, b1, s1, in1, t1)
    net.set_conv("c2", w2, b2, s2, t1, t2)
    net.set_conv("c3", w3, b3, s3, t2)
    np.testing.assert_array_equal(net.scale_in("c1", 16).view(np.int32), oracle.scale_in(s1, in1).view(np.int32))
    y1 = oracle.conv_layer_forward(x, w1, s1, in1, pad=(1, 1), bias=b1, top_scale=t1, int8_out=True, act_type=1)
    y2 = oracle.conv_layer_forward(y1, w2, s2, t1, stride=(2, 2), pad=(1, 1), groups=16, bias=b2, top_scale=t2,
                                   int8_out=True, act_type=3)
    y3 = oracle.conv_layer_forward(y2, w3, s3, t2, bias=b3)
    np.testing.assert_array_equal(net.run("data", x, "c1"), y1)
    np.testing.assert_array_equal(net.run("data", x, "c2"), y2)
    np.testing.assert_allclose(net.run("data", x, "c3"), y3, rtol=1e-5, atol=1e-30)


@pytest.mark.gpu
def test_net_runs_a_stack_of_same_shape_3x3_layers_as_one_launch(oracle):
    """Input -> 3x3 conv to 72 channels (int8 out) -> three more 3x3 convs 72 -> 72 (int8 out) -> 1x1 conv (fp32 out).
    The three 72 -> 72 layers are one run for the chain entry point (the first layer
    changes the channel count and stays by itself); the Net must give the oracle's blobs whether the run goes
    through in one launch (only its last blob asked for) or layer by layer (a blob inside the run asked for first)."""
    rng = np.random.default_rng(15)
    N, C0, C, H, W = 3, 16, 72, 13, 26
    x = rng.uniform(-1, 1, (N, C0, H, W)).astype(np.float32)
    names = ["c0", "c1", "c2", "c3"]
    chans = [C0, C, C, C, C]
    net = hostnet.Net()
    net.add_layer(type="Input", name="data", batchsize=N, channel=C0, height=H, width=W)
    for i, nm in enumerate(names):
        net.add_layer(type="Convolution", name=nm, out_channels=chans[i + 1], kernel=3, padding=1, int8_scale_term=102,
                      activation="Relu")
    net.add_layer(type="Convolution", name="head", out_channels=8, kernel=1, int8_scale_term=2)
    net.compile()
    scale = np.float32(127) / np.abs(x).max()
    want, cur = {}, x
    for i, nm in enumerate(names):
        w, s = _qweights(rng, chans[i + 1], chans[i], 3)
        b = rng.normal(0, 0.05, chans[i + 1]).astype(np.float32)
        top = np.float32(rng.uniform(15, 30))
        net.set_conv(nm, w, b, s, scale, top)
        cur = oracle.conv_layer_forward(cur, w, s, scale, pad=(1, 1), bias=b, top_scale=top, int8_out=True, act_type=1)
        want[nm] = cur
        scale = top
    wh, sh = _qweights(rng, 8, C, 1)
    bh = rng.normal(0, 0.05, 8).astype(np.float32)
    net.set_conv("head", wh, bh, sh, scale)
    want["head"] = oracle.conv_layer_forward(cur, wh, sh, scale, bias=bh)

    # (the library takes the single launch only for large problems by default: lift the threshold for this small one)
    from tensor_amd import capi
    int8lib = capi.load_cdll()
    old_threshold = int8lib.otter_hip_conv_chain_set_min_tiles(0)
    # (Net.run makes two passes: one for the shape, one for the data)
    before = hostnet.chain_forward_count()
    np.testing.assert_allclose(net.run("data", x, "head"), want["head"], rtol=1e-5, atol=1e-30)
    assert hostnet.chain_forward_count() == before + 2   # c1..c3 in one launch per pass
    np.testing.assert_array_equal(net.run("data", x, "c3"), want["c3"])
    assert hostnet.chain_forward_count() == before + 4
    # a blob inside the run: every pass computes from scratch, the layers up to that blob one by one
    np.testing.assert_array_equal(net.run("data", x, "c2"), want["c2"])
    np.testing.assert_array_equal(net.run("data", x, "c1"), want["c1"])
    assert hostnet.chain_forward_count() == before + 4
    int8lib.otter_hip_conv_chain_set_min_tiles(old_threshold)
    np.testing.assert_array_equal(net.run("data", x, "c3"), want["c3"])   # now layer by layer
    assert hostnet.chain_forward_count() == before + 4


@pytest.mark.gpu
def test_net_residual_block_with_auto_split(oracle):
    """A MobileNetV2-style inverted residual: the block input feeds the expand conv AND the element-wise add, so the
    graph builder must insert a Split; the project conv feeds the add, so it stays fp32."""
    rng = np.random.default_rng(6)
    C, E = 16, 96
    x = rng.uniform(0, 1, (2, C, 14, 14)).astype(np.float32)
    we, se = _qweights(rng, E, C, 1)
    wd, sd = _qweights(rng, E, 1, 3)
    wp, sp = _qweights(rng, C, E, 1)
    be, bd, bp = (rng.normal(0, 0.1, n).astype(np.float32) for n in (E, E, C))
    in_e = np.float32(127) / np.abs(x).max()
    te = td = np.float32(127.0 / 6.0)
    net = hostnet.Net()
    net.add_layer(type="Input", name="data", batchsize=2, channel=C, height=14, width=14)
    net.add_layer(type="Convolution", name="expand", input="data", out_channels=E, kernel=1, int8_scale_term=102,
                  activation="Relu6")
    net.add_layer(type="Convolution", name="dw", out_channels=E, kernel=3, padding=1, groups=E, int8_scale_term=101,
                  activation="Relu6")
    net.add_layer(type="Convolution", name="project", out_channels=C, kernel=1, int8_scale_term=2)
    net.add_layer(type="Eltwise", name="add", input="data,project")
    net.add_layer(type="GlobalAvgPool", name="pool")
    net.add_layer(type="InnerProduct", name="fc", out_features=10)
    net.compile()
    net.set_conv("expand", we, be, se, in_e, te)
    net.set_conv("dw", wd, bd, sd, te, td)
    net.set_conv("project", wp, bp, sp, td)
    wfc = rng.normal(0, 0.1, (10, C)).astype(np.float32)
    bfc = rng.normal(0, 0.1, 10).astype(np.float32)
    net.set_inner_product("fc", wfc, bfc)
    y = oracle.conv_layer_forward(x, we, se, in_e, bias=be, top_scale=te, int8_out=True, act_type=3)
    y = oracle.conv_layer_forward(y, wd, sd, te, pad=(1, 1), groups=E, bias=bd, top_scale=td, int8_out=True, act_type=3)
    y = oracle.conv_layer_forward(y, wp, sp, td, bias=bp)
    s = y + x
    np.testing.assert_allclose(net.run("data", x, "add"), s, rtol=1e-5, atol=1e-30)
    want = oracle.inner_product(oracle.global_avgpool(s), wfc, bfc)
    got = net.run("data", x, "fc").reshape(2, 10)
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("same_scale", [True, False], ids=["readers_agree", "readers_disagree"])
def test_sum_feeding_int8_convolutions_is_quantized_on_the_way(oracle, same_scale):
    """An Eltwise sum read by int8 convolutions (here two, behind an automatic Split, plus a second Eltwise that needs
    the fp32 sum itself) carries its own quantization when the readers agree on the input scale; whether they do or
    not, every blob equals the oracle's layer-by-layer computation."""
    rng = np.random.default_rng(17)
    C, K = 24, 16
    x = rng.uniform(-1, 1, (3, C, 9, 11)).astype(np.float32)
    wp, sp = _qweights(rng, C, C, 1)
    wa, sa = _qweights(rng, K, C, 3)
    wb, sb = _qweights(rng, C, C, 1)
    bp, ba, bb = (rng.normal(0, 0.1, n).astype(np.float32) for n in (C, K, C))
    in_p = np.float32(127) / np.abs(x).max()
    net = hostnet.Net(lightmode=False)
    net.add_layer(type="Input", name="data", batchsize=3, channel=C, height=9, width=11)
    net.add_layer(type="Convolution", name="p", input="data", out_channels=C, kernel=1, int8_scale_term=2)
    net.add_layer(type="Eltwise", name="sum", input="data,p")
    net.add_layer(type="Convolution", name="a", input="sum", out_channels=K, kernel=3, padding=1, int8_scale_term=102,
                  activation="Relu")
    net.add_layer(type="Convolution", name="b", input="sum", out_channels=C, kernel=1, int8_scale_term=2)
    net.add_layer(type="Eltwise", name="sum2", input="sum,b")
    net.compile()
    yp = oracle.conv_layer_forward(x, wp, sp, in_p, bias=bp)
    s1 = yp + x
    in_a = np.float32(127) / np.abs(s1).max()
    in_b = in_a if same_scale else np.float32(in_a * 0.75)
    net.set_conv("p", wp, bp, sp, in_p)
    net.set_conv("a", wa, ba, sa, in_a, 9.0)
    net.set_conv("b", wb, bb, sb, in_b)
    ya = oracle.conv_layer_forward(s1, wa, sa, in_a, pad=(1, 1), bias=ba, top_scale=9.0, int8_out=True, act_type=1)
    yb = oracle.conv_layer_forward(s1, wb, sb, in_b, bias=bb)
    np.testing.assert_allclose(net.run("data", x, "sum"), s1, rtol=1e-5, atol=1e-30)
    np.testing.assert_array_equal(net.run("data", x, "a"), ya)
    np.testing.assert_allclose(net.run("data", x, "b"), yb, rtol=1e-5, atol=1e-30)
    np.testing.assert_allclose(net.run("data", x, "sum2"), s1 + yb, rtol=1e-5, atol=1e-30)


@pytest.mark.gpu
@pytest.mark.parametrize("k", [1, 3], ids=["pointwise_producer", "3x3_producer"])
@pytest.mark.parametrize("same_scale", [True, False], ids=["readers_agree", "readers_disagree"])
def test_fp32_convolution_feeding_int8_convolutions_is_quantized_on_the_way(oracle, same_scale, k):
    """The MobileNetV2 pattern at the head of a residual chain: a project convolution whose fp32 result is read by the
    shortcut sum and by the next expand convolutions. The producer writes the readers' quantization itself when they
    agree on the scale; every blob equals the oracle's layer-by-layer computation either way."""
    rng = np.random.default_rng(23 + k)
    C, K = 24, 32
    x = rng.uniform(-1, 1, (3, C, 9, 11)).astype(np.float32)
    wp, sp = _qweights(rng, C, C, k)
    wa, sa = _qweights(rng, K, C, 1)
    wb, sb = _qweights(rng, C, C, 1)
    bp, ba, bb = (rng.normal(0, 0.1, n).astype(np.float32) for n in (C, K, C))
    in_p = np.float32(127) / np.abs(x).max()
    net = hostnet.Net(lightmode=False)
    net.add_layer(type="Input", name="data", batchsize=3, channel=C, height=9, width=11)
    net.add_layer(type="Convolution", name="p", input="data", out_channels=C, kernel=k, padding=k // 2,
                  int8_scale_term=2)
    net.add_layer(type="Convolution", name="a", input="p", out_channels=K, kernel=1, int8_scale_term=102,
                  activation="Relu6")
    net.add_layer(type="Convolution", name="b", input="p", out_channels=C, kernel=1, int8_scale_term=2)
    net.add_layer(type="Eltwise", name="sum", input="p,b")
    net.compile()
    yp = oracle.conv_layer_forward(x, wp, sp, in_p, pad=(k // 2, k // 2), bias=bp)
    in_a = np.float32(127) / np.abs(yp).max() * np.float32(1.2)
    in_b = in_a if same_scale else np.float32(in_a * 0.75)
    net.set_conv("p", wp, bp, sp, in_p)
    net.set_conv("a", wa, ba, sa, in_a, 9.0)
    net.set_conv("b", wb, bb, sb, in_b)
    ya = oracle.conv_layer_forward(yp, wa, sa, in_a, bias=ba, top_scale=9.0, int8_out=True, act_type=3)
    yb = oracle.conv_layer_forward(yp, wb, sb, in_b, bias=bb)
    np.testing.assert_allclose(net.run("data", x, "p"), yp, rtol=1e-5, atol=1e-30)
    np.testing.assert_array_equal(net.run("data", x, "a"), ya)
    np.testing.assert_allclose(net.run("data", x, "b"), yb, rtol=1e-5, atol=1e-30)
    np.testing.assert_allclose(net.run("data", x, "sum"), yp + yb, rtol=1e-5, atol=1e-30)


@pytest.mark.gpu
@pytest.mark.parametrize("k", [1, 3], ids=["pointwise_project", "3x3_project"])
@pytest.mark.parametrize("ask_inner_first", [False, True], ids=["fused", "inner_blob_requested"])
def test_residual_block_tail_runs_as_one_launch_with_the_same_blobs(oracle, k, ask_inner_first):
    """A residual block: the project convolution's fp32 result is read by the Eltwise sum alone, and the sum by an
    int8 convolution and a second sum. Convolution + sum (+ the reader's quantization) run as one launch; asking for
    the convolution's own blob first makes the layers run one by one. Same blobs either way."""
    rng = np.random.default_rng(31 + k)
    C, K = 24, 16
    x = rng.uniform(-1, 1, (3, C, 9, 11)).astype(np.float32)
    wp, sp = _qweights(rng, C, C, k)
    wa, sa = _qweights(rng, K, C, 1)
    wb, sb = _qweights(rng, C, C, 1)
    bp, ba, bb = (rng.normal(0, 0.1, n).astype(np.float32) for n in (C, K, C))
    in_p = np.float32(127) / np.abs(x).max()
    net = hostnet.Net(lightmode=False)
    net.add_layer(type="Input", name="data", batchsize=3, channel=C, height=9, width=11)
    net.add_layer(type="Convolution", name="p", input="data", out_channels=C, kernel=k, padding=k // 2,
                  int8_scale_term=2)
    net.add_layer(type="Eltwise", name="sum", input="data,p")
    net.add_layer(type="Convolution", name="a", input="sum", out_channels=K, kernel=1, int8_scale_term=102,
                  activation="Relu")
    net.add_layer(type="Convolution", name="b", input="sum", out_channels=C, kernel=1, int8_scale_term=2)
    net.add_layer(type="Eltwise", name="sum2", input="b,sum")
    net.compile()
    yp = oracle.conv_layer_forward(x, wp, sp, in_p, pad=(k // 2, k // 2), bias=bp)
    s1 = x + yp
    in_a = np.float32(127) / np.abs(s1).max()
    net.set_conv("p", wp, bp, sp, in_p)
    net.set_conv("a", wa, ba, sa, in_a, 9.0)
    net.set_conv("b", wb, bb, sb, in_a)
    ya = oracle.conv_layer_forward(s1, wa, sa, in_a, bias=ba, top_scale=9.0, int8_out=True, act_type=1)
    yb = oracle.conv_layer_forward(s1, wb, sb, in_a, bias=bb)

    def last_of(names, shape, dtype):
        """one extractor, the blobs extracted in this order; the last one comes back"""
        s = net.session("data", x, ",".join(names))
        s.run()
        out = s.fetch(shape, dtype)
        s.close()
        return out

    first = ["p"] if ask_inner_first else []
    np.testing.assert_allclose(last_of(first + ["sum"], s1.shape, np.float32), s1, rtol=1e-5, atol=1e-30)
    np.testing.assert_array_equal(last_of(first + ["a"], ya.shape, np.int8), ya)
    np.testing.assert_allclose(last_of(first + ["sum2"], s1.shape, np.float32), yb + s1, rtol=1e-5, atol=1e-30)
    np.testing.assert_allclose(last_of(first + ["sum", "p"], yp.shape, np.float32), yp, rtol=1e-5, atol=1e-30)


@pytest.mark.gpu
@pytest.mark.parametrize("glue", ["Concat", "ShortCut", "Concat+ChannelShuffle"])
@pytest.mark.parametrize("same_scale", [True, False], ids=["readers_agree", "readers_disagree"])
def test_concat_and_shortcut_feeding_int8_convolutions_quantize_on_the_way(oracle, glue, same_scale):
    """Two fp32 convolution results joined by a Concat (channels) or a ShortCut (sum) and read by two int8
    convolutions: the joining layer writes the readers' int8 input itself when they agree on the scale."""
    rng = np.random.default_rng(41 + len(glue))
    C, K = 16, 24   # 2K = 48 channels: a multiple of 16, as the quantizing shuffle needs
    x = rng.uniform(-1, 1, (2, C, 9, 11)).astype(np.float32)
    w1, s1 = _qweights(rng, K, C, 1)
    w2, s2 = _qweights(rng, K, C, 3)
    b1, b2 = (rng.normal(0, 0.1, K).astype(np.float32) for _ in range(2))
    in_x = np.float32(127) / np.abs(x).max()
    J = K if glue == "ShortCut" else 2 * K
    wa, sa = _qweights(rng, K, J, 1)
    wb, sb = _qweights(rng, 8, J, 3)
    ba, bb = rng.normal(0, 0.1, K).astype(np.float32), rng.normal(0, 0.1, 8).astype(np.float32)
    net = hostnet.Net(lightmode=False)
    net.add_layer(type="Input", name="data", batchsize=2, channel=C, height=9, width=11)
    net.add_layer(type="Convolution", name="c1", input="data", out_channels=K, kernel=1, int8_scale_term=2)
    net.add_layer(type="Convolution", name="c2", input="data", out_channels=K, kernel=3, padding=1, int8_scale_term=2,
                  activation="Relu")
    if glue == "Concat+ChannelShuffle":
        net.add_layer(type="Concat", name="cat", input="c1,c2")
        net.add_layer(type="ChannelShuffle", name="j", input="cat", groups=2)
    else:
        net.add_layer(type=glue, name="j", input="c1,c2")
    net.add_layer(type="Convolution", name="a", input="j", out_channels=K, kernel=1, int8_scale_term=102, activation="Relu6")
    net.add_layer(type="Convolution", name="b", input="j", out_channels=8, kernel=3, padding=1, int8_scale_term=2)
    net.compile()
    y1 = oracle.conv_layer_forward(x, w1, s1, in_x, bias=b1)
    y2 = oracle.conv_layer_forward(x, w2, s2, in_x, pad=(1, 1), bias=b2, act_type=1)
    j = y1 + y2 if glue == "ShortCut" else np.concatenate([y1, y2], axis=1)
    if glue == "Concat+ChannelShuffle":
        j = j.reshape(2, 2, K, 9, 11).transpose(0, 2, 1, 3, 4).reshape(2, 2 * K, 9, 11)
    in_a = np.float32(127) / np.abs(j).max() * np.float32(1.1)
    in_b = in_a if same_scale else np.float32(in_a * 0.8)
    net.set_conv("c1", w1, b1, s1, in_x)
    net.set_conv("c2", w2, b2, s2, in_x)
    net.set_conv("a", wa, ba, sa, in_a, 11.0)
    net.set_conv("b", wb, bb, sb, in_b)
    ya = oracle.conv_layer_forward(j, wa, sa, in_a, bias=ba, top_scale=11.0, int8_out=True, act_type=3)
    yb = oracle.conv_layer_forward(j, wb, sb, in_b, pad=(1, 1), bias=bb)
    np.testing.assert_allclose(net.run("data", x, "j"), j, rtol=1e-5, atol=1e-30)
    np.testing.assert_array_equal(net.run("data", x, "a"), ya)
    np.testing.assert_allclose(net.run("data", x, "b"), yb, rtol=1e-5, atol=1e-30)


@pytest.mark.gpu
def test_functional_api_matches_oracle(oracle):
    rng = np.random.default_rng(8)
    for (C, K, k, s, p, g, i8) in [(16, 16, 3, 1, 1, 1, True), (32, 32, 3, 2, 1, 32, True), (8, 12, 1, 1, 0, 1, False)]:
        x = rng.uniform(-1, 1, (2, C, 11, 9)).astype(np.float32)
        wq, ws = _qweights(rng, K, C // g, k)
        bias = rng.normal(0, 0.2, K).astype(np.float32)
        in_scale = np.float32(127) / np.abs(x).max()
        want, acc_want = oracle.conv_layer_forward(x, wq, ws, in_scale, stride=(s, s), pad=(p, p), groups=g, bias=bias,
                                                   top_scale=13.0, int8_out=i8, act_type=1 if i8 else 0, want_acc=True)
        acc, out = hostnet.functional_chain(x, in_scale, wq, oracle.scale_in(ws, in_scale), bias, stride=s, pad=p,
                                            groups=g, int8_out=i8, top_scale=13.0, act=1 if i8 else 0)
        np.testing.assert_array_equal(acc, acc_want)
        if i8:
            np.testing.assert_array_equal(out, want)
        else:
            np.testing.assert_allclose(out, want, rtol=1e-5, atol=1e-30)


@pytest.mark.gpu
def test_error_conventions():
    net = hostnet.Net()
    net.add_layer(type="Input", name="data", batchsize=1, channel=8, height=4, width=4)
    net.add_layer(type="NoSuchLayer", name="bad")
    with pytest.raises(hostnet.HostError):
        net.compile()
    net2 = hostnet.Net()
    net2.add_layer(type="Input", name="data", batchsize=1, channel=8, height=4, width=4)
    net2.add_layer(type="Convolution", name="c", out_channels=8, kernel=3, padding=1, int8_scale_term=2)
    net2.compile()
    with pytest.raises(hostnet.HostError):  # pipeline never built: forward returns the reference's -1
        net2.run("data", np.zeros((1, 8, 4, 4), np.float32), "c")
