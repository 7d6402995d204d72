"""The benchmark configurations at their FULL sizes, through the C ABI.

The CPU oracle cannot chew through 59 GOP per layer in test time, so full-size runs are checked by (a) the oracle on a
few whole images of the batch (first, last, one in the middle: the ends of the persistent tile walk and of the
batch-linear pixel tiling), (b) properties that hold at any size: a batch is N independent images (the full-batch result
equals the images run one at a time, bit for bit), int32 accumulators are linear in the weights
(conv(x, w1) + conv(x, w2) == conv(x, w1 + w2) while nothing saturates), and an all-zero input gives requantize(bias).
"""
import zlib

import numpy as np
import pytest

from tensor_amd import capi
from gpu_util import run_conv, mobilenet_oracle_forward

FP32_RTOL = 1e-5  # the bar for fp32 results

pytestmark = pytest.mark.gpu


def _problem(rng, N, C, K, k, groups, H, W, in_i8=True):
    wq = rng.integers(-127, 128, size=(K, C // groups, k, k)).astype(np.int8)
    ws = rng.uniform(80, 300, K).astype(np.float32)
    x = rng.integers(-127, 128, size=(N, C, H, W)).astype(np.int8) if in_i8 else \
        rng.uniform(-1, 1, (N, C, H, W)).astype(np.float32)
    bias = rng.normal(0, 0.3, K).astype(np.float32)
    return x, wq, ws, bias


CONFIGS = [
    # name, N, C, K, k, stride, pad, groups, H, W, act, int8_out, expected kernel family
    ("c3_layer", 64, 128, 128, 3, 1, 1, 1, 56, 56, 1, True, 3),
    ("c1_s1", 8, 256, 256, 3, 1, 1, 256, 112, 112, 3, True, 2),
    ("c1_s2", 8, 256, 256, 3, 2, 1, 256, 112, 112, 3, True, 2),
    ("c2", 32, 256, 512, 1, 1, 0, 1, 28, 28, 1, False, 1),
]


@pytest.mark.parametrize("cfg", CONFIGS, ids=[c[0] for c in CONFIGS])
def test_full_size_layer(hip, oracle, cfg):
    name, N, C, K, k, s, p, g, H, W, act, int8_out, family = cfg
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    x, wq, ws, bias = _problem(rng, N, C, K, k, g, H, W)
    in_scale, top_scale = 40.0, 15.0
    kw = dict(stride=s, pad=p, groups=g, bias=bias, top_scale=top_scale, act=act,
              out_kind=capi.OUT_I8 if int8_out else capi.OUT_F32)
    full, kind = run_conv(hip, oracle, x, wq, ws, in_scale, **kw)
    assert kind == family

    # (a) whole images against the oracle
    for n in (0, N // 2, N - 1):
        want = oracle.conv_layer_forward(x[n:n + 1], wq, ws, in_scale, stride=(s, s), pad=(p, p), groups=g, bias=bias,
                                         top_scale=top_scale, int8_out=int8_out, act_type=act)
        if int8_out:
            np.testing.assert_array_equal(full[n:n + 1], want, err_msg="image %d" % n)
        else:
            np.testing.assert_allclose(full[n:n + 1], want, rtol=1e-5, atol=1e-6, err_msg="image %d" % n)

    # (b1) a batch is N independent images: every image alone reproduces its slice of the batch result bit for bit
    for n in (1, N - 2):
        one, _ = run_conv(hip, oracle, x[n:n + 1], wq, ws, in_scale, **kw)
        np.testing.assert_array_equal(one, full[n:n + 1], err_msg="image %d alone" % n)

    # (b2) zero input: the accumulators vanish, the output is the epilogue of the bias alone
    zero, _ = run_conv(hip, oracle, np.zeros_like(x[:2]), wq, ws, in_scale, **kw)
    v = bias.astype(np.float32)
    v = np.maximum(v, 0) if act == 1 else (np.clip(v, 0, 6) if act == 3 else v)
    if int8_out:
        t = v * np.float32(top_scale)
        want0 = np.clip(np.trunc(t + np.copysign(np.float32(0.5), t)), -127, 127).astype(np.int8)
        np.testing.assert_array_equal(zero, np.broadcast_to(want0[None, :, None, None], zero.shape))
    else:
        np.testing.assert_array_equal(zero, np.broadcast_to(v[None, :, None, None], zero.shape))


@pytest.mark.parametrize("cfg", CONFIGS, ids=[c[0] for c in CONFIGS])
def test_full_size_accumulators_are_linear_in_the_weights(hip, oracle, cfg):
    name, N, C, K, k, s, p, g, H, W, act, int8_out, family = cfg
    rng = np.random.default_rng(7 + zlib.crc32(name.encode()))
    n_img = min(N, 16)  # int32 outputs are 4x the bytes; 16 images still span several tile rounds
    x = rng.integers(-127, 128, size=(n_img, C, H, W)).astype(np.int8)
    w1 = rng.integers(-60, 61, size=(K, C // g, k, k)).astype(np.int8)
    w2 = rng.integers(-60, 61, size=(K, C // g, k, k)).astype(np.int8)
    ws = np.ones(K, np.float32)
    kw = dict(stride=s, pad=p, groups=g, out_kind=capi.OUT_I32)
    a1, _ = run_conv(hip, oracle, x, w1, ws, 1.0, **kw)
    a2, _ = run_conv(hip, oracle, x, w2, ws, 1.0, **kw)
    a12, _ = run_conv(hip, oracle, x, (w1.astype(np.int16) + w2).astype(np.int8), ws, 1.0, **kw)
    np.testing.assert_array_equal(a1.astype(np.int64) + a2, a12)
    # and a checksum over everything against the oracle's accumulators of one image
    want = oracle.conv_layer_forward(x[:1], w1, ws, 1.0, stride=(s, s), pad=(p, p), groups=g, want_acc=True)[1]
    np.testing.assert_array_equal(a1[:1], want)


# ---------------------------------------------------------------------------------------------------------------
# The benchmark configurations exactly as they are stated (input dtype, distributions, scales, bias, activation)
# ---------------------------------------------------------------------------------------------------------------

def _quantize_weights(wf):
    K = wf.shape[0]
    ws = (np.float32(127) / np.abs(wf).reshape(K, -1).max(axis=1)).astype(np.float32)
    wq = np.clip(np.round(wf * ws[:, None, None, None]), -127, 127).astype(np.int8)
    return wq, ws


def test_c0_as_stated(hip, oracle):
    """Single 3x3 s1 p1 convolution 64->64 on 1x64x56x56 fp32 ~U(-1,1), seed 0, weights ~N(0,0.05), per-channel weight
    scales 127/max|w_c|, input scale 127/max|x|, NO bias, no activation, dequantized fp32 output; through the fp32
    Float8 blob the reference's Net hands the layer, the quantize pass and the LDS-halo kernel."""
    rng = np.random.default_rng(0)
    x = rng.uniform(-1, 1, (1, 64, 56, 56)).astype(np.float32)
    wq, ws = _quantize_weights(rng.normal(0, 0.05, (64, 64, 3, 3)).astype(np.float32))
    in_scale = np.float32(127) / np.abs(x).max()
    got, kind = run_conv(hip, oracle, x, wq, ws, in_scale, pad=1, out_kind=capi.OUT_F32)
    assert kind == 3
    want, acc_want = oracle.conv_layer_forward(x, wq, ws, in_scale, pad=(1, 1), want_acc=True)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-30)
    np.testing.assert_array_equal(got.view(np.int32), want.view(np.int32))
    acc, _ = run_conv(hip, oracle, x, wq, ws, in_scale, pad=1, out_kind=capi.OUT_I32)
    np.testing.assert_array_equal(acc, acc_want)
    # closed form on the way: the dequantized output is acc / (in_scale * w_scale) to fp32 rounding
    np.testing.assert_allclose(got, acc_want / (np.float64(in_scale) * ws.astype(np.float64))[None, :, None, None],
                               rtol=1e-6, atol=1e-30)


@pytest.mark.parametrize("stride", [1, 2])
def test_c1_as_stated_fp32_input(hip, oracle, stride):
    """Depthwise 3x3 p1 on 8x256x112x112 fp32 ~U(-1,1): quantize (127/max|x|) -> depthwise -> bias ~N(0,0.01) ->
    ReLU6 -> requantize with 127/6 -> int8, the fp32 blob handed over as Float8."""
    rng = np.random.default_rng(10 + stride)
    N, C, H, W = 8, 256, 112, 112
    x = rng.uniform(-1, 1, (N, C, H, W)).astype(np.float32)
    wq, ws = _quantize_weights(rng.normal(0, 0.1, (C, 1, 3, 3)).astype(np.float32))
    bias = rng.normal(0, 0.01, C).astype(np.float32)
    in_scale = np.float32(127) / np.abs(x).max()
    top = np.float32(127.0 / 6.0)
    kw = dict(stride=stride, pad=1, groups=C, bias=bias, top_scale=top, act=3, out_kind=capi.OUT_I8)
    full, kind = run_conv(hip, oracle, x, wq, ws, in_scale, **kw)
    assert kind == 2
    for n in (0, 3, N - 1):
        want = oracle.conv_layer_forward(x[n:n + 1], wq, ws, in_scale, stride=(stride, stride), pad=(1, 1), groups=C,
                                         bias=bias, top_scale=top, int8_out=True, act_type=3)
        np.testing.assert_array_equal(full[n:n + 1], want, err_msg="image %d" % n)
    one, _ = run_conv(hip, oracle, x[5:6], wq, ws, in_scale, **kw)
    np.testing.assert_array_equal(one, full[5:6])
    assert full.min() >= 0 and full.max() <= 127  # ReLU6 then 127/6: the output range of the configuration


def test_c2_as_stated_fp32_input(hip, oracle):
    """1x1 convolution 256->512 on 32x256x28x28 fp32 ~U(0,1) (GEMM 512 x 25088 x 256): quantize -> int32 accumulate ->
    bias ~N(0,0.01) -> dequantize + ReLU -> fp32."""
    rng = np.random.default_rng(20)
    N, C, K, H, W = 32, 256, 512, 28, 28
    x = rng.uniform(0, 1, (N, C, H, W)).astype(np.float32)
    wq, ws = _quantize_weights(rng.normal(0, 0.03, (K, C, 1, 1)).astype(np.float32))
    bias = rng.normal(0, 0.01, K).astype(np.float32)
    in_scale = np.float32(127) / np.abs(x).max()
    kw = dict(bias=bias, act=1, out_kind=capi.OUT_F32)
    full, kind = run_conv(hip, oracle, x, wq, ws, in_scale, **kw)
    assert kind == 6   # quantize + convolution in one launch that reads the fp32 blob once
    two, _ = run_conv(hip, oracle, x, wq, ws, in_scale, tile=(-6, 0), **kw)   # the reference's order: two launches
    assert full.tobytes() == two.tobytes()
    for n in (0, 17, N - 1):
        want = oracle.conv_layer_forward(x[n:n + 1], wq, ws, in_scale, bias=bias, act_type=1)
        np.testing.assert_allclose(full[n:n + 1], want, rtol=1e-5, atol=1e-30, err_msg="image %d" % n)
        np.testing.assert_array_equal(full[n:n + 1].view(np.int32), want.view(np.int32))
    one, _ = run_conv(hip, oracle, x[9:10], wq, ws, in_scale, **kw)
    np.testing.assert_array_equal(one, full[9:10])
    assert full.min() >= 0


def test_c3_as_stated_four_layer_chain(hip, oracle):
    """Four chained 128->128 3x3 s1 p1 layers at 56x56, batch 64, int8 ~U[-127,127] in, weights ~N(0,0.04), bias
    ~N(0,0.01), fused requantize + ReLU, each layer's output scale 127/max(activation) on a seeded calibration batch
    of 16 (the rule bench.py uses), the next layer's input scale = that output scale. The oracle follows three
    sampled images through all four layers."""
    rng = np.random.default_rng(0)
    N, C, H, W, L = 64, 128, 56, 56, 4
    x = rng.integers(-127, 128, size=(N, C, H, W), dtype=np.int8)
    xc = rng.integers(-127, 128, size=(16, C, H, W), dtype=np.int8)
    xd = hip.to_device(capi.pack_np(x, 8))
    cal = hip.to_device(capi.pack_np(xc, 8))
    in_scale = np.float32(127.0)
    params, convs = [], []
    for l in range(L):
        wq, ws = _quantize_weights(rng.normal(0, 0.04, (C, C, 3, 3)).astype(np.float32))
        bias = rng.normal(0, 0.01, C).astype(np.float32)
        si = (np.float32(1.0) / (np.float32(in_scale) * ws)).astype(np.float32)
        probe = hip.conv(wq=wq, scale_in=si, bias=bias, pad=(1, 1), act=1, out_kind=capi.OUT_F32)
        amax = float(probe.forward(cal, capi.I8_P8, 16, H, W).abs().max().item())
        probe.close()
        out_scale = np.float32(127.0) / np.float32(amax)
        conv = hip.conv(wq=wq, scale_in=si, bias=bias, out_scale=[out_scale], pad=(1, 1), act=1,
                        out_kind=capi.OUT_I8, out_round=capi.ROUND_SSE)
        assert conv.kernel_kind(capi.I8_P8, N, H, W, capi.I8_P8) == 3
        cal = conv.forward(cal, capi.I8_P8, 16, H, W)
        convs.append(conv)
        params.append((wq, ws, bias, float(in_scale), float(out_scale)))
        in_scale = out_scale
    # calibration reached the top of the int8 range in every layer: the scale rule is what the configuration states
    cur = xd
    outs = []
    for conv in convs:
        cur = conv.forward(cur, capi.I8_P8, N, H, W, capi.I8_P8)
        outs.append(cur)
    hip.torch.cuda.synchronize()
    got = [capi.unpack_np(o.cpu().numpy(), 8, (N, C, H, W)) for o in outs]
    for n in (0, 31, N - 1):
        ref = x[n:n + 1]
        for l, (wq, ws, bias, ins, outs_) in enumerate(params):
            ref = oracle.conv_layer_forward(ref, wq, ws, ins, pad=(1, 1), bias=bias, top_scale=outs_, int8_out=True,
                                            act_type=1)
            np.testing.assert_array_equal(got[l][n:n + 1], ref, err_msg="image %d layer %d" % (n, l))
    assert all(g.max() >= 100 for g in got)  # the calibrated scales use the int8 range
    for conv in convs:
        conv.close()


def test_c4_as_stated_batch_64_at_224(hip, oracle):
    """The MobileNetV2-style network at 64x3x224x224 through otter::Net: images are independent (an image alone
    reproduces its slice of the batch bit for bit, at the logits and at an int8 blob in the middle), and the first
    image matches the oracle's walk through all 52 convolutions, the adds, the pooling and the inner product."""
    from tensor_amd import hostnet, mobilenet
    rng = np.random.default_rng(0)
    batch, hw = 64, 224
    layers = mobilenet.describe()
    params = mobilenet.init_weights(layers, rng)
    mobilenet.calibrate(hip, capi, layers, params, rng.uniform(0, 1, (32, 3, hw, hw)).astype(np.float32))
    x = rng.uniform(0, 1, (batch, 3, hw, hw)).astype(np.float32)
    net = mobilenet.build_net(hostnet, layers, params, batch, hw)
    logits = net.run("data", x, "fc").reshape(batch, -1)
    mid = net.run("data", x, "b7_dw")
    assert mid.dtype == np.int8
    net1 = mobilenet.build_net(hostnet, layers, params, 1, hw)
    for n in (0, 40, batch - 1):
        np.testing.assert_array_equal(net1.run("data", x[n:n + 1], "fc").reshape(1, -1), logits[n:n + 1])
        np.testing.assert_array_equal(net1.run("data", x[n:n + 1], "b7_dw"), mid[n:n + 1])
    want = mobilenet_oracle_forward(oracle, layers, params, x[:1])
    np.testing.assert_array_equal(mid[:1], want["b7_dw"])
    # Behind the blocks that run as one launch under the DEFAULT policy at this size (the 28x28, 14x14 and 7x7 blocks,
    # the 7x7 ones with a band's expanded channels dealt to several workgroups whose partial sums meet in memory): the
    # last block's int8 result bit for bit, the head convolution's fp32 result and the pooled features at 1e-5.
    blocks = hostnet.block_forward_count()
    prj = net.run("data", x, "b16_project")
    assert hostnet.block_forward_count() >= blocks + 11  # (asking for a block's own result keeps it one launch)
    assert prj.dtype == np.int8
    np.testing.assert_array_equal(prj[:1], want["b16_project"])
    np.testing.assert_array_equal(prj[40:41], net1.run("data", x[40:41], "b16_project"))
    np.testing.assert_allclose(net.run("data", x, "head")[:1], want["head"], rtol=FP32_RTOL, atol=1e-30)
    pooled = net.run("data", x, "pool").reshape(batch, -1)
    np.testing.assert_allclose(pooled[:1], want["pool"].reshape(1, -1), rtol=FP32_RTOL, atol=1e-30)
    # The logits are 1280-term fp32 dot products whose terms cancel; the GPU adds them in another order than the oracle
    # (sixteen partial sums on the matrix cores), so the bound that holds is relative to the sum of the terms' magnitudes,
    # not to the (possibly much smaller) result: |got - exact| <= 1e-5 * (|w| . |x| + |b|), exact in float64 from the
    # GPU's own pooled features; and the oracle's logits lie inside the same bound.
    fc = params["fc"]
    w64, p64 = fc["w"].astype(np.float64), pooled[:1].astype(np.float64)
    exact = p64 @ w64.T + fc["bias"].astype(np.float64)
    bound = FP32_RTOL * (np.abs(p64) @ np.abs(w64).T + np.abs(fc["bias"].astype(np.float64)))
    assert (np.abs(logits[:1] - exact) <= bound).all()
    assert (np.abs(want["fc"] - exact) <= 2 * bound).all()
