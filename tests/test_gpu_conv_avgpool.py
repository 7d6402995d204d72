"""otter_hip_conv_forward_avgpool: a convolution with an fp32 result and the mean over the image of that result (the
tail of a classifier). As one launch (pointwise layer, Byte8 input, at most 64 pixels) the convolution's own blob is not
made; the means must equal those of the oracle's layer + pooling within the fp32 tolerance of a sum of H*W terms, and
those of the two launches."""
import numpy as np
import pytest

from tensor_amd import capi

pytestmark = pytest.mark.gpu

MEAN_RTOL = 1e-5  # (49 fp32 additions in another order than the oracle's double sum)

CASES = [
    # C, K, N, H, W, k, pad, act, bias, launches
    (320, 1280, 4, 7, 7, 1, 0, 3, True, 1),   # MobileNetV2's head
    (64, 40, 3, 8, 8, 1, 0, 0, True, 1),      # 64 pixels, K not a multiple of 32, signed values
    (24, 8, 2, 1, 1, 1, 0, 1, False, 1),      # one pixel, one octet of results
    (136, 100, 2, 5, 9, 1, 0, 2, True, 1),    # LeakyReLU, K % 4 == 0 only, 17 input octets
    (448, 64, 2, 4, 4, 1, 0, 3, True, 1),     # seven reduction steps (the looped form of the kernel, odd count)
    (384, 32, 1, 3, 5, 1, 0, 0, False, 1),    # six reduction steps
    (32, 64, 2, 9, 9, 1, 0, 3, True, 2),      # 81 pixels: the layer and the pooling one after the other
    (16, 32, 2, 6, 6, 3, 1, 1, True, 2),      # a 3x3 layer
]


@pytest.mark.parametrize("C,K,N,H,W,k,pad,act,with_bias,launches", CASES)
def test_conv_avgpool_equals_layer_then_pooling(hip, oracle, C, K, N, H, W, k, pad, act, with_bias, launches):
    rng = np.random.default_rng(C + K + H)
    wf = rng.normal(0, 1.0 / np.sqrt(C * k * k), (K, C, k, k)).astype(np.float32)
    ws = (np.float32(127) / np.abs(wf).reshape(K, -1).max(axis=1)).astype(np.float32)
    wq = np.clip(np.round(wf * ws[:, None, None, None]), -127, 127).astype(np.int8)
    in_scale = np.float32(25.0)
    bias = rng.normal(0, 0.5, K).astype(np.float32) if with_bias else None
    conv = hip.conv(wq=wq, scale_in=(np.float32(1) / (in_scale * ws)).astype(np.float32), bias=bias, in_scale=float(in_scale),
                    pad=(pad, pad), act=act, act_p0=0.1 if act == 2 else 0.0, out_kind=capi.OUT_F32)
    assert conv.avgpool_launches(capi.I8_P8, N, H, W) == launches
    x = rng.integers(-127, 128, (N, C, H, W)).astype(np.int8)
    xd = hip.to_device(capi.pack_np(x, 8))
    got = conv.forward_avgpool(xd, capi.I8_P8, N, H, W).cpu().numpy().reshape(N, K)
    # the oracle's layer, then its pooling
    blob = oracle.conv_layer_forward(x, wq, ws, float(in_scale), stride=(1, 1), pad=(pad, pad), bias=bias, int8_out=False,
                                     act_type=act, act_params=[0.1] if act == 2 else None)
    want = blob.reshape(N, K, -1).astype(np.float64).mean(axis=2)
    np.testing.assert_allclose(got, want, rtol=MEAN_RTOL, atol=1e-30 if act in (1, 3) else 1e-6)
    # the layer's own blob through the library, then the library's pooling
    oh, ow = conv.out_hw(H, W)
    layout = capi.F32_P4 if K % 4 == 0 else capi.F32
    b2 = conv.forward(xd, capi.I8_P8, N, H, W, layout)
    two = hip.global_avgpool(b2, layout, N, K, oh, ow).cpu().numpy().reshape(N, K)
    np.testing.assert_allclose(got, two, rtol=MEAN_RTOL, atol=1e-30 if act in (1, 3) else 1e-6)
    conv.close()


def test_conv_avgpool_refuses_an_int8_layer(hip):
    rng = np.random.default_rng(1)
    wq = rng.integers(-127, 128, (16, 16, 1, 1)).astype(np.int8)
    conv = hip.conv(wq=wq, scale_in=np.full(16, 0.01, np.float32), bias=None, in_scale=10.0, out_scale=[20.0], out_kind=capi.OUT_I8)
    assert hip.lib.otter_hip_conv_avgpool_launches(conv.h, capi.I8_P8, 1, 4, 4) == -2
    conv.close()
