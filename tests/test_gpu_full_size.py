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
from gpu_util import run_conv

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
