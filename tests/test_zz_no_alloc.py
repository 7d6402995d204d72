"""GPU: the allocation-free entry point otter_hip_conv_forward_static against otter_hip_conv_forward, through the C ABI.

The static variant takes its workspace (the quantized copy of an fp32 input, or the channel-padded copy of a blob whose
channel count is not a multiple of 8) from a device array the library holds; every call on a GPU shares it and it keeps
the last call's contents, so each case runs two calls in a row, the second on a smaller input, and both must equal the
ordinary entry point bit for bit. Inputs that need more than the array holds are refused.
"""
import ctypes as C

import numpy as np
import pytest

from gpu_util import host_scale_in, in_layout_for
from tensor_amd import capi

pytestmark = pytest.mark.gpu

STATIC_BYTES = 32 << 20


def _layer(hip, oracle, rng, C_, K, k, s, p, g, act, out_kind):
    wq = rng.integers(-127, 128, size=(K, C_ // g, k, k)).astype(np.int8)
    ws = rng.uniform(50, 400, K).astype(np.float32)
    bias = rng.normal(0, 0.5, K).astype(np.float32)
    in_scale = 90.0
    return hip.conv(wq=wq, scale_in=host_scale_in(ws, in_scale), bias=bias, in_scale=in_scale,
                    out_scale=[9.0] if out_kind == capi.OUT_I8 else None, stride=(s, s), pad=(p, p), groups=g, act=act,
                    out_kind=out_kind, out_round=oracle.requantize_round_mode(C_, K, g, True),
                    in_round=oracle.quantize_round_mode(C_, True))


CASES = [
    # C, K, k, stride, pad, groups, act, out kind, (N, H, W) of the first call, (N, H, W) of the second (smaller)
    (256, 512, 1, 1, 0, 1, 1, capi.OUT_F32, (8, 28, 28), (3, 14, 20)),      # fp32 in -> quantize -> implicit GEMM
    (64, 64, 3, 1, 1, 1, 1, capi.OUT_I8, (4, 56, 56), (1, 20, 22)),         # fp32 in -> quantize -> LDS-halo kernel
    (64, 64, 3, 2, 1, 64, 3, capi.OUT_I8, (4, 56, 56), (2, 17, 13)),        # fp32 in -> quantize -> depthwise
    (12, 16, 3, 1, 1, 1, 0, capi.OUT_F32, (3, 30, 31), (1, 9, 8)),          # C % 8 != 0: channel-padded copy
    (3, 32, 3, 2, 1, 1, 3, capi.OUT_I8, (2, 64, 64), (1, 33, 35)),          # image stem: needs no workspace
]


@pytest.mark.parametrize("case", CASES, ids=["c%d_k%d_%dx%d_s%d_g%d" % c[:6] for c in CASES])
def test_static_forward_equals_forward_twice_in_a_row(hip, oracle, case):
    C_, K, k, s, p, g, act, out_kind, first, second = case
    rng = np.random.default_rng(C_ * 31 + K)
    conv = _layer(hip, oracle, rng, C_, K, k, s, p, g, act, out_kind)
    for (n, h, w) in (first, second):
        x = rng.uniform(-1.4, 1.4, (n, C_, h, w)).astype(np.float32)  # 1.4 * 90 = 126
        layout = in_layout_for(x, C_)
        xd = hip.to_device(capi.pack_np(x, capi.layout_pack(layout)))
        want = conv.forward(xd, layout, n, h, w)
        got = conv.forward_static(xd, layout, n, h, w)
        hip.torch.cuda.synchronize()
        assert got.dtype == want.dtype and got.numel() == want.numel()
        np.testing.assert_array_equal(got.cpu().numpy().view(np.uint8), want.cpu().numpy().view(np.uint8))
        assert want.cpu().numpy().any()
    conv.close()


def test_static_forward_int8_input_needs_no_workspace(hip, oracle):
    rng = np.random.default_rng(5)
    conv = _layer(hip, oracle, rng, 128, 128, 3, 1, 1, 1, 1, capi.OUT_I8)
    # 40 MB of int8 input: more than the static array, but an int8 blob is convolved in place
    n, h, w = 100, 56, 56
    x = hip.torch.randint(-127, 128, (n * 128 * h * w,), dtype=hip.torch.int8, device=hip.device)
    assert hip.lib.otter_hip_conv_workspace_bytes(conv.h, capi.I8_P8, n, h, w) == 0
    want = conv.forward(x, capi.I8_P8, n, h, w)
    got = conv.forward_static(x, capi.I8_P8, n, h, w)
    assert hip.torch.equal(got, want)
    conv.close()


def test_static_forward_refuses_what_does_not_fit(hip, oracle):
    rng = np.random.default_rng(6)
    conv = _layer(hip, oracle, rng, 256, 256, 3, 1, 1, 256, 3, capi.OUT_I8)
    n, h, w = 11, 112, 112  # 35 MB quantized copy
    assert hip.lib.otter_hip_conv_workspace_bytes(conv.h, capi.F32_P8, n, h, w) > STATIC_BYTES
    x = hip.torch.zeros(n * 256 * h * w, dtype=hip.torch.float32, device=hip.device)
    out = hip.empty(n * 256 * h * w, np.int8)
    rc = hip.lib.otter_hip_conv_forward_static(conv.h, hip.ptr(x), capi.F32_P8, n, h, w, hip.ptr(out), capi.I8_P8,
                                               hip.stream())
    assert rc == -1
    assert b"static" in hip.lib.otter_hip_last_error()
    # the largest batch that fits still runs, and equals the ordinary entry point
    n = 10
    assert hip.lib.otter_hip_conv_workspace_bytes(conv.h, capi.F32_P8, n, h, w) <= STATIC_BYTES
    xs = hip.torch.rand(n * 256 * h * w, dtype=hip.torch.float32, device=hip.device)
    assert hip.torch.equal(conv.forward_static(xs, capi.F32_P8, n, h, w), conv.forward(xs, capi.F32_P8, n, h, w))
    conv.close()
