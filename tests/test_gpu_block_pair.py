"""otter_hip_conv_block_forward where the block does not run as the single launch: the pointwise layer and its depthwise
reader as ONE launch (the expanded rows only ever in LDS), the last layer by itself. The result must be, bit for bit,
what the three layers give one by one through otter_hip_conv_forward (+ _residual / _twin) and what the oracle gives
for the three layers."""
import numpy as np
import pytest

from tensor_amd import capi
from test_gpu_block import FP32_RTOL, make_block, one_by_one

pytestmark = pytest.mark.gpu

CASES = [
    # cin, ce, cout, N, H, W, act, stride, dw_pad, f32_out, residual, twin, strip rows
    (16, 96, 24, 2, 112, 112, 3, 2, 1, True, False, True, 0),   # MobileNetV2's first stride-2 block: 7 pixel groups a row
    (24, 144, 24, 2, 56, 56, 3, 1, 1, True, True, True, 0),     # stride 1 at 56x56, 24 input channels (three octets)
    (24, 144, 32, 2, 56, 56, 3, 2, 1, True, False, True, 0),
    (32, 192, 64, 3, 28, 28, 3, 2, 1, True, False, False, 0),
    (96, 576, 160, 3, 14, 14, 3, 2, 1, True, False, True, 0),   # two reduction steps, one pixel group
    (40, 144, 24, 2, 11, 13, 0, 1, 1, True, False, False, 0),   # five input octets, signed blobs, odd sizes
    (8, 16, 8, 1, 1, 1, 3, 1, 1, True, True, True, 0),          # a single pixel
    (16, 96, 24, 1, 37, 100, 1, 2, 1, False, False, False, 5),  # ReLU, odd height, strips of five rows, int8 result
    (32, 64, 16, 2, 30, 128, 3, 1, 1, True, False, False, 4),   # the widest row: eight pixel groups, two column chunks
    (128, 256, 32, 1, 9, 64, 3, 2, 1, True, False, False, 0),   # 128 input channels at the widest row they take
    (64, 128, 32, 2, 19, 33, 0, 2, 0, True, False, True, 3),    # no padding in the depthwise layer, three pixel groups
    (16, 48, 16, 2, 40, 17, 3, 1, 0, True, False, False, 7),    # no padding, stride 1
    (8, 32, 8, 3, 23, 90, 0, 1, 1, False, False, False, 2),     # six pixel groups (rounded up to seven), strips of two rows
]


@pytest.mark.parametrize("cin,ce,cout,N,H,W,act,stride,dw_pad,f32_out,with_res,with_twin,strip", CASES)
def test_pair_launch_equals_the_three_layers(hip, oracle, cin, ce, cout, N, H, W, act, stride, dw_pad, f32_out, with_res,
                                             with_twin, strip):
    rng = np.random.default_rng(cin * 1000 + ce + H + stride)
    layers = make_block(hip, rng, cin, ce, cout, act, f32_out, stride=stride, dw_pad=dw_pad)
    e, d, p = (l["conv"] for l in layers)
    if strip:
        e.set_block_plan(strip, 0, 0)
    always = hip.conv_block_set_always(0)
    pair = hip.conv_block_set_pair(1)  # wherever the kernel takes the shapes, not only where it was measured faster
    try:
        launches = hip.conv_block_launches(e, d, p, N, H, W)
        if launches == 1:
            pytest.skip("this shape runs as the single launch")
        assert launches == 2
        x = rng.integers(-127, 128, (N, cin, H, W)).astype(np.int8)
        xd = hip.to_device(capi.pack_np(x, 8))
        oh, ow = d.out_hw(H, W)
        res = resd = None
        if with_res:
            res = rng.normal(0, 1, (N, cout, oh, ow)).astype(np.float32)
            resd = hip.to_device(capi.pack_np(res, 4))
        q_scale = 21.5 if with_twin else None
        for _ in range(2):  # twice: nothing may depend on what the previous call left in LDS or memory
            got, got_q = hip.conv_block(e, d, p, xd, N, H, W, residual=resd, q_scale=q_scale)
            hip.torch.cuda.synchronize()
            want, want_q = one_by_one(hip, layers, xd, N, H, W, resd, q_scale)
            hip.torch.cuda.synchronize()
            assert hip.torch.equal(got, want)
            if with_twin:
                assert hip.torch.equal(got_q, want_q)
        # the layers one by one behind the same call give the same
        hip.conv_block_set_pair(-1)
        assert hip.conv_block_launches(e, d, p, N, H, W) == 3
        got3, _ = hip.conv_block(e, d, p, xd, N, H, W, residual=resd, q_scale=q_scale)
        assert hip.torch.equal(got3, got)
    finally:
        hip.conv_block_set_always(always)
        hip.conv_block_set_pair(pair)
    # against the oracle, layer by layer
    cur = x
    for l in layers:
        cur = oracle.conv_layer_forward(cur, l["wq"], l["ws"], l["in_scale"], stride=(l["stride"],) * 2, pad=(l["pad"],) * 2,
                                        groups=l["groups"], bias=l["bias"], top_scale=l["out_scale"], int8_out=l["int8_out"],
                                        act_type=l["act"])
    if with_res:
        cur = oracle.eltwise_add(cur, res)
    out = capi.unpack_np(got.cpu().numpy(), 4 if f32_out else 8, (N, cout, oh, ow))
    if f32_out:
        np.testing.assert_allclose(out, cur, rtol=FP32_RTOL, atol=0)
        assert (out.view(np.int32) == cur.view(np.int32)).all()
        if with_twin:
            q = oracle.quantize(cur, np.float32(q_scale), capi.ROUND_SSE)
            assert (capi.unpack_np(got_q.cpu().numpy(), 8, (N, cout, oh, ow)) == q).all()
    else:
        assert (out == cur).all()
    for l in layers:
        l["conv"].close()


def test_pair_launch_with_the_exact_rounding_mode(hip):
    """Layers that round with 0.49999997 (the reference's unpacked route) keep that constant in both requantizations of
    the shared launch."""
    rng = np.random.default_rng(5)
    layers = make_block(hip, rng, 24, 144, 32, 3, False, stride=2, out_round=capi.ROUND_EXACT)
    e, d, p = (l["conv"] for l in layers)
    N, H, W = 2, 30, 44
    assert hip.conv_block_launches(e, d, p, N, H, W) == 2  # (a stride-2 depthwise layer: taken by default)
    x = rng.integers(-127, 128, (N, 24, H, W)).astype(np.int8)
    xd = hip.to_device(capi.pack_np(x, 8))
    got, _ = hip.conv_block(e, d, p, xd, N, H, W)
    want, _ = one_by_one(hip, layers, xd, N, H, W, None, None)
    assert hip.torch.equal(got, want)
    for l in layers:
        l["conv"].close()


def test_pair_launch_random_shapes(hip):
    """Seeded random blocks (channel counts, image sizes, strides, padding, activations, result kinds, strip heights):
    wherever the launch of the first two layers takes the shape it equals the three layers one by one, bit for bit."""
    rng = np.random.default_rng(77)
    always = hip.conv_block_set_always(2)  # (never the single launch: every block here goes to the pair or to three)
    pair = hip.conv_block_set_pair(1)
    taken = 0
    try:
        for case in range(48):
            cin = 8 * int(rng.integers(1, 17))
            ce = 16 * int(rng.integers(1, 13))
            cout = 8 * int(rng.integers(1, 9))
            stride = int(rng.choice([1, 2]))
            dw_pad = int(rng.choice([0, 1, 1]))
            N, H = int(rng.integers(1, 4)), int(rng.integers(3, 40))
            W = int(rng.integers(3, 129 if cin <= 32 else 65))
            act = int(rng.choice([0, 1, 3]))
            f32_out = bool(rng.integers(0, 2))
            layers = make_block(hip, rng, cin, ce, cout, act, f32_out, stride=stride, dw_pad=dw_pad)
            e, d, p = (l["conv"] for l in layers)
            strip = int(rng.choice([0, 0, 1, 2, 3, 5, 9]))
            if strip:
                e.set_block_plan(strip, 0, 0)
                hip.conv_block_set_always(2)
            launches = hip.conv_block_launches(e, d, p, N, H, W)
            x = rng.integers(-127, 128, (N, cin, H, W)).astype(np.int8)
            xd = hip.to_device(capi.pack_np(x, 8))
            q_scale = 17.0 if f32_out and rng.integers(0, 2) else None
            got, got_q = hip.conv_block(e, d, p, xd, N, H, W, q_scale=q_scale)
            want, want_q = one_by_one(hip, layers, xd, N, H, W, None, q_scale)
            hip.torch.cuda.synchronize()
            assert hip.torch.equal(got, want), (case, cin, ce, cout, stride, dw_pad, N, H, W, act, strip, launches)
            if q_scale is not None:
                assert hip.torch.equal(got_q, want_q), case
            taken += launches == 2
            for l in layers:
                l["conv"].close()
    finally:
        hip.conv_block_set_always(always)
        hip.conv_block_set_pair(pair)
    assert taken >= 30
