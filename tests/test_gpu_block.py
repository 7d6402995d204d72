"""otter_hip_conv_block_forward: an inverted-residual block (1x1 expand -> depthwise 3x3 -> 1x1 project, optionally
+ shortcut and the quantized twin of the result) as one launch that keeps the expanded tensor in LDS. The result must
be, bit for bit, what the three layers give one by one through otter_hip_conv_forward (+ _residual / _twin), and what
the oracle gives for the three layers (int8 blobs bit-exact, the fp32 result within FP32_RTOL, in fact bitwise)."""
import numpy as np
import pytest

from tensor_amd import capi

pytestmark = pytest.mark.gpu

FP32_RTOL = 1e-5


@pytest.fixture(autouse=True)
def every_qualifying_block_as_one_launch(hip):
    """By default the single launch is only taken for the shapes it was measured faster on; the tests here exercise it
    on every shape it can run."""
    before = hip.conv_block_set_always(1)
    yield
    hip.conv_block_set_always(before)


def quantize_weights(wf):
    K = wf.shape[0]
    ws = (np.float32(127) / np.abs(wf).reshape(K, -1).max(axis=1)).astype(np.float32)
    wq = np.clip(np.round(wf * ws[:, None, None, None]), -127, 127).astype(np.int8)
    return wq, ws


def make_block(hip, rng, cin, ce, cout, act, f32_out, stride=1, out_round=capi.ROUND_SSE, dw_pad=1):
    """The three layers as a MobileNetV2 block has them: expand and depthwise with `act` and int8 results, a linear
    project layer with an fp32 or int8 result."""
    layers = []
    in_scale = np.float32(rng.uniform(20, 60))
    specs = [(cin, ce, 1, 1, 0, 1, act, True), (ce, ce, 3, stride, dw_pad, ce, act, True), (ce, cout, 1, 1, 0, 1, 0, not f32_out)]
    for (ci, co, k, s, pad, groups, a, i8) in specs:
        wq, ws = quantize_weights(rng.normal(0, 0.3 if groups > 1 else 2.0 / np.sqrt(ci), (co, ci // groups, k, k)).astype(np.float32))
        bias = rng.normal(0, 0.05, co).astype(np.float32)
        out_scale = np.float32(rng.uniform(15, 40))
        si = (np.float32(1.0) / (in_scale * ws)).astype(np.float32)
        conv = hip.conv(wq=wq, scale_in=si, bias=bias, in_scale=float(in_scale), out_scale=[out_scale] if i8 else None,
                        stride=(s, s), pad=(pad, pad), groups=groups, act=a,
                        out_kind=capi.OUT_I8 if i8 else capi.OUT_F32, out_round=out_round)
        layers.append(dict(conv=conv, wq=wq, ws=ws, bias=bias, in_scale=float(in_scale), out_scale=float(out_scale), k=k,
                           stride=s, pad=pad, groups=groups, act=a, int8_out=i8))
        in_scale = out_scale
    return layers


def one_by_one(hip, layers, xd, n, h, w, residual, q_scale):
    e, d, p = (l["conv"] for l in layers)
    t = e.forward(xd, capi.I8_P8, n, h, w, capi.I8_P8)
    t = d.forward(t, capi.I8_P8, n, h, w, capi.I8_P8)
    oh, ow = d.out_hw(h, w)
    if residual is not None:
        return p.forward_residual(t, capi.I8_P8, n, oh, ow, residual, q_scale=q_scale)
    if q_scale is not None:
        return p.forward_twin(t, capi.I8_P8, n, oh, ow, q_scale, capi.ROUND_SSE)
    return p.forward(t, capi.I8_P8, n, oh, ow), None


CASES = [
    # cin, ce, cout, N, H, W, act, f32_out, residual, twin, plan
    (64, 384, 64, 5, 14, 14, 3, True, True, True, None),      # a 14x14 MobileNetV2 block, automatic plan
    (64, 384, 64, 3, 14, 14, 3, True, True, True, (4, 128)),  # four bands, 128-channel slices
    (64, 384, 64, 3, 14, 14, 3, True, True, True, (8, 64)),   # two bands of unequal height
    (160, 960, 160, 3, 7, 7, 3, True, True, True, None),      # 7x7: one band, three reduction steps in the expand layer
    (160, 960, 320, 2, 7, 7, 3, False, False, False, None),   # int8 result, ten channel pairs in the project layer
    (32, 192, 32, 3, 28, 28, 3, True, True, True, None),      # 28x28
    (24, 144, 24, 2, 56, 56, 3, True, True, True, None),      # 56x56, 24 channels (padded reduction), 144 = 2.25 slices
    (96, 576, 96, 3, 14, 14, 1, True, True, False, None),     # ReLU, 4.5 slices of 128, no twin
    (64, 384, 96, 3, 14, 14, 3, True, False, True, None),     # no shortcut (channel count changes), twin only
    (40, 136, 24, 2, 11, 13, 0, True, False, False, None),    # no activation (signed blobs), odd sizes, nothing fused behind
    (16, 96, 24, 2, 9, 64, 3, True, False, False, None),      # the widest image the launch takes
    (8, 48, 8, 1, 1, 1, 3, True, True, True, None),           # a single pixel
    (160, 960, 160, 5, 7, 7, 3, True, True, True, (0, 0, 4)),  # a band's slices dealt to four workgroups
    (64, 384, 64, 3, 14, 14, 3, True, True, True, (4, 64, 3)),  # six slices over three workgroups per band
    (160, 960, 320, 3, 7, 7, 3, False, False, False, (0, 128, 8)),  # one slice per workgroup, int8 result
    (32, 200, 32, 2, 10, 12, 0, True, True, False, (0, 64, 3)),  # four slices over three workgroups: the last takes none... two
]


@pytest.mark.parametrize("cin,ce,cout,N,H,W,act,f32_out,with_res,with_twin,plan", CASES)
def test_block_equals_the_three_layers(hip, oracle, cin, ce, cout, N, H, W, act, f32_out, with_res, with_twin, plan):
    rng = np.random.default_rng(cin * 1000 + ce + H)
    layers = make_block(hip, rng, cin, ce, cout, act, f32_out)
    e, d, p = (l["conv"] for l in layers)
    if plan is not None:
        e.set_block_plan(*plan)
    assert hip.conv_block_launches(e, d, p, N, H, W) == 1
    x = rng.integers(-127, 128, (N, cin, H, W)).astype(np.int8)
    xd = hip.to_device(capi.pack_np(x, 8))
    res = resd = None
    if with_res:
        res = rng.normal(0, 1, (N, cout, H, W)).astype(np.float32)
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
    # against the oracle, layer by layer
    cur = x
    for l in layers:
        cur = oracle.conv_layer_forward(cur, l["wq"], l["ws"], l["in_scale"], stride=(l["stride"],) * 2, pad=(l["pad"],) * 2,
                                        groups=l["groups"], bias=l["bias"], top_scale=l["out_scale"], int8_out=l["int8_out"],
                                        act_type=l["act"])
    if with_res:
        cur = oracle.eltwise_add(cur, res)
    out = capi.unpack_np(got.cpu().numpy(), 4 if f32_out else 8, (N, cout, H, W))
    if f32_out:
        np.testing.assert_allclose(out, cur, rtol=FP32_RTOL, atol=0)
        assert (out.view(np.int32) == cur.view(np.int32)).all()
        if with_twin:
            q = oracle.quantize(cur, np.float32(q_scale), capi.ROUND_SSE)
            assert (capi.unpack_np(got_q.cpu().numpy(), 8, (N, cout, H, W)) == q).all()
    else:
        assert (out == cur).all()
    for l in layers:
        l["conv"].close()


@pytest.mark.parametrize("act,f32_out", [(3, True), (0, False)])
def test_block_with_the_exact_rounding_mode(hip, act, f32_out):
    """Layers that round with 0.49999997 (the reference's unpacked route) keep that constant inside the single launch,
    in both requantizations, the int8 result and the quantized twin."""
    rng = np.random.default_rng(11 + act)
    layers = make_block(hip, rng, 64, 384, 64, act, f32_out, out_round=capi.ROUND_EXACT)
    e, d, p = (l["conv"] for l in layers)
    N, H, W = 3, 14, 14
    assert hip.conv_block_launches(e, d, p, N, H, W) == 1
    x = rng.integers(-127, 128, (N, 64, H, W)).astype(np.int8)
    xd = hip.to_device(capi.pack_np(x, 8))
    q_scale = 17.25 if f32_out else None
    got, got_q = hip.conv_block(e, d, p, xd, N, H, W, q_scale=q_scale, q_round_mode=capi.ROUND_EXACT)
    t = e.forward(xd, capi.I8_P8, N, H, W, capi.I8_P8)
    t = d.forward(t, capi.I8_P8, N, H, W, capi.I8_P8)
    if f32_out:
        want, want_q = p.forward_twin(t, capi.I8_P8, N, H, W, q_scale, capi.ROUND_EXACT)
    else:
        want, want_q = p.forward(t, capi.I8_P8, N, H, W), None
    hip.torch.cuda.synchronize()
    assert hip.torch.equal(got, want)
    if f32_out:
        assert hip.torch.equal(got_q, want_q)
    for l in layers:
        l["conv"].close()


@pytest.mark.parametrize("cin,ce,cout,H,split,f32_out", [(160, 960, 160, 7, 4, True), (160, 960, 320, 7, 8, False),
                                                         (64, 384, 64, 14, 3, True)])
def test_split_bands_on_changing_inputs_sharing_one_workspace(hip, cin, ce, cout, H, split, f32_out):
    """Bands whose slices are dealt to several workgroups hand their partial sums over through the workspace. Launches
    on DIFFERENT inputs, back to back on one stream and one workspace with no synchronisation in between: a partial sum
    that the last workgroup of a band picked up before its store had landed would be the previous launch's (a different
    number here), so every result must equal the three layers one by one bit for bit."""
    torch = hip.torch
    rng = np.random.default_rng(77 + H + split)
    N, W = 6, H
    layers = make_block(hip, rng, cin, ce, cout, 3, f32_out)
    e, d, p = (l["conv"] for l in layers)
    e.set_block_plan(0, 0, split)
    assert hip.conv_block_launches(e, d, p, N, H, W) == 1
    import ctypes
    plan = (ctypes.c_int * 6)()
    assert hip.lib.otter_hip_conv_block_plan(cin, ce, cout, N, H, W, 0, 0, split, plan) == 0
    assert plan[4] > 1 and plan[5] > 0  # several workgroups per band, partial sums in the workspace
    xs = [hip.to_device(capi.pack_np(rng.integers(-127, 128, (N, cin, H, W)).astype(np.int8), 8)) for _ in range(8)]
    wants = [one_by_one(hip, layers, x, N, H, W, None, None)[0].clone() for x in xs]
    ws = hip.empty(hip.lib.otter_hip_conv_block_workspace_bytes(e.h, d.h, p.h, N, H, W), np.int8)
    outs = [hip.empty(N * cout * H * W, np.float32 if f32_out else np.int8) for _ in xs]
    torch.cuda.synchronize()
    for rep in range(4):
        for x, out in zip(xs, outs):
            hip.conv_block(e, d, p, x, N, H, W, out=out, workspace=ws)
        torch.cuda.synchronize()
        for out, want in zip(outs, wants):
            assert torch.equal(out, want.view(-1))
            out.zero_()
    for l in layers:
        l["conv"].close()


def test_block_replayed_from_a_captured_graph(hip):
    """A launch whose bands are dealt to several workgroups, captured into a graph and replayed on new inputs, with eager
    launches in between: the arrival counters it was captured with are left at zero by every launch, so each replay
    equals the three layers one by one."""
    torch = hip.torch
    rng = np.random.default_rng(23)
    N, H, W = 5, 7, 7
    layers = make_block(hip, rng, 160, 960, 160, 3, True)
    e, d, p = (l["conv"] for l in layers)
    e.set_block_plan(0, 0, 4)
    assert hip.conv_block_launches(e, d, p, N, H, W) == 1
    xs = [hip.to_device(capi.pack_np(rng.integers(-127, 128, (N, 160, H, W)).astype(np.int8), 8)) for _ in range(3)]
    res = hip.to_device(capi.pack_np(rng.normal(0, 1, (N, 160, H, W)).astype(np.float32), 4))
    wants = [tuple(t.clone() for t in one_by_one(hip, layers, x, N, H, W, res, 21.5)) for x in xs]
    x_static = xs[0].clone()
    out = hip.empty(N * 160 * H * W, np.float32)
    q = hip.empty(N * 160 * H * W, np.int8)
    ws = hip.empty(hip.lib.otter_hip_conv_block_workspace_bytes(e.h, d.h, p.h, N, H, W), np.int8)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):  # (the first launch of a kernel raises its LDS limit: not inside a capture)
        hip.conv_block(e, d, p, x_static, N, H, W, residual=res, q_scale=21.5, out=out, q=q, workspace=ws)
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        hip.conv_block(e, d, p, x_static, N, H, W, residual=res, q_scale=21.5, out=out, q=q, workspace=ws)
    for rep in range(2):
        for x, (want, want_q) in zip(xs, wants):
            x_static.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, want.view(-1)) and torch.equal(q, want_q.view(-1))
            with torch.cuda.stream(side):
                eager, eager_q = hip.conv_block(e, d, p, x, N, H, W, residual=res, q_scale=21.5)
            side.synchronize()
            assert torch.equal(eager, want) and torch.equal(eager_q, want_q)
    for l in layers:
        l["conv"].close()


def test_default_policy_takes_the_measured_shapes_only(hip):
    hip.conv_block_set_always(0)
    rng = np.random.default_rng(3)
    for (cin, ce, cout, n, hw, want) in [(64, 384, 64, 64, 14, 1), (32, 192, 32, 64, 28, 1), (24, 144, 24, 64, 56, 2),
                                          (160, 960, 160, 64, 7, 1), (160, 960, 320, 64, 7, 1), (96, 576, 96, 64, 14, 1), (64, 384, 64, 4, 14, 3),
                                          (64, 384, 64, 16, 14, 1)]:
        layers = make_block(hip, rng, cin, ce, cout, 3, True)
        e, d, p = (l["conv"] for l in layers)
        assert hip.conv_block_launches(e, d, p, n, hw, hw) == want
        for l in layers:
            l["conv"].close()


def test_block_falls_back_to_three_launches(hip):
    """A stride-2 depthwise layer is not what the single launch takes, and 160 input channels are more than the launch
    of the first two layers takes: the same call runs the layers one by one."""
    rng = np.random.default_rng(5)
    layers = make_block(hip, rng, 160, 192, 64, 3, True, stride=2)
    e, d, p = (l["conv"] for l in layers)
    N, H, W = 2, 28, 28
    assert hip.conv_block_launches(e, d, p, N, H, W) == 3
    x = rng.integers(-127, 128, (N, 160, H, W)).astype(np.int8)
    xd = hip.to_device(capi.pack_np(x, 8))
    got, got_q = hip.conv_block(e, d, p, xd, N, H, W, q_scale=30.0)
    t = e.forward(xd, capi.I8_P8, N, H, W, capi.I8_P8)
    t = d.forward(t, capi.I8_P8, N, H, W, capi.I8_P8)
    want, want_q = p.forward_twin(t, capi.I8_P8, N, 14, 14, 30.0, capi.ROUND_SSE)
    hip.torch.cuda.synchronize()
    assert hip.torch.equal(got, want) and hip.torch.equal(got_q, want_q)
    for l in layers:
        l["conv"].close()


def test_block_random_shapes(hip):
    """Seeded random blocks (channel counts, image sizes, activations, result kinds, plans): wherever the single launch
    takes the shape it equals the three layers one by one, bit for bit."""
    rng = np.random.default_rng(2024)
    taken = 0
    for case in range(40):
        cin = 8 * int(rng.integers(1, 25))
        ce = 8 * int(rng.integers(1, min(6 * cin // 8, 144) + 1))
        cout = 8 * int(rng.integers(1, 21))
        N, H, W = int(rng.integers(1, 4)), int(rng.integers(1, 21)), int(rng.integers(1, 31))
        act = int(rng.choice([0, 1, 3]))
        f32_out = bool(rng.integers(0, 2))
        with_res = f32_out and cin == cout and bool(rng.integers(0, 2))
        with_twin = f32_out and bool(rng.integers(0, 2))
        layers = make_block(hip, rng, cin, ce, cout, act, f32_out)
        e, d, p = (l["conv"] for l in layers)
        if rng.integers(0, 2):
            e.set_block_plan(int(rng.integers(0, H + 1)), int(rng.choice([0, 64, 128])), int(rng.integers(0, 5)))
        if hip.conv_block_launches(e, d, p, N, H, W) == 1:
            taken += 1
            xd = hip.to_device(capi.pack_np(rng.integers(-127, 128, (N, cin, H, W)).astype(np.int8), 8))
            resd = hip.to_device(capi.pack_np(rng.normal(0, 1, (N, cout, H, W)).astype(np.float32), 4)) if with_res else None
            q_scale = 19.0 if with_twin else None
            got, got_q = hip.conv_block(e, d, p, xd, N, H, W, residual=resd, q_scale=q_scale)
            want, want_q = one_by_one(hip, layers, xd, N, H, W, resd, q_scale)
            hip.torch.cuda.synchronize()
            assert hip.torch.equal(got, want), (case, cin, ce, cout, N, H, W, act, f32_out)
            if with_twin:
                assert hip.torch.equal(got_q, want_q), (case, cin, ce, cout, N, H, W)
        for l in layers:
            l["conv"].close()
    assert taken >= 20
