"""otter_hip_conv_chain_forward: a chain of int8 -> int8 convolution layers. Where the layers are the same 3x3 "same"
geometry the chain is one persistent launch whose workgroups hand tiles from layer to layer through flags; the result
must be, bit for bit, what the layers give one by one (and what the oracle gives on sampled images), call after call,
with no workgroup ever giving up a wait. Other chains run layer by layer behind the same entry point."""
import numpy as np
import pytest

from tensor_amd import capi

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def every_qualifying_chain_as_one_launch(hip):
    """By default the single launch is only taken for problems large enough to gain from it; the tests here exercise it
    on small shapes, so the threshold is lifted for their duration."""
    before = hip.conv_chain_set_min_tiles(0)
    yield
    hip.conv_chain_set_min_tiles(before)


def quantize_weights(wf):
    K = wf.shape[0]
    ws = (np.float32(127) / np.abs(wf).reshape(K, -1).max(axis=1)).astype(np.float32)
    wq = np.clip(np.round(wf * ws[:, None, None, None]), -127, 127).astype(np.int8)
    return wq, ws


def _layers(hip, rng, chans, k=3, pad=1, act=1, stride=1):
    convs, params = [], []
    in_scale = np.float32(127.0)
    for cin, cout in zip(chans[:-1], chans[1:]):
        wq, ws = quantize_weights(rng.normal(0, 0.05, (cout, cin, k, k)).astype(np.float32))
        bias = rng.normal(0, 0.02, cout).astype(np.float32)
        out_scale = np.float32(rng.uniform(20, 60))
        si = (np.float32(1.0) / (in_scale * ws)).astype(np.float32)
        convs.append(hip.conv(wq=wq, scale_in=si, bias=bias, out_scale=[out_scale], stride=(stride, stride), pad=(pad, pad),
                              act=act, out_kind=capi.OUT_I8, out_round=capi.ROUND_SSE))
        params.append(dict(wq=wq, ws=ws, bias=bias, in_scale=float(in_scale), out_scale=float(out_scale)))
        in_scale = out_scale
    return convs, params


def _one_by_one(hip, convs, xd, n, h, w):
    cur = xd
    for c in convs:
        cur = c.forward(cur, capi.I8_P8, n, h, w, capi.I8_P8)
        h, w = c.out_hw(h, w)
    return cur


@pytest.mark.parametrize("C,N,H,W,L,act", [
    (128, 16, 28, 28, 4, 1),     # whole tiles, two images per XCD, ReLU
    (72, 19, 13, 26, 3, 3),      # padded channels, ragged tiles, images not a multiple of the XCDs, clip
    (128, 64, 56, 56, 4, 1),     # the benchmark's chain
    (96, 9, 15, 55, 2, 0),       # odd width, no activation (signed results)
    (128, 3, 56, 56, 8, 1),      # fewer images than XCDs, the longest chain one launch takes
    (64, 16, 28, 28, 4, 1),      # 64 channels: the 1 x 4 wave layout (64 channels x 64*FN pixels per tile)
    (40, 5, 17, 30, 3, 0),       # 40 channels padded to 64 rows, ragged tiles, signed results
    (64, 11, 56, 56, 2, 3),      # 64 channels at the benchmark's image size
])
def test_same_shape_chain_is_one_launch_and_equals_the_layers_one_by_one(hip, oracle, C, N, H, W, L, act):
    rng = np.random.default_rng(C + N + H + L)
    convs, params = _layers(hip, rng, [C] * (L + 1), act=act)
    x = rng.integers(-127, 128, size=(N, C, H, W), dtype=np.int8)
    xd = hip.to_device(capi.pack_np(x, 8))
    want = _one_by_one(hip, convs, xd, N, H, W).cpu().numpy()
    assert not hip.conv_chain_gave_up()
    assert hip.conv_chain_launches(convs, N, H, W) == 1
    for rep in range(3):  # the flags and queue counters carry over from launch to launch
        got = hip.conv_chain(convs, xd, N, H, W)
        assert not hip.conv_chain_gave_up()
        np.testing.assert_array_equal(got.cpu().numpy(), want, err_msg="call %d" % rep)
    # and the oracle through all layers on two images
    for n in (0, N - 1):
        cur = x[n:n + 1]
        for p in params:
            cur = oracle.conv_layer_forward(cur, p["wq"], p["ws"], p["in_scale"], pad=(1, 1), bias=p["bias"],
                                            top_scale=p["out_scale"], int8_out=True, act_type=act)
        got_n = capi.unpack_np(got.cpu().numpy(), 8, (N, C, H, W))[n:n + 1]
        np.testing.assert_array_equal(got_n, cur)


def test_other_chains_run_layer_by_layer(hip, oracle):
    rng = np.random.default_rng(5)
    # channel counts change along the chain, and a 1x1 in the middle
    convs, _ = _layers(hip, rng, [32, 64], k=3)
    c2, _ = _layers(hip, rng, [64, 64], k=1, pad=0)
    c3, _ = _layers(hip, rng, [64, 24], k=3, stride=2)
    chain = convs + c2 + c3
    N, H, W = 3, 17, 20
    x = rng.integers(-127, 128, size=(N, 32, H, W), dtype=np.int8)
    xd = hip.to_device(capi.pack_np(x, 8))
    want = _one_by_one(hip, chain, xd, N, H, W).cpu().numpy()
    assert hip.conv_chain_launches(chain, N, H, W) == 3
    got = hip.conv_chain(chain, xd, N, H, W).cpu().numpy()
    np.testing.assert_array_equal(got, want)
    assert not hip.conv_chain_gave_up()


def test_same_shape_chain_that_needs_two_lds_stages_runs_layer_by_layer(hip):
    """72 channels at 13x22: a tile's rows of all 128 padded channels do not fit LDS at once, which the one-launch
    kernel requires; the entry point runs the layers one after the other and the result is the same."""
    rng = np.random.default_rng(8)
    convs, _ = _layers(hip, rng, [72] * 4, act=3)
    N, H, W = 5, 13, 22
    x = rng.integers(-127, 128, size=(N, 72, H, W), dtype=np.int8)
    xd = hip.to_device(capi.pack_np(x, 8))
    want = _one_by_one(hip, convs, xd, N, H, W).cpu().numpy()
    assert hip.conv_chain_launches(convs, N, H, W) == 3
    np.testing.assert_array_equal(hip.conv_chain(convs, xd, N, H, W).cpu().numpy(), want)


def test_chains_on_several_streams_at_once(hip):
    """A GPU has four flag sets; a stream without one takes a free set or an idle one (least recently used, last launch
    completed), so launches on different streams may overlap. Six streams each run their own chain, enqueued back to
    back without a synchronisation in between: the first four are one launch each (the device is idle when they start,
    whoever owned the sets before), the last two are one launch if a set has come free by then and layer by layer if
    not - every result equals the layers one by one."""
    torch = hip.torch
    rng = np.random.default_rng(21)
    N, C, H, W, L = 8, 128, 28, 28, 4
    jobs = []
    for j in range(6):
        convs, _ = _layers(hip, rng, [C] * (L + 1), act=1)
        x = rng.integers(-127, 128, size=(N, C, H, W), dtype=np.int8)
        xd = hip.to_device(capi.pack_np(x, 8))
        want = _one_by_one(hip, convs, xd, N, H, W).cpu().numpy()
        jobs.append((convs, xd, want, torch.cuda.Stream()))
    torch.cuda.synchronize()
    outs = []
    for rep in range(3):
        outs = []
        for j, (convs, xd, want, st) in enumerate(jobs):
            with torch.cuda.stream(st):
                outs.append(hip.conv_chain(convs, xd, N, H, W))
            made = hip.conv_chain_last_launches()
            assert made in (1, L)
            if rep == 0 and j < 4:
                assert made == 1
        torch.cuda.synchronize()
    assert not hip.conv_chain_gave_up()  # (synchronizes the device)
    for (convs, xd, want, st), got in zip(jobs, outs):
        np.testing.assert_array_equal(got.cpu().numpy(), want)


def test_default_rule_takes_the_single_launch_for_large_problems_only(hip):
    """With the default threshold a chain is one launch only where a layer's share of an XCD's tile list is long (the
    benchmark's stack: 8 images x 14 tiles = 112); small stacks of the same geometry run layer by layer."""
    rng = np.random.default_rng(30)
    convs, _ = _layers(hip, rng, [128] * 5, act=1)
    hip.conv_chain_set_min_tiles(96)
    assert hip.conv_chain_launches(convs, 64, 56, 56) == 1
    assert hip.conv_chain_launches(convs, 16, 28, 28) == 4
    assert hip.conv_chain_launches(convs, 8, 56, 56) == 4
    hip.conv_chain_set_min_tiles(0)
    assert hip.conv_chain_launches(convs, 16, 28, 28) == 1


def test_chain_replayed_from_a_captured_graph(hip):
    """The single launch captured into a graph and replayed: every replay must take a fresh epoch number (it lives in
    device memory, not in the kernel arguments), so replays on new inputs, with eager work and synchronisations in
    between, all equal the layers one by one."""
    torch = hip.torch
    rng = np.random.default_rng(40)
    N, C, H, W, L = 16, 128, 28, 28, 3
    convs, _ = _layers(hip, rng, [C] * (L + 1), act=1)
    xs = [hip.to_device(capi.pack_np(rng.integers(-127, 128, size=(N, C, H, W), dtype=np.int8), 8)) for _ in range(3)]
    wants = [_one_by_one(hip, convs, x, N, H, W).clone() for x in xs]
    x_static = xs[0].clone()
    out = hip.empty(N * C * H * W, np.int8)
    ws = hip.empty(2 * N * C * H * W + 1024, np.int8)
    assert hip.conv_chain_launches(convs, N, H, W) == 1
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        hip.conv_chain(convs, x_static, N, H, W, out=out, workspace=ws)  # (first call on this stream: takes a flag set)
    assert hip.conv_chain_last_launches() == 1  # the persistent kernel, not the layers one by one
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        hip.conv_chain(convs, x_static, N, H, W, out=out, workspace=ws)
        assert hip.conv_chain_last_launches() == 1
    for rep in range(2):
        for x, want in zip(xs, wants):
            x_static.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert bool((out == want.view(-1)).all().item())
            # eager work on the same flag set between replays
            with torch.cuda.stream(side):
                eager = hip.conv_chain(convs, x, N, H, W)
            assert hip.conv_chain_last_launches() == 1
            side.synchronize()
            assert bool((eager == want.view(-1)).all().item())
    assert not hip.conv_chain_gave_up()


def test_chain_argument_checks(hip):
    rng = np.random.default_rng(6)
    convs, _ = _layers(hip, rng, [16, 32])
    other, _ = _layers(hip, rng, [16, 16])
    x = hip.to_device(np.zeros(2 * 16 * 8 * 8, np.int8))
    with pytest.raises(capi.HipError):
        hip.conv_chain(convs + other, x, 2, 8, 8)  # 32 channels out, 16 in
    f32 = hip.conv(wq=np.zeros((16, 16, 3, 3), np.int8), scale_in=np.ones(16, np.float32), pad=(1, 1), out_kind=capi.OUT_F32)
    with pytest.raises(capi.HipError):
        hip.conv_chain(other + [f32], x, 2, 8, 8)  # an fp32 result inside a chain
