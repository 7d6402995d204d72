"""The boundary's threading promise: one otter_hip_conv_t (and one otter::Net) used from several host threads at once,
each thread on its own stream with its own workspaces and blobs (the reference: one const Net, an Extractor per thread,
Tensor/Net.cpp:668-736). Every result must equal the single-threaded one."""
import threading

import numpy as np
import pytest

from tensor_amd import capi, hostnet
from test_gpu_block import make_block, one_by_one

pytestmark = pytest.mark.gpu


def _qweights(rng, K, Cg, k):
    wf = rng.normal(0, 0.05, (K, Cg, k, k)).astype(np.float32)
    ws = (np.float32(127) / np.abs(wf).reshape(K, -1).max(axis=1)).astype(np.float32)
    return np.clip(np.round(wf * ws[:, None, None, None]), -127, 127).astype(np.int8), ws


def _run_threads(workers):
    errors = []

    def guarded(fn):
        try:
            fn()
        except BaseException as e:  # noqa: BLE001 (the assertion of a worker must reach the test)
            errors.append(e)

    threads = [threading.Thread(target=guarded, args=(w,)) for w in workers]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
        assert not t.is_alive(), "a worker thread did not finish"
    if errors:
        raise errors[0]


def test_shared_handles_from_two_threads(hip):
    """Two threads share a 3x3 layer, a chain of three such layers (one persistent launch each: the per-stream flag sets
    and the lock around their launches) and an inverted-residual block whose bands are dealt to four workgroups (the
    arrival counters); each thread has its own stream, inputs, outputs and workspaces."""
    torch = hip.torch
    rng = np.random.default_rng(91)
    C, N, H, W = 128, 16, 28, 28
    convs = []
    scale = np.float32(30.0)
    for _ in range(3):
        wq, ws = _qweights(rng, C, C, 3)
        top = np.float32(rng.uniform(15, 30))
        convs.append(hip.conv(wq=wq, scale_in=(np.float32(1) / (scale * ws)).astype(np.float32),
                              bias=rng.normal(0, 0.05, C).astype(np.float32), in_scale=float(scale), out_scale=[top],
                              pad=(1, 1), act=1, out_kind=capi.OUT_I8))
        scale = top
    layers = make_block(hip, rng, 160, 960, 160, 3, True)
    e, d, p = (l["conv"] for l in layers)
    e.set_block_plan(0, 0, 4)
    BN, BH = 5, 7
    always = hip.conv_block_set_always(1)
    old_tiles = hip.conv_chain_set_min_tiles(0)
    try:
        assert hip.conv_chain_launches(convs, N, H, W) == 1
        assert hip.conv_block_launches(e, d, p, BN, BH, BH) == 1
        jobs = []
        for t in range(2):
            xs = [hip.to_device(capi.pack_np(rng.integers(-127, 128, (N, C, H, W)).astype(np.int8), 8)) for _ in range(3)]
            bx = [hip.to_device(capi.pack_np(rng.integers(-127, 128, (BN, 160, BH, BH)).astype(np.int8), 8)) for _ in range(3)]
            want_layer = [convs[0].forward(x, capi.I8_P8, N, H, W, capi.I8_P8).clone() for x in xs]
            want_chain = []
            for x in xs:
                cur = x
                for c in convs:
                    cur = c.forward(cur, capi.I8_P8, N, H, W, capi.I8_P8)
                want_chain.append(cur.clone())
            want_block = [one_by_one(hip, layers, x, BN, BH, BH, None, None)[0].clone() for x in bx]
            jobs.append((xs, bx, want_layer, want_chain, want_block, torch.cuda.Stream()))
        torch.cuda.synchronize()
        chain_launches = [[], []]

        def worker(t):
            xs, bx, want_layer, want_chain, want_block, stream = jobs[t]
            ws_chain = hip.empty(2 * N * C * H * W + 1024, np.int8)
            ws_block = hip.empty(hip.lib.otter_hip_conv_block_workspace_bytes(e.h, d.h, p.h, BN, BH, BH), np.int8)
            with torch.cuda.stream(stream):
                for rep in range(12):
                    outs = []
                    for i in range(3):
                        a = convs[0].forward(xs[i], capi.I8_P8, N, H, W, capi.I8_P8)
                        b = hip.conv_chain(convs, xs[i], N, H, W, workspace=ws_chain)
                        chain_launches[t].append(hip.conv_chain_last_launches())
                        c, _ = hip.conv_block(e, d, p, bx[i], BN, BH, BH, workspace=ws_block)
                        outs.append((a, b, c))
                    stream.synchronize()
                    for i, (a, b, c) in enumerate(outs):
                        assert torch.equal(a, want_layer[i]), "layer, thread %d" % t
                        assert torch.equal(b, want_chain[i]), "chain, thread %d" % t
                        assert torch.equal(c, want_block[i]), "block, thread %d" % t

        _run_threads([lambda: worker(0), lambda: worker(1)])
        assert not hip.conv_chain_gave_up()
        # two streams, four flag sets: every chain call was the single persistent launch
        assert set(chain_launches[0]) == {1} and set(chain_launches[1]) == {1}
    finally:
        hip.conv_chain_set_min_tiles(old_tiles)
        hip.conv_block_set_always(always)
        for c in convs:
            c.close()
        for l in layers:
            l["conv"].close()


def test_one_net_two_extractors_in_two_threads(hip, oracle):
    """One otter::Net (a run of 3x3 layers that goes through the chain entry point, then an inverted-residual block with
    its shortcut sum that goes through the block entry point), two threads that each run their own passes over it on
    their own input: each gets what a single-threaded pass over that input gives."""
    rng = np.random.default_rng(92)
    N, C0, C, E, H, W = 4, 16, 64, 384, 14, 14
    net = hostnet.Net()
    net.add_layer(type="Input", name="data", batchsize=N, channel=C0, height=H, width=W)
    names = ["c0", "c1", "c2", "c3"]  # c0 reads the fp32 image and changes the channel count; c1..c3 are the run
    for nm in names:
        net.add_layer(type="Convolution", name=nm, out_channels=C, kernel=3, padding=1, int8_scale_term=102, activation="Relu")
    net.add_layer(type="Convolution", name="stem", out_channels=C, kernel=1, int8_scale_term=2)
    net.add_layer(type="Convolution", name="expand", input="stem", out_channels=E, kernel=1, int8_scale_term=102,
                  activation="Relu6")
    net.add_layer(type="Convolution", name="dw", out_channels=E, kernel=3, padding=1, groups=E, int8_scale_term=101,
                  activation="Relu6")
    net.add_layer(type="Convolution", name="project", out_channels=C, kernel=1, int8_scale_term=2)
    net.add_layer(type="Eltwise", name="add", input="stem,project")
    net.compile()
    scale = np.float32(127.0)
    for nm in names:
        w, s = _qweights(rng, C, C0 if nm == "c0" else C, 3)
        top = np.float32(rng.uniform(15, 30))
        net.set_conv(nm, w, rng.normal(0, 0.05, C).astype(np.float32), s, scale, top)
        scale = top
    w, s = _qweights(rng, C, C, 1)
    net.set_conv("stem", w, rng.normal(0, 0.05, C).astype(np.float32), s, scale)
    t6 = np.float32(127.0 / 6.0)
    we, se = _qweights(rng, E, C, 1)
    wd, sd = _qweights(rng, E, 1, 3)
    wp, sp = _qweights(rng, C, E, 1)
    net.set_conv("expand", we, rng.normal(0, 0.1, E).astype(np.float32), se, np.float32(40.0), t6)
    net.set_conv("dw", wd, rng.normal(0, 0.1, E).astype(np.float32), sd, t6, t6)
    net.set_conv("project", wp, rng.normal(0, 0.1, C).astype(np.float32), sp, t6)
    always = hip.conv_block_set_always(1)
    old_tiles = hip.conv_chain_set_min_tiles(0)
    try:
        xs = [rng.uniform(-1, 1, (N, C0, H, W)).astype(np.float32) for _ in range(2)]
        chains, blocks = hostnet.chain_forward_count(), hostnet.block_forward_count()
        wants = [net.run("data", x, "add") for x in xs]
        assert hostnet.chain_forward_count() > chains and hostnet.block_forward_count() > blocks  # both entry points in play
        assert np.abs(wants[0] - wants[1]).max() > 0.1
        results = [[], []]

        def worker(t):
            sess = net.session("data", xs[t], "add")
            for _ in range(15):
                sess.run()
                results[t].append(sess.fetch(wants[t].shape, np.float32))
            sess.close()

        _run_threads([lambda: worker(0), lambda: worker(1)])
        for t in range(2):
            assert len(results[t]) == 15
            for r in results[t]:
                np.testing.assert_array_equal(r.view(np.int32), wants[t].view(np.int32))
    finally:
        hip.conv_chain_set_min_tiles(old_tiles)
        hip.conv_block_set_always(always)
        net.close()
