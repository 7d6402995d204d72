"""The calibration utility: fp32 weights + a calibration batch -> int8 weights and scales, on a generated description
with every kind of convolution the path has (fp32-out stem, depthwise int8-out with per-channel and with single weight
scale, pointwise int8-out, fp32-out head, a shortcut). Checked against a plain torch fp32 network (CPU) for accuracy,
against the scale definition (the calibration batch reaches exactly +-127 in every int8 blob and saturates nowhere
else), and through the files: the written `.bin` read back by Net::load_weight -- and by the compiled reference's Net --
gives the calibrated network again."""
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from tensor_amd import calibration, hostnet

pytestmark = pytest.mark.gpu


def _conv(name, inp, k_out, k, s, p, term, groups=1, act=None):
    o = 'Convolution {\n name: %s\n input: %s\n output: %s\n' % (name, inp, name)
    if act:
        o += ' activation: %s\n' % act
    o += (' Param {\n  out_channels: %d\n  kernel: %d\n  stride: %d\n  padding: %d\n  groups: %d\n  int8_scale_term: %d\n'
          '  bias_term: true\n' % (k_out, k, s, p, groups, term))
    if act == "LRelu":
        o += '  activation_params: 0.100000\n'
    return o + ' }\n}\n'


OTTER = ('name: "calibration"\nInput {\n name: data\n output: data\n Param {\n  height: 40\n  width: 40\n  channel: 3\n }\n}\n' +
         _conv("stem", "data", 16, 3, 2, 1, 2, act="LRelu") +
         _conv("dw1", "stem", 16, 3, 1, 1, 101, groups=16, act="Relu") +
         _conv("pw1", "dw1", 32, 1, 1, 0, 101, act="Relu") +
         _conv("dw2", "pw1", 32, 3, 2, 1, 102, groups=32) +
         _conv("pw2", "dw2", 32, 1, 1, 0, 1, act="Relu") +
         _conv("pw3", "pw2", 32, 3, 1, 1, 1) +
         'ShortCut {\n name: add\n input: "pw2, pw3"\n output: add\n}\n')
SPEC = [("stem", 3, 16, 3, 2, 1, 1, "lrelu"), ("dw1", 16, 16, 3, 1, 1, 16, "relu"), ("pw1", 16, 32, 1, 1, 0, 1, "relu"),
        ("dw2", 32, 32, 3, 2, 1, 32, None), ("pw2", 32, 32, 1, 1, 0, 1, "relu"), ("pw3", 32, 32, 3, 1, 1, 1, None)]


def _float_net(weights, x):
    t = torch.from_numpy(x)
    out = {}
    cur = t
    for name, _c, _k, _ks, s, p, g, act in SPEC:
        w, b = weights[name]
        src = out["pw2"] if name == "pw3" else cur
        y = F.conv2d(src, torch.from_numpy(w), torch.from_numpy(b), stride=s, padding=p, groups=g)
        y = F.leaky_relu(y, 0.1) if act == "lrelu" else (F.relu(y) if act == "relu" else y)
        out[name] = y
        cur = y
    return (out["pw2"] + out["pw3"]).numpy()


def test_calibrated_network(ref, tmp_path):
    rng = np.random.default_rng(21)
    weights = {}
    for name, c, k, ks, _s, _p, g, _act in SPEC:
        fan = c // g * ks * ks
        weights[name] = (rng.normal(0, np.sqrt(2.0 / fan), (k, c // g, ks, ks)).astype(np.float32),
                         rng.normal(0, 0.05, k).astype(np.float32))
    path = str(tmp_path / "cal.otter")
    with open(path, "w") as f:
        f.write(OTTER)
    x_cal = rng.uniform(-1, 1, (8, 3, 40, 40)).astype(np.float32)
    net = hostnet.Net(lightmode=False)
    net.load_otter(path)
    records, blobs = calibration.calibrate_net(net, weights, {"data": x_cal})

    # the scale definition: every int8 blob of the calibration batch touches +-127 and nothing saturates beyond it
    int8_blobs = [n for n, b in blobs.items() if b.dtype == np.int8]
    assert sorted(int8_blobs) == ["dw1", "dw2", "pw1"]
    for n in int8_blobs:
        assert np.abs(blobs[n]).max() == 127
        assert (np.abs(blobs[n]) == 127).mean() < 0.01
    # an int8 blob's consumer reads it with the producer's scale
    assert records["pw1"]["bottom_scale"] == records["dw1"]["top_scale"]
    assert records["dw2"]["weight_scales"].shape == (1,) and records["dw1"]["weight_scales"].shape == (16,)

    # accuracy against the fp32 network
    want = _float_net(weights, x_cal)
    got = net.eval({"data": x_cal}, "add")
    rel = np.linalg.norm(got - want) / np.linalg.norm(want)
    assert rel < 0.05, rel

    # through the files: our loader and the reference's both give the calibrated network again
    bin_path = str(tmp_path / "cal.bin")
    with open(bin_path, "wb") as f:
        f.write(calibration.to_bin(net, records))
    net2 = hostnet.Net()
    net2.load_otter(path)
    net2.load_weight(bin_path, ncnn=True)
    np.testing.assert_array_equal(net2.eval({"data": x_cal}, "add"), got)
    rnet = ref.net(path, bin_path)
    for i in (0, 7):
        r = rnet.run("data", x_cal[i:i + 1], ["add"])[0]["add"]
        np.testing.assert_allclose(got[i:i + 1], r, rtol=1e-5, atol=1e-6)
