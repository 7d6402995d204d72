"""MobileNetV2-style int8 network through the C++ host layer against the CPU oracle, at reduced resolution."""
import numpy as np
import pytest

from gpu_util import mobilenet_oracle_forward
from tensor_amd import capi, hostnet, mobilenet


def test_description_matches_the_configuration():
    layers = mobilenet.describe()
    convs = [l for l in layers if l["kind"] == "conv"]
    assert len(convs) == 52 and sum(l["kind"] == "add" for l in layers) == 10
    # 299.49 MMAC of convolution + 1.28 MMAC inner product per 224x224 image
    assert abs(mobilenet.conv_macs_per_image(layers, 224) - 300.77e6) < 0.05e6
    # a convolution writes int8 exactly when no element-wise add (or the pooling) consumes its output
    feeds_add = {l["a"] for l in layers if l["kind"] == "add"} | {l["b"] for l in layers if l["kind"] == "add"}
    for l in convs:
        assert l["int8_out"] == (l["name"] not in feeds_add and l["name"] != "head")


@pytest.mark.gpu
def test_network_matches_oracle_layer_by_layer(hip, oracle):
    rng = np.random.default_rng(0)
    hw, batch = 64, 2
    layers = mobilenet.describe(num_classes=50)
    params = mobilenet.init_weights(layers, rng)
    mobilenet.calibrate(hip, capi, layers, params, rng.uniform(0, 1, (4, 3, hw, hw)).astype(np.float32))
    net = mobilenet.build_net(hostnet, layers, params, batch, hw, num_classes=50)
    x = rng.uniform(0, 1, (batch, 3, hw, hw)).astype(np.float32)
    want = mobilenet_oracle_forward(oracle, layers, params, x)
    for name in ("stem", "b0_project", "b1_dw", "b2_add", "b5_project", "b9_add", "b16_project", "head"):
        got = net.run("data", x, name)
        if got.dtype == np.int8:
            np.testing.assert_array_equal(got, want[name], err_msg=name)
        else:
            np.testing.assert_allclose(got, want[name], rtol=1e-5, atol=1e-30, err_msg=name)
    got = net.run("data", x, "fc").reshape(batch, -1)
    np.testing.assert_allclose(got, want["fc"], rtol=1e-4, atol=1e-5)


@pytest.mark.gpu
def test_network_with_blocks_as_single_launches(hip, oracle):
    """The same network with every inverted-residual block that qualifies by shape run as one launch
    (otter_hip_conv_block_forward through Net's block units): the blobs behind the blocks equal the oracle's and, bit
    for bit, those of the layers one by one; a blob asked for inside a block still comes from the layers one by one."""
    rng = np.random.default_rng(0)
    hw, batch = 64, 2
    layers = mobilenet.describe(num_classes=50)
    params = mobilenet.init_weights(layers, rng)
    mobilenet.calibrate(hip, capi, layers, params, rng.uniform(0, 1, (4, 3, hw, hw)).astype(np.float32))
    net = mobilenet.build_net(hostnet, layers, params, batch, hw, num_classes=50)
    x = rng.uniform(0, 1, (batch, 3, hw, hw)).astype(np.float32)
    want = mobilenet_oracle_forward(oracle, layers, params, x)
    names = ("b2_add", "b5_add", "b9_add", "b10_project", "b12_add", "b15_add", "b16_project", "head")
    plain = {name: net.run("data", x, name) for name in names}
    before = hip.conv_block_set_always(1)
    try:
        count0 = hostnet.block_forward_count()
        for name in names:
            got = net.run("data", x, name)
            assert got.tobytes() == plain[name].tobytes(), name
            if got.dtype == np.int8:
                np.testing.assert_array_equal(got, want[name], err_msg=name)
            else:
                np.testing.assert_allclose(got, want[name], rtol=1e-5, atol=1e-30, err_msg=name)
        # every block with an expand layer goes through the block entry point, b1..b16 = 16 of them up to the head: the
        # stride-1 ones as one launch, the stride-2 ones as one launch for the first two layers and one for the last
        # (Net.run makes two passes: one for the shape, one to fetch)
        count1 = hostnet.block_forward_count()
        assert count1 > count0
        net.run("data", x, "head")
        assert hostnet.block_forward_count() - count1 == 2 * 16
        # a blob inside a block: the layers run one by one up to it, same bytes as before
        inner = net.run("data", x, "b8_dw")
        np.testing.assert_array_equal(inner, want["b8_dw"])
    finally:
        hip.conv_block_set_always(before)
