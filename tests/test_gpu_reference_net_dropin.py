"""The drop-in, proved on the REFERENCE's own Net: oracle/ref_hip_layer.cpp is the binding a maintainer of the reference
would add (a ConvolutionLayer subclass over include/otter_hip_int8.h, registered with LayerRegistry::AddCreator under
"Convolution", Tensor/LayerRegistry.hpp:27-33). It is compiled against the reference's headers into
oracle/_ref/libotter_ref_hip.so together with the reference itself. Here the reference's Net reads its own int8
detection model description and an ncnn `.bin`, once with its stock layers and once with the GPU layer registered,
and the blobs are compared: everything but the 110 convolutions (graph, weight loading, layout conversion, every glue
layer, the Extractor) is the reference's own code in both runs."""
import os

import numpy as np
import pytest

from tensor_amd import hostnet, modelfile

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
NANODET = os.path.join(GOLDEN, "nanodet-plus-m-1.5x_416_int8_fused.otter")
# the reference's other int8 description (benchmark/benchotter.cpp:88-90 runs both): the same network with conv_1 kept
# in fp32 (int8_scale_term 0)
NANODET_MIXED = os.path.join(GOLDEN, "nanodet-plus-m-1.5x_416_int8_mixed.otter")
HEADS = ["conv_95", "conv_100", "conv_105", "conv_110"]  # what feeds the detection post-processing


@pytest.fixture(scope="module")
def ref_hip():
    from oracle.binding import Ref, ref_hip_available
    if not ref_hip_available():
        pytest.skip("oracle/_ref/libotter_ref_hip.so not built (needs /root/reference)")
    return Ref(hip=True)


@pytest.mark.parametrize("description,n_gpu", [(NANODET, 110), (NANODET_MIXED, 109)], ids=["int8_fused", "int8_mixed"])
def test_reference_net_with_the_gpu_convolution_layer_registered(ref_hip, tmp_path, description, n_gpu):
    """int8_mixed: the fp32 conv_1 must fall through to the stock ConvolutionLayer inside the GPU layer (its
    create_pipeline makes no handle for an fp32 layer), the other 109 convolutions go through the C ABI."""
    rng = np.random.default_rng(23)
    probe = hostnet.Net(lightmode=False)  # only to enumerate the layers for the synthetic weight file
    probe.load_otter(NANODET)             # (the two descriptions differ in conv_1's int8_scale_term only)
    layers = probe.describe()
    if description == NANODET_MIXED:
        assert layers[1][0] == "Convolution" and layers[1][1] == "conv_1"
        layers[1][4]["int8_scale_term"] = 0
    blob, _ = modelfile.synthetic_int8_weights(layers, rng)
    path = str(tmp_path / "nanodet_int8.bin")
    with open(path, "wb") as f:
        f.write(blob)
    probe.close()
    # some int8 blobs inside the net as well as the four fp32 heads
    int8_convs = [l[1] for l in layers if l[0] == "Convolution" and l[4]["int8_scale_term"] > 100]
    names = HEADS + int8_convs[::6]
    x = rng.uniform(0, 1, (1, 3, 416, 416)).astype(np.float32)

    stock = ref_hip.net(description, path)
    want, _ = stock.run("data_1", x, names)

    ref_hip.use_hip_convolution(True)
    try:
        gpu = ref_hip.net(description, path)  # compiled now: its 110 "Convolution" layers come from the new creator
    finally:
        ref_hip.use_hip_convolution(False)
    before = ref_hip.hip_forward_count()
    got, _ = gpu.run("data_1", x, names)
    assert ref_hip.hip_forward_count() - before == n_gpu  # every int8 convolution of the net went through the C ABI

    n_int8 = 0
    for n in names:
        assert got[n].shape == want[n].shape and got[n].dtype == want[n].dtype, n
        if got[n].dtype == np.int8:
            n_int8 += 1
            # the two nets diverge nowhere upstream (int8 blobs are bit-exact layer by layer), so neither here
            np.testing.assert_array_equal(got[n], want[n], err_msg=n)
            assert np.abs(want[n]).max() > 20
        else:
            np.testing.assert_allclose(got[n], want[n], rtol=1e-5, atol=1e-5, err_msg=n)
    assert n_int8 >= 8

    # the stock creator is back: a net compiled now runs on the CPU again
    before = ref_hip.hip_forward_count()
    again = ref_hip.net(description, path)
    again.run("data_1", x, HEADS[:1])
    assert ref_hip.hip_forward_count() == before

