"""Which rounding primitive a layer ends in, on the GPU, against layer results of the compiled reference that sit exactly
on +-0.49999997f (cases.TIE_ROUTE_CASES: the one value float2int8_sse and float2int8 round differently,
Tensor/VecIntrinsic.hpp:71-95). Three ways in, each with the rounding modes chosen by the code a user of that way
gets: the host layer's own rule (otter::ConvolutionLayer::create_pipeline_int8 in tensor_amd/host), the reference-side
binding's rule (oracle/ref_hip_layer.cpp inside the reference's own layer machinery), and the bare C ABI with the modes
the oracle's routing functions name. A layer that took the other primitive would differ from the vector in dozens of
positions (asserted on the CPU side, tests/test_oracle_golden.py)."""
import numpy as np
import pytest

from cases import TIE_ROUTE_CASES, layer_options, make_tie_inputs
from gpu_util import ACT, run_conv
from tensor_amd import capi, hostnet

pytestmark = pytest.mark.gpu

IDS = [c[0] for c in TIE_ROUTE_CASES]


@pytest.mark.parametrize("case", TIE_ROUTE_CASES, ids=IDS)
def test_host_layer_takes_the_reference_rounding_primitive(tie_golden, case):
    name, C, K, k, s, p, d, g, H, W, N, in_i8, i8_out, bias, act, act_params, packing = case
    t = make_tie_inputs(case)
    net = hostnet.Net(use_packing_layout=packing)
    net.add_layer(type="Input", name="data", batchsize=N, channel=C, height=H, width=W)
    opts = layer_options(case[:16])
    opts.pop("in_channels")
    net.add_layer(name="conv", **opts)
    net.compile()
    net.set_conv("conv", t["wq"], t["bias"], t["w_scales"], float(t["in_scale"]), float(t["top_scale"]))
    np.testing.assert_array_equal(net.scale_in("conv", K).view(np.int32), tie_golden[name + "/scale_in"].view(np.int32))
    got = net.run("data", t["x"], "conv")
    np.testing.assert_array_equal(got, tie_golden[name + "/out"])
    net.close()


@pytest.mark.parametrize("case", TIE_ROUTE_CASES, ids=IDS)
def test_c_abi_with_the_modes_the_routing_names(hip, oracle, tie_golden, case):
    name, C, K, k, s, p, d, g, H, W, N, in_i8, i8_out, bias, act, act_params, packing = case
    t = make_tie_inputs(case)
    got, _ = run_conv(hip, oracle, t["x"], t["wq"], t["w_scales"], t["in_scale"], stride=s, pad=p, dil=d, groups=g,
                      bias=t["bias"], top_scale=float(t["top_scale"]), out_kind=capi.OUT_I8, act=ACT[act],
                      use_packing=packing)
    np.testing.assert_array_equal(got, tie_golden[name + "/out"])


@pytest.fixture(scope="module")
def ref_hip():
    from oracle.binding import Ref, ref_hip_available
    if not ref_hip_available():
        pytest.skip("oracle/_ref/libotter_ref_hip.so not built (needs /root/reference)")
    return Ref(hip=True)


@pytest.mark.parametrize("case", TIE_ROUTE_CASES, ids=IDS)
def test_reference_side_binding_takes_the_reference_rounding_primitive(ref_hip, tie_golden, case):
    """The reference's own layer machinery (parse_param, load_param, Net's layout conversion in front of forward) around
    the GPU layer of oracle/ref_hip_layer.cpp, created through the reference's LayerRegistry."""
    name, C, H, W, packing = case[0], case[1], case[8], case[9], case[16]
    t = make_tie_inputs(case)
    before = ref_hip.hip_forward_count()
    ref_hip.use_hip_convolution(True)
    try:
        layer = ref_hip.conv_layer(layer_options(case[:16]), (1, C, H, W), t["wq"], t["bias"], t["w_scales"],
                                   float(t["in_scale"]), float(t["top_scale"]), packing)
    finally:
        ref_hip.use_hip_convolution(False)
    got, _ = layer.forward(t["x"])
    layer.close()
    assert ref_hip.hip_forward_count() == before + t["x"].shape[0]  # one GPU forward per image (the reference loops a batch)
    np.testing.assert_array_equal(got, tie_golden[name + "/out"])
