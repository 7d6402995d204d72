"""Sigmoid (4) and mish (5) in the int8 epilogues against vectors written by the compiled reference
(tests/golden/make_activation_fixtures.py). The reference evaluates them with polynomial exp / log and an
approximate-reciprocal division (-Ofast), so its own values depend on the CPU model: int8 results may differ by one
step where the scaled value sits at a rounding tie, fp32 results within a relative 1e-5."""
import os

import numpy as np
import pytest

from gpu_util import host_scale_in, run_conv
from oracle.binding import ROUND_EXACT, ROUND_SSE
from tensor_amd import capi

HERE = os.path.dirname(os.path.abspath(__file__))
MAX_TIE_FRACTION = 2e-3

REQUANT = [(act, packing, K) for act in (4, 5) for packing in (True, False) for K in (8, 4, 6)]
LAYERS = [(True, 16, 16, 3, 1), (True, 8, 12, 1, 1), (True, 16, 16, 3, 16), (False, 16, 16, 3, 1), (False, 8, 12, 1, 1)]


@pytest.fixture(scope="module")
def act_golden():
    return dict(np.load(os.path.join(HERE, "golden", "activation_golden.npz"), allow_pickle=False))


def assert_int8_within_one_step(got, want):
    d = got.astype(np.int32) - want.astype(np.int32)
    assert np.abs(d).max() <= 1
    assert np.count_nonzero(d) <= max(1, int(MAX_TIE_FRACTION * d.size))


def _requant_case(g, act, packing, K):
    tag = "requant/act%d_pack%d_K%d" % (act, int(packing), K)
    mode = ROUND_SSE if (packing and K % 4 == 0) else ROUND_EXACT
    return g[tag + "/acc"], g[tag + "/si"], g[tag + "/so"], g[tag + "/bias"], g[tag + "/q"], mode


def _layer_case(g, int8_out, C, K, k, groups):
    tag = "layer/sigmoid_i8%d_C%d_K%d_k%d_g%d" % (int(int8_out), C, K, k, groups)
    return (g[tag + "/x"], g[tag + "/wq"], g[tag + "/ws"], g[tag + "/bias"], float(g[tag + "/in_scale"]), g[tag + "/y"])


@pytest.mark.parametrize("act,packing,K", REQUANT)
def test_oracle_requantize_sigmoid_mish(oracle, act_golden, act, packing, K):
    acc, si, so, bias, want, mode = _requant_case(act_golden, act, packing, K)
    assert_int8_within_one_step(oracle.requantize(acc, si, so, bias, act, None, mode), want)
    assert len(np.unique(want)) > 20  # the vectors exercise the curve, not a saturated plateau


@pytest.mark.parametrize("int8_out,C,K,k,groups", LAYERS)
def test_oracle_layer_sigmoid(oracle, act_golden, int8_out, C, K, k, groups):
    x, wq, ws, bias, in_scale, want = _layer_case(act_golden, int8_out, C, K, k, groups)
    got = oracle.conv_layer_forward(x, wq, ws, in_scale, pad=(k // 2, k // 2), groups=groups, bias=bias, top_scale=120.0,
                                    int8_out=int8_out, act_type=4, use_packing=int8_out)
    if int8_out:
        assert_int8_within_one_step(got, want)
    else:
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-30)


@pytest.mark.parametrize("act,packing,K", REQUANT)
def test_reference_reproduces_its_vectors(ref, act_golden, act, packing, K):
    """Where the compiled reference is present: on the machine that wrote the vectors this is exact, on another CPU
    model it is the same one-step bound."""
    acc, si, so, bias, want, _ = _requant_case(act_golden, act, packing, K)
    assert_int8_within_one_step(ref.requantize(acc, si, so, bias, act, None, packing=packing), want)


@pytest.mark.gpu
@pytest.mark.parametrize("act,packing,K", REQUANT)
def test_gpu_requantize_sigmoid_mish(hip, act_golden, act, packing, K):
    acc, si, so, bias, want, mode = _requant_case(act_golden, act, packing, K)
    for sp in ((1, 4, 8) if K % 8 == 0 else (1, 4) if K % 4 == 0 else (1,)):
        dp = 8 if K % 8 == 0 else 1
        q = hip.requantize(hip.to_device(capi.pack_np(acc, sp)), capi.layout_for(np.int32, sp), acc.shape,
                           hip.to_device(si), hip.to_device(so), hip.to_device(bias), act, 0.0, mode,
                           capi.layout_for(np.int8, dp))
        assert_int8_within_one_step(capi.unpack_np(q.cpu().numpy(), dp, acc.shape), want)


@pytest.mark.gpu
@pytest.mark.parametrize("int8_out,C,K,k,groups", LAYERS)
def test_gpu_layer_sigmoid(hip, oracle, act_golden, int8_out, C, K, k, groups):
    x, wq, ws, bias, in_scale, want = _layer_case(act_golden, int8_out, C, K, k, groups)
    got, _ = run_conv(hip, oracle, x, wq, ws, in_scale, pad=k // 2, groups=groups, bias=bias, top_scale=120.0, act=4,
                      out_kind=capi.OUT_I8 if int8_out else capi.OUT_F32)
    if int8_out:
        assert_int8_within_one_step(got, want)
    else:
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-30)
