"""CPU: the C restatement in oracle/ replayed against vectors produced by the compiled reference
(tests/golden/make_golden.py). Every function of the oracle is pinned here, bit for bit."""
import numpy as np
import pytest

from cases import LAYER_CASES, TIE_ROUTE_CASES, UNPACKED_LAYER_CASES, make_tie_inputs
from oracle.binding import ROUND_EXACT, ROUND_SSE

ACT = {"": 0, "Relu": 1, "LRelu": 2, "Relu6": 3}


def _g(golden, tag, key):
    return golden.get(tag + "/" + key)


@pytest.mark.parametrize("case", LAYER_CASES, ids=[c[0] for c in LAYER_CASES])
def test_layer_forward_matches_reference(oracle, golden, case):
    name, C, K, k, s, p, d, g, H, W, N, in_i8, i8_out, bias, act, act_params = case
    x, wq = _g(golden, name, "x"), _g(golden, name, "wq")
    out, acc = oracle.conv_layer_forward(
        x, wq, _g(golden, name, "w_scales"), float(_g(golden, name, "in_scale")), stride=(s, s), pad=(p, p),
        dil=(d, d), groups=g, bias=_g(golden, name, "bias"), top_scale=float(_g(golden, name, "top_scale")),
        int8_out=i8_out, act_type=ACT[act], act_params=act_params, use_packing=True, want_acc=True)
    np.testing.assert_array_equal(acc, _g(golden, name, "acc"))
    np.testing.assert_array_equal(
        oracle.scale_in(_g(golden, name, "w_scales"), float(_g(golden, name, "in_scale"))).view(np.int32),
        _g(golden, name, "scale_in").view(np.int32))
    want = _g(golden, name, "out")
    if i8_out:
        np.testing.assert_array_equal(out, want)
    else:
        # fp32 results are reproduced bitwise as well (fused multiply-add, same order)
        np.testing.assert_array_equal(out.view(np.int32), want.view(np.int32))


@pytest.mark.parametrize("case", UNPACKED_LAYER_CASES, ids=[c[0] for c in UNPACKED_LAYER_CASES])
def test_unpacked_layer_forward_matches_reference(oracle, golden, case):
    """use_packing_layout = false: the unpacked sgemm route with the scalar float2int8 in quantize / requantize
    (Tensor/ConvolutionMM2DInt8X86.cpp:1182-1262, Tensor/QuantizeX86.cpp:617-641)."""
    name, C, K, k, s, p, d, g, H, W, N, in_i8, i8_out, bias, act, act_params = case
    x, wq = _g(golden, name, "x"), _g(golden, name, "wq")
    if not in_i8:
        xq = oracle.quantize(x, [_g(golden, name, "in_scale")], oracle.quantize_round_mode(C, False))
        np.testing.assert_array_equal(xq, _g(golden, name, "xq"))
    out, acc = oracle.conv_layer_forward(
        x, wq, _g(golden, name, "w_scales"), float(_g(golden, name, "in_scale")), stride=(s, s), pad=(p, p),
        dil=(d, d), groups=g, bias=_g(golden, name, "bias"), top_scale=float(_g(golden, name, "top_scale")),
        int8_out=i8_out, act_type=ACT[act], act_params=act_params, use_packing=False, want_acc=True)
    np.testing.assert_array_equal(acc, _g(golden, name, "acc"))
    want = _g(golden, name, "out")
    if i8_out:
        np.testing.assert_array_equal(out, want)
    else:
        np.testing.assert_array_equal(out.view(np.int32), want.view(np.int32))


def test_layer_quantized_input_matches_reference(oracle, golden):
    for case in LAYER_CASES:
        name, C = case[0], case[1]
        if case[11]:
            continue
        xq = oracle.quantize(_g(golden, name, "x"), [_g(golden, name, "in_scale")],
                             oracle.quantize_round_mode(C, True))
        np.testing.assert_array_equal(xq, _g(golden, name, "xq"))


@pytest.mark.parametrize("C,packing", [(8, True), (8, False), (4, True), (4, False), (3, True), (3, False)])
def test_quantize_near_ties(oracle, golden, C, packing):
    tag = "quant_ties/C%d_pack%d" % (C, int(packing))
    x, want = golden[tag + "/x"], golden[tag + "/q"]
    mode = oracle.quantize_round_mode(C, packing)
    np.testing.assert_array_equal(oracle.quantize(x, [1.0], mode), want)
    # the other rounding primitive must NOT reproduce the vectors: the fixture discriminates the two
    assert (oracle.quantize(x, [1.0], 1 - mode) != want).any()


def test_quantize_per_channel(oracle, golden):
    q = oracle.quantize(golden["quant_perchannel/x"], golden["quant_perchannel/scales"], ROUND_SSE)
    np.testing.assert_array_equal(q, golden["quant_perchannel/q"])


@pytest.mark.parametrize("C", [8, 4, 6])
@pytest.mark.parametrize("packing", [True, False])
@pytest.mark.parametrize("j", [0, 1, 2, 3])
def test_requantize_exact_ties(oracle, golden, C, packing, j):
    tag = "requant_ties/C%d_pack%d_b%d" % (C, int(packing), j)
    mode = ROUND_SSE if (packing and C % 4 == 0) else ROUND_EXACT
    q = oracle.requantize(golden[tag + "/acc"], golden[tag + "/scale_in"], golden[tag + "/scale_out"],
                          golden.get(tag + "/bias"), 0, None, mode)
    np.testing.assert_array_equal(q, golden[tag + "/q"])


@pytest.mark.parametrize("act", [0, 1, 2, 3])
@pytest.mark.parametrize("C,packing", [(8, True), (12, True), (6, True), (8, False)])
def test_requantize_random(oracle, golden, act, C, packing):
    tag = "requant_rand/act%d_C%d_pack%d" % (act, C, int(packing))
    mode = ROUND_SSE if (packing and C % 4 == 0) else ROUND_EXACT
    q = oracle.requantize(golden[tag + "/acc"], golden[tag + "/scale_in"], golden[tag + "/scale_out"],
                          golden[tag + "/bias"], act, golden.get(tag + "/act_params"), mode)
    np.testing.assert_array_equal(q, golden[tag + "/q"])


@pytest.mark.parametrize("C,packing", [(8, True), (4, True), (8, False)])
@pytest.mark.parametrize("j", [0, 1])
def test_dequantize_bitwise(oracle, golden, C, packing, j):
    tag = "dequant/C%d_pack%d_b%d" % (C, int(packing), j)
    acc, scale, bias = golden[tag + "/acc"], golden[tag + "/scale"], golden.get(tag + "/bias")
    y = oracle.dequantize(acc, scale, bias)
    np.testing.assert_array_equal(y.view(np.int32), golden[tag + "/y"].view(np.int32))
    if bias is not None:
        # a two-rounding multiply-then-add does not reproduce the vectors: the fixture pins the fused form
        two = (acc.astype(np.float32) * scale[None, :, None, None]).astype(np.float32) + bias[None, :, None, None]
        assert (two.view(np.int32) != golden[tag + "/y"].view(np.int32)).any()


def test_conv_int32_against_independent_einsum(oracle):
    """Closed form: exact integer arithmetic is order independent, so an int64 einsum over explicitly
    zero-padded, strided windows pins the accumulator completely (transposed operand / wrong stride or
    dilation index / dropped tap all fail here)."""
    rng = np.random.default_rng(7)
    for (C, K, kh, kw, sh, sw, ph, pw, dh, dw, g, H, W) in [
            (8, 8, 3, 3, 1, 1, 1, 1, 1, 1, 1, 9, 7), (6, 4, 3, 2, 2, 1, 1, 0, 1, 2, 2, 11, 9),
            (16, 16, 3, 3, 2, 2, 1, 1, 1, 1, 16, 9, 8), (3, 8, 5, 3, 2, 2, 2, 1, 1, 1, 1, 12, 10),
            (12, 12, 1, 1, 1, 1, 0, 0, 1, 1, 4, 5, 5)]:
        x = rng.integers(-128, 128, size=(2, C, H, W)).astype(np.int8)
        w = rng.integers(-128, 128, size=(K, C // g, kh, kw)).astype(np.int8)
        got = oracle.conv_int32(x, w, (sh, sw), (ph, pw), (dh, dw), g)
        xp = np.pad(x.astype(np.int64), ((0, 0), (0, 0), (ph, ph), (pw, pw)))
        OH, OW = got.shape[2], got.shape[3]
        want = np.zeros((2, K, OH, OW), np.int64)
        cg, kg = C // g, K // g
        for gi in range(g):
            for u in range(kh):
                for v in range(kw):
                    win = xp[:, gi * cg:(gi + 1) * cg, u * dh:u * dh + sh * (OH - 1) + 1:sh,
                             v * dw:v * dw + sw * (OW - 1) + 1:sw]
                    want[:, gi * kg:(gi + 1) * kg] += np.einsum("nchw,kc->nkhw", win,
                                                                w[gi * kg:(gi + 1) * kg, :, u, v].astype(np.int64))
        np.testing.assert_array_equal(got.astype(np.int64), want)


def test_pack_roundtrip_and_layout(oracle):
    a = np.arange(2 * 16 * 3 * 5, dtype=np.int32).reshape(2, 16, 3, 5)
    for p in (4, 8):
        pk = oracle.pack(a, p)
        np.testing.assert_array_equal(pk, a.reshape(2, 16 // p, p, 3, 5).transpose(0, 1, 3, 4, 2))
        np.testing.assert_array_equal(oracle.unpack(pk), a)


def test_global_avgpool_against_closed_form(oracle):
    """The mean over H*W per (image, channel), against a float64 mean and against cases with a known answer: a constant
    plane returns the constant, a plane that is 1 at one pixel returns 1/(H*W) for that channel only (an index that
    strides over channels instead of pixels, or a divisor of C instead of H*W, fails)."""
    rng = np.random.default_rng(11)
    x = rng.normal(0, 3, (3, 5, 7, 4)).astype(np.float32)
    got = oracle.global_avgpool(x)
    assert got.shape == (3, 5) and got.dtype == np.float32
    np.testing.assert_allclose(got, x.astype(np.float64).mean(axis=(2, 3)), rtol=1e-6, atol=1e-7)
    c = np.broadcast_to(np.arange(10, dtype=np.float32).reshape(2, 5, 1, 1), (2, 5, 3, 9))
    np.testing.assert_array_equal(oracle.global_avgpool(c), np.arange(10, dtype=np.float32).reshape(2, 5))
    one = np.zeros((2, 3, 4, 8), np.float32)
    one[1, 2, 3, 5] = 1.0
    want = np.zeros((2, 3), np.float32)
    want[1, 2] = 1.0 / 32
    np.testing.assert_array_equal(oracle.global_avgpool(one), want)


def test_inner_product_against_closed_form(oracle):
    """y[n][o] = sum_i x[n][i] * W[o][i] + b[o] (Tensor/InnerProductLayer.cpp:176-): a float64 matmul with a
    NON-symmetric, non-square weight (a transposed weight index cannot even be evaluated consistently), unit vectors
    that pick out single weight entries exactly, and the bias alone on a zero input."""
    rng = np.random.default_rng(12)
    n, in_f, out_f = 3, 37, 11
    x = rng.normal(0, 1, (n, in_f)).astype(np.float32)
    w = rng.normal(0, 1, (out_f, in_f)).astype(np.float32)
    b = rng.normal(0, 1, out_f).astype(np.float32)
    got = oracle.inner_product(x, w, b)
    assert got.shape == (n, out_f) and got.dtype == np.float32
    want = x.astype(np.float64) @ w.astype(np.float64).T + b.astype(np.float64)
    np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(oracle.inner_product(x, w, None), want - b, rtol=1e-6, atol=1e-6)
    # square but non-symmetric weight: e_i picks column i of W, i.e. y[o] = W[o][i] exactly
    ws = rng.normal(0, 1, (6, 6)).astype(np.float32)
    eye = np.eye(6, dtype=np.float32)
    np.testing.assert_array_equal(oracle.inner_product(eye, ws, None), ws.T)
    assert not np.array_equal(ws, ws.T)
    np.testing.assert_array_equal(oracle.inner_product(np.zeros((2, in_f), np.float32), w, b), np.stack([b, b]))


def test_eltwise_add_is_the_fp32_sum(oracle):
    rng = np.random.default_rng(13)
    a = rng.normal(0, 1e3, 1001).astype(np.float32)
    b = rng.normal(0, 1e-3, 1001).astype(np.float32)
    np.testing.assert_array_equal(oracle.eltwise_add(a, b), a + b)


@pytest.mark.parametrize("case", TIE_ROUTE_CASES, ids=[c[0] for c in TIE_ROUTE_CASES])
def test_layer_routing_of_the_rounding_primitive_matches_reference(oracle, tie_golden, case):
    """Which rounding primitive a layer ends in (otter_oracle_quantize_round_mode / otter_oracle_requantize_round_mode
    inside otter_oracle_conv_layer_forward) against layer results of the compiled reference that sit exactly on
    +-0.49999997f, the one value the two primitives round differently. The layer as a whole must reproduce the vector;
    put together from its steps with the OTHER primitive in the step under test it must not (so the vector does
    discriminate), and with the primitive the routing function names it must."""
    name, C, K, k, s, p, d, g, H, W, N, in_i8, i8_out, bias, act, act_params, packing = case
    t = make_tie_inputs(case)
    want = tie_golden[name + "/out"]
    np.testing.assert_array_equal(oracle.scale_in(t["w_scales"], float(t["in_scale"])).view(np.int32),
                                  tie_golden[name + "/scale_in"].view(np.int32))
    out = oracle.conv_layer_forward(t["x"], t["wq"], t["w_scales"], float(t["in_scale"]), stride=(s, s), pad=(p, p),
                                    dil=(d, d), groups=g, bias=t["bias"], top_scale=float(t["top_scale"]), int8_out=True,
                                    act_type=ACT[act], use_packing=packing)
    np.testing.assert_array_equal(out, want)

    def by_steps(q_mode, r_mode):
        xq = t["x"] if in_i8 else oracle.quantize(t["x"], [t["in_scale"]], q_mode)
        acc = oracle.conv_int32(xq, t["wq"], (s, s), (p, p), (d, d), g)
        return oracle.requantize(acc, oracle.scale_in(t["w_scales"], float(t["in_scale"])), [t["top_scale"]], t["bias"],
                                 ACT[act], None, r_mode)

    other = {ROUND_SSE: ROUND_EXACT, ROUND_EXACT: ROUND_SSE}
    q_mode, r_mode = oracle.quantize_round_mode(C, packing), oracle.requantize_round_mode(C, K, g, packing)
    np.testing.assert_array_equal(by_steps(q_mode, r_mode), want)
    if in_i8:
        assert (by_steps(q_mode, other[r_mode]) != want).any(), "the vector does not tell the requantize primitives apart"
    else:
        assert (by_steps(other[q_mode], r_mode) != want).any(), "the vector does not tell the quantize primitives apart"


def test_tie_route_cases_cover_both_primitives_on_both_sides(oracle):
    """The case table meets every branch of the routing: SIMD and scalar rounding, in quantize and in requantize."""
    seen = set()
    for case in TIE_ROUTE_CASES:
        C, K, g, in_i8, packing = case[1], case[2], case[7], case[11], case[16]
        seen.add(("requantize", oracle.requantize_round_mode(C, K, g, packing)) if in_i8 else
                 ("quantize", oracle.quantize_round_mode(C, packing)))
    assert seen == {("quantize", ROUND_SSE), ("quantize", ROUND_EXACT), ("requantize", ROUND_SSE), ("requantize", ROUND_EXACT)}
