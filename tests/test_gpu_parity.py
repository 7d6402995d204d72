"""GPU parity tests proper: the HIP path, called through the C ABI, against (a) the golden vectors produced by
the compiled reference and (b) the CPU oracle on seeded inputs. int32 accumulators and int8 outputs must be
bit-exact; fp32 outputs within 1e-5 relative (they are in fact reproduced bitwise, which is asserted too)."""
import numpy as np
import pytest

from cases import LAYER_CASES, UNPACKED_LAYER_CASES
from gpu_util import ACT, host_scale_in, run_conv
from oracle.binding import ROUND_EXACT, ROUND_SSE
from tensor_amd import capi

pytestmark = pytest.mark.gpu

FP32_RTOL = 1e-5


def assert_f32_close(got, want):
    np.testing.assert_allclose(got, want, rtol=FP32_RTOL, atol=1e-30)


def _g(golden, tag, key):
    return golden.get(tag + "/" + key)


@pytest.mark.parametrize("case", LAYER_CASES, ids=[c[0] for c in LAYER_CASES])
def test_layer_against_reference_vectors(hip, oracle, golden, case):
    name, C, K, k, s, p, d, g, H, W, N, in_i8, i8_out, bias, act, act_params = case
    x, wq = _g(golden, name, "x"), _g(golden, name, "wq")
    common = dict(stride=s, pad=p, dil=d, groups=g, bias=_g(golden, name, "bias"),
                  top_scale=float(_g(golden, name, "top_scale")), act=ACT[act],
                  act_p0=float(act_params[0]) if act_params else 0.0)
    ws, ins = _g(golden, name, "w_scales"), float(_g(golden, name, "in_scale"))
    # raw accumulators (what otter::convolution returns)
    acc, kind = run_conv(hip, oracle, x, wq, ws, ins, out_kind=capi.OUT_I32, **common)
    np.testing.assert_array_equal(acc, _g(golden, name, "acc"))
    # the layer output, in the reference's default packed layout and unpacked
    want = _g(golden, name, "out")
    kind_out = capi.OUT_I8 if i8_out else capi.OUT_F32
    for out_layout in (None, capi.I8 if i8_out else capi.F32):
        out, _ = run_conv(hip, oracle, x, wq, ws, ins, out_kind=kind_out, out_layout=out_layout, **common)
        if i8_out:
            np.testing.assert_array_equal(out, want)
        else:
            assert_f32_close(out, want)
            np.testing.assert_array_equal(out.view(np.int32), want.view(np.int32))
    # the fast kernels must be the ones that ran, not the scalar fallback
    if C % 8 == 0 and (g == 1 or g == C == K):
        assert kind in (1, 2, 3)


@pytest.mark.parametrize("case", UNPACKED_LAYER_CASES, ids=[c[0] for c in UNPACKED_LAYER_CASES])
def test_unpacked_mode_layer_against_reference_vectors(hip, oracle, golden, case):
    """use_packing_layout = false (the reference's unpacked sgemm_conv2d_int8_x86 route,
    Tensor/ConvolutionMM2DInt8X86.cpp:1182-1262): every blob elempack 1, the scalar float2int8 in quantize and
    requantize. Vectors written by the compiled reference's ConvolutionLayer::forward in that mode."""
    name, C, K, k, s, p, d, g, H, W, N, in_i8, i8_out, bias, act, act_params = case
    x, wq = _g(golden, name, "x"), _g(golden, name, "wq")
    common = dict(stride=s, pad=p, dil=d, groups=g, bias=_g(golden, name, "bias"),
                  top_scale=float(_g(golden, name, "top_scale")), act=ACT[act],
                  act_p0=float(act_params[0]) if act_params else 0.0, use_packing=False)
    ws, ins = _g(golden, name, "w_scales"), float(_g(golden, name, "in_scale"))
    acc, _ = run_conv(hip, oracle, x, wq, ws, ins, out_kind=capi.OUT_I32, **common)
    np.testing.assert_array_equal(acc, _g(golden, name, "acc"))
    want = _g(golden, name, "out")
    out, _ = run_conv(hip, oracle, x, wq, ws, ins, out_kind=capi.OUT_I8 if i8_out else capi.OUT_F32, **common)
    if i8_out:
        np.testing.assert_array_equal(out, want)
    else:
        assert_f32_close(out, want)
        np.testing.assert_array_equal(out.view(np.int32), want.view(np.int32))


def test_layer_unpacked_input_layouts(hip, oracle, golden):
    """The same blob handed over unpacked (fp32 NCHW / int8 NCHW) gives the same answer."""
    for case in LAYER_CASES[:3] + LAYER_CASES[14:16]:
        name, C, K, k, s, p, d, g, H, W, N, in_i8, i8_out, bias, act, act_params = case
        x = _g(golden, name, "x")
        out, _ = run_conv(hip, oracle, x, _g(golden, name, "wq"), _g(golden, name, "w_scales"),
                          float(_g(golden, name, "in_scale")), stride=s, pad=p, dil=d, groups=g,
                          bias=_g(golden, name, "bias"), top_scale=float(_g(golden, name, "top_scale")), act=ACT[act],
                          out_kind=capi.OUT_I8 if i8_out else capi.OUT_F32,
                          in_layout=capi.I8 if in_i8 else capi.F32)
        want = _g(golden, name, "out")
        if i8_out:
            np.testing.assert_array_equal(out, want)
        else:
            assert_f32_close(out, want)


# ---- standalone quantize / requantize / dequantize against the reference's fine-print vectors ----------

@pytest.mark.parametrize("C,packing", [(8, True), (8, False), (4, True), (4, False), (3, True), (3, False)])
def test_quantize_near_ties(hip, oracle, golden, C, packing):
    tag = "quant_ties/C%d_pack%d" % (C, int(packing))
    x, want = golden[tag + "/x"], golden[tag + "/q"]
    # |x*scale| >= 2^31 is outside the supported domain (x86 integer-indefinite artefact)
    ok = np.abs(x) < 2.0 ** 31
    mode = oracle.quantize_round_mode(C, packing)
    sp = (8 if C % 8 == 0 else 4 if C % 4 == 0 else 1) if packing else 1
    dp = 8 if (packing and C % 8 == 0) else 1
    src = hip.to_device(capi.pack_np(x, sp))
    scales = hip.to_device(np.ones(1, np.float32))
    q = hip.quantize(src, capi.layout_for(np.float32, sp), x.shape, scales, mode, capi.layout_for(np.int8, dp))
    got = capi.unpack_np(q.cpu().numpy(), dp, x.shape)
    np.testing.assert_array_equal(got[ok], want[ok])


def test_quantize_per_channel(hip, golden):
    x, ps = golden["quant_perchannel/x"], golden["quant_perchannel/scales"]
    for sp in (1, 4, 8):
        for dp in (1, 8):
            q = hip.quantize(hip.to_device(capi.pack_np(x, sp)), capi.layout_for(np.float32, sp), x.shape,
                             hip.to_device(ps), ROUND_SSE, capi.layout_for(np.int8, dp))
            np.testing.assert_array_equal(capi.unpack_np(q.cpu().numpy(), dp, x.shape), golden["quant_perchannel/q"])


@pytest.mark.parametrize("C", [8, 4, 6])
@pytest.mark.parametrize("packing", [True, False])
def test_requantize_exact_ties(hip, golden, C, packing):
    for j in range(4):
        tag = "requant_ties/C%d_pack%d_b%d" % (C, int(packing), j)
        mode = ROUND_SSE if (packing and C % 4 == 0) else ROUND_EXACT
        acc = golden[tag + "/acc"]
        sp = 4 if (packing and C % 4 == 0) else 1
        dp = 8 if (packing and C % 8 == 0) else 1
        bias = golden.get(tag + "/bias")
        q = hip.requantize(hip.to_device(capi.pack_np(acc, sp)), capi.layout_for(np.int32, sp), acc.shape,
                           hip.to_device(golden[tag + "/scale_in"]), hip.to_device(golden[tag + "/scale_out"]),
                           None if bias is None else hip.to_device(bias), 0, 0.0, mode, capi.layout_for(np.int8, dp))
        np.testing.assert_array_equal(capi.unpack_np(q.cpu().numpy(), dp, acc.shape), golden[tag + "/q"])


@pytest.mark.parametrize("act", [0, 1, 2, 3])
@pytest.mark.parametrize("C,packing", [(8, True), (12, True), (6, True), (8, False)])
def test_requantize_random(hip, golden, act, C, packing):
    tag = "requant_rand/act%d_C%d_pack%d" % (act, C, int(packing))
    mode = ROUND_SSE if (packing and C % 4 == 0) else ROUND_EXACT
    acc = golden[tag + "/acc"]
    ap = golden.get(tag + "/act_params")
    for sp in ((1, 4, 8) if C % 8 == 0 else (1, 4) if C % 4 == 0 else (1,)):
        for dp in ((1, 8) if C % 8 == 0 else (1,)):
            q = hip.requantize(hip.to_device(capi.pack_np(acc, sp)), capi.layout_for(np.int32, sp), acc.shape,
                               hip.to_device(golden[tag + "/scale_in"]), hip.to_device(golden[tag + "/scale_out"]),
                               hip.to_device(golden[tag + "/bias"]), act, float(ap[0]) if ap is not None else 0.0,
                               mode, capi.layout_for(np.int8, dp))
            np.testing.assert_array_equal(capi.unpack_np(q.cpu().numpy(), dp, acc.shape), golden[tag + "/q"])


@pytest.mark.parametrize("C,packing", [(8, True), (4, True), (8, False)])
def test_dequantize_bitwise(hip, golden, C, packing):
    for j in (0, 1):
        tag = "dequant/C%d_pack%d_b%d" % (C, int(packing), j)
        acc, bias = golden[tag + "/acc"], golden.get(tag + "/bias")
        for sp in ((1, 4, 8) if C % 8 == 0 else (1, 4)):
            for dp in ((1, 4, 8) if C % 8 == 0 else (1, 4)):
                y = hip.dequantize(hip.to_device(capi.pack_np(acc, sp)), capi.layout_for(np.int32, sp), acc.shape,
                                   hip.to_device(golden[tag + "/scale"]),
                                   None if bias is None else hip.to_device(bias), capi.layout_for(np.float32, dp))
                got = capi.unpack_np(y.cpu().numpy(), dp, acc.shape)
                assert_f32_close(got, golden[tag + "/y"])
                np.testing.assert_array_equal(got.view(np.int32), golden[tag + "/y"].view(np.int32))


def test_repack_roundtrip(hip):
    rng = np.random.default_rng(3)
    a = rng.integers(-100, 100, size=(2, 16, 5, 7)).astype(np.int8)
    for sp in (1, 8):
        for dp in (1, 8):
            r = hip.repack(hip.to_device(capi.pack_np(a, sp)), capi.layout_for(np.int8, sp), a.shape,
                           capi.layout_for(np.int8, dp))
            np.testing.assert_array_equal(capi.unpack_np(r.cpu().numpy(), dp, a.shape), a)
    f = rng.normal(size=(2, 16, 5, 7)).astype(np.float32)
    for sp in (1, 4, 8):
        for dp in (1, 4, 8):
            r = hip.repack(hip.to_device(capi.pack_np(f, sp)), capi.layout_for(np.float32, sp), f.shape,
                           capi.layout_for(np.float32, dp))
            np.testing.assert_array_equal(capi.unpack_np(r.cpu().numpy(), dp, f.shape), f)


# ---- seeded random shapes against the oracle: every MFMA tile shape, ragged pixel counts, odd channels ----

def _rand_problem(rng, C, K, k, g, N, H, W, in_i8=True):
    wq = rng.integers(-127, 128, size=(K, C // g, k, k)).astype(np.int8)
    ws = rng.uniform(50, 400, K).astype(np.float32)
    x = rng.integers(-127, 128, size=(N, C, H, W)).astype(np.int8) if in_i8 else \
        rng.uniform(-1, 1, (N, C, H, W)).astype(np.float32)
    bias = rng.normal(0, 0.5, K).astype(np.float32)
    return x, wq, ws, bias


TILES = [(128, 256), (128, 128), (128, 64), (64, 256), (64, 128), (64, 64), (32, 256), (32, 128), (32, 64)]


@pytest.mark.parametrize("stage", [1, 2], ids=["chunkwise", "staged"])
@pytest.mark.parametrize("tile", TILES, ids=["%dx%d" % t for t in TILES])
def test_igemm_every_tile_shape(hip, oracle, tile, stage):
    """Every tile shape in both variants of the kernel (one 64-deep slice of the reduction per stage, or several):
    accumulators, the int8 epilogue with ReLU, without activation and with LeakyReLU, the fp32 epilogue with ReLU and
    LeakyReLU. The reductions are 9, 1 and 18 slices long: shorter than, equal to and not a multiple of a stage."""
    rng = np.random.default_rng(tile[0] * 1000 + tile[1])
    tile = (tile[0], tile[1] + stage)
    # K = 128 divides every row tile; 2 x 19 x 23 pixels leaves a ragged last pixel tile
    for (C, K, k, s, p) in [(64, 128, 3, 1, 1), (24, 128, 1, 1, 0), (72, 128, 3, 2, 1)]:
        x, wq, ws, bias = _rand_problem(rng, C, K, k, 1, 2, 19, 23)
        in_scale = 31.75
        want, acc_want = oracle.conv_layer_forward(x, wq, ws, in_scale, stride=(s, s), pad=(p, p), bias=bias,
                                                   top_scale=9.0, int8_out=True, act_type=1, want_acc=True)
        acc, kind = run_conv(hip, oracle, x, wq, ws, in_scale, stride=s, pad=p, out_kind=capi.OUT_I32, tile=tile)
        assert kind == 1
        np.testing.assert_array_equal(acc, acc_want)
        out, _ = run_conv(hip, oracle, x, wq, ws, in_scale, stride=s, pad=p, bias=bias, top_scale=9.0, act=1,
                          out_kind=capi.OUT_I8, tile=tile)
        np.testing.assert_array_equal(out, want)
        for act, int8_out in [(0, True), (2, True), (1, False), (2, False)]:
            want = oracle.conv_layer_forward(x, wq, ws, in_scale, stride=(s, s), pad=(p, p), bias=bias, top_scale=9.0,
                                             int8_out=int8_out, act_type=act, act_params=[0.1])
            out, _ = run_conv(hip, oracle, x, wq, ws, in_scale, stride=s, pad=p, bias=bias, top_scale=9.0, act=act,
                              act_p0=0.1, out_kind=capi.OUT_I8 if int8_out else capi.OUT_F32, tile=tile)
            if int8_out:
                np.testing.assert_array_equal(out, want)
            else:
                np.testing.assert_allclose(out, want, rtol=FP32_RTOL, atol=0)


@pytest.mark.parametrize("fn", [4, 5, 6, 7])
def test_halo3x3_every_fragment_count(hip, oracle, fn):
    """The 3x3 stride-1 LDS-halo MFMA kernel: wide (K > 64) and narrow wave layouts, padded channel counts, pad 0 and 1,
    ragged last tile, several channel blocks (C = 320 at 30 columns does not fit LDS at once), the three LDS line pitches
    (up to 60, 124 and 252 columns), several tiles per workgroup, odd image widths (the last pixel pair of a row is
    half padding: both pitches, the widest rows of either, the last row of the tensor, an odd octet count)."""
    rng = np.random.default_rng(fn)
    for (C, K, p, N, H, W) in [(128, 128, 1, 2, 19, 22), (64, 64, 1, 1, 56, 56), (72, 24, 0, 2, 11, 10),
                               (16, 160, 1, 1, 7, 8), (320, 96, 1, 1, 14, 30), (8, 16, 1, 1, 9, 66),
                               (16, 136, 1, 3, 5, 124), (128, 128, 1, 2, 13, 55), (24, 64, 1, 3, 9, 59),
                               (64, 40, 0, 1, 7, 123), (8, 32, 1, 2, 5, 7), (32, 96, 0, 1, 6, 61),
                               (64, 128, 1, 1, 6, 125), (16, 72, 1, 2, 5, 252), (128, 64, 0, 1, 4, 201),
                               (24, 32, 1, 1, 3, 130)]:
        x, wq, ws, bias = _rand_problem(rng, C, K, 3, 1, N, H, W)
        in_scale = 25.0
        for int8_out in (True, False):
            want, acc_want = oracle.conv_layer_forward(x, wq, ws, in_scale, pad=(p, p), bias=bias, top_scale=7.0,
                                                       int8_out=int8_out, act_type=1, want_acc=True)
            out, kind = run_conv(hip, oracle, x, wq, ws, in_scale, pad=p, bias=bias, top_scale=7.0, act=1,
                                 out_kind=capi.OUT_I8 if int8_out else capi.OUT_F32, tile=(-1, fn))
            assert kind == 3
            if int8_out:
                np.testing.assert_array_equal(out, want)
            else:
                assert_f32_close(out, want)
        # raw accumulators take the generic implicit-GEMM kernel
        acc, kind = run_conv(hip, oracle, x, wq, ws, in_scale, pad=p, out_kind=capi.OUT_I32, tile=(-1, fn))
        assert kind == 1
        np.testing.assert_array_equal(acc, acc_want)


@pytest.mark.parametrize("fn", [4, 5, 6, 7])
def test_halo3x3_stride2_and_dilation2(hip, oracle, fn):
    """The strided and the dilated variant of the LDS-halo kernel (row blocks of 64 channels and more): paddings 0 up
    to the dilation, both wave layouts, both line pitches, odd and even widths and heights, ragged last tiles, several
    channel blocks per tile, several tiles per workgroup. K <= 32 stays on the implicit-GEMM kernel."""
    rng = np.random.default_rng(100 + fn)
    cases = [  # C, K, stride, dilation, pad, N, H, W
        (128, 128, 2, 1, 1, 2, 56, 56), (64, 128, 2, 1, 1, 2, 33, 51), (72, 40, 2, 1, 0, 2, 11, 13),
        (16, 160, 2, 1, 1, 1, 9, 124), (128, 72, 2, 1, 1, 2, 40, 60), (192, 256, 2, 1, 0, 1, 30, 53),
        (128, 128, 1, 2, 2, 2, 19, 22), (64, 64, 1, 2, 2, 1, 56, 56), (72, 40, 1, 2, 0, 2, 11, 13),
        (16, 160, 1, 2, 1, 1, 9, 123), (320, 96, 1, 2, 2, 1, 14, 30), (24, 136, 1, 2, 2, 3, 7, 59),
    ]
    for (C, K, s, d, p, N, H, W) in cases:
        x, wq, ws, bias = _rand_problem(rng, C, K, 3, 1, N, H, W)
        in_scale = 25.0
        for int8_out in (True, False):
            want = oracle.conv_layer_forward(x, wq, ws, in_scale, stride=(s, s), dil=(d, d), pad=(p, p), bias=bias,
                                             top_scale=7.0, int8_out=int8_out, act_type=1)
            out, kind = run_conv(hip, oracle, x, wq, ws, in_scale, stride=s, dil=d, pad=p, bias=bias, top_scale=7.0,
                                 act=1, out_kind=capi.OUT_I8 if int8_out else capi.OUT_F32, tile=(-1, fn))
            assert kind == 3, (C, K, s, d, p)
            if int8_out:
                np.testing.assert_array_equal(out, want)
            else:
                assert_f32_close(out, want)
    # 32 output channels, or a stride-2 tile whose input rows do not fit LDS: the implicit-GEMM kernel
    for (C, K, s, d, p, H, W) in [(64, 32, 2, 1, 1, 12, 12), (64, 32, 1, 2, 2, 12, 12), (128, 128, 2, 1, 1, 19, 22)]:
        x, wq, ws, bias = _rand_problem(rng, C, K, 3, 1, 1, H, W)
        want = oracle.conv_layer_forward(x, wq, ws, 25.0, stride=(s, s), dil=(d, d), pad=(p, p), bias=bias, top_scale=7.0,
                                         int8_out=True, act_type=1)
        out, kind = run_conv(hip, oracle, x, wq, ws, 25.0, stride=s, dil=d, pad=p, bias=bias, top_scale=7.0, act=1,
                             out_kind=capi.OUT_I8)
        assert kind == 1
        np.testing.assert_array_equal(out, want)


def test_halo3x3_ragged_last_tile_then_full_tile_in_one_workgroup(hip, oracle):
    """Tiles of whole image rows (128 pixels = 8 rows of 16) on an image that is not a whole number of tiles (20 rows:
    the third tile of an image has 4 rows), with so many output channels that the persistent grid is shorter than the
    tile list: some workgroups start on a ragged tile and go on to a full one, whose lanes past the ragged tile's end
    need their own LDS offsets."""
    rng = np.random.default_rng(77)
    C, K, N, H, W = 8, 1024, 32, 20, 16
    x, wq, ws, bias = _rand_problem(rng, C, K, 3, 1, N, H, W)
    out, kind = run_conv(hip, oracle, x, wq, ws, 25.0, pad=1, bias=bias, top_scale=7.0, act=1, out_kind=capi.OUT_I8,
                         tile=(-1, 4))
    assert kind == 3
    want = oracle.conv_layer_forward(x, wq, ws, 25.0, pad=(1, 1), bias=bias, top_scale=7.0, int8_out=True, act_type=1)
    np.testing.assert_array_equal(out, want)


@pytest.mark.parametrize("C,K,k,s,p,d,g,N,H,W", [
    (16, 24, 1, 1, 0, 1, 1, 3, 14, 14),     # MobileNetV2 project: K % 32 != 0
    (96, 160, 1, 1, 0, 1, 1, 2, 7, 7),
    (320, 1280, 1, 1, 0, 1, 1, 1, 7, 7),
    (144, 24, 1, 1, 0, 1, 1, 2, 9, 9),
    (8, 20, 3, 1, 1, 1, 1, 1, 9, 9),        # K % 8 != 0, K % 4 == 0 -> Int4 / Byte
    (8, 10, 3, 2, 1, 1, 1, 2, 9, 7),        # K % 4 != 0 -> unpacked outputs
    (32, 32, 3, 1, 2, 2, 1, 1, 11, 11),     # dilation
    (16, 16, 3, 1, 1, 1, 2, 1, 8, 8),       # grouped, non-depthwise: a group per grid slice of the implicit GEMM
    (6, 6, 3, 1, 1, 1, 6, 1, 8, 8),         # depthwise with C % 8 != 0: channels zero-padded to an octet
    (12, 8, 3, 1, 1, 1, 1, 1, 8, 8),        # C % 8 != 0
    (64, 64, 3, 1, 1, 1, 64, 2, 17, 13),    # depthwise 3x3 s1, ragged strips
    (64, 64, 3, 2, 1, 1, 64, 2, 17, 13),    # depthwise 3x3 s2
    (16, 16, 3, 1, 1, 1, 16, 11, 7, 7),     # depthwise, narrow image: 9 images share a wave, ragged last group
    (24, 24, 3, 1, 1, 1, 24, 5, 14, 14),    # 4 images per wave
    (16, 16, 3, 2, 1, 1, 16, 5, 28, 28),    # stride 2 to 14 columns: 4 images per wave
    (8, 8, 3, 1, 1, 1, 8, 3, 9, 32),        # 2 images per wave, full wave
    (8, 8, 3, 1, 0, 1, 8, 3, 9, 33),        # 33 columns: one image per wave again; pad 0
    (16, 16, 7, 1, 3, 1, 16, 1, 12, 12),    # depthwise 7x7
    (16, 16, 3, 1, 2, 2, 16, 1, 12, 12),    # depthwise dilated -> generic depthwise kernel
    (128, 128, 3, 1, 1, 1, 1, 4, 56, 56),   # the c3 layer at reduced batch
])
def test_random_shapes_against_oracle(hip, oracle, C, K, k, s, p, d, g, N, H, W):
    rng = np.random.default_rng(C * 7 + K * 3 + k + s + g)
    x, wq, ws, bias = _rand_problem(rng, C, K, k, g, N, H, W)
    in_scale = 20.0
    for int8_out, act in ((True, 3), (False, 1), (True, 2)):
        want, acc_want = oracle.conv_layer_forward(x, wq, ws, in_scale, stride=(s, s), pad=(p, p), dil=(d, d),
                                                   groups=g, bias=bias, top_scale=11.0, int8_out=int8_out,
                                                   act_type=act, act_params=[0.25], want_acc=True)
        acc, _ = run_conv(hip, oracle, x, wq, ws, in_scale, stride=s, pad=p, dil=d, groups=g,
                          out_kind=capi.OUT_I32)
        np.testing.assert_array_equal(acc, acc_want)
        out, _ = run_conv(hip, oracle, x, wq, ws, in_scale, stride=s, pad=p, dil=d, groups=g, bias=bias,
                          top_scale=11.0, act=act, act_p0=0.25,
                          out_kind=capi.OUT_I8 if int8_out else capi.OUT_F32)
        if int8_out:
            np.testing.assert_array_equal(out, want)
        else:
            assert_f32_close(out, want)


@pytest.mark.parametrize("groups_slices", [(0, 0), (4, 1), (2, 2), (2, 3), (2, 1), (4, 5)],
                         ids=["auto", "g4s1", "g2s2", "g2s3", "g2s1", "g4s5"])
def test_streamed_pointwise_kernel(hip, oracle, groups_slices):
    """The streamed 1x1 int8 -> int8 kernel (at most 256 input channels): 1 to 8 input octets (a half-used operand
    register, a full one), four reduction steps (200..256 channels, the last step partly filled) on blobs of at least
    20 000 pixels, output channel counts that end inside a pair of row tiles (8, 24, 40, 144) and on one, pixel
    counts that are not whole groups of 16 (and images smaller than one group), every epilogue the fast int8 path has
    (none, ReLU, clip, LeakyReLU), with and without bias, forced pixel groups per wave and channel slices. fp32
    output, 72..192 input channels, and four reduction steps over few pixels, stay on the implicit-GEMM kernel."""
    G, S = groups_slices
    rng = np.random.default_rng(100 + 8 * G + S)
    for (C, K, N, H, W) in [(16, 96, 2, 19, 23), (24, 144, 1, 28, 28), (32, 16, 3, 9, 11), (8, 8, 2, 3, 3),
                            (64, 384, 1, 14, 14), (40, 24, 2, 16, 16), (56, 40, 1, 5, 41), (32, 192, 2, 1, 70),
                            (256, 24, 7, 56, 56), (200, 72, 21, 31, 31), (232, 40, 2, 100, 101)]:
        pairs = (K + 31) // 32
        tile = (-5, G | min(S, pairs) << 3) if G else None
        x, wq, ws, bias = _rand_problem(rng, C, K, 1, 1, N, H, W)
        in_scale = 25.0
        for act, b in [(0, bias), (1, bias), (3, None), (2, bias)]:
            want = oracle.conv_layer_forward(x, wq, ws, in_scale, bias=b, top_scale=11.0, int8_out=True, act_type=act,
                                             act_params=[0.1] if act == 2 else [0.0, 6.0])
            out, kind = run_conv(hip, oracle, x, wq, ws, in_scale, bias=b, top_scale=11.0, act=act, act_p0=0.1,
                                 out_kind=capi.OUT_I8, tile=tile)
            assert kind == 5, (C, K, act)
            np.testing.assert_array_equal(out, want)
        out, kind = run_conv(hip, oracle, x, wq, ws, in_scale, bias=bias, act=1, out_kind=capi.OUT_F32)
        assert kind == 1
    x, wq, ws, bias = _rand_problem(rng, 72, 32, 1, 1, 1, 6, 6)
    _, kind = run_conv(hip, oracle, x, wq, ws, 25.0, bias=bias, top_scale=11.0, act=1, out_kind=capi.OUT_I8)
    assert kind == 1


@pytest.mark.parametrize("seed", range(6))
def test_drawn_geometries_against_oracle(hip, oracle, seed):
    """Eight geometries per seed drawn from the whole domain of the layer (kernel 1..5, stride 1..2, dilation 1..2,
    padding 0..dilation*(k/2), dense / grouped / depthwise, channel counts that are and are not multiples of 8 and 4,
    int8 and fp32 inputs, odd sizes), whatever kernel each one routes to: int8 result bit for bit, fp32 within 1e-5."""
    rng = np.random.default_rng(1000 + seed)
    done = 0
    while done < 8:
        k = int(rng.choice([1, 3, 3, 3, 5]))
        s = int(rng.integers(1, 3))
        d = 1 if k == 1 else int(rng.integers(1, 3))
        p = int(rng.integers(0, d * (k // 2) + 1))
        kind = rng.choice(["dense", "dense", "grouped", "depthwise"])
        if kind == "dense":
            C, K, g = int(rng.choice([8, 16, 24, 40, 64, 72, 128, 12, 3])), int(rng.choice([8, 16, 20, 32, 64, 96, 136, 10])), 1
        elif kind == "grouped":
            g = int(rng.choice([2, 4]))
            C, K = g * int(rng.choice([8, 16, 4])), g * int(rng.choice([8, 16, 12]))
        else:
            C = K = g = int(rng.choice([8, 16, 24, 64, 6]))
        N, H, W = int(rng.integers(1, 4)), int(rng.integers(5, 30)), int(rng.integers(5, 70))
        if (H + 2 * p - d * (k - 1) - 1) // s + 1 < 1 or (W + 2 * p - d * (k - 1) - 1) // s + 1 < 1:
            continue
        done += 1
        x, wq, ws, bias = _rand_problem(rng, C, K, k, g, N, H, W, in_i8=bool(rng.integers(0, 2)))
        in_scale = 20.0 if x.dtype == np.int8 else 100.0
        act = int(rng.choice([0, 1, 2, 3]))
        int8_out = bool(rng.integers(0, 2))
        what = (C, K, k, s, p, d, g, N, H, W, str(x.dtype), act, int8_out)
        want = oracle.conv_layer_forward(x, wq, ws, in_scale, stride=(s, s), pad=(p, p), dil=(d, d), groups=g, bias=bias,
                                         top_scale=11.0, int8_out=int8_out, act_type=act, act_params=[0.25])
        out, _ = run_conv(hip, oracle, x, wq, ws, in_scale, stride=s, pad=p, dil=d, groups=g, bias=bias, top_scale=11.0,
                          act=act, act_p0=0.25, out_kind=capi.OUT_I8 if int8_out else capi.OUT_F32)
        if int8_out:
            np.testing.assert_array_equal(out, want, err_msg=str(what))
        else:
            np.testing.assert_allclose(out, want, rtol=FP32_RTOL, atol=1e-30, err_msg=str(what))


@pytest.mark.parametrize("shift", [0, 1, 2])
@pytest.mark.parametrize("s", [1, 2])
@pytest.mark.parametrize("family", [-2, -3], ids=["mfma", "valu"])
def test_depthwise3x3_every_strip_height(hip, oracle, family, s, shift):
    """The depthwise 3x3 kernels (matrix-core and vector-ALU family) are instantiated for three strip heights per
    stride, chosen from the problem size: force each on shapes with ragged last strips, narrow images sharing a
    wave, more than 64 columns, a channel count that ends on a single octet, pad 0, and every fast epilogue."""
    rng = np.random.default_rng(10 * s + shift)
    for (C, N, H, W, p) in [(16, 3, 19, 70, 1), (8, 7, 13, 9, 1), (24, 5, 8, 8, 0), (40, 3, 9, 5, 1),
                            (8, 1, 33, 64, 1)]:
        x, wq, ws, bias = _rand_problem(rng, C, C, 3, C, N, H, W)
        for act, int8_out in ((3, True), (0, True), (1, False)):
            want = oracle.conv_layer_forward(x, wq, ws, 20.0, stride=(s, s), pad=(p, p), groups=C, bias=bias,
                                             top_scale=9.0, int8_out=int8_out, act_type=act)
            out, kind = run_conv(hip, oracle, x, wq, ws, 20.0, stride=s, pad=p, groups=C, bias=bias, top_scale=9.0,
                                 act=act, out_kind=capi.OUT_I8 if int8_out else capi.OUT_F32, tile=(family, shift))
            assert kind == 2
            if int8_out:
                np.testing.assert_array_equal(out, want)
            else:
                assert_f32_close(out, want)


@pytest.mark.parametrize("s", [1, 2])
@pytest.mark.parametrize("family", [-2, -3], ids=["mfma", "valu"])
def test_depthwise5x5_and_wide_padding(hip, oracle, family, s):
    """The matrix-core depthwise kernel also takes a 5x5 window with pad 2 (the 8 input pixels of a column cover it)
    and a 3x3 window with pad 2; checked like the 3x3 case, forced strips included, against the oracle and against
    the vector-ALU family."""
    rng = np.random.default_rng(50 + s)
    for (C, N, H, W, k, p) in [(16, 2, 19, 70, 5, 2), (8, 5, 13, 9, 5, 2), (40, 3, 9, 21, 5, 2), (24, 2, 26, 26, 5, 2),
                               (16, 2, 11, 12, 3, 2)]:
        x, wq, ws, bias = _rand_problem(rng, C, C, k, C, N, H, W)
        for act, int8_out, shift in ((3, True, 0), (0, True, 1), (2, False, 2)):
            want = oracle.conv_layer_forward(x, wq, ws, 20.0, stride=(s, s), pad=(p, p), groups=C, bias=bias,
                                             top_scale=9.0, int8_out=int8_out, act_type=act,
                                             act_params=[0.1] if act == 2 else None)
            out, kind = run_conv(hip, oracle, x, wq, ws, 20.0, stride=s, pad=p, groups=C, bias=bias, top_scale=9.0,
                                 act=act, act_p0=0.1, out_kind=capi.OUT_I8 if int8_out else capi.OUT_F32,
                                 tile=(family, shift))
            assert kind == 2
            if int8_out:
                np.testing.assert_array_equal(out, want, err_msg=str((C, N, H, W, k, act)))
            else:
                assert_f32_close(out, want)


@pytest.mark.parametrize("C,K,k,s,p,g,N,H,W,kind", [
    (64, 96, 3, 1, 1, 1, 2, 14, 16, 3),     # 3x3 LDS-halo kernel
    (80, 72, 1, 1, 0, 1, 2, 13, 11, 1),     # 1x1 implicit GEMM
    (48, 72, 1, 1, 0, 1, 2, 13, 11, 5),     # 1x1 streamed (int8 result; the fp32 one takes the implicit GEMM)
    (32, 64, 3, 2, 1, 1, 2, 15, 15, 1),     # 3x3 stride 2 implicit GEMM
    (40, 40, 3, 1, 1, 40, 3, 12, 20, 2),    # depthwise stride 1
    (24, 24, 3, 2, 1, 24, 3, 13, 18, 2),    # depthwise stride 2
])
def test_leaky_relu_fast_epilogues(hip, oracle, C, K, k, s, p, g, N, H, W, kind):
    """LeakyReLU 0.1 is the activation of the reference's own int8 models (benchmark/nanodet-plus-m-1.5x_416_int8_*.otter):
    the fused epilogues evaluate it as max(v, v * slope); int8 and fp32 outputs against the oracle."""
    rng = np.random.default_rng(C + K + k + s)
    x, wq, ws, bias = _rand_problem(rng, C, K, k, g, N, H, W)
    for int8_out in (True, False):
        want = oracle.conv_layer_forward(x, wq, ws, 18.0, stride=(s, s), pad=(p, p), groups=g, bias=bias, top_scale=13.0,
                                         int8_out=int8_out, act_type=2, act_params=[0.1])
        out, got_kind = run_conv(hip, oracle, x, wq, ws, 18.0, stride=s, pad=p, groups=g, bias=bias, top_scale=13.0,
                                 act=2, act_p0=0.1, out_kind=capi.OUT_I8 if int8_out else capi.OUT_F32)
        assert got_kind == (1 if kind == 5 and not int8_out else kind)
        if int8_out:
            np.testing.assert_array_equal(out, want)
        else:
            assert_f32_close(out, want)


@pytest.mark.parametrize("C,K,k,s,p,g,N,H,W,kind_i8,kind_f32", [
    (16, 16, 3, 1, 1, 2, 2, 9, 11, 1, 1),       # two groups of 8 -> 8
    (64, 128, 3, 1, 1, 4, 3, 14, 14, 1, 1),     # four groups of 16 -> 32
    (32, 48, 1, 1, 0, 2, 2, 13, 7, 1, 1),       # pointwise, groups of 16 -> 24
    (48, 24, 3, 2, 1, 3, 2, 15, 17, 1, 1),      # stride 2, three groups of 16 -> 8
    (16, 8, 3, 1, 1, 2, 2, 8, 8, 0, 1),         # groups of 8 -> 4: whole Float4 elements, but half a Byte8 element
    (24, 24, 3, 1, 1, 2, 1, 8, 8, 0, 0),        # groups of 12 channels: not whole octets -> the scalar catch-all
    (6, 6, 3, 1, 1, 6, 2, 9, 10, 2, 2),         # depthwise, C % 8 != 0
    (20, 20, 3, 2, 1, 20, 3, 13, 15, 2, 2),     # depthwise stride 2, C % 4 == 0
    (12, 12, 5, 1, 2, 12, 2, 11, 11, 2, 2),     # depthwise 5x5
])
def test_grouped_and_odd_depthwise_routes(hip, oracle, C, K, k, s, p, g, N, H, W, kind_i8, kind_f32):
    """Grouped non-depthwise convolutions (Tensor/Convolution.cpp:396-408: the reference slices the channels and runs
    a convolution per group) run as one launch of the implicit-GEMM kernel with the group on grid.z when a group is
    whole octets in and whole elements out; depthwise layers whose channel count is not a multiple of 8 run on the
    depthwise kernels over a zero-padded octet. Accumulators, int8 and fp32 results against the oracle."""
    rng = np.random.default_rng(C * 5 + K + k + s + g)
    x, wq, ws, bias = _rand_problem(rng, C, K, k, g, N, H, W)
    in_scale = 23.0
    want_acc = oracle.conv_layer_forward(x, wq, ws, in_scale, stride=(s, s), pad=(p, p), groups=g, bias=bias,
                                         top_scale=12.0, int8_out=True, act_type=1, want_acc=True)[1]
    acc, _ = run_conv(hip, oracle, x, wq, ws, in_scale, stride=s, pad=p, groups=g, out_kind=capi.OUT_I32)
    np.testing.assert_array_equal(acc, want_acc)
    for int8_out, act, kind in ((True, 1, kind_i8), (True, 0, kind_i8), (False, 3, kind_f32)):
        want = oracle.conv_layer_forward(x, wq, ws, in_scale, stride=(s, s), pad=(p, p), groups=g, bias=bias,
                                         top_scale=12.0, int8_out=int8_out, act_type=act)
        out, got_kind = run_conv(hip, oracle, x, wq, ws, in_scale, stride=s, pad=p, groups=g, bias=bias, top_scale=12.0,
                                 act=act, out_kind=capi.OUT_I8 if int8_out else capi.OUT_F32)
        assert got_kind == kind
        if int8_out:
            np.testing.assert_array_equal(out, want)
        else:
            assert_f32_close(out, want)


@pytest.mark.parametrize("C,K,s,p,N,H,W,in_i8,act,int8_out", [
    (3, 32, 2, 1, 3, 30, 46, False, 3, True),    # the MobileNetV2 stem: fp32 image, ReLU6, int8 out
    (3, 24, 2, 1, 2, 33, 21, False, 2, False),   # the detection model's stem: LeakyReLU, fp32 out, 1.5 tiles of channels
    (1, 16, 1, 0, 2, 9, 19, False, 0, True),     # one channel, no padding
    (4, 40, 1, 1, 2, 12, 17, True, 1, True),     # int8 planar input, 2.5 tiles
    (5, 64, 2, 0, 1, 15, 16, True, 0, False),    # the widest reduction (45 of 64 bytes), 4 tiles
    (3, 8, 1, 1, 5, 8, 8, False, 1, False),      # half a tile
    (3, 16, 2, 1, 1, 10, 420, False, 1, True),   # a wide image: the strip's rows are loaded in two rounds of 16-byte loads
    (3, 16, 1, 1, 2, 9, 16, True, 0, True),      # int8 planar rows of whole 4-byte units, signed result
    (2, 8, 2, 0, 1, 11, 23, False, 3, True),     # two channels, no padding, odd width: scalar loads, clip at six
    (4, 32, 2, 1, 2, 3, 4, True, 2, True),       # fewer output rows than a strip, one 4-pixel unit per row
])
def test_few_channel_3x3_stem_kernel(hip, oracle, C, K, s, p, N, H, W, in_i8, act, int8_out):
    """3x3 on a blob with at most 5 channels goes straight from the unpacked blob (quantized on the way) to the
    packed output; the same layer forced through the channel-padded copy and the generic kernel must agree bit for
    bit, and both equal the oracle."""
    rng = np.random.default_rng(1000 * C + K)
    x, wq, ws, bias = _rand_problem(rng, C, K, 3, 1, N, H, W, in_i8=in_i8)
    kw = dict(stride=s, pad=p, bias=bias, top_scale=11.0, act=act, act_p0=0.1,
              out_kind=capi.OUT_I8 if int8_out else capi.OUT_F32)
    want = oracle.conv_layer_forward(x, wq, ws, 25.0, stride=(s, s), pad=(p, p), bias=bias, top_scale=11.0,
                                     int8_out=int8_out, act_type=act, act_params=[0.1] if act == 2 else None)
    out, kind = run_conv(hip, oracle, x, wq, ws, 25.0, **kw)
    assert kind == 4
    via_copy, kind2 = run_conv(hip, oracle, x, wq, ws, 25.0, tile=(-4, 0), **kw)
    assert kind2 == 1
    if int8_out:
        np.testing.assert_array_equal(out, want)
    else:
        assert_f32_close(out, want)
    np.testing.assert_array_equal(out, via_copy)


@pytest.mark.parametrize("C,K,k,s,p,g,N,H,W,act,kind", [
    (96, 24, 1, 1, 0, 1, 3, 14, 13, 0, 1),     # pointwise project, ragged pixel tile: twin from the epilogue
    (32, 16, 1, 1, 0, 1, 2, 9, 9, 1, 1),
    (144, 40, 1, 2, 0, 1, 2, 9, 9, 3, 1),      # K % 32 != 0
    (64, 64, 3, 1, 1, 1, 1, 10, 12, 1, 3),     # halo kernel: quantize pass behind it
    (16, 16, 3, 1, 1, 16, 2, 9, 9, 0, 2),      # depthwise
    (24, 24, 1, 1, 0, 1, 1, 5, 5, 4, 1),       # sigmoid: generic epilogue, quantize pass
])
@pytest.mark.parametrize("round_mode", [capi.ROUND_SSE, capi.ROUND_EXACT], ids=["sse", "exact"])
def test_forward_twin_equals_forward_then_quantize(hip, oracle, C, K, k, s, p, g, N, H, W, act, kind, round_mode):
    """otter_hip_conv_forward_twin: the fp32 blob is bit-identical to otter_hip_conv_forward's, and the Byte8 twin
    is bit-identical to the oracle's quantize_to_int8 of that blob, whichever kernel produced it."""
    rng = np.random.default_rng(C + K * 5 + k + act)
    x, wq, ws, bias = _rand_problem(rng, C, K, k, g, N, H, W)
    in_scale = 20.0
    conv = hip.conv(wq=wq, scale_in=host_scale_in(ws, in_scale), bias=bias, in_scale=in_scale, out_scale=None,
                    stride=(s, s), pad=(p, p), dil=(1, 1), groups=g, act=act, act_p0=0.0, out_kind=capi.OUT_F32,
                    out_round=0, in_round=oracle.quantize_round_mode(C, True))
    xd = hip.to_device(capi.pack_np(x, 8))
    assert conv.kernel_kind(capi.I8_P8, N, H, W, capi.F32_P4) == kind
    plain = conv.forward(xd, capi.I8_P8, N, H, W, capi.F32_P4).cpu().numpy()
    q_scale = 127.0 / max(float(np.abs(plain).max()), 1e-6) * 1.3   # some values saturate
    out, q = conv.forward_twin(xd, capi.I8_P8, N, H, W, q_scale, round_mode, capi.F32_P4)
    hip.torch.cuda.synchronize()
    oh, ow = conv.out_hw(H, W)
    np.testing.assert_array_equal(out.cpu().numpy().view(np.uint32), plain.view(np.uint32))
    y = capi.unpack_np(plain, 4, (N, K, oh, ow))
    want = oracle.quantize(y, np.float32(q_scale), round_mode)
    np.testing.assert_array_equal(capi.unpack_np(q.cpu().numpy(), 8, (N, K, oh, ow)), want)
    conv.close()


@pytest.mark.parametrize("C,K,k,s,p,g,N,H,W,act,kind", [
    (96, 24, 1, 1, 0, 1, 3, 14, 13, 0, 1),     # pointwise project of a residual block: sum from the epilogue
    (192, 32, 1, 1, 0, 1, 2, 9, 9, 1, 1),
    (144, 20, 1, 1, 0, 1, 2, 7, 7, 0, 1),      # K % 8 != 0: the sum alone
    (64, 64, 3, 1, 1, 1, 1, 10, 12, 1, 3),     # halo kernel: add (+ quantize) pass behind it
    (16, 16, 3, 1, 1, 16, 2, 9, 9, 0, 2),      # depthwise
    (24, 24, 1, 1, 0, 1, 1, 5, 5, 4, 1),       # sigmoid: generic epilogue
])
@pytest.mark.parametrize("with_q", [True, False], ids=["sum_and_twin", "sum_only"])
def test_forward_residual_equals_forward_then_add(hip, oracle, C, K, k, s, p, g, N, H, W, act, kind, with_q):
    """otter_hip_conv_forward_residual: the sum is bit-identical to otter_hip_conv_forward's blob plus the shortcut (one
    fp32 addition per element), and the twin to the oracle's quantize_to_int8 of that sum."""
    rng = np.random.default_rng(C * 3 + K + k + act)
    x, wq, ws, bias = _rand_problem(rng, C, K, k, g, N, H, W)
    in_scale = 20.0
    conv = hip.conv(wq=wq, scale_in=host_scale_in(ws, in_scale), bias=bias, in_scale=in_scale, out_scale=None,
                    stride=(s, s), pad=(p, p), dil=(1, 1), groups=g, act=act, act_p0=0.0, out_kind=capi.OUT_F32,
                    out_round=0, in_round=oracle.quantize_round_mode(C, True))
    xd = hip.to_device(capi.pack_np(x, 8))
    assert conv.kernel_kind(capi.I8_P8, N, H, W, capi.F32_P4) == kind
    oh, ow = conv.out_hw(H, W)
    plain = capi.unpack_np(conv.forward(xd, capi.I8_P8, N, H, W, capi.F32_P4).cpu().numpy(), 4, (N, K, oh, ow))
    short = (rng.normal(0, 1, plain.shape) * np.abs(plain).mean()).astype(np.float32)
    want = plain + short
    with_q = with_q and K % 8 == 0
    q_scale = 127.0 / float(np.abs(want).max()) * 1.3 if with_q else None   # some values saturate
    out, q = conv.forward_residual(xd, capi.I8_P8, N, H, W, hip.to_device(capi.pack_np(short, 4)), q_scale,
                                   capi.ROUND_SSE, capi.F32_P4)
    hip.torch.cuda.synchronize()
    got = capi.unpack_np(out.cpu().numpy(), 4, (N, K, oh, ow))
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    if with_q:
        np.testing.assert_array_equal(capi.unpack_np(q.cpu().numpy(), 8, (N, K, oh, ow)),
                                      oracle.quantize(want, np.float32(q_scale), capi.ROUND_SSE))
    conv.close()


@pytest.mark.parametrize("s", [1, 2])
def test_depthwise3x3_from_an_fp32_blob_in_one_launch(hip, oracle, s):
    """A depthwise 3x3 layer on an fp32 Float8 blob of 17..128 columns runs quantize_to_int8 and the convolution as ONE
    launch (every value quantized once, through the wave's LDS lines). Against the oracle's layer, and bit for bit
    against the two launches (set_tile(-6, 0)): both column-chunk counts, odd widths, widths that end inside and on a
    chunk, ragged and forced strips (one row per strip, more rows than the image), pad 0, batch > 1, values on rounding
    ties and beyond saturation, both rounding primitives, every fast epilogue."""
    rng = np.random.default_rng(300 + s)
    shapes = [(16, 3, 19, 70, 1), (8, 2, 13, 17, 1), (24, 2, 8, 64, 0), (8, 1, 33, 65, 1), (8, 2, 9, 128, 1), (16, 1, 30, 112, 1),
              (8, 2, 5, 33, 0), (32, 2, 3, 40, 1)]
    for i, (C, N, H, W, p) in enumerate(shapes):
        x, wq, ws, bias = _rand_problem(rng, C, C, 3, C, N, H, W, in_i8=False)
        in_scale = np.float32(100.0)
        # some values exactly on a tie of the quantization, on the value the two primitives round differently, and
        # beyond saturation
        flat = x.reshape(-1)
        flat[::7] = (rng.integers(-140, 141, flat[::7].size) + 0.5) / in_scale
        flat[3::11] = np.nextafter(np.float32(0.5), np.float32(0)) / in_scale * rng.choice([-1, 1], flat[3::11].size)
        for act, int8_out, tile in ((3, True, None), (0, True, (-2, 1)), (1, False, (-2, 200)), (2, True, (-2, 5))):
            kw = dict(stride=(s, s), pad=(p, p), groups=C, bias=bias, top_scale=9.0, int8_out=int8_out, act_type=act,
                      act_params=[0.1] if act == 2 else None)
            want = oracle.conv_layer_forward(x, wq, ws, in_scale, **kw)
            args = dict(stride=s, pad=p, groups=C, bias=bias, top_scale=9.0, act=act, act_p0=0.1,
                        out_kind=capi.OUT_I8 if int8_out else capi.OUT_F32)
            out, kind = run_conv(hip, oracle, x, wq, ws, in_scale, tile=tile, **args)
            two, _ = run_conv(hip, oracle, x, wq, ws, in_scale, tile=(-6, 0), **args)
            assert kind == 2
            what = str((C, N, H, W, p, act, int8_out, tile))
            assert out.tobytes() == two.tobytes(), what
            if int8_out:
                np.testing.assert_array_equal(out, want, err_msg=what)
            else:
                assert_f32_close(out, want)
    # the scalar rounding primitive on the input side (what an unpacked net would ask for) through the same launch; with a
    # power-of-two input scale a fifth of the values land exactly on the one float the two primitives round differently
    x, wq, ws, bias = _rand_problem(rng, 8, 8, 3, 8, 2, 9, 40, in_i8=False)
    x.reshape(-1)[::5] = np.nextafter(np.float32(0.5), np.float32(0)) / np.float32(128.0)
    si = (np.float32(1.0) / (np.float32(128.0) * ws)).astype(np.float32)
    outs = {}
    for mode in (capi.ROUND_SSE, capi.ROUND_EXACT):
        conv = hip.conv(wq=wq, scale_in=si, bias=bias, in_scale=128.0, out_scale=[900.0], stride=(s, s), pad=(1, 1), groups=8,
                        act=0, out_kind=capi.OUT_I8, in_round=mode)
        xq = oracle.quantize(x, [np.float32(128.0)], mode)
        want = oracle.requantize(oracle.conv_int32(xq, wq, (s, s), (1, 1), (1, 1), 8), si, [900.0], bias, 0, None, capi.ROUND_SSE)
        got = conv.forward(hip.to_device(capi.pack_np(x, 8)), capi.F32_P8, 2, 9, 40, capi.I8_P8)
        oh, ow = conv.out_hw(9, 40)
        outs[mode] = capi.unpack_np(got.cpu().numpy(), 8, (2, 8, oh, ow))
        np.testing.assert_array_equal(outs[mode], want)
        conv.close()
    assert (outs[capi.ROUND_SSE] != outs[capi.ROUND_EXACT]).any()


def _fp32_blob_with_ties(rng, shape, in_scale):
    """fp32 values with some exactly on a tie of the quantization, on the float the two rounding primitives round
    differently, and beyond saturation."""
    x = rng.uniform(-1, 1, shape).astype(np.float32)
    flat = x.reshape(-1)
    flat[::7] = (rng.integers(-140, 141, flat[::7].size) + 0.5) / in_scale
    flat[3::11] = np.nextafter(np.float32(0.5), np.float32(0)) / in_scale * rng.choice([-1, 1], flat[3::11].size)
    return x


@pytest.mark.parametrize("C,K,N,H,W,int8_out,tile_shape,small", [
    (72, 512, 2, 9, 11, True, "128x64", True),
    (72, 512, 1, 7, 7, False, "128x64", True),
    (136, 64, 1, 30, 30, True, "64x64", True),
    (72, 64, 8, 128, 128, True, "64x128", False),
    (8, 64, 8, 256, 256, False, "64x256", False),
    (80, 24, 2, 9, 11, True, "32x64", True),
    (80, 32, 2, 128, 128, True, "32x128", False),
    (8, 16, 8, 256, 256, False, "32x256", False),
    (200, 100, 3, 5, 13, False, "64x64", True),    # channel octets that end inside a 64-deep step, K % 8 != 0
])
def test_pointwise_from_an_fp32_blob_in_the_igemm_loader(hip, oracle, C, K, N, H, W, int8_out, tile_shape, small):
    """A pointwise layer of the implicit-GEMM kernel on an fp32 Float8 blob quantizes in the kernel's loader (one launch,
    no int8 copy of the blob; set_tile(-4, 0) keeps the layers on this kernel that would otherwise go to the kernel of
    the next test). Bit for bit against the two launches (set_tile(-6, 0)) at every tile shape the launcher picks --
    values on rounding ties, on the float the two primitives round differently and beyond saturation, every packed
    epilogue -- and, at the sizes the oracle finishes in seconds, against the oracle's layer."""
    rng = np.random.default_rng(C * 7 + K)
    _, wq, ws, bias = _rand_problem(rng, C, K, 1, 1, N, H, W, in_i8=False)
    in_scale = np.float32(100.0)
    x = _fp32_blob_with_ties(rng, (N, C, H, W), in_scale)
    for act in ((3, 0, 2) if int8_out else (1, 2)):
        args = dict(bias=bias, top_scale=9.0, act=act, act_p0=0.1, out_kind=capi.OUT_I8 if int8_out else capi.OUT_F32)
        out, kind = run_conv(hip, oracle, x, wq, ws, in_scale, tile=(-4, 0), **args)
        two, _ = run_conv(hip, oracle, x, wq, ws, in_scale, tile=(-6, 0), **args)
        assert kind == 1
        assert out.tobytes() == two.tobytes(), (act, tile_shape)
        if small:
            want = oracle.conv_layer_forward(x, wq, ws, in_scale, bias=bias, top_scale=9.0, int8_out=int8_out, act_type=act,
                                             act_params=[0.1] if act == 2 else None)
            if int8_out:
                np.testing.assert_array_equal(out, want)
            else:
                assert_f32_close(out, want)


@pytest.mark.parametrize("C,K,N,H,W,int8_out,auto,small", [
    (72, 512, 2, 9, 11, True, True, True),        # two reduction steps, the second one 8 channels; four LDS rounds
    (256, 136, 1, 7, 7, False, True, True),       # K % 32 != 0: a pair with one live tile and a half
    (64, 128, 3, 5, 13, True, True, True),        # one reduction step; 65 pixels: a wave with one live pixel
    (200, 100, 3, 5, 13, False, False, True),     # K % 8 != 0 (fp32 out only), channel octets ending inside a step
    (8, 16, 2, 9, 11, True, False, True),         # one octet, one output tile
    (40, 24, 2, 17, 3, True, False, True),
    (136, 264, 1, 30, 30, True, True, True),      # three steps, 9 pairs: a last round of one pair
    (256, 512, 32, 28, 28, False, True, False),   # the benchmark layer: one group per wave by the launcher's choice
    (128, 128, 64, 28, 28, True, True, False),    # two groups per wave by the launcher's choice
    (8, 4, 1, 1, 1, False, False, True),          # one pixel, one Float4 element of output
    (16, 8, 5, 1, 3, True, False, True),          # three pixels per image, one Byte8 element
    (256, 128, 1, 1, 1, True, True, True),        # one pixel, every reduction step
])
def test_pointwise_from_an_fp32_blob_read_once(hip, oracle, C, K, N, H, W, int8_out, auto, small):
    """conv_pw_f32in_kernel: a pointwise layer of up to 256 input channels on an fp32 Float8 blob, the blob read once, all
    output channels walked per pixel group through LDS rounds of weights. Taken by itself from 64 input and 128 output
    channels on (`auto`), forced otherwise (set_tile(-7, groups | pairs << 3)). Bit for bit against the two launches with
    one and two pixel groups per wave and with rounds of one, two and the default number of pairs; against the oracle's
    layer at the sizes it finishes in seconds."""
    rng = np.random.default_rng(C * 11 + K)
    _, wq, ws, bias = _rand_problem(rng, C, K, 1, 1, N, H, W, in_i8=False)
    in_scale = np.float32(100.0)
    x = _fp32_blob_with_ties(rng, (N, C, H, W), in_scale)
    for act in ((3, 0, 2) if int8_out else (1, 2)):
        args = dict(bias=bias, top_scale=9.0, act=act, act_p0=0.1, out_kind=capi.OUT_I8 if int8_out else capi.OUT_F32)
        two, _ = run_conv(hip, oracle, x, wq, ws, in_scale, tile=(-6, 0), **args)
        tiles = [None] if auto else []
        tiles += [(-7, 1), (-7, 2)] + ([(-7, 1 | 1 << 3), (-7, 2 | 2 << 3)] if small else [])
        for tile in tiles:
            out, kind = run_conv(hip, oracle, x, wq, ws, in_scale, tile=tile, **args)
            assert kind == 6, tile
            assert out.tobytes() == two.tobytes(), (act, tile)
        if small:
            want = oracle.conv_layer_forward(x, wq, ws, in_scale, bias=bias, top_scale=9.0, int8_out=int8_out, act_type=act,
                                             act_params=[0.1] if act == 2 else None)
            if int8_out:
                np.testing.assert_array_equal(two, want)
            else:
                assert_f32_close(two, want)


@pytest.mark.parametrize("seed", range(4))
def test_pointwise_from_an_fp32_blob_drawn_shapes(hip, oracle, seed):
    """Eight pointwise layers per seed on fp32 Float8 blobs, drawn over channel counts (8..256 in, 4..520 out), image
    sizes, batch, activation and output kind, through whichever launch the library picks and through both one-launch
    kernels forced (set_tile(-4, 0): the implicit-GEMM loader; set_tile(-7, g): the read-once kernel where it takes the
    shape): bit for bit equal to the two launches, and equal to the oracle's layer."""
    rng = np.random.default_rng(4000 + seed)
    for _ in range(8):
        C = 8 * int(rng.integers(1, 33))
        int8_out = bool(rng.integers(0, 2))
        K = (8 if int8_out else 4) * int(rng.integers(1, 66 if int8_out else 131))
        N, H, W = int(rng.integers(1, 4)), int(rng.integers(1, 20)), int(rng.integers(1, 40))
        act = int(rng.choice([0, 1, 2, 3]))
        _, wq, ws, bias = _rand_problem(rng, C, K, 1, 1, N, H, W, in_i8=False)
        in_scale = np.float32(100.0)
        x = _fp32_blob_with_ties(rng, (N, C, H, W), in_scale)
        what = (C, K, N, H, W, act, int8_out)
        args = dict(bias=bias, top_scale=11.0, act=act, act_p0=0.25, out_kind=capi.OUT_I8 if int8_out else capi.OUT_F32)
        want = oracle.conv_layer_forward(x, wq, ws, in_scale, bias=bias, top_scale=11.0, int8_out=int8_out, act_type=act,
                                         act_params=[0.25])
        two, _ = run_conv(hip, oracle, x, wq, ws, in_scale, tile=(-6, 0), **args)
        if int8_out:
            np.testing.assert_array_equal(two, want, err_msg=str(what))
        else:
            np.testing.assert_allclose(two, want, rtol=FP32_RTOL, atol=1e-30, err_msg=str(what))
        for tile in (None, (-4, 0), (-7, 1), (-7, 2)):
            out, kind = run_conv(hip, oracle, x, wq, ws, in_scale, tile=tile, **args)
            assert out.tobytes() == two.tobytes(), (what, tile, kind)


def test_pointwise_from_an_fp32_blob_read_once_exact_rounding(hip, oracle):
    """The scalar rounding primitive on the input side through conv_pw_f32in_kernel: with a power-of-two input scale a fifth
    of the values land exactly on the one float the two primitives round differently."""
    rng = np.random.default_rng(91)
    C, K, N, H, W = 64, 128, 2, 9, 20
    x, wq, ws, bias = _rand_problem(rng, C, K, 1, 1, N, H, W, in_i8=False)
    x.reshape(-1)[::5] = np.nextafter(np.float32(0.5), np.float32(0)) / np.float32(128.0)
    si = (np.float32(1.0) / (np.float32(128.0) * ws)).astype(np.float32)
    outs = {}
    for mode in (capi.ROUND_SSE, capi.ROUND_EXACT):
        conv = hip.conv(wq=wq, scale_in=si, bias=bias, in_scale=128.0, out_scale=[900.0], act=0, out_kind=capi.OUT_I8, in_round=mode)
        assert conv.kernel_kind(capi.F32_P8, N, H, W, capi.I8_P8) == 6
        xq = oracle.quantize(x, [np.float32(128.0)], mode)
        want = oracle.requantize(oracle.conv_int32(xq, wq, (1, 1), (0, 0), (1, 1), 1), si, [900.0], bias, 0, None, capi.ROUND_SSE)
        got = conv.forward(hip.to_device(capi.pack_np(x, 8)), capi.F32_P8, N, H, W, capi.I8_P8)
        outs[mode] = capi.unpack_np(got.cpu().numpy(), 8, (N, K, H, W))
        np.testing.assert_array_equal(outs[mode], want)
        conv.close()
    assert (outs[capi.ROUND_SSE] != outs[capi.ROUND_EXACT]).any()


@pytest.mark.parametrize("C,K,kind", [(96, 24, 1), (96, 136, 6)])
@pytest.mark.parametrize("mode", [capi.ROUND_SSE, capi.ROUND_EXACT], ids=["sse", "exact"])
def test_pointwise_from_an_fp32_blob_twin_and_shortcut(hip, oracle, mode, C, K, kind):
    """A pointwise layer on an fp32 blob with the shortcut sum and the quantized twin (the implicit-GEMM launch writes both
    from its epilogue, also for a layer whose plain forward takes the read-once kernel), and with either rounding
    primitive on the input side: against the oracle's quantize -> convolution -> dequantize -> add -> quantize."""
    rng = np.random.default_rng(77 + mode)
    N, H, W = 3, 14, 13
    x, wq, ws, bias = _rand_problem(rng, C, K, 1, 1, N, H, W, in_i8=False)
    x.reshape(-1)[::5] = np.nextafter(np.float32(0.5), np.float32(0)) / np.float32(128.0)
    si = (np.float32(1.0) / (np.float32(128.0) * ws)).astype(np.float32)
    conv = hip.conv(wq=wq, scale_in=si, bias=bias, in_scale=128.0, out_scale=None, stride=(1, 1), pad=(0, 0), groups=1,
                    act=0, out_kind=capi.OUT_F32, in_round=mode)
    xq = oracle.quantize(x, [np.float32(128.0)], mode)
    plain_want = oracle.dequantize(oracle.conv_int32(xq, wq, (1, 1), (0, 0), (1, 1), 1), si, bias)
    xd = hip.to_device(capi.pack_np(x, 8))
    assert conv.kernel_kind(capi.F32_P8, N, H, W, capi.F32_P4) == kind
    plain = capi.unpack_np(conv.forward(xd, capi.F32_P8, N, H, W, capi.F32_P4).cpu().numpy(), 4, (N, K, H, W))
    assert_f32_close(plain, plain_want)
    short = (rng.normal(0, 1, plain.shape) * np.abs(plain).mean()).astype(np.float32)
    want = plain + short
    q_scale = 127.0 / float(np.abs(want).max()) * 1.3
    out, q = conv.forward_residual(xd, capi.F32_P8, N, H, W, hip.to_device(capi.pack_np(short, 4)), q_scale, capi.ROUND_SSE,
                                   capi.F32_P4)
    hip.torch.cuda.synchronize()
    got = capi.unpack_np(out.cpu().numpy(), 4, (N, K, H, W))
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    np.testing.assert_array_equal(capi.unpack_np(q.cpu().numpy(), 8, (N, K, H, W)),
                                  oracle.quantize(want, np.float32(q_scale), capi.ROUND_SSE))
    out2, q2 = conv.forward_twin(xd, capi.F32_P8, N, H, W, q_scale, capi.ROUND_EXACT, capi.F32_P4)
    hip.torch.cuda.synchronize()
    got2 = capi.unpack_np(out2.cpu().numpy(), 4, (N, K, H, W))
    np.testing.assert_array_equal(got2.view(np.uint32), plain.view(np.uint32))
    np.testing.assert_array_equal(capi.unpack_np(q2.cpu().numpy(), 8, (N, K, H, W)),
                                  oracle.quantize(plain, np.float32(q_scale), capi.ROUND_EXACT))
    conv.close()


def test_fp32_input_is_quantized_like_the_reference(hip, oracle):
    rng = np.random.default_rng(11)
    for C in (3, 4, 8, 32):
        x, wq, ws, bias = _rand_problem(rng, C, 16, 3, 1, 2, 9, 10, in_i8=False)
        in_scale = np.float32(127) / np.abs(x).max()
        want = oracle.conv_layer_forward(x, wq, ws, in_scale, pad=(1, 1), bias=bias, top_scale=15.0, int8_out=True,
                                         act_type=1)
        out, _ = run_conv(hip, oracle, x, wq, ws, in_scale, pad=1, bias=bias, top_scale=15.0, act=1,
                          out_kind=capi.OUT_I8)
        np.testing.assert_array_equal(out, want)


def test_error_codes(hip):
    wq = np.zeros((8, 8, 3, 3), np.int8)
    conv = hip.conv(wq=wq, scale_in=np.ones(8, np.float32), out_kind=capi.OUT_F32, pad=(1, 1))
    x = hip.to_device(np.zeros(8 * 5 * 5, np.int8))
    with pytest.raises(capi.HipError) as e:
        conv.forward(x, capi.I8_P8, 1, 5, 5, out_layout=capi.I8_P8)  # element type does not match out_kind
    assert e.value.code == -2
    with pytest.raises(capi.HipError) as e:
        conv.forward(x, capi.I32_P4, 1, 5, 5, out_layout=capi.F32_P4)  # int32 input
    assert e.value.code == -2
    with pytest.raises(capi.HipError) as e:
        hip.conv(wq=np.zeros((9, 4, 3, 3), np.int8), scale_in=np.ones(9, np.float32), groups=2)  # K % groups != 0
    assert e.value.code == -2
    with pytest.raises(capi.HipError) as e:
        hip.conv(wq=wq, scale_in=np.ones(8, np.float32), out_kind=capi.OUT_I8)  # int8 output without output scale
    assert e.value.code == -2
