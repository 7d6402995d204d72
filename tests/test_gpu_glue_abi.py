"""The fp32 glue entry points of the C ABI called directly, with every combination of source and destination layout
(elempack 1, 4, 8), against numpy / torch definitions: the host layer only ever uses a few of these combinations."""
import itertools

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from tensor_amd import capi

pytestmark = pytest.mark.gpu

F32 = {1: capi.F32, 4: capi.F32_P4, 8: capi.F32_P8}


def _dev(hip, a, p):
    return hip.to_device(capi.pack_np(a, p))


def _host(t, p, shape):
    return capi.unpack_np(t.cpu().numpy(), p, shape)


@pytest.mark.parametrize("ps,pd", list(itertools.product([1, 4, 8], repeat=2)))
def test_copy_channels_every_layout_pair(hip, ps, pd):
    rng = np.random.default_rng(10 * ps + pd)
    N, Cs, Cd, H, W = 3, 24, 40, 5, 7
    src = rng.normal(0, 1, (N, Cs, H, W)).astype(np.float32)
    base = rng.normal(0, 1, (N, Cd, H, W)).astype(np.float32)
    for s0, d0, cnt in [(0, 0, 24), (8, 16, 16), (4, 8, 8), (3, 5, 7), (0, 39, 1)]:
        dst = _dev(hip, base, pd)
        hip.copy_channels(_dev(hip, src, ps), F32[ps], Cs, s0, dst, F32[pd], Cd, d0, cnt, N, H, W)
        want = base.copy()
        want[:, d0:d0 + cnt] = src[:, s0:s0 + cnt]
        np.testing.assert_array_equal(_host(dst, pd, base.shape), want, err_msg=str((s0, d0, cnt)))


@pytest.mark.parametrize("ps,pd", list(itertools.product([1, 4, 8], repeat=2)))
@pytest.mark.parametrize("groups", [2, 3, 8])
def test_channel_shuffle(hip, ps, pd, groups):
    rng = np.random.default_rng(groups)
    shape = (2, 48, 6, 5)
    x = rng.normal(0, 1, shape).astype(np.float32)
    got = _host(hip.channel_shuffle(_dev(hip, x, ps), F32[ps], shape, groups, F32[pd]), pd, shape)
    want = F.channel_shuffle(torch.from_numpy(x), groups).numpy()
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("ps,pd", [(1, 1), (4, 8), (8, 4), (8, 8), (1, 8)])
@pytest.mark.parametrize("k,s,p,d,ceil", [((3, 3), (2, 2), (1, 1), (1, 1), False), ((2, 2), (2, 2), (0, 0), (1, 1), False),
                                          ((3, 2), (1, 2), (1, 0), (2, 1), False), ((3, 3), (2, 2), (1, 1), (1, 1), True)])
def test_maxpool_both_paddings(hip, ps, pd, k, s, p, d, ceil):
    rng = np.random.default_rng(3)
    shape = (2, 16, 11, 14)
    x = (rng.normal(0, 1, shape) - 1.5).astype(np.float32)  # mostly negative: the padding value shows
    t = torch.from_numpy(x)
    want_inf = F.max_pool2d(t, k, s, p, d, ceil_mode=ceil).numpy()
    oh, ow = want_inf.shape[2:]
    got = _host(hip.maxpool2d(_dev(hip, x, ps), F32[ps], shape, k, s, p, d, (oh, ow), -np.inf, F32[pd]), pd, want_inf.shape)
    np.testing.assert_array_equal(got, want_inf)
    if not ceil and d == (1, 1):
        # zero padding = pooling the explicitly zero-padded blob without padding
        want_zero = F.max_pool2d(F.pad(t, (p[1], p[1], p[0], p[0])), k, s, 0, d).numpy()
        got0 = _host(hip.maxpool2d(_dev(hip, x, ps), F32[ps], shape, k, s, p, d, (oh, ow), 0.0, F32[pd]), pd, want_zero.shape)
        np.testing.assert_array_equal(got0, want_zero)


@pytest.mark.parametrize("ps,pd", [(1, 1), (4, 8), (8, 8)])
def test_upsample_against_torch(hip, ps, pd):
    """Bilinear with half-pixel centres and nearest by floor(d * in/out) are torch's definitions too; bilinear agrees to
    rounding (the reference's operation order is reproduced exactly, torch's differs), nearest exactly."""
    rng = np.random.default_rng(4)
    shape = (2, 8, 5, 7)
    x = rng.normal(0, 1, shape).astype(np.float32)
    t = torch.from_numpy(x)
    for oh, ow in [(10, 14), (15, 21), (7, 9)]:
        got = _host(hip.upsample2d(_dev(hip, x, ps), F32[ps], shape, (oh, ow), 2, False, F32[pd]), pd, (2, 8, oh, ow))
        want = F.interpolate(t, size=(oh, ow), mode="bilinear", align_corners=False).numpy()
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)  # torch weights the taps in another order
        gotn = _host(hip.upsample2d(_dev(hip, x, ps), F32[ps], shape, (oh, ow), 1, False, F32[pd]), pd, (2, 8, oh, ow))
        wantn = F.interpolate(t, size=(oh, ow), mode="nearest").numpy()
        np.testing.assert_array_equal(gotn, wantn)
    got = _host(hip.upsample2d(_dev(hip, x, ps), F32[ps], shape, (10, 14), 2, True, F32[pd]), pd, (2, 8, 10, 14))
    want = F.interpolate(t, size=(10, 14), mode="bilinear", align_corners=True).numpy()
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)  # torch weights the taps in another order


@pytest.mark.parametrize("p", [4, 8])
@pytest.mark.parametrize("mode", [capi.ROUND_SSE, capi.ROUND_EXACT])
def test_eltwise_add_quantize(hip, oracle, p, mode):
    rng = np.random.default_rng(p)
    shape = (3, 24, 7, 9)
    a = rng.normal(0, 1, shape).astype(np.float32)
    b = rng.normal(0, 1, shape).astype(np.float32)
    b.reshape(-1)[:64] = (np.arange(64) - 32 + 0.5) / np.float32(37.5) - a.reshape(-1)[:64]  # sums on rounding ties
    out, q = hip.eltwise_add_quantize(_dev(hip, a, p), _dev(hip, b, p), F32[p], shape, 37.5, mode)
    s = a + b
    np.testing.assert_array_equal(_host(out, p, shape), s)
    want_q = oracle.quantize(s, [37.5], mode)
    np.testing.assert_array_equal(_host(q, 8, shape), want_q)


@pytest.mark.parametrize("ps,pd", list(itertools.product([4, 8], repeat=2)))
@pytest.mark.parametrize("mode", [capi.ROUND_SSE, capi.ROUND_EXACT])
def test_copy_channels_quantize_builds_the_concat_and_its_int8_blob(hip, oracle, ps, pd, mode):
    """A Concat of three blobs (24 + 8 + 16 channels; 4 channels from the middle of a blob at the end when the
    destination packs allow it): the fp32 result equals numpy's, the Byte8 blob the oracle's quantize of it, rounding
    ties included."""
    rng = np.random.default_rng(ps * 10 + pd + mode)
    N, H, W, scale = 2, 5, 7, 37.5
    parts = [rng.normal(0, 1, (N, c, H, W)).astype(np.float32) for c in (24, 8, 16)]
    parts[1].reshape(-1)[:64] = (np.arange(64) - 32 + 0.5) / np.float32(scale)   # exact ties
    ranges = [(0, 24), (0, 8), (4, 8) if pd == 8 else (4, 4)]   # (first source channel, count)
    Cd = sum(r[1] for r in ranges)
    Cd += (-Cd) % 8
    dst = hip.to_device(np.zeros(N * Cd * H * W, np.float32))
    q = hip.to_device(np.zeros(N * Cd * H * W, np.int8))
    want = np.zeros((N, Cd, H, W), np.float32)
    at = 0
    for part, (s0, cnt) in zip(parts, ranges):
        hip.copy_channels_quantize(_dev(hip, part, ps), F32[ps], part.shape[1], s0, dst, F32[pd], Cd, at, cnt, N, H, W, q,
                                   scale, mode)
        want[:, at:at + cnt] = part[:, s0:s0 + cnt]
        at += cnt
    np.testing.assert_array_equal(_host(dst, pd, want.shape), want)
    np.testing.assert_array_equal(_host(q, 8, want.shape), oracle.quantize(want, [scale], mode))


@pytest.mark.parametrize("packs", [(4, 4, 4, 4), (8, 8, 8, 8), (4, 8, 8, 4), (8, 4, 4, 8)], ids=str)
@pytest.mark.parametrize("with_q", [False, True], ids=["plain", "quantized"])
def test_concat_channels_in_one_launch(hip, oracle, packs, with_q):
    """otter_hip_concat_channels: three sources (layouts packs[0..2]) into a destination of layout packs[3], equal to
    numpy's concatenate; with a scale also the oracle's quantize of the result, rounding ties included."""
    rng = np.random.default_rng(sum(p * (i + 1) for i, p in enumerate(packs)))
    N, H, W, scale = 2, 5, 7, 37.5
    parts = [rng.normal(0, 1, (N, c, H, W)).astype(np.float32) for c in (24, 8, 16)]
    parts[1].reshape(-1)[:64] = (np.arange(64) - 32 + 0.5) / np.float32(scale)   # exact ties
    want = np.concatenate(parts, axis=1)
    dst, q = hip.concat_channels([_dev(hip, a, p) for a, p in zip(parts, packs)], [F32[p] for p in packs[:3]],
                                 [a.shape[1] for a in parts], N, H, W, F32[packs[3]], scale if with_q else None, capi.ROUND_SSE)
    np.testing.assert_array_equal(_host(dst, packs[3], want.shape), want)
    if with_q:
        np.testing.assert_array_equal(_host(q, 8, want.shape), oracle.quantize(want, [scale], capi.ROUND_SSE))


@pytest.mark.parametrize("mode", [capi.ROUND_SSE, capi.ROUND_EXACT])
def test_channel_shuffle_quantize(hip, oracle, mode):
    rng = np.random.default_rng(5 + mode)
    shape, scale = (3, 48, 6, 7), 29.5
    x = rng.normal(0, 1, shape).astype(np.float32)
    x.reshape(-1)[:64] = (np.arange(64) - 32 + 0.5) / np.float32(scale)   # exact ties
    dst, q = hip.channel_shuffle_quantize(_dev(hip, x, 8), shape, 2, scale, mode)
    want = x.reshape(3, 2, 24, 6, 7).transpose(0, 2, 1, 3, 4).reshape(shape)
    np.testing.assert_array_equal(_host(dst, 8, shape), want)
    np.testing.assert_array_equal(_host(q, 8, shape), oracle.quantize(want, [scale], mode))
    with pytest.raises(capi.HipError):
        hip.channel_shuffle_quantize(_dev(hip, x, 8), shape, 3, scale, mode)      # the two-group kernel only


def test_shuffle2_split_is_concat_shuffle_and_two_crops(hip):
    rng = np.random.default_rng(9)
    N, Ch, H, W = 3, 24, 5, 9
    a = rng.normal(0, 1, (N, Ch, H, W)).astype(np.float32)
    b = rng.normal(0, 1, (N, Ch, H, W)).astype(np.float32)
    c1, c2 = hip.shuffle2_split(_dev(hip, a, 8), _dev(hip, b, 8), N, Ch, H, W)
    s = F.channel_shuffle(torch.from_numpy(np.concatenate([a, b], 1)), 2).numpy()
    np.testing.assert_array_equal(_host(c1, 8, a.shape), s[:, :Ch])
    np.testing.assert_array_equal(_host(c2, 8, a.shape), s[:, Ch:])
    c1, c2, q2 = hip.shuffle2_split(_dev(hip, a, 8), _dev(hip, b, 8), N, Ch, H, W, scale=41.0, round_mode=capi.ROUND_SSE)
    np.testing.assert_array_equal(_host(c2, 8, a.shape), s[:, Ch:])
    t = s[:, Ch:] * np.float32(41.0)
    np.testing.assert_array_equal(_host(q2, 8, a.shape), np.clip(np.trunc(t + np.copysign(np.float32(0.5), t)), -127, 127))
    c1, c2 = hip.shuffle2_split(_dev(hip, a, 4), _dev(hip, b, 8), N, Ch, H, W, a_layout=capi.F32_P4)
    np.testing.assert_array_equal(_host(c1, 8, a.shape), s[:, :Ch])
    np.testing.assert_array_equal(_host(c2, 8, a.shape), s[:, Ch:])
    with pytest.raises(capi.HipError):
        hip.shuffle2_split(_dev(hip, a[:, :12], 4), _dev(hip, b[:, :12], 4), N, 12, H, W)


def test_glue_argument_errors(hip):
    x = hip.to_device(np.zeros(8 * 16, np.float32))
    with pytest.raises(capi.HipError):
        hip.copy_channels(x, capi.F32, 8, 4, x, capi.F32, 8, 0, 8, 1, 4, 4)          # range beyond the source
    with pytest.raises(capi.HipError):
        hip.channel_shuffle(x, capi.F32, (1, 8, 4, 4), 3, capi.F32)                  # groups do not divide C
    with pytest.raises(capi.HipError):
        hip.upsample2d(x, capi.F32, (1, 8, 4, 4), (8, 8), 3, False, capi.F32)        # bicubic is not supported
    with pytest.raises(capi.HipError):
        hip.maxpool2d(x, capi.F32, (1, 8, 4, 4), (3, 3), (2, 2), (1, 1), (1, 1), (9, 9), 0.0, capi.F32)  # output too large
    with pytest.raises(capi.HipError):
        hip.eltwise_add_quantize(x, x, capi.F32, (1, 8, 4, 4), 1.0, capi.ROUND_SSE)  # unpacked blobs
    q = hip.to_device(np.zeros(8 * 16, np.int8))
    with pytest.raises(capi.HipError):
        hip.copy_channels_quantize(x, capi.F32, 8, 0, x, capi.F32_P8, 8, 0, 8, 1, 4, 4, q, 1.0, capi.ROUND_SSE)   # unpacked source
    with pytest.raises(capi.HipError):
        hip.copy_channels_quantize(x, capi.F32_P4, 8, 0, x, capi.F32_P4, 12, 0, 8, 1, 2, 2, q, 1.0, capi.ROUND_SSE)  # dst_c % 8
    with pytest.raises(capi.HipError):
        hip.concat_channels([x, x], [capi.F32, capi.F32_P4], [4, 4], 1, 2, 2, capi.F32_P4)   # an unpacked source
    with pytest.raises(capi.HipError):
        hip.concat_channels([x] * 9, [capi.F32_P4] * 9, [4] * 9, 1, 1, 1, capi.F32_P4)       # more than 8 sources


@pytest.mark.parametrize("N,IN,OUT,bias", [(64, 1280, 1000, True), (17, 64, 5, True), (100, 96, 33, False),
                                           (16, 1280, 1000, True), (3, 1280, 10, True), (40, 72, 16, True)])
def test_inner_product_against_float64(hip, N, IN, OUT, bias):
    """Both kernels behind otter_hip_inner_product (the matrix-core one takes IN % 16 == 0 from 64 inputs on, the vector
    one the rest): y = x w^T + b against a float64 product, to fp32 summation accuracy. The weight is not symmetric and
    x has a distinct row per image, so a transposed operand or a misplaced row fails. A row's result does not depend
    on the batch it sits in."""
    rng = np.random.default_rng(N + IN)
    x = rng.normal(0, 1, (N, IN)).astype(np.float32)
    w = rng.normal(0, 0.05, (OUT, IN)).astype(np.float32)
    b = rng.normal(0, 1, OUT).astype(np.float32) if bias else None
    y = hip.inner_product(hip.to_device(x), N, IN, hip.to_device(w), hip.to_device(b) if bias else None, OUT)
    want = x.astype(np.float64) @ w.astype(np.float64).T + (b.astype(np.float64) if bias else 0.0)
    got = y.cpu().numpy().reshape(N, OUT)
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)
    alone = hip.inner_product(hip.to_device(x[N - 1:]), 1, IN, hip.to_device(w), hip.to_device(b) if bias else None, OUT)
    np.testing.assert_array_equal(alone.cpu().numpy().reshape(1, OUT), got[N - 1:])
