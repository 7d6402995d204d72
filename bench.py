#!/usr/bin/env python3
"""Benchmark of the int8 convolution path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3|c1s1|c1s2|c1s1i8|c1s2i8|c1s1valu|c1s2valu|c2|c2i8|c0|c0n64|c4|det|blk14|blk112s2|dil2|grp8|s2|odd55|w224|copy]
                    [--no-cpu] [--no-also]

Prints ONE JSON line. The headline workload is the fourth benchmark configuration (the MFMA-bound case the metric's
"int8 conv TOPS (% MFMA peak)" is quoted on): four chained int8-in/int8-out 3x3 convolutions 128->128 at
56x56, batch 64, fused requantize+ReLU. One step = the four layers back to back on device-resident int8
activations. The other single-GPU configurations (depthwise c1 at stride 1 and 2 with its HBM roofline, the
1x1 GEMM c2 and its int8-output variant, the single-image c0 and the same layer at batch 64, the MobileNetV2-style
network c4, the reference's detection model file, two inverted-residual blocks and five single layers outside the tuned
shapes) are measured the same way and reported under "also", followed by a plain device-to-device copy of 256 MiB ("copy": what a copy reaches on
the box the line was measured on). A bandwidth-bound kernel's roofline figure comes from a loop that rotates over enough
buffer sets to exceed the 256 MB last-level cache; the figure of the loop over one (cache-resident) set is reported
beside it as "roofline_resident".

Timing: HIP events recorded on the stream the kernels are launched on (torch's current stream is handed to the
C ABI as the launch stream), inputs resident in HBM before the timed region. Every timed loop is preceded by an
untimed run-in of SETTLE_S seconds of the same step (the shader clock needs tens of milliseconds of load to reach its
steady state), then the W warm-up steps, then exactly K timed steps.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0  # MI355X dense int8 MFMA, TOP/s
PEAK_HBM_GBS = 8000.0    # MI355X HBM3E, GB/s


def quantize_weights(wf):
    K = wf.shape[0]
    ws = (np.float32(127) / np.abs(wf).reshape(K, -1).max(axis=1)).astype(np.float32)
    wq = np.clip(np.round(wf * ws[:, None, None, None]), -127, 127).astype(np.int8)
    return wq, ws


def host_scale_in(ws, in_scale):
    return (np.float32(1.0) / (np.float32(in_scale) * ws)).astype(np.float32)


SETTLE_S = 0.15  # untimed run-in before the warm-up steps, seconds of the workload's own step


class Timer:
    def __init__(self, torch, hip=None):
        self.torch = torch
        self.hip = hip  # the library binding, for the clock measurement behind a matrix-bound loop

    def run(self, fn, steps, warmup, settle=None):
        """fn: a closure, or a list of closures taken in turn (the same launch over different buffer sets, so that the
        loop's footprint exceeds the caches)."""
        t = self.torch
        if isinstance(fn, (list, tuple)):
            fns, state = list(fn), [0]

            def fn():
                fns[state[0] % len(fns)]()
                state[0] += 1
        settle = SETTLE_S if settle is None else settle
        # The shader clock ramps up over the first tens of milliseconds of load (measured: the same 4-layer step
        # takes 135 us in its first 100 iterations after an idle period and 120 us from then on), so the step runs
        # untimed for SETTLE_S first; the W warm-up steps and the K timed steps follow as the contract has them.
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < settle:
            for _ in range(10):
                fn()
            t.cuda.synchronize()
        for _ in range(warmup):
            fn()
        t.cuda.synchronize()
        e0, e1 = t.cuda.Event(enable_timing=True), t.cuda.Event(enable_timing=True)
        wall0 = time.perf_counter()
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        t.cuda.synchronize()
        wall = (time.perf_counter() - wall0) * 1e3 / steps
        return e0.elapsed_time(e1) / steps, wall


# ------------------------------------------------------------------------------------------------------
# workloads
# ------------------------------------------------------------------------------------------------------

COLD_BYTES = 320 << 20  # footprint of a rotating loop: above the 256 MB of the last-level (Infinity) cache


def cold_sets(bytes_per_set):
    return max(2, -(-COLD_BYTES // bytes_per_set))


def build_c3(hip, capi, rng):
    """configs[3]: 4 x (128->128 3x3 s1 p1) at 56x56, batch 64, int8 in / int8 out, requantize+ReLU. The output
    scale of each layer is 127/max(activation) on a seeded calibration batch of 16, computed with the fp32-output
    variant of the same GPU layer; the next layer's input scale is that output scale."""
    torch = hip.torch
    N, C, H, W, L = 64, 128, 56, 56, 4
    x = rng.integers(-127, 128, size=(N, C, H, W), dtype=np.int8)
    xc = rng.integers(-127, 128, size=(16, C, H, W), dtype=np.int8)
    xd = hip.to_device(capi.pack_np(x, 8))
    cal = hip.to_device(capi.pack_np(xc, 8))
    in_scale = np.float32(127.0)
    layers, params = [], []
    for l in range(L):
        wq, ws = quantize_weights(rng.normal(0, 0.04, (C, C, 3, 3)).astype(np.float32))
        bias = rng.normal(0, 0.01, C).astype(np.float32)
        si = host_scale_in(ws, in_scale)
        probe = hip.conv(wq=wq, scale_in=si, bias=bias, pad=(1, 1), act=1, out_kind=capi.OUT_F32)
        amax = float(probe.forward(cal, capi.I8_P8, 16, H, W).abs().max().item())
        probe.close()
        out_scale = np.float32(127.0) / np.float32(amax)
        conv = hip.conv(wq=wq, scale_in=si, bias=bias, out_scale=[out_scale], pad=(1, 1), act=1,
                        out_kind=capi.OUT_I8, out_round=capi.ROUND_SSE)
        cal = conv.forward(cal, capi.I8_P8, 16, H, W)
        layers.append(conv)
        params.append(dict(wq=wq, ws=ws, bias=bias, in_scale=float(in_scale), out_scale=float(out_scale)))
        in_scale = out_scale
    bufs = [hip.empty(N * C * H * W, np.int8) for _ in range(2)]

    def step_layers():
        src = xd
        for l, conv in enumerate(layers):
            dst = bufs[l & 1]
            conv.forward(src, capi.I8_P8, N, H, W, capi.I8_P8, out=dst)
            src = dst
        return src

    # the chain through the entry point that takes consecutive layers at once (one persistent launch for this chain)
    chain_ws = hip.empty(3 * N * C * H * W + 1024, np.int8)
    chain_out = hip.empty(N * C * H * W, np.int8)

    def step():
        return hip.conv_chain(layers, xd, N, H, W, out=chain_out, workspace=chain_ws)

    ops_layer = 2.0 * N * C * C * 9 * H * W
    launches = hip.conv_chain_launches(layers, N, H, W)
    layer_fn = lambda: layers[1].forward(bufs[0], capi.I8_P8, N, H, W, capi.I8_P8, out=bufs[1])  # noqa: E731
    # the dominant kernel is the chain's one launch (all four layers' operations); when the library runs the chain
    # layer by layer it is one layer's launch
    one = launches == 1
    return dict(name="c3", step=step, step_layers=step_layers, layer_fn=layer_fn, layers=layers, ops=L * ops_layer, launches=launches,
                dom_ops=L * ops_layer if one else ops_layer,
                dom_bytes=2 * N * C * H * W + C * C * 9, bound="mfma",
                workload="4 x int8 3x3 conv 128->128 s1 p1 @56x56, batch 64, int8 in/out, requantize+ReLU",
                dom_kernel="conv3x3_chain_kernel (the 4 layers in one persistent launch)" if one
                else "conv 3x3 128->128 (MFMA implicit GEMM)",
                dom_fn=step if one else layer_fn, layer_ops=ops_layer,
                x=x, params=params, shape=(N, C, H, W))


def build_c1(hip, capi, rng, stride, variant=""):
    """configs[1]: depthwise 3x3 p1 on 8x256x112x112 fp32, bias, ReLU6, requantize to int8 with 127/6. The step is the
    configuration as stated: the layer on the fp32 Float8 blob, ONE launch that quantizes on the way in
    (conv_dw3x3_f32in_kernel). The layer on an int8 blob (what a depthwise layer inside a network sees) and the
    standalone quantize pass are timed beside it. variant "i8": the step is the layer on the int8 blob (matrix-core
    kernel); "valu": the same on the vector-ALU kernels (v_dot4_i32_i8), kept for comparison."""
    N, C, H, W = 8, 256, 112, 112
    x = rng.uniform(-1, 1, (N, C, H, W)).astype(np.float32)
    wq, ws = quantize_weights(rng.normal(0, 0.1, (C, 1, 3, 3)).astype(np.float32))
    bias = rng.normal(0, 0.01, C).astype(np.float32)
    in_scale = np.float32(127) / np.abs(x).max()
    out_scale = np.float32(127.0 / 6.0)
    conv = hip.conv(wq=wq, scale_in=host_scale_in(ws, in_scale), bias=bias, in_scale=float(in_scale),
                    out_scale=[out_scale], stride=(stride, stride), pad=(1, 1), groups=C, act=3,
                    out_kind=capi.OUT_I8)
    xd = hip.to_device(capi.pack_np(x, 8))          # Float8, what Net::convert_layout hands the layer
    oh, ow = conv.out_hw(H, W)
    xq = hip.empty(N * C * H * W, np.int8)
    out = hip.empty(N * C * oh * ow, np.int8)
    scale_dev = hip.to_device(np.array([in_scale], np.float32))

    def step():
        conv.forward(xd, capi.F32_P8, N, H, W, capi.I8_P8, out=out, workspace=xq)
        return out

    in_b, out_b = N * C * H * W, N * C * oh * ow
    # the same launches over enough buffer sets that nothing a launch reads is still in a cache from the last time
    hip.quantize(xd, capi.F32_P8, (N, C, H, W), scale_dev, capi.ROUND_SSE, capi.I8_P8, dst=xq)
    n_dom = cold_sets(4 * in_b + out_b)
    xds, outs = [xd.clone() for _ in range(n_dom)], [hip.empty(out_b, np.int8) for _ in range(n_dom)]
    dom_cold = [lambda i=i: conv.forward(xds[i], capi.F32_P8, N, H, W, capi.I8_P8, out=outs[i], workspace=xq) for i in range(n_dom)]
    n_i8 = cold_sets(in_b + out_b)
    xqs, outs8 = [xq.clone() for _ in range(n_i8)], [hip.empty(out_b, np.int8) for _ in range(n_i8)]
    i8_cold = [lambda i=i: conv.forward(xqs[i], capi.I8_P8, N, H, W, capi.I8_P8, out=outs8[i]) for i in range(n_i8)]
    xq2 = [hip.empty(in_b, np.int8) for _ in range(n_dom)]
    q_cold = [lambda i=i: hip.quantize(xds[i], capi.F32_P8, (N, C, H, W), scale_dev, capi.ROUND_SSE, capi.I8_P8, dst=xq2[i])
              for i in range(n_dom)]
    if variant:
        if variant == "valu":
            conv.set_tile(-3, 0)
        fn = lambda: conv.forward(xq, capi.I8_P8, N, H, W, capi.I8_P8, out=out)  # noqa: E731
        kern = "conv_dw3x3_mfma_kernel (matrix cores)" if variant == "i8" else "conv_dw3x3_i8_kernel (vector ALU, v_dot4_i32_i8)"
        return dict(name="c1s%d%s" % (stride, variant), step=fn, dom_fn_cold=i8_cold, ops=2.0 * N * C * 9 * oh * ow, launches=1,
                    bytes=in_b + out_b, dom_ops=2.0 * N * C * 9 * oh * ow, dom_bytes=in_b + out_b, bound="hbm",
                    workload="depthwise int8 3x3 s%d p1 on an int8 Byte8 blob 8x256x112x112 -> conv + bias + ReLU6 + "
                             "requantize -> int8" % stride,
                    dom_kernel=kern + ": depthwise 3x3 s%d + requantize (int8 in -> int8 out)" % stride, dom_fn=fn,
                    x=x, params=[dict(wq=wq, ws=ws, bias=bias, in_scale=float(in_scale), out_scale=float(out_scale))],
                    shape=(N, C, H, W), stride=stride, int8_in=True)
    return dict(name="c1s%d" % stride, step=step, dom_fn_cold=dom_cold, ops=2.0 * N * C * 9 * oh * ow, launches=1,
                bytes=4 * in_b + out_b, dom_ops=2.0 * N * C * 9 * oh * ow, dom_bytes=4 * in_b + out_b, bound="hbm",
                workload="depthwise int8 3x3 s%d p1, 8x256x112x112 fp32 in -> quantize + conv + bias + ReLU6 + requantize "
                         "-> int8, one launch" % stride,
                dom_kernel="conv_dw3x3_f32in_kernel: quantize + depthwise 3x3 s%d + requantize (fp32 Float8 in -> int8 "
                           "out)" % stride,
                dom_fn=step,
                aux=[dict(kernel="conv_dw3x3_mfma_kernel: the same layer on an int8 Byte8 blob (int8 in -> int8 out)",
                          bytes=in_b + out_b, fn_cold=i8_cold,
                          fn=lambda: conv.forward(xq, capi.I8_P8, N, H, W, capi.I8_P8, out=out)),
                     dict(kernel="quantize fp32 Float8 -> Byte8 as a pass of its own", bytes=5 * in_b, fn_cold=q_cold,
                          fn=lambda: hip.quantize(xd, capi.F32_P8, (N, C, H, W), scale_dev, capi.ROUND_SSE, capi.I8_P8,
                                                  dst=xq))],
                x=x, params=[dict(wq=wq, ws=ws, bias=bias, in_scale=float(in_scale), out_scale=float(out_scale))],
                shape=(N, C, H, W), stride=stride)


def build_c2(hip, capi, rng, int8_out=False):
    """configs[2]: 1x1 conv 256->512 on 32x256x28x28 (GEMM M=512, N=25088, K=256), bias, dequantize+ReLU, fp32. The step
    is the configuration as stated: the layer on the fp32 Float8 blob, ONE launch that quantizes on the way in and reads
    the blob once (conv_pw_f32in_kernel). The layer on an int8 blob (what a pointwise layer inside a network sees) and the standalone quantize
    pass are timed beside it.
    int8_out: the same layer requantizing to int8 (a fixed output scale), which takes the fp32 result off the bus."""
    N, C, K, H, W = 32, 256, 512, 28, 28
    x = rng.uniform(0, 1, (N, C, H, W)).astype(np.float32)
    wq, ws = quantize_weights(rng.normal(0, 0.03, (K, C, 1, 1)).astype(np.float32))
    bias = rng.normal(0, 0.01, K).astype(np.float32)
    in_scale = np.float32(127) / np.abs(x).max()
    out_scale = np.float32(20.0)
    if int8_out:
        conv = hip.conv(wq=wq, scale_in=host_scale_in(ws, in_scale), bias=bias, in_scale=float(in_scale), act=1,
                        out_scale=[out_scale], out_kind=capi.OUT_I8, out_round=capi.ROUND_SSE)
    else:
        conv = hip.conv(wq=wq, scale_in=host_scale_in(ws, in_scale), bias=bias, in_scale=float(in_scale), act=1,
                        out_kind=capi.OUT_F32)
    out_layout, out_dt, out_esz = (capi.I8_P8, np.int8, 1) if int8_out else (capi.F32_P4, np.float32, 4)
    xd = hip.to_device(capi.pack_np(x, 8))
    xq = hip.empty(N * C * H * W, np.int8)
    out = hip.empty(N * K * H * W, out_dt)
    scale_dev = hip.to_device(np.array([in_scale], np.float32))

    def step():
        conv.forward(xd, capi.F32_P8, N, H, W, out_layout, out=out, workspace=xq)
        return out

    step()
    hip.quantize(xd, capi.F32_P8, (N, C, H, W), scale_dev, capi.ROUND_SSE, capi.I8_P8, dst=xq)
    in_b, out_b = N * C * H * W, out_esz * N * K * H * W
    dom_bytes = 4 * in_b + K * C + out_b
    n_dom = cold_sets(dom_bytes)
    xds, outs = [xd.clone() for _ in range(n_dom)], [hip.empty(N * K * H * W, out_dt) for _ in range(n_dom)]
    dom_cold = [lambda i=i: conv.forward(xds[i], capi.F32_P8, N, H, W, out_layout, out=outs[i], workspace=xq) for i in range(n_dom)]
    n_i8 = cold_sets(in_b + K * C + out_b)
    xqs, outs8 = [xq.clone() for _ in range(n_i8)], [hip.empty(N * K * H * W, out_dt) for _ in range(n_i8)]
    i8_cold = [lambda i=i: conv.forward(xqs[i], capi.I8_P8, N, H, W, out_layout, out=outs8[i]) for i in range(n_i8)]
    xq2 = [hip.empty(in_b, np.int8) for _ in range(n_dom)]
    q_cold = [lambda i=i: hip.quantize(xds[i], capi.F32_P8, (N, C, H, W), scale_dev, capi.ROUND_SSE, capi.I8_P8, dst=xq2[i])
              for i in range(n_dom)]
    ops = 2.0 * N * K * C * H * W
    tail = "requantize + ReLU -> int8" if int8_out else "dequantize + ReLU -> fp32"
    i8_kernel = "conv_pw_stream_kernel" if conv.kernel_kind(capi.I8_P8, N, H, W, out_layout) == 5 else "conv_igemm_kernel"
    return dict(name="c2i8" if int8_out else "c2", step=step, ops=ops, launches=1, dom_ops=ops, dom_fn_cold=dom_cold,
                dom_bytes=dom_bytes, bound="hbm",
                workload="int8 1x1 conv 256->512 @28x28 batch 32 (GEMM 512x25088x256), fp32 in -> quantize + conv + bias + "
                         + tail + ", one launch",
                dom_kernel="%s: quantize + conv 1x1 256->512 (fp32 Float8 in -> %s out)"
                           % ("conv_pw_f32in_kernel" if conv.kernel_kind(capi.F32_P8, N, H, W, out_layout) == 6
                              else "conv_igemm_kernel, fp32-input loader", "int8" if int8_out else "fp32"),
                dom_fn=step,
                aux=[dict(kernel=i8_kernel + ": the same layer on an int8 Byte8 blob", bytes=in_b + K * C + out_b,
                          fn_cold=i8_cold, fn=lambda: conv.forward(xq, capi.I8_P8, N, H, W, out_layout, out=out)),
                     dict(kernel="quantize fp32 Float8 -> Byte8 as a pass of its own", bytes=5 * in_b, fn_cold=q_cold,
                          fn=lambda: hip.quantize(xd, capi.F32_P8, (N, C, H, W), scale_dev, capi.ROUND_SSE, capi.I8_P8,
                                                  dst=xq))],
                x=x, params=[dict(wq=wq, ws=ws, bias=bias, in_scale=float(in_scale), out_scale=float(out_scale))],
                shape=(N, C, H, W), int8_out=int8_out)


def build_c0(hip, capi, rng, batch=1):
    """configs[0]: one 3x3 s1 p1 conv 64->64 on 1x64x56x56 fp32, no bias, dequantize to fp32 (batch 64: the same layer
    with enough work to fill the chip)."""
    N, C, K, H, W = batch, 64, 64, 56, 56
    x = rng.uniform(-1, 1, (N, C, H, W)).astype(np.float32)
    wq, ws = quantize_weights(rng.normal(0, 0.05, (K, C, 3, 3)).astype(np.float32))
    in_scale = np.float32(127) / np.abs(x).max()
    conv = hip.conv(wq=wq, scale_in=host_scale_in(ws, in_scale), in_scale=float(in_scale), pad=(1, 1),
                    out_kind=capi.OUT_F32)
    xd = hip.to_device(capi.pack_np(x, 8))
    ws_buf = hip.empty(N * C * H * W, np.int8)
    out = hip.empty(N * K * H * W, np.float32)

    def step():
        conv.forward(xd, capi.F32_P8, N, H, W, capi.F32_P4, out=out, workspace=ws_buf)
        return out

    ops = 2.0 * N * K * C * 9 * H * W
    if batch > 1:
        # the convolution alone on the quantized blob; 64 fp32 bytes out per int8 pixel in: bound by the writes
        step()
        xq = hip.empty(N * C * H * W, np.int8)
        scale_dev = hip.to_device(np.array([in_scale], np.float32))
        hip.quantize(xd, capi.F32_P8, (N, C, H, W), scale_dev, capi.ROUND_SSE, capi.I8_P8, dst=xq)
        dom_bytes = N * C * H * W + K * C * 9 + 4 * N * K * H * W
        n_dom = cold_sets(dom_bytes)
        xqs, outs = [xq.clone() for _ in range(n_dom)], [hip.empty(N * K * H * W, np.float32) for _ in range(n_dom)]
        return dict(name="c0n%d" % batch, step=step, ops=ops, launches=2, dom_ops=ops, dom_bytes=dom_bytes, bound="hbm",
                    workload="int8 3x3 conv 64->64 s1 p1, %dx64x56x56 fp32 in -> quantize -> conv -> fp32 out" % batch,
                    dom_kernel="conv 3x3 64->64 (MFMA, LDS halo, fp32 out)",
                    dom_fn=lambda: conv.forward(xq, capi.I8_P8, N, H, W, capi.F32_P4, out=out),
                    dom_fn_cold=[lambda i=i: conv.forward(xqs[i], capi.I8_P8, N, H, W, capi.F32_P4, out=outs[i])
                                 for i in range(n_dom)],
                    x=x, params=[dict(wq=wq, ws=ws, bias=None, in_scale=float(in_scale))], shape=(N, C, H, W))
    return dict(name="c0", step=step, ops=ops, launches=2, dom_ops=ops,
                dom_bytes=N * C * H * W + K * C * 9 + 4 * N * K * H * W, bound="mfma",
                workload="single int8 3x3 conv 64->64 s1 p1, 1x64x56x56 fp32 in -> fp32 out (latency-bound)",
                dom_kernel="conv 3x3 64->64 (MFMA, %s, fp32 out)" % (
                    "LDS halo" if conv.kernel_kind(capi.I8_P8, N, H, W, capi.F32_P4) == 3 else "implicit GEMM"),
                dom_fn=None, x=x, params=[dict(wq=wq, ws=ws, bias=None, in_scale=float(in_scale))],
                shape=(N, C, H, W))


LAYER_SHAPES = {
    # name: (C, K, kernel, stride, pad, dilation, groups, N, H, W, what)
    "dil2": (128, 128, 3, 1, 2, 2, 1, 64, 56, 56, "dilated (2) 3x3 128->128"),
    "grp8": (256, 256, 3, 1, 1, 1, 8, 64, 28, 28, "grouped (8 groups of 32->32) 3x3 256->256"),
    "s2": (128, 128, 3, 2, 1, 1, 1, 64, 56, 56, "3x3 stride 2 128->128"),
    "odd55": (128, 128, 3, 1, 1, 1, 1, 64, 55, 55, "3x3 128->128 on an odd image width"),
    "w224": (64, 64, 3, 1, 1, 1, 1, 8, 224, 224, "3x3 64->64 on 224-pixel rows"),
}


def build_layer(hip, capi, rng, name):
    """One int8-in / int8-out convolution layer (bias, ReLU, requantize) of a shape outside the tuned benchmark
    configurations: the variants of the path (dilation, groups, stride 2, odd widths)."""
    C, K, k, s, p, d, g, N, H, W, what = LAYER_SHAPES[name]
    x = rng.integers(-127, 128, size=(N, C, H, W), dtype=np.int8)
    wq, ws = quantize_weights(rng.normal(0, 0.04, (K, C // g, k, k)).astype(np.float32))
    bias = rng.normal(0, 0.01, K).astype(np.float32)
    conv = hip.conv(wq=wq, scale_in=host_scale_in(ws, np.float32(127.0)), bias=bias, out_scale=[np.float32(40.0)],
                    stride=(s, s), pad=(p, p), dil=(d, d), groups=g, act=1, out_kind=capi.OUT_I8, out_round=capi.ROUND_SSE)
    xd = hip.to_device(capi.pack_np(x, 8))
    oh, ow = conv.out_hw(H, W)
    out = hip.empty(N * K * oh * ow, np.int8)

    def step():
        conv.forward(xd, capi.I8_P8, N, H, W, capi.I8_P8, out=out)
        return out

    ops = 2.0 * N * K * (C // g) * k * k * oh * ow
    nbytes = N * C * H * W + N * K * oh * ow + K * (C // g) * k * k
    kind = conv.kernel_kind(capi.I8_P8, N, H, W, capi.I8_P8)
    bound = "mfma" if ops / nbytes > PEAK_INT8_TOPS * 1e12 / (PEAK_HBM_GBS * 1e9) else "hbm"
    return dict(name=name, step=step, ops=ops, launches=1, dom_ops=ops, dom_bytes=nbytes, bound=bound,
                workload="int8 %s s%d p%d @%dx%d, batch %d, int8 in/out, requantize+ReLU (kernel family %d)"
                         % (what, s, p, H, W, N, kind),
                dom_kernel="the layer's one launch", dom_fn=None, x=x,
                params=[dict(wq=wq, ws=ws, bias=bias, in_scale=127.0, out_scale=40.0)], shape=(N, C, H, W),
                layer=(C, K, k, s, p, d, g))


def build_block(hip, capi, rng, N=64, cin=64, ce=384, cout=64, hw=14, stride=1, name="blk14"):
    """One inverted-residual block of the MobileNetV2-style network (1x1 expand, depthwise 3x3, 1x1 project, shortcut sum
    where the shapes allow one, int8 twin of the result): a step is otter_hip_conv_block_forward (blk14, 14x14 stride 1:
    one launch; blk112s2, 112x112 with a stride-2 depthwise layer: one launch for the first two layers, one for the
    last); the same block as three launches (forward, forward, forward_residual / _twin) is timed beside it."""
    layers = []
    in_scale = np.float32(40.0)
    for (ci, co, k, pad, groups, act, i8) in [(cin, ce, 1, 0, 1, 3, True), (ce, ce, 3, 1, ce, 3, True), (ce, cout, 1, 0, 1, 0, False)]:
        wq, ws = quantize_weights(rng.normal(0, 0.3 if groups > 1 else 2.0 / np.sqrt(ci), (co, ci // groups, k, k)).astype(np.float32))
        bias = rng.normal(0, 0.05, co).astype(np.float32)
        out_scale = np.float32(25.0)
        conv = hip.conv(wq=wq, scale_in=host_scale_in(ws, in_scale), bias=bias, in_scale=float(in_scale),
                        out_scale=[out_scale] if i8 else None, stride=(stride, stride) if groups > 1 else (1, 1), pad=(pad, pad),
                        groups=groups, act=act, out_kind=capi.OUT_I8 if i8 else capi.OUT_F32, out_round=capi.ROUND_SSE)
        layers.append(dict(conv=conv, wq=wq, ws=ws, bias=bias, in_scale=float(in_scale), out_scale=float(out_scale), k=k,
                           pad=pad, groups=groups, act=act, int8_out=i8, stride=stride if groups > 1 else 1))
        in_scale = out_scale
    e, d, p = (l["conv"] for l in layers)
    x = rng.integers(-127, 128, size=(N, cin, hw, hw), dtype=np.int8)
    xd = hip.to_device(capi.pack_np(x, 8))
    oh, _ = d.out_hw(hw, hw)
    with_res = stride == 1 and cin == cout
    res = hip.to_device(capi.pack_np(rng.normal(0, 1, (N, cout, oh, oh)).astype(np.float32), 4)) if with_res else None
    out = hip.empty(N * cout * oh * oh, np.float32)
    q = hip.empty(N * cout * oh * oh, np.int8)
    t0 = hip.empty(N * ce * hw * hw, np.int8)
    t1 = hip.empty(N * ce * oh * oh, np.int8)
    ws_bytes = hip.lib.otter_hip_conv_block_workspace_bytes(e.h, d.h, p.h, N, hw, hw)
    ws = hip.empty(ws_bytes, np.int8) if ws_bytes else None
    launches = hip.conv_block_launches(e, d, p, N, hw, hw)

    def step():
        return hip.conv_block(e, d, p, xd, N, hw, hw, residual=res, q_scale=20.0, out=out, q=q, workspace=ws)[0]

    def three():
        e.forward(xd, capi.I8_P8, N, hw, hw, capi.I8_P8, out=t0)
        d.forward(t0, capi.I8_P8, N, hw, hw, capi.I8_P8, out=t1)
        if with_res:
            return p.forward_residual(t1, capi.I8_P8, N, oh, oh, res, q_scale=20.0)[0]
        return p.forward_twin(t1, capi.I8_P8, N, oh, oh, 20.0, capi.ROUND_SSE)[0]

    px, opx = N * hw * hw, N * oh * oh
    ops = 2.0 * (px * cin * ce + opx * (9 * ce + ce * cout))
    # in, (shortcut,) out, twin, weights: what the block must move; the blobs between its layers are not in it
    nbytes = px * cin + opx * ((4 * cout if with_res else 0) + 4 * cout + cout) + cin * ce + 9 * ce + ce * cout
    how = {1: "one launch", 2: "one launch for the first two layers, one for the last", 3: "three launches"}[launches]
    return dict(name=name, step=step, ops=ops, launches=launches, dom_ops=ops, dom_bytes=nbytes, bound="hbm",
                workload="inverted-residual block %d->%d->%d (1x1 ReLU6, depthwise 3x3 stride %d ReLU6, 1x1 linear%s, + int8 "
                         "twin) @%dx%d, batch %d, through otter_hip_conv_block_forward (%s)"
                         % (cin, ce, cout, stride, ", + shortcut" if with_res else "", hw, hw, N, how),
                dom_kernel="conv_block_kernel (the block's one launch)" if launches == 1 else
                           "conv_xdw_kernel (pointwise + depthwise layer) and the last layer's launch",
                dom_fn=None, x=x, step_layers=three, params=layers, shape=(N, cin, hw, hw), _keep=(xd, res, out, q, t0, t1, ws))


def build_det(hip, capi, rng, batch=16):
    """The reference's own int8 detection model description (benchmark/nanodet-plus-m-1.5x_416_int8_fused.otter, a data
    file kept under tests/golden) read by Net::load_otter, with synthetic int8 weights written as an ncnn .bin and read by
    Net::load_weight: 110 int8 convolutions and the fp32 glue between them, from the image to the four head blobs."""
    import tempfile
    from tensor_amd import hostnet, modelfile
    otter = os.path.join(ROOT, "tests", "golden", "nanodet-plus-m-1.5x_416_int8_fused.otter")
    net = hostnet.Net()
    net.load_otter(otter)
    layers = net.describe()
    blob, _ = modelfile.synthetic_int8_weights(layers, rng)
    tmp = tempfile.mkdtemp(prefix="otter_det_")
    bin_path = os.path.join(tmp, "nanodet_int8.bin")
    with open(bin_path, "wb") as f:
        f.write(blob)
    net.load_weight(bin_path, ncnn=True)
    x = rng.uniform(0, 1, (batch, 3, 416, 416)).astype(np.float32)
    sess = net.session("data_1", x, "conv_95,conv_100,conv_105,conv_110")
    n_layers = sum(l[0] not in ("Input", "Split", "NanodetPlusDetectionOutput") for l in layers)
    # algorithmic work per image: convolution MACs; bytes = every layer's output written once and read once per
    # consumer (int8 where the convolution requantizes, fp32 elsewhere) + the image
    alias = {t: l[2][0] for l in layers if l[0] == "Split" for t in l[3]}
    readers = {}
    for l in layers:
        if l[0] != "Split":
            for b in l[2]:
                readers[alias.get(b, b)] = readers.get(alias.get(b, b), 0) + 1
    macs = 0
    act_bytes = 4 * 3 * 416 * 416
    for typ, _name, _bottoms, tops, c, (_, C, H, W) in layers:
        if typ in ("Input", "Split", "NanodetPlusDetectionOutput"):
            continue
        esz = 1 if (c and c["int8_scale_term"] > 100) else 4
        act_bytes += C * H * W * esz * (1 + max(1, readers.get(tops[0], 1)))
        if c:
            macs += c["K"] * (c["C"] // c["groups"]) * c["kh"] * c["kw"] * H * W
    return dict(name="det", step=sess.run, ops=2.0 * macs * batch, launches=n_layers, images=batch,
                dom_ops=2.0 * macs * batch, dom_bytes=float(act_bytes) * batch,
                bound="hbm", workload="nanodet-plus-m-1.5x int8 (the reference's .otter description, synthetic ncnn .bin "
                "weights), %dx3x416x416 fp32 in, through otter::Net: 110 int8 convolutions + %d fp32 glue layers, to the "
                "four head blobs" % (batch, n_layers - 110), dom_kernel="whole network (all kernels of one forward pass)",
                dom_fn=None, x=x, params=[], shape=(batch, 3, 416, 416), otter=otter, bin=bin_path, _keep=(net, sess))


def build_copy(hip, capi, rng):
    """Calibration workload for the rocprofv3 FETCH_SIZE / WRITE_SIZE counters: a plain device copy of 256 MiB."""
    torch = hip.torch
    n = 256 << 20
    src = torch.zeros(n, dtype=torch.int8, device=hip.device)
    dst = torch.empty_like(src)
    return dict(name="copy", step=lambda: dst.copy_(src), ops=0.0, launches=1, bytes=2 * n, dom_ops=0.0, dom_bytes=2 * n,
                bound="hbm", workload="device-to-device copy of 256 MiB (counter calibration; what a plain copy reaches on this box)", dom_kernel="copy",
                dom_fn=None, x=None, params=[], shape=(n,))


# ------------------------------------------------------------------------------------------------------
# CPU baseline: the reference itself (oracle/_ref, kind "reference") or the C restatement (kind "port")
# ------------------------------------------------------------------------------------------------------

def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(wl, budget_s=15.0):
    r = _cpu_baseline(wl, budget_s)
    if isinstance(r, dict) and "cpu" not in r:
        r["cpu"] = cpu_model()
    return r


def _cpu_baseline(wl, budget_s=15.0):
    from oracle import binding
    name = wl["name"]
    if name == "copy":  # the counter calibration: nothing of the reference to time
        return None
    p = wl["params"]
    N, C, H, W = wl["shape"]
    x = wl["x"]
    try:
        R = binding.Ref() if binding.ref_available() else None
    except OSError:
        R = None
    if name == "c3":
        n_img = 16  # about 1.5 s on 16 threads over the five repetitions: some 20 core-seconds
        xs = x[:n_img]
        if R is not None:
            t_total = 0.0
            cur = xs
            for l in range(4):
                opts = {"type": "Convolution", "in_channels": C, "out_channels": C, "kernel": 3, "stride": 1,
                        "padding": 1, "int8_scale_term": 102, "activation": "Relu"}
                L = R.conv_layer(opts, (1, C, H, W), p[l]["wq"], p[l]["bias"], p[l]["ws"], p[l]["in_scale"],
                                 p[l]["out_scale"], True)
                cur, t = L.forward(cur, repeat=5)
                L.close()
                t_total += t
            ops = 4 * 2.0 * n_img * C * C * 9 * H * W
            return dict(value=ops / t_total / 1e12, unit="TOPS", cores=R.num_threads(), kind="reference",
                        sample="%d of 64 images through the 4 layers, reference ConvolutionLayer::forward per image "
                               "(weights pre-packed), min of 5" % n_img)
        O = binding.Oracle()
        t0 = time.perf_counter()
        O.conv_layer_forward(xs[:1], p[0]["wq"], p[0]["ws"], p[0]["in_scale"], pad=(1, 1), bias=p[0]["bias"],
                             top_scale=p[0]["out_scale"], int8_out=True, act_type=1)
        t = time.perf_counter() - t0
        return dict(value=2.0 * C * C * 9 * H * W / t / 1e12, unit="TOPS", cores=O.num_threads(), kind="port",
                    sample="1 image, layer 1, scalar C restatement")
    if name.startswith("c1"):
        s = wl["stride"]
        n_img = 4
        oh = (H + 2 - 3) // s + 1
        algo_bytes = n_img * C * (H * W * 5 + H * W + oh * oh)
        if R is not None:
            opts = {"type": "Convolution", "in_channels": C, "out_channels": C, "kernel": 3, "stride": s, "padding": 1,
                    "groups": C, "int8_scale_term": 101, "activation": "Relu6"}
            L = R.conv_layer(opts, (1, C, H, W), p[0]["wq"], p[0]["bias"], p[0]["ws"], p[0]["in_scale"],
                             p[0]["out_scale"], True)
            _, t = L.forward(x[:n_img], repeat=5, want_out=False)
            L.close()
            return dict(value=algo_bytes / t / 1e9, unit="GB/s", cores=R.num_threads(), kind="reference",
                        sample="%d of 8 images, reference layer forward (quantize + depthwise + requantize), min of 5, "
                               "algorithmic bytes" % n_img)
        O = binding.Oracle()
        t0 = time.perf_counter()
        O.conv_layer_forward(x[:n_img], p[0]["wq"], p[0]["ws"], p[0]["in_scale"], stride=(s, s), pad=(1, 1), groups=C,
                             bias=p[0]["bias"], top_scale=p[0]["out_scale"], int8_out=True, act_type=3)
        t = time.perf_counter() - t0
        return dict(value=algo_bytes / t / 1e9, unit="GB/s", cores=O.num_threads(), kind="port",
                    sample="%d images, scalar C restatement" % n_img)
    if name.startswith("blk"):
        n_img = 4
        if R is not None:
            cur, t_all = x[:n_img], 0.0
            for l in p:
                co, cg, k, _ = l["wq"].shape
                opts = {"type": "Convolution", "in_channels": cg * l["groups"], "out_channels": co, "kernel": k, "stride": l["stride"],
                        "padding": l["pad"], "groups": l["groups"], "int8_scale_term": (101 if l["groups"] > 1 else 102) if l["int8_out"] else 2}
                if l["act"] == 3:
                    opts["activation"] = "Relu6"
                L = R.conv_layer(opts, (1,) + cur.shape[1:], l["wq"], l["bias"], l["ws"], l["in_scale"], l["out_scale"], True)
                cur, t = L.forward(cur, repeat=5, want_out=True)
                L.close()
                t_all += t
            return dict(value=wl["ops"] * n_img / N / t_all / 1e12, unit="TOPS", cores=R.num_threads(), kind="reference",
                        sample="%d images, the three reference layers' forward one after the other, min of 5 each" % n_img)
        O = binding.Oracle()
        t0 = time.perf_counter()
        cur = x[:1]
        for l in p:
            cur = O.conv_layer_forward(cur, l["wq"], l["ws"], l["in_scale"], stride=(l["stride"],) * 2, pad=(l["pad"],) * 2,
                                       groups=l["groups"], bias=l["bias"], top_scale=l["out_scale"], int8_out=l["int8_out"],
                                       act_type=l["act"])
        t = time.perf_counter() - t0
        return dict(value=wl["ops"] / N / t / 1e12, unit="TOPS", cores=O.num_threads(), kind="port",
                    sample="1 image, C restatement of the three layers")
    if name == "copy":
        return None
    if name == "det":
        # the reference's own Net on the same two files, one image at a time, in a child process
        import subprocess
        r = subprocess.run([sys.executable, os.path.abspath(__file__), "--det-cpu-child", wl["otter"], wl["bin"]],
                           capture_output=True, text=True, timeout=300)
        if r.returncode != 0:
            raise RuntimeError("det CPU child failed (%d): %s" % (r.returncode, r.stderr[-200:]))
        return json.loads(r.stdout.strip().splitlines()[-1])
    if name == "c4":
        # the reference layer by layer in a child process (a crash or hang in it must not take the GPU figures along)
        import subprocess
        r = subprocess.run([sys.executable, os.path.abspath(__file__), "--c4-cpu-child"], capture_output=True, text=True,
                           timeout=300)
        if r.returncode != 0:
            raise RuntimeError("c4 CPU child failed (%d): %s" % (r.returncode, r.stderr[-200:]))
        return json.loads(r.stdout.strip().splitlines()[-1])
    if name in LAYER_SHAPES:
        Cc, K, k, st, pd, dl, gr = wl["layer"]
        if R is None or gr > 1:
            # (the compiled reference's packed int8 path stops on an assertion for a grouped, non-depthwise layer:
            # Tensor/ExpandUtils.cpp:75 under Tensor/Convolution.cpp:396-408; the C restatement stands in)
            O = binding.Oracle()
            t0 = time.perf_counter()
            O.conv_layer_forward(x[:1], p[0]["wq"], p[0]["ws"], p[0]["in_scale"], stride=(st, st), pad=(pd, pd),
                                 dil=(dl, dl), groups=gr, bias=p[0]["bias"], top_scale=p[0]["out_scale"], int8_out=True,
                                 act_type=1)
            t = time.perf_counter() - t0
            return dict(value=wl["ops"] / N / t / 1e12, unit="TOPS", cores=O.num_threads(), kind="port",
                        sample="1 image, C restatement of the layer")
        n_img = 4
        opts = {"type": "Convolution", "in_channels": Cc, "out_channels": K, "kernel": k, "stride": st, "padding": pd,
                "dilation": dl, "groups": gr, "int8_scale_term": 102, "activation": "Relu"}
        L = R.conv_layer(opts, (1, Cc, H, W), p[0]["wq"], p[0]["bias"], p[0]["ws"], p[0]["in_scale"], p[0]["out_scale"], True)
        _, t = L.forward(x[:n_img], repeat=5, want_out=False)
        L.close()
        return dict(value=wl["ops"] * n_img / N / t / 1e12, unit="TOPS", cores=R.num_threads(), kind="reference",
                    sample="%d images, reference layer forward, min of 5" % n_img)
    if name in ("c2", "c0", "c2i8") or name.startswith("c0n"):
        n_img = min(4, N)
        K = p[0]["wq"].shape[0]
        k = p[0]["wq"].shape[2]
        ops = 2.0 * n_img * K * C * k * k * H * W
        if R is not None:
            int8_out = bool(wl.get("int8_out"))
            opts = {"type": "Convolution", "in_channels": C, "out_channels": K, "kernel": k, "stride": 1,
                    "padding": k // 2, "int8_scale_term": 102 if int8_out else 2,
                    "bias_term": "true" if p[0]["bias"] is not None else "false"}
            if name.startswith("c2"):
                opts["activation"] = "Relu"
            L = R.conv_layer(opts, (1, C, H, W), p[0]["wq"], p[0]["bias"], p[0]["ws"], p[0]["in_scale"],
                             p[0].get("out_scale", 1.0), True)
            _, t = L.forward(x[:n_img], repeat=5, want_out=False)
            L.close()
            return dict(value=ops / t / 1e12, unit="TOPS", cores=R.num_threads(), kind="reference",
                        sample="%d images, reference layer forward, min of 5" % n_img)
    return None


def c4_cpu_child():
    """Times the reference's ConvolutionLayer::forward for each of the 52 convolutions of the c4 network on ONE image
    (synthetic inputs of each layer's shape and dtype, weights pre-packed, min of 3) and prints images/s of their sum.
    The glue layers (adds, pooling, inner product) are left out: the reference has no int8 path for them."""
    from oracle import binding
    from tensor_amd import mobilenet
    R = binding.Ref()
    rng = np.random.default_rng(0)
    layers = mobilenet.describe()
    params = mobilenet.init_weights(layers, rng)
    size, int8_blob = {"data": 224}, {"data": False}
    total = 0.0
    for l in layers:
        if l["kind"] == "add":
            size[l["name"]], int8_blob[l["name"]] = size[l["a"]], False
            continue
        if l["kind"] != "conv":
            continue
        hin = size[l["input"]]
        hout = (hin + 2 * (l["k"] // 2) - l["k"]) // l["stride"] + 1
        size[l["name"]], int8_blob[l["name"]] = hout, l["int8_out"]
        pr = params[l["name"]]
        dw = l["groups"] == l["cin"] == l["cout"]
        opts = {"type": "Convolution", "in_channels": l["cin"], "out_channels": l["cout"], "kernel": l["k"],
                "stride": l["stride"], "padding": l["k"] // 2, "groups": l["groups"],
                "int8_scale_term": (1 if dw else 2) + (100 if l["int8_out"] else 0)}
        if l["act"]:
            opts["activation"] = l["act"]
        if int8_blob[l["input"]]:
            x = rng.integers(-127, 128, (1, l["cin"], hin, hin)).astype(np.int8)
        else:
            x = rng.uniform(0, 1, (1, l["cin"], hin, hin)).astype(np.float32)
        L = R.conv_layer(opts, (1, l["cin"], hin, hin), pr["wq"], pr["bias"], pr["ws"], 100.0, 20.0, True)
        _, t = L.forward(x, repeat=3, want_out=False)
        L.close()
        total += t
    print(json.dumps(dict(value=1.0 / total, unit="images/s", cores=R.num_threads(), kind="reference",
                          sample="1 image: the 52 convolution layers through the reference ConvolutionLayer::forward, one "
                                 "by one (weights pre-packed, synthetic layer inputs), min of 3 each; glue layers not "
                                 "included")))


def det_cpu_child(otter, bin_path):
    """Times the compiled reference's Net (load_otter + load_weight, then Extractor::extract of the four heads) on a
    few images, one at a time as the reference runs them."""
    from oracle import binding
    R = binding.Ref()
    net = R.net(otter, bin_path)
    rng = np.random.default_rng(1)
    heads = ["conv_95", "conv_100", "conv_105", "conv_110"]
    best = None
    for _ in range(6):
        x = rng.uniform(0, 1, (1, 3, 416, 416)).astype(np.float32)
        t0 = time.perf_counter()
        net.run("data_1", x, heads)
        t = time.perf_counter() - t0
        best = t if best is None else min(best, t)
    print(json.dumps(dict(value=1.0 / best, unit="images/s", cores=R.num_threads(), kind="reference",
                          sample="6 single images through the reference's Net (same .otter and .bin), min")))


def measured_traffic(name):
    """HBM bytes per launch of the workload's dominant kernel, from the committed rocprofv3 --pmc summary
    (profiles/hbm_traffic.json: FETCH_SIZE / WRITE_SIZE scaled by a copy-kernel calibration); None if not profiled."""
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            return json.load(f).get(name, {}).get("traffic_bytes")
    except (OSError, ValueError):
        return None


def measure(wl, timer, steps, warmup, unit_main):
    ms, wall_ms = timer.run(wl["step"], steps, warmup)
    res = dict(workload=wl["workload"], ms_per_step=ms, wall_ms_per_step=wall_ms)
    if wl["bound"] == "mfma" or unit_main == "TOPS":
        res["tops"] = wl["ops"] / (ms * 1e-3) / 1e12
    if "bytes" in wl:
        res["gbs"] = wl["bytes"] / (ms * 1e-3) / 1e9
    # dominant kernel alone, back to back
    if wl.get("dom_fn") is not None:
        kms, _ = timer.run(wl["dom_fn"], max(steps * 4, 50), 5)
    else:
        kms = ms
    # a bandwidth-bound kernel is priced on a loop that rotates over buffer sets larger than the last-level cache;
    # the figure of the loop over ONE set (operands still cached from the previous launch) is reported beside it
    kms_resident = None
    if wl.get("dom_fn_cold"):
        kms_resident = kms
        kms, _ = timer.run(wl["dom_fn_cold"], max(steps * 4, 50), 2 * len(wl["dom_fn_cold"]))
    if wl["bound"] == "mfma":
        ach = wl["dom_ops"] / (kms * 1e-3) / 1e12
        res["roofline"] = dict(bound="mfma", achieved=ach, peak=PEAK_INT8_TOPS, unit="TOP/s", frac=ach / PEAK_INT8_TOPS,
                               traffic=measured_traffic(wl["name"]), kernel=wl["dom_kernel"], kernel_ms=kms)
        # The published peak assumes the maximum engine clock. What the matrix cores can do on THIS box: compute units
        # x 4 SIMDs x 2048 int8 operations per cycle x the shader clock it holds under matrix load, measured right behind
        # the timed loop (the clock is in its loaded state then).
        hipl = timer.hip
        if hipl is not None:
            info = hipl.device_info()
            # (the chain launch times itself with the shader-cycle counter; other kernels get the clock of a millisecond
            # of bare matrix instructions, which is an upper bound: a kernel that also keeps the vector ALU and LDS busy
            # holds a lower clock)
            mhz = hipl.conv_chain_clock_mhz() if wl["name"] == "c3" else 0.0
            res["roofline"]["shader_clock_source"] = "the timed kernel's own cycle counter" if mhz > 0 else "a bare matrix-instruction loop"
            if mhz <= 0:
                mhz = hipl.shader_clock_mhz()
            peak_clk = info["compute_units"] * 4 * 2048 * mhz * 1e6 / 1e12
            res["roofline"].update(shader_clock_mhz=mhz, max_clock_mhz=info["clock_mhz"], compute_units=info["compute_units"],
                                   peak_at_shader_clock=peak_clk, frac_of_peak_at_shader_clock=ach / peak_clk)
    else:
        ach = wl["dom_bytes"] / (kms * 1e-3) / 1e9
        res["roofline"] = dict(bound="hbm", achieved=ach, peak=PEAK_HBM_GBS, unit="GB/s", frac=ach / PEAK_HBM_GBS,
                               traffic=measured_traffic(wl["name"]), kernel=wl["dom_kernel"], kernel_ms=kms)
        res["roofline"]["tops"] = wl["dom_ops"] / (kms * 1e-3) / 1e12
        if kms_resident is not None:
            res["roofline"]["working_set"] = "%d buffer sets in turn, %d MB per loop" % (
                len(wl["dom_fn_cold"]), len(wl["dom_fn_cold"]) * wl["dom_bytes"] >> 20)
            res["roofline_resident"] = dict(kernel_ms=kms_resident, achieved=wl["dom_bytes"] / (kms_resident * 1e-3) / 1e9,
                                            frac=wl["dom_bytes"] / (kms_resident * 1e-3) / 1e9 / PEAK_HBM_GBS,
                                            working_set="one buffer set, %d MB (cache-resident)" % (wl["dom_bytes"] >> 20))
    for aux in wl.get("aux", []):
        ams_res, _ = timer.run(aux["fn"], max(steps * 4, 50), 5)
        ams = ams_res
        if aux.get("fn_cold"):
            ams, _ = timer.run(aux["fn_cold"], max(steps * 4, 50), 2 * len(aux["fn_cold"]))
        res.setdefault("aux_kernels", []).append(
            dict(kernel=aux["kernel"], kernel_ms=ams, gbs=aux["bytes"] / (ams * 1e-3) / 1e9,
                 frac_hbm=aux["bytes"] / (ams * 1e-3) / 1e9 / PEAK_HBM_GBS, resident_kernel_ms=ams_res,
                 resident_frac_hbm=aux["bytes"] / (ams_res * 1e-3) / 1e9 / PEAK_HBM_GBS))
    return res


def main():
    if "--c4-cpu-child" in sys.argv:
        c4_cpu_child()
        return
    if "--det-cpu-child" in sys.argv:
        i = sys.argv.index("--det-cpu-child")
        det_cpu_child(sys.argv[i + 1], sys.argv[i + 2])
        return
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c3")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-also", action="store_true")
    ap.add_argument("--per-layer", action="store_true",
                    help="print one JSON line with every convolution layer of the c4 network timed by itself, and exit")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build runs on one GPU only (the path shards by batch: images are independent); "
              "--gpus %d is not supported" % a.gpus, file=sys.stderr)
        sys.exit(2)
    if int(os.environ.get("WORLD_SIZE", "1")) > 1:
        print("bench.py: one process, one GPU", file=sys.stderr)
        sys.exit(2)

    from tensor_amd import capi
    hip = capi.Library(0)
    timer = Timer(hip.torch, hip)
    if a.per_layer:
        from tensor_amd import mobilenet
        rows = mobilenet.per_layer(hip, capi, np.random.default_rng(0),
                                   lambda fn: timer.run(fn, max(a.steps * 2, 100), a.warmup, settle=0.02)[0])
        for r in rows:
            r["frac_hbm"] = r["gbs"] / PEAK_HBM_GBS
            r["frac_mfma"] = r["tops"] / PEAK_INT8_TOPS
        print(json.dumps({"workload": "c4 layers one by one, batch 64", "sum_us": sum(r["us"] for r in rows),
                          "layers": rows}))
        return
    builders = {"c3": lambda r: build_c3(hip, capi, r), "c1s1": lambda r: build_c1(hip, capi, r, 1),
                "c1s2": lambda r: build_c1(hip, capi, r, 2), "c2": lambda r: build_c2(hip, capi, r),
                "c1s1i8": lambda r: build_c1(hip, capi, r, 1, "i8"), "c1s2i8": lambda r: build_c1(hip, capi, r, 2, "i8"),
                "c1s1valu": lambda r: build_c1(hip, capi, r, 1, "valu"), "c1s2valu": lambda r: build_c1(hip, capi, r, 2, "valu"),
                "c0": lambda r: build_c0(hip, capi, r), "copy": lambda r: build_copy(hip, capi, r),
                "c2i8": lambda r: build_c2(hip, capi, r, int8_out=True), "c0n64": lambda r: build_c0(hip, capi, r, batch=64)}
    try:
        from tensor_amd import mobilenet  # noqa: F401
        builders["c4"] = lambda r: mobilenet.build_bench(hip, capi, r)
    except ImportError:
        pass
    builders["det"] = lambda r: build_det(hip, capi, r)
    for lname in LAYER_SHAPES:
        builders[lname] = lambda r, lname=lname: build_layer(hip, capi, r, lname)
    builders["blk14"] = lambda r: build_block(hip, capi, r)
    builders["blk112s2"] = lambda r: build_block(hip, capi, r, cin=16, ce=96, cout=24, hw=112, stride=2, name="blk112s2")
    if a.workload not in builders:
        print("unknown workload %s (have %s)" % (a.workload, sorted(builders)), file=sys.stderr)
        sys.exit(2)

    wl = builders[a.workload](np.random.default_rng(0))
    unit = "images/s" if wl["name"] in ("c4", "det") else ("GB/s" if "bytes" in wl else "TOPS")
    no_settle = None
    if wl["name"] == "c3":
        # the same measurement without the run-in, after an idle second (the clock at rest): reported beside the line
        hip.torch.cuda.synchronize()
        time.sleep(1.0)
        ms0, _ = timer.run(wl["step"], a.steps, a.warmup, settle=0.0)
        time.sleep(1.0)
        k0, _ = timer.run(wl["dom_fn"], max(a.steps * 4, 50), 5, settle=0.0)
        no_settle = dict(ms_per_step=ms0, tops=wl["ops"] / (ms0 * 1e-3) / 1e12, kernel_ms=k0,
                         frac=wl["dom_ops"] / (k0 * 1e-3) / 1e12 / PEAK_INT8_TOPS,
                         note="same loops with settle_s = 0, each after one idle second")
        # the same four layers as four launches of the per-layer entry point, and one of those launches alone
        msl, _ = timer.run(wl["step_layers"], a.steps, a.warmup)
        kl, _ = timer.run(wl["layer_fn"], max(a.steps * 4, 50), 5)
        # the chain launch ran some thousand times above: its result must still be the four launches' result, and no
        # workgroup may have given up a wait
        same = bool((wl["step"]().cpu() == wl["step_layers"]().cpu()).all().item())
        gave_up = hip.conv_chain_gave_up()
        layer_by_layer = dict(ms_per_step=msl, tops=wl["ops"] / (msl * 1e-3) / 1e12, launches_per_step=4,
                              chain_equals_layers=same, chain_gave_up=gave_up,
                              kernel="conv3x3_halo_kernel (one layer per launch)", kernel_ms=kl,
                              frac=wl["layer_ops"] / (kl * 1e-3) / 1e12 / PEAK_INT8_TOPS)
    res = measure(wl, timer, a.steps, a.warmup, unit)
    if wl["name"] == "c4":
        value = wl["images"] / (res["ms_per_step"] * 1e-3)
        metric = "MobileNetV2-style int8 net images/sec b64"
    elif wl["name"] == "det":
        value = wl["images"] / (res["ms_per_step"] * 1e-3)
        metric = "int8 detection model (reference .otter description) images/sec b16"
    elif unit == "TOPS":
        value = res["tops"]
        metric = "int8 conv TOPS"
    else:
        value = res["gbs"]
        metric = "depthwise int8 HBM GB/s (quantize + depthwise layer, algorithmic bytes)"
    line = {"metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
            "ms_per_step": res["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "int8 x int8 -> int32 (fp32 epilogue)", "data": "synthetic, seeded (numpy default_rng(0))",
            "config": {"workload": wl["workload"],
                       # the networks run fewer launches than layers (fused layer groups): count the layers there
                       ("layers_per_step" if wl["name"] in ("c4", "det") else "launches_per_step"): wl["launches"],
                       "settle_s": SETTLE_S},
            "roofline": res["roofline"], "wall_ms_per_step": res["wall_ms_per_step"]}
    if "aux_kernels" in res:
        line["aux_kernels"] = res["aux_kernels"]
    if "roofline_resident" in res:
        line["roofline_resident"] = res["roofline_resident"]
    if no_settle is not None:
        line["no_settle"] = no_settle
        line["layer_by_layer"] = layer_by_layer
    if not a.no_cpu:
        try:
            line["cpu_baseline"] = cpu_baseline(wl)
        except Exception as e:  # the baseline is a reported figure, never the measured path
            line["cpu_baseline"] = {"error": str(e)[:200]}
    if not a.no_also:
        also = []
        for name in ("c1s1", "c1s2", "c2", "c2i8", "c0", "c0n64", "c4", "det", "blk14", "blk112s2") + tuple(LAYER_SHAPES) + ("copy",):
            if name == a.workload or name not in builders:
                continue
            w2 = builders[name](np.random.default_rng(0))
            r2 = measure(w2, timer, max(10, a.steps // 2), a.warmup, "")
            entry = dict(name=name, **r2)
            if name.startswith("blk"):  # the same block as three launches, in the same run
                ms3, _ = timer.run(w2["step_layers"], max(10, a.steps // 2), a.warmup)
                entry["three_launches_ms_per_step"] = ms3
            if name in ("c4", "det"):
                entry["images_per_s"] = w2["images"] / (r2["ms_per_step"] * 1e-3)
            if not a.no_cpu:
                try:
                    entry["cpu_baseline"] = cpu_baseline(w2)
                except Exception as e:
                    entry["cpu_baseline"] = {"error": str(e)[:200]}
            also.append(entry)
            del w2
        line["also"] = also
    print(json.dumps(line))


if __name__ == "__main__":
    main()
