"""Writes tests/golden/int8_conv_golden.npz from the *compiled reference* (oracle/_ref/libotter_ref.so,
built from /root/reference by `make -C oracle ref`). Run in the build container only:

    python tests/golden/make_golden.py

The file holds, per case, the inputs and the reference's outputs (layer level through a real
otter::ConvolutionLayer; function level for the quantize / requantize / dequantize rounding fine print with
adversarial near-tie values). The tests replay them against oracle/otter_int8_oracle.c on any machine and
against the GPU library on the GPU box.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, HERE)

from oracle.binding import Ref, out_size  # noqa: E402
from cases import LAYER_CASES, UNPACKED_LAYER_CASES, layer_options, make_inputs  # noqa: E402


def near_tie_values(rng, n):
    ks = rng.integers(-130, 131, size=n).astype(np.float32)
    base = ks + np.float32(0.5) * np.where(ks >= 0, 1, -1).astype(np.float32)
    out = []
    for b in base:
        out += [b, np.nextafter(b, np.float32(1e9), dtype=np.float32), np.nextafter(b, np.float32(-1e9), dtype=np.float32)]
    out += [0.49999997, -0.49999997, 0.5, -0.5, 0.0, -0.0, 127.49999, 127.5, -127.5, 128.7, -300.0, 126.5, -126.5,
            1e6, -1e6, 2.0e9, -2.0e9]
    return np.array(out, np.float32)


def main():
    R = Ref()
    rng = np.random.default_rng(1234)
    G = {}
    # ---- layer level -------------------------------------------------------------------------------
    for i, case in enumerate(LAYER_CASES):
        name = case[0]
        C, K, k, s, p, d, g = case[1:8]
        N = case[10]
        t = make_inputs(case, seed=100 + i)
        H, W = case[8], case[9]
        L = R.conv_layer(layer_options(case), (1, C, H, W), t["wq"], t["bias"], t["w_scales"], float(t["in_scale"]),
                         float(t["top_scale"]), True)
        out, _ = L.forward(t["x"])
        G[name + "/scale_in"] = L.scale_in()
        L.close()
        xq = t["x"] if t["x"].dtype == np.int8 else R.quantize(t["x"], [t["in_scale"]], True)
        acc = R.conv_int32(xq, t["wq"], (s, s), (p, p), (d, d), g, True)
        for key, v in t.items():
            if v is not None:
                G[name + "/" + key] = np.asarray(v)
        G[name + "/xq"] = xq
        G[name + "/acc"] = acc
        G[name + "/out"] = out
        print("%-32s out %s %s" % (name, out.dtype, out.shape))
    # ---- layer level, use_packing_layout = false ---------------------------------------------------------
    for i, case in enumerate(UNPACKED_LAYER_CASES):
        name = case[0]
        C, K, k, s, p, d, g = case[1:8]
        H, W = case[8], case[9]
        t = make_inputs(case, seed=300 + i)
        L = R.conv_layer(layer_options(case), (1, C, H, W), t["wq"], t["bias"], t["w_scales"], float(t["in_scale"]),
                         float(t["top_scale"]), False)
        out, _ = L.forward(t["x"])
        G[name + "/scale_in"] = L.scale_in()
        L.close()
        xq = t["x"] if t["x"].dtype == np.int8 else R.quantize(t["x"], [t["in_scale"]], False)
        acc = R.conv_int32(xq, t["wq"], (s, s), (p, p), (d, d), g, False)
        for key, v in t.items():
            if v is not None:
                G[name + "/" + key] = np.asarray(v)
        G[name + "/xq"] = xq
        G[name + "/acc"] = acc
        G[name + "/out"] = out
        print("%-32s out %s %s (unpacked)" % (name, out.dtype, out.shape))
    # ---- quantize fine print -----------------------------------------------------------------------
    for C in (8, 4, 3):
        v = near_tie_values(rng, 120)
        hw = (v.size + C - 1) // C
        x = np.resize(v, (1, C, hw, 1)).astype(np.float32)
        for packing in (True, False):
            tag = "quant_ties/C%d_pack%d" % (C, int(packing))
            G[tag + "/x"] = x
            G[tag + "/q"] = R.quantize(x, [1.0], packing)
    x = rng.uniform(-1, 1, (2, 16, 9, 7)).astype(np.float32)
    ps = rng.uniform(50, 200, 16).astype(np.float32)
    G["quant_perchannel/x"], G["quant_perchannel/scales"] = x, ps
    G["quant_perchannel/q"] = R.quantize(x, ps, True)
    # ---- requantize fine print: exact .5 ties, +-1ulp bias nudges, fused multiply-add ------------------
    for C in (8, 4, 6):
        for packing in (True, False):
            acc = rng.integers(-300, 300, size=(1, C, 13, 11)).astype(np.int32)
            si = np.ones(C, np.float32)
            so = np.array([0.5], np.float32)
            for j, bias in enumerate((None, np.zeros(C, np.float32), np.full(C, 2.0 ** -24, np.float32),
                                      np.full(C, -2.0 ** -24, np.float32))):
                tag = "requant_ties/C%d_pack%d_b%d" % (C, int(packing), j)
                G[tag + "/acc"], G[tag + "/scale_in"], G[tag + "/scale_out"] = acc, si, so
                if bias is not None:
                    G[tag + "/bias"] = bias
                G[tag + "/q"] = R.requantize(acc, si, so, bias, 0, None, packing)
    for act in (0, 1, 2, 3):
        for C, packing in ((8, True), (12, True), (6, True), (8, False)):
            acc = rng.integers(-20000, 20000, size=(1, C, 12, 12)).astype(np.int32)
            si = rng.uniform(1e-4, 1e-3, C).astype(np.float32)
            so = np.array([rng.uniform(20, 40)], np.float32)
            bias = rng.normal(0, 0.05, C).astype(np.float32)
            ap = np.array([0.1], np.float32) if act == 2 else None
            tag = "requant_rand/act%d_C%d_pack%d" % (act, C, int(packing))
            G[tag + "/acc"], G[tag + "/scale_in"], G[tag + "/scale_out"], G[tag + "/bias"] = acc, si, so, bias
            if ap is not None:
                G[tag + "/act_params"] = ap
            G[tag + "/q"] = R.requantize(acc, si, so, bias, act, ap, packing)
    # ---- dequantize: bitwise, with the magnitudes where fma and mul+add part ways -------------------
    for C, packing in ((8, True), (4, True), (8, False)):
        acc = rng.integers(-2000000, 2000000, size=(2, C, 8, 8)).astype(np.int32)  # H*W % 4 == 0: the reference's unpacked dequantize leaves a ragged tail unwritten
        si = rng.uniform(1e-6, 1e-5, C).astype(np.float32)
        bias = rng.normal(0, 1, C).astype(np.float32)
        for j, b in enumerate((None, bias)):
            tag = "dequant/C%d_pack%d_b%d" % (C, int(packing), j)
            G[tag + "/acc"], G[tag + "/scale"] = acc, si
            if b is not None:
                G[tag + "/bias"] = b
            G[tag + "/y"] = R.dequantize(acc, si, b, packing)
    path = os.path.join(HERE, "int8_conv_golden.npz")
    np.savez_compressed(path, **G)
    print("wrote", path, os.path.getsize(path), "bytes,", len(G), "arrays")


if __name__ == "__main__":
    main()
