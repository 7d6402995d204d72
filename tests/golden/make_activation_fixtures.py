"""Writes tests/golden/activation_golden.npz from the *compiled reference* (oracle/_ref/libotter_ref.so, built from
/root/reference by `make -C oracle ref`). Run in the build container only:

    python tests/golden/make_activation_fixtures.py

Inputs and the reference's outputs for the two transcendental activations of the int8 epilogues (sigmoid = type 4,
mish = type 5; Tensor/QuantizeX86.hpp:72-106): the standalone requantize with packed and unpacked blobs, and a real
otter::ConvolutionLayer with `activation=Sigmoid`, int8 and fp32 result (the layer has no option string for mish,
Tensor/ConvolutionLayer.cpp:107-118). The fp32 cases run unpacked: on a packed fp32 blob the reference's Sigmoid
layer stops with '"neg_cpu" not implemented for Float4' (Tensor/SigmoidLayer.cpp:22-26).

These vectors are exact for the machine that wrote them only: the reference build (-Ofast -ffast-math) evaluates
exp / log with polynomials and turns the division of the sigmoid into an approximate-reciprocal instruction plus one
Newton step, whose result differs between CPU models. The tests therefore allow one int8 step at rounding ties and a
relative 1e-5 on fp32 values.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle.binding import Ref  # noqa: E402


def main():
    R = Ref()
    rng = np.random.default_rng(4242)
    G = {}
    for act, so in ((4, 100.0), (5, 6.0)):
        for packing in (True, False):
            for K in (8, 4, 6):
                tag = "requant/act%d_pack%d_K%d" % (act, int(packing), K)
                acc = rng.integers(-200000, 200000, size=(2, K, 24, 20)).astype(np.int32)
                acc[0, 0, 0, :8] = [0, 1, -1, 2 ** 24, -2 ** 24, 10 ** 6, -10 ** 6, 12345]   # v = 0, tiny, +-1677, +-100
                si = rng.uniform(0.5e-4, 1.5e-4, K).astype(np.float32)   # v within about +-30
                bias = rng.normal(0, 0.1, K).astype(np.float32)
                so_v = np.full(1, so, np.float32)
                G[tag + "/acc"], G[tag + "/si"], G[tag + "/so"], G[tag + "/bias"] = acc, si, so_v, bias
                G[tag + "/q"] = R.requantize(acc, si, so_v, bias, act, None, packing=packing)
    for int8_out in (True, False):
        for (C, K, k, g) in ((16, 16, 3, 1), (8, 12, 1, 1), (16, 16, 3, 16)):
            if g > 1 and not int8_out:
                continue  # the reference's unpacked depthwise path does not take a batch dimension
            tag = "layer/sigmoid_i8%d_C%d_K%d_k%d_g%d" % (int(int8_out), C, K, k, g)
            x = rng.uniform(-1, 1, (1, C, 10, 12)).astype(np.float32)
            w = rng.normal(0, 0.3, (K, C // g, k, k)).astype(np.float32)
            ws = (127.0 / np.abs(w).reshape(K, -1).max(axis=1)).astype(np.float32)
            wq = np.clip(np.rint(w * ws[:, None, None, None]), -127, 127).astype(np.int8)
            bias = rng.normal(0, 0.5, K).astype(np.float32)
            in_scale = np.float32(127.0) / np.abs(x).max()
            opts = {"out_channels": K, "kernel": k, "padding": k // 2, "groups": g, "bias_term": "true",
                    "int8_scale_term": (101 if g == 1 else 102) if int8_out else (1 if g == 1 else 2), "activation": "Sigmoid"}
            L = R.conv_layer(opts, (1, C, 10, 12), wq, bias, ws, float(in_scale), top_scale=120.0, use_packing=int8_out)
            y, _ = L.forward(x)
            L.close()
            G[tag + "/x"], G[tag + "/wq"], G[tag + "/ws"], G[tag + "/bias"] = x, wq, ws, bias
            G[tag + "/in_scale"], G[tag + "/y"] = np.float32(in_scale), y
    out = os.path.join(HERE, "activation_golden.npz")
    np.savez_compressed(out, **G)
    print("wrote", out, os.path.getsize(out), "bytes,", len(G), "arrays")


if __name__ == "__main__":
    main()
