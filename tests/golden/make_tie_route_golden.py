"""Writes tests/golden/tie_route_golden.npz from the *compiled reference* (oracle/_ref/libotter_ref.so, built from
/root/reference by `make -C oracle ref`). Run in the build container only:

    python tests/golden/make_tie_route_golden.py

Per case of cases.TIE_ROUTE_CASES: the output of a real otter::ConvolutionLayer (parse_param -> load_param ->
create_pipeline -> forward behind Net's layout conversion) on inputs whose results sit exactly on +-0.49999997f, the one
value that float2int8_sse and float2int8 round differently. The inputs are not stored: cases.make_tie_inputs rebuilds
them. The vectors pin which rounding primitive a layer ends in for its (C, K, groups, packing)."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, HERE)

from oracle.binding import Ref  # noqa: E402
from cases import TIE_ROUTE_CASES, layer_options, make_tie_inputs  # noqa: E402


def main():
    R = Ref()
    G = {}
    for case in TIE_ROUTE_CASES:
        name, C, H, W, packing = case[0], case[1], case[8], case[9], case[16]
        t = make_tie_inputs(case)
        L = R.conv_layer(layer_options(case[:16]), (1, C, H, W), t["wq"], t["bias"], t["w_scales"], float(t["in_scale"]),
                         float(t["top_scale"]), packing)
        out, _ = L.forward(t["x"])
        G[name + "/scale_in"] = L.scale_in()
        G[name + "/out"] = out
        L.close()
        vals, counts = np.unique(out, return_counts=True)
        print("%-34s %s" % (name, dict(zip(vals.tolist(), counts.tolist()))))
    path = os.path.join(HERE, "tie_route_golden.npz")
    np.savez_compressed(path, **G)
    print("wrote", path, os.path.getsize(path), "bytes,", len(G), "arrays")


if __name__ == "__main__":
    main()
