"""CPU: the launch plan of the inverted-residual block launch (host arithmetic of the GPU library, no GPU needed).

A workgroup owns a band of output rows of one image and, where a batch has few bands, a share of the band's slices of
expanded channels. The plan must cover every row and every slice exactly once, stay inside the LDS of a compute unit
and the project-tile budget of a workgroup, and size the workspace of the shared accumulators; the automatic choice is
checked on the shapes it was tuned on."""
import ctypes as C

import pytest

from tensor_amd import capi


def block_plan(lib, cin, ce, cout, n, h, w, rb=0, sl=0, split=0):
    plan = (C.c_int * 6)()
    rc = lib.otter_hip_conv_block_plan(cin, ce, cout, n, h, w, rb, sl, split, plan)
    if rc != 0:
        return None
    return dict(zip(("rb", "bands", "sl", "lds", "split", "ws_words"), list(plan)))


SHAPES = [(64, 384, 64, 64, 14, 14), (96, 576, 96, 64, 14, 14), (32, 192, 32, 64, 28, 28), (160, 960, 160, 64, 7, 7),
          (160, 960, 320, 64, 7, 7), (24, 144, 24, 64, 56, 56), (64, 384, 64, 3, 14, 14), (8, 48, 8, 1, 1, 1),
          (16, 96, 24, 2, 9, 64), (40, 136, 24, 2, 11, 13), (64, 384, 64, 1000, 14, 14)]


@pytest.mark.parametrize("cin,ce,cout,n,h,w", SHAPES)
@pytest.mark.parametrize("force", [(0, 0, 0), (0, 64, 0), (0, 128, 3), (2, 64, 2), (100, 0, 100)])
def test_plan_covers_rows_and_slices_within_the_budgets(cin, ce, cout, n, h, w, force):
    lib = capi.load_cdll()
    p = block_plan(lib, cin, ce, cout, n, h, w, *force)
    if p is None:
        # a forced plan may not fit; the automatic one must exist for every shape listed
        assert force != (0, 0, 0)
        return
    assert 1 <= p["rb"] <= h and p["bands"] == -(-h // p["rb"])
    # bands of nearly equal height: band b owns rows [b * h // bands, (b + 1) * h // bands), none taller than rb
    edges = [b * h // p["bands"] for b in range(p["bands"] + 1)]
    assert edges[0] == 0 and edges[-1] == h and max(b - a for a, b in zip(edges, edges[1:])) <= p["rb"]
    assert min(b - a for a, b in zip(edges, edges[1:])) >= 1
    assert p["sl"] in (64, 128) and (force[1] == 0 or p["sl"] == force[1])
    assert 0 < p["lds"] <= 160 * 1024
    # the slices dealt to `split` workgroups, spp consecutive ones each: every slice once, nobody empty-handed
    slices = -(-ce // p["sl"])
    spp = -(-slices // p["split"])
    assert 1 <= p["split"] <= slices and p["split"] * spp >= slices and (p["split"] - 1) * spp < slices
    # project tiles (32 channels x 16 pixels) of a band: at most 48 per workgroup; their accumulators (512 words each)
    # per workgroup in the workspace when there are several workgroups per band
    tiles = -(-cout // 32) * -(-(p["rb"] * w) // 16)
    assert tiles <= 48
    assert p["ws_words"] == (n * p["bands"] * p["split"] * tiles * 512 if p["split"] > 1 else 0)


def test_automatic_plans_of_the_tuned_shapes():
    lib = capi.load_cdll()
    # 14x14 at batch 64: four bands of 3..4 rows = one workgroup per compute unit, 128-channel slices, no split
    p = block_plan(lib, 64, 384, 64, 64, 14, 14)
    assert (p["rb"], p["bands"], p["sl"], p["split"]) == (4, 4, 128, 1)
    # 28x28: four bands of 7 rows
    p = block_plan(lib, 32, 192, 32, 64, 28, 28)
    assert (p["rb"], p["bands"], p["sl"], p["split"]) == (7, 4, 64, 1)  # (192 channels: three slices of 64, not 128 + 64)
    # 7x7: one band per image, the eight slices of 960 channels dealt to four workgroups
    p = block_plan(lib, 160, 960, 160, 64, 7, 7)
    assert (p["rb"], p["bands"], p["sl"], p["split"]) == (7, 1, 128, 4)
    # 7x7 with 320 output channels: one band would hold 40 project tiles; two bands of 20, each dealt to two workgroups
    p = block_plan(lib, 160, 960, 320, 64, 7, 7)
    assert (p["rb"], p["bands"], p["sl"], p["split"]) == (4, 2, 128, 2)
    # a small batch: the slices split as far as they go
    p = block_plan(lib, 64, 384, 64, 4, 14, 14)
    assert p["split"] == 3
    # shapes the launch does not take
    assert block_plan(lib, 64, 384, 64, 8, 14, 65) is None      # wider than 64 pixels
    assert block_plan(lib, 200, 384, 64, 8, 14, 14) is None     # more than 192 input channels
    assert block_plan(lib, 64, 384, 1600, 8, 14, 14) is None    # more project tiles than a workgroup holds
