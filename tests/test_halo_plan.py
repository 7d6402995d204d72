"""CPU: the launch plan of the 3x3 LDS-halo kernel (host arithmetic of the GPU library, no GPU needed).

A persistent workgroup walks over tiles of `pt` consecutive output pixels of one image and may keep the per-lane LDS
offsets of its first tile for its later tiles. That is only right when every tile the workgroup meets covers the same
pixels relative to its first row. The walk is replayed here from the plan the library reports, with the kernel's tile
order, and every later tile's offsets are compared with the first tile's.
"""
import ctypes as C

import numpy as np
import pytest

from tensor_amd import capi


def halo_plan(lib, c, k, pad, n, h, w, force_fn=0):
    plan = (C.c_int * 8)()
    rc = lib.otter_hip_conv3x3_halo_plan(c, k, pad, n, h, w, force_fn, plan)
    if rc != 0:
        return None
    keys = ("fn", "pt", "tiles_per_img", "grid_x", "grid_y", "tile_inv", "r_max", "cb")
    return dict(zip(keys, list(plan)))


def tile_of(t, total, tiles_per_img, pt):
    """The kernel's tile order: consecutive tiles go to the same XCD."""
    per = total // 8
    if per > 0 and t < per * 8:
        t = (t % 8) * per + t // 8
    return t // tiles_per_img, (t % tiles_per_img) * pt


def lane_offsets(p0, pt, OW, OHW, pad):
    """(row within the tile's LDS rows, column) of every pixel slot of a tile; slots past the image end are clamped to
    the last pixel as the kernel does (their results are never stored)."""
    pix = np.minimum(p0 + np.arange(pt), OHW - 1)
    return pix // OW - p0 // OW, pix % OW - pad + 2, p0 + np.arange(pt) < OHW


SHAPES = [
    # C, K, pad, N, H, W
    (64, 128, 1, 256, 64, 64),   # 192-pixel tiles = 3 rows, 4096 % 192 != 0, several tiles per workgroup
    (64, 256, 1, 128, 64, 64),
    (8, 1024, 1, 32, 20, 16),    # the GPU regression case of test_gpu_parity
    (128, 128, 1, 64, 56, 56),   # the benchmark layer: whole tiles
    (64, 64, 1, 1, 56, 56),
    (16, 160, 1, 3, 7, 8),
    (72, 24, 0, 2, 11, 10),
    (128, 128, 1, 40, 32, 32),
]


@pytest.mark.parametrize("shape", SHAPES, ids=["%dx%d_p%d_n%d_%dx%d" % s for s in SHAPES])
@pytest.mark.parametrize("force_fn", [0, 4, 5, 6, 7])
def test_reused_offsets_are_right_for_every_tile_of_the_walk(shape, force_fn):
    lib = capi.load_cdll()
    c, k, pad, n, h, w = shape
    pl = halo_plan(lib, c, k, pad, n, h, w, force_fn)
    assert pl is not None
    OH, OW = h + 2 * pad - 2, w + 2 * pad - 2
    OHW = OH * OW
    assert pl["tiles_per_img"] == -(-OHW // pl["pt"])
    total = n * pl["tiles_per_img"]
    assert 1 <= pl["grid_x"] <= total
    seen = np.zeros(total, bool)
    for b in range(pl["grid_x"]):
        first = None
        for t in range(b, total, pl["grid_x"]):
            img, p0 = tile_of(t, total, pl["tiles_per_img"], pl["pt"])
            assert 0 <= img < n and p0 < OHW
            seen[img * pl["tiles_per_img"] + p0 // pl["pt"]] = True
            row, col, live = lane_offsets(p0, pl["pt"], OW, OHW, pad)
            assert row[live].max() + 3 <= pl["r_max"]  # rows touched + the two halo rows fit the LDS tile
            if first is None or not pl["tile_inv"]:
                first = (row, col)
            # what the kernel would use for this tile: the cached offsets of the workgroup's first tile
            np.testing.assert_array_equal(first[0][live], row[live])
            np.testing.assert_array_equal(first[1][live], col[live])
    assert seen.all()  # the swizzled walk covers every tile exactly


def test_offsets_are_only_reused_without_a_ragged_last_tile():
    lib = capi.load_cdll()
    # 192-pixel tiles on a 64x64 image: whole rows, but 4096 = 21 * 192 + 64
    pl = halo_plan(lib, 64, 128, 1, 256, 64, 64, 6)
    assert pl["pt"] == 192 and pl["tile_inv"] == 0
    # 224-pixel tiles on 56x56: whole rows and 3136 = 14 * 224
    pl = halo_plan(lib, 128, 128, 1, 64, 56, 56, 7)
    assert pl["pt"] == 224 and pl["tile_inv"] == 1
    # tiles that are not whole rows never reuse
    pl = halo_plan(lib, 128, 128, 1, 2, 19, 22, 4)
    assert pl["tile_inv"] == 0


def test_plan_refuses_what_the_kernel_does_not_take():
    lib = capi.load_cdll()
    assert halo_plan(lib, 64, 64, 1, 1, 56, 200) is None  # rows wider than an LDS line
    assert lib.otter_hip_conv3x3_halo_plan(64, 64, 1, 0, 56, 56, 0, (C.c_int * 8)()) == -2
