"""``htgs_extract_ranges`` also writes the order in which the blend kernels take the tiles: groups of sixteen neighbouring
tiles (strips of four tile rows, column by column, cut into runs of sixteen), the groups with the longest lists first,
binned by total length with four bins per power of two, and a group's tiles at the workgroup indices that one
accelerator die is given (8 (16 p + t) + x).  The order must be a permutation of the tiles with that structure, and no
result may depend on it."""
import numpy as np
import pytest
import torch

from htgs_amd.synthetic import make_scene
from htgs_amd.torch_bindings import FrameBuffers, RasterizerMode
from util import u32

pytestmark = pytest.mark.gpu


def length_bin(length: np.ndarray) -> np.ndarray:
    """four bins per power of two; 0 for an empty list"""
    length = length.astype(np.int64)
    p = np.floor(np.log2(np.maximum(length, 1))).astype(np.int64)
    sub = np.where(p >= 2, (length >> np.maximum(p - 2, 0)) & 3, (length << np.maximum(2 - p, 0)) & 3)
    return np.where(length > 0, 4 * p + sub + 1, 0)


def strip_order(grid_w: int, grid_h: int) -> np.ndarray:
    """the tiles, strip by strip of four tile rows, column by column inside a strip"""
    out = []
    for y0 in range(0, grid_h, 4):
        rows = min(4, grid_h - y0)
        for x in range(grid_w):
            out.extend((y0 + r) * grid_w + x for r in range(rows))
    return np.array(out, np.int64)


def check_order(fb, mode):
    order = u32(fb.tile_order)[:fb.n_tiles].astype(np.int64)
    assert np.array_equal(np.sort(order), np.arange(fb.n_tiles))
    ranges = u32(fb.ranges).astype(np.int64)
    length = ranges[:, 1] - ranges[:, 0]
    tile = 16 if mode == 2 else 8
    grid_w, grid_h = -(-fb.width // tile), -(-fb.height // tile)
    strip = strip_order(grid_w, grid_h)
    assert np.array_equal(np.sort(strip), np.arange(fb.n_tiles))
    n_groups = fb.n_tiles // 16
    interleaved = n_groups // 8 * 8
    group_of_tile = np.empty(fb.n_tiles, np.int64)
    group_of_tile[strip] = np.arange(fb.n_tiles) // 16
    totals = []
    for place in range(n_groups):
        at = (8 * (16 * (place // 8) + np.arange(16)) + place % 8) if place < interleaved else 16 * place + np.arange(16)
        tiles = order[at]
        group = group_of_tile[tiles[0]]
        assert np.array_equal(tiles, strip[16 * group:16 * group + 16])        # one group, its tiles in strip order
        totals.append(length[tiles].sum())
    assert np.array_equal(order[16 * n_groups:], strip[16 * n_groups:])          # the tiles that fill no group
    if totals:
        assert (np.diff(length_bin(np.array(totals))) <= 0).all()


@pytest.mark.parametrize("config,n,mode", [(0, 10_000, 0), (1, 60_000, 0), (1, 60_000, 2), (3, 40_000, 0), (0, 0, 0)])
def test_order_is_a_permutation_with_the_longest_lists_first(cuda, config, n, mode):
    print(f"case config={config} n={n} mode={mode}", flush=True)
    scene = make_scene(config, max(n, 1))
    if n == 0:                                     # nothing visible: every list is empty
        scene.positions[:, 2] = -5.0
    scene = scene.to(cuda)
    fb = FrameBuffers(*scene.gaussians(), scene.settings(RasterizerMode(mode), 4), True, False)
    fb.run()
    torch.cuda.synchronize()
    check_order(fb, mode)


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_results_do_not_depend_on_the_order(cuda, mode):
    print(f"case mode={mode}", flush=True)
    scene = make_scene(1, 60_000).to(cuda)
    settings = scene.settings(RasterizerMode(mode), 16)
    with_order = FrameBuffers(*scene.gaussians(), settings, True, False)
    with_order.run()
    in_tile_order = FrameBuffers(*scene.gaussians(), settings, True, False, pool=None, order_tiles=False)
    in_tile_order.run()
    torch.cuda.synchronize()
    assert with_order.tile_order is not None and in_tile_order.tile_order is None
    assert torch.equal(with_order.image, in_tile_order.image)
    assert torch.equal(with_order.depth, in_tile_order.depth)


@pytest.mark.parametrize("width,height", [(8, 8), (24, 16), (100, 52), (130, 70), (33, 200)])
@pytest.mark.parametrize("mode", [0, 2])
def test_order_on_grids_that_fill_no_whole_groups_or_strips(cuda, width, height, mode):
    """Images whose tile grids have fewer than sixteen tiles, leave tiles over after the last whole group, or end in a strip
    of fewer than four tile rows: the order is still a permutation of the stated structure and changes nothing."""
    import dataclasses
    from htgs_amd.synthetic import pinhole
    print(f"case {width}x{height} mode={mode}", flush=True)
    scene = make_scene(0, 4000)
    M, VPM, cam = pinhole(width, height, 0.6 * width, 0.6 * width, width / 2, height / 2, scene.near_plane, scene.far_plane)
    scene = dataclasses.replace(scene, M=M, VPM=VPM, cam_position=cam, width=width, height=height).to(cuda)
    settings = scene.settings(RasterizerMode(mode), 4)
    fb = FrameBuffers(*scene.gaussians(), settings, True, False)
    fb.run()
    plain = FrameBuffers(*scene.gaussians(), settings, True, False, pool=None, order_tiles=False)
    plain.run()
    torch.cuda.synchronize()
    check_order(fb, mode)
    assert float(fb.image.max()) > 0.0
    assert torch.equal(fb.image, plain.image) and torch.equal(fb.depth, plain.depth)
