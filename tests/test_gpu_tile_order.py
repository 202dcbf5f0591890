"""``htgs_extract_ranges`` also writes the order in which the blend kernels take the tiles: longest lists first, binned by
length with four bins per power of two.  The order must be a permutation of the tiles with non-increasing bins, and no
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
    order = u32(fb.tile_order)[:fb.n_tiles].astype(np.int64)
    assert np.array_equal(np.sort(order), np.arange(fb.n_tiles))
    ranges = u32(fb.ranges).astype(np.int64)
    bins = length_bin(ranges[order, 1] - ranges[order, 0])
    assert (np.diff(bins) <= 0).all()


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
