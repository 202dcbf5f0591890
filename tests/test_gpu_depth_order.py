"""ALPHA_BLEND_GLOBAL_ORDERING with the Gaussians sorted by depth before the instances are made (htgs_frame.depth_order):
the instance keys then hold the tile alone, and the stable sort by tile leaves every tile's list in the order of the
reference's sort of tile | depth keys (cub::DeviceRadixSort over both, R/src/alpha_blend_global_ordering/inference.cu:117-124).
The sorted primitive indices and the ranges must be the oracle's, the image the one of the frame with the reference's keys."""
import numpy as np
import pytest
import torch

from htgs_amd.synthetic import make_scene
from htgs_amd.torch_bindings import FrameBuffers, RasterizerMode, rasterize
from util import gpu_stages, oracle_render

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("config,n,K", [(0, 3000, 4), (1, 60_000, 16), (2, 200_000, 16), (3, 100_000, 16), (4, 50_000, 8)])
def test_depth_order_gives_the_reference_lists(cuda, config, n, K):
    print(f"case config={config} n={n} K={K}", flush=True)
    scene = make_scene(config, n)
    ref = oracle_render(scene, 2, K)
    got = gpu_stages(scene.to(cuda), 2, K, order_gaussians=True)
    keyed = gpu_stages(scene.to(cuda), 2, K, order_gaussians=False)
    assert got["fb"].key_bytes == 2 and keyed["fb"].key_bytes == 8
    assert got["n_instances"] == len(ref["keys"])
    np.testing.assert_array_equal(got["n_touched"], ref["pre"]["n_touched"])
    np.testing.assert_array_equal(got["sorted_vals"], ref["sorted_vals"])
    np.testing.assert_array_equal(got["sorted_keys"], ref["sorted_keys"] >> np.uint64(32))
    np.testing.assert_array_equal(got["ranges"], ref["ranges"])
    assert np.array_equal(got["image"], keyed["image"]) and np.array_equal(got["depth"], keyed["depth"])
    assert np.abs(got["image"] - ref["image"]).max() <= 1e-4 and np.abs(got["depth"] - ref["depth"]).max() <= 1e-4
    # offsets: the prefix sums of the counts in depth order (culled Gaussians last)
    fb = got["fb"]
    order = fb.depth_order[fb.lib.htgs_depth_order_result_word(fb._ref):][:n].cpu().numpy().view(np.uint32)
    depth = got["MT3"][:, 3]
    seen = got["n_touched"][order] > 0
    assert not seen[np.argmin(seen):].any() if not seen.all() else True
    d = depth[order][seen]
    assert (np.diff(d) >= 0).all()
    same = np.diff(d) == 0
    assert (np.diff(order[seen].astype(np.int64))[same] > 0).all()      # equal depths: ascending index (stable)
    np.testing.assert_array_equal(got["offsets"], np.cumsum(got["n_touched"][order].astype(np.uint64)).astype(np.uint32))


def test_depth_order_with_equal_depths(cuda):
    """Coincident Gaussians (equal depths by the thousand): the order inside a depth is the index order, as in the
    reference's stable sort of equal keys."""
    scene = make_scene(0, 1000)
    rep = lambda t: t.repeat(4, *([1] * (t.dim() - 1))).contiguous()
    import dataclasses
    g = torch.Generator().manual_seed(3)
    scene = dataclasses.replace(scene, name="cfg0-copies", positions=rep(scene.positions), scales=rep(scene.scales), rotations=rep(scene.rotations),
                                opacities=rep(scene.opacities), sh_0=(rep(scene.sh_0) + 0.3 * torch.randn(4000, *scene.sh_0.shape[1:], generator=g)).contiguous(),
                                sh_rest=rep(scene.sh_rest))
    ref = oracle_render(scene, 2, 4)
    got = gpu_stages(scene.to(cuda), 2, 4, order_gaussians=True)
    np.testing.assert_array_equal(got["sorted_vals"], ref["sorted_vals"])
    np.testing.assert_array_equal(got["ranges"], ref["ranges"])
    assert np.abs(got["image"] - ref["image"]).max() <= 1e-4


def test_depth_order_empty_and_all_culled(cuda):
    scene = make_scene(0, 500).to(cuda)
    s = scene.settings(RasterizerMode.ALPHA_BLEND_GLOBAL_ORDERING, 4)
    g = list(scene.gaussians())
    g[0] = g[0].clone(); g[0][:, 2] = -5.0                     # everything behind the camera
    image, depth = rasterize(*g, s, True, False)
    assert float(image.abs().max()) == 0.0
    empty = [t[:0].contiguous() for t in scene.gaussians()]
    image, depth = rasterize(*empty, s, True, False)
    assert float(image.abs().max()) == 0.0


def test_rasterize_takes_the_depth_order(cuda):
    scene = make_scene(1, 100_000).to(cuda)
    s = scene.settings(RasterizerMode.ALPHA_BLEND_GLOBAL_ORDERING, 16)
    fb = FrameBuffers(*scene.gaussians(), s, True, False)
    assert fb.depth_order is not None and fb.key_bytes == 2
    image, depth = rasterize(*scene.gaussians(), s, True, False)
    keyed = FrameBuffers(*scene.gaussians(), s, True, False, order_gaussians=False)
    keyed.run()
    torch.cuda.synchronize()
    assert torch.equal(image, keyed.image) and torch.equal(depth.reshape(keyed.depth.shape), keyed.depth)


@pytest.mark.parametrize("near,far", [(0.2, 1000.0), (1e-3, 1e6), (0.0, 100.0), (0.5, float("inf"))])
def test_depth_order_key_ranges(cuda, near, far):
    """The depth keys are taken relative to the near plane's bit pattern and are as wide as the far plane makes them
    (three or four digit passes); without a positive near plane or with an infinite far plane they are the full 32 bits."""
    import dataclasses
    print(f"case near={near} far={far}", flush=True)
    scene = dataclasses.replace(make_scene(0, 4000), near_plane=near, far_plane=far)
    ref = oracle_render(scene, 2, 8)
    got = gpu_stages(scene.to(cuda), 2, 8, order_gaussians=True)
    np.testing.assert_array_equal(got["sorted_vals"], ref["sorted_vals"])
    np.testing.assert_array_equal(got["ranges"], ref["ranges"])
    assert np.abs(got["image"] - ref["image"]).max() <= 1e-4


@pytest.mark.parametrize("n", [1, 5, 257, 4097])
def test_depth_order_small_counts(cuda, n):
    """Counts that are no multiple of the buffers' alignment or of a sort block."""
    print(f"case n={n}", flush=True)
    scene = make_scene(0, n)
    ref = oracle_render(scene, 2, 4)
    got = gpu_stages(scene.to(cuda), 2, 4, order_gaussians=True)
    assert got["n_instances"] == len(ref["keys"])
    np.testing.assert_array_equal(got["sorted_vals"], ref["sorted_vals"])
    np.testing.assert_array_equal(got["ranges"], ref["ranges"])
    assert np.abs(got["image"] - ref["image"]).max() <= 1e-4


def test_depth_that_is_not_a_number_sorts_behind_the_valid_ones(cuda):
    """A camera row with a NaN makes a Gaussian's depth NaN while its screen rectangle stays finite; the depth cull
    (``z < near || z > far``, R/include/kernel_utils.cuh:89-90) lets it through.  With the reference's tile | depth keys
    its bit pattern sorts behind every valid depth, equal patterns in index order; the frame with depth_order must list
    the same instances in the same order (its key is held just below the key of a culled Gaussian).  Also one NaN
    position, which both paths cull."""
    import dataclasses
    scene = make_scene(0, 3000)
    pos = scene.positions.clone()
    pos[17] = float("nan")
    scene = dataclasses.replace(scene, positions=pos)
    for nan_row in (False, True):
        print(f"case nan_row={nan_row}", flush=True)
        sc = scene
        if nan_row:
            M = scene.M.clone()
            M[2, 3] = float("nan")
            sc = dataclasses.replace(scene, M=M)
        got = gpu_stages(sc.to(cuda), 2, 4, order_gaussians=True)
        keyed = gpu_stages(sc.to(cuda), 2, 4, order_gaussians=False)
        assert got["n_instances"] == keyed["n_instances"] > 0
        np.testing.assert_array_equal(got["n_touched"], keyed["n_touched"])
        assert got["n_touched"][17] == 0
        np.testing.assert_array_equal(got["sorted_vals"], keyed["sorted_vals"])
        np.testing.assert_array_equal(got["ranges"], keyed["ranges"])
        assert np.array_equal(got["image"], keyed["image"], equal_nan=True)


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("config,n", [(0, 5000), (1, 60_000), (3, 60_000)])
def test_fast_path_lists_are_the_reference_lists_roughly_front_to_back(cuda, config, n, mode):
    """The image-only fast path of the two modes with a sorted core sorts the Gaussians by eight bits of their depth keys
    before the instances are made: every tile's list must hold exactly the instances of the oracle's list, and along a
    list the depths may fall only by what one step of the coarse keys is worth (a key step is at most 2^19 steps of the
    depth's bit pattern for near / far planes within the usual eight powers of two, 6.3 % of the depth)."""
    print(f"case config={config} n={n} mode={mode}", flush=True)
    scene = make_scene(config, n)
    ref = oracle_render(scene, mode, 16)
    sg = scene.to(cuda)
    fb = FrameBuffers(*sg.gaussians(), sg.settings(RasterizerMode(mode), 16), True, False, fast=True)
    assert fb.depth_order is not None
    fb.run()
    torch.cuda.synchronize()
    exact = FrameBuffers(*sg.gaussians(), sg.settings(RasterizerMode(mode), 16), True, False)
    assert exact.depth_order is None                                   # the exact path keeps the reference's order
    from util import u32
    assert fb.lib.htgs_frame_depth_sort_passes(fb._ref) == 1
    ranges = u32(fb.ranges).astype(np.int64)
    np.testing.assert_array_equal(ranges, ref["ranges"])
    vals = u32(fb.vals[fb.selector])[:fb.n_instances].astype(np.int64)
    assert len(vals) == len(ref["sorted_vals"])
    depth = ref["pre"]["MT3"][:, 3].astype(np.float64)                 # camera-space depth of the centre
    worst = 0.0
    for a, b in ranges[ranges[:, 1] > ranges[:, 0]]:
        assert np.array_equal(np.sort(vals[a:b]), ref["sorted_vals"][a:b].astype(np.int64))
        d = depth[vals[a:b]]
        worst = max(worst, float(np.max(np.maximum.accumulate(d) / d)))
    assert worst <= 1.07
    image = fb.image.cpu().numpy()
    diff = np.abs(image - ref["image"])
    assert float((diff > 1e-5).mean()) < 1e-3 and float(diff.max()) <= 5e-2


@pytest.mark.parametrize("near,far", [(1e-3, 1e6), (0.0, 100.0), (0.5, float("inf")), (3.0, 5.5)])
@pytest.mark.parametrize("n", [1, 300, 4097, 9000])
def test_fast_path_coarse_order_with_other_planes_and_counts(cuda, near, far, n):
    """The fast path's coarse depth keys for near / far planes that make the full keys wide (or 32 bits: no positive near
    plane, an infinite far plane) or narrow, and for counts that are no multiple of a sort block: every tile's list holds
    the oracle's instances, the lists run front to back up to what a key step is worth, the image stays within the fast
    path's bounds."""
    import dataclasses
    from util import u32
    print(f"case near={near} far={far} n={n}", flush=True)
    scene = dataclasses.replace(make_scene(0, n), near_plane=near, far_plane=far)
    ref = oracle_render(scene, 0, 8)
    sg = scene.to(cuda)
    fb = FrameBuffers(*sg.gaussians(), sg.settings(RasterizerMode(0), 8), True, False, fast=True)
    fb.run()
    torch.cuda.synchronize()
    ranges = u32(fb.ranges).astype(np.int64)
    np.testing.assert_array_equal(ranges, ref["ranges"])
    vals = u32(fb.vals[fb.selector])[:fb.n_instances].astype(np.int64) if fb.n_instances else np.zeros(0, np.int64)
    depth = ref["pre"]["MT3"][:, 3].astype(np.float64)
    # what one step of an eight-bit key is worth at most: the keys span the bit patterns from the near plane (or 0) to the far
    # plane (or the largest pattern), 2^23 patterns per power of two
    lo = np.float32(near).view(np.uint32) if near > 0.0 and np.isfinite(far) else np.uint32(0)
    hi = np.float32(far).view(np.uint32) if near > 0.0 and np.isfinite(far) else np.uint32(0xfffffffe)
    shift = 0
    while ((int(hi) - int(lo)) >> shift) + 1 >= 256:
        shift += 1
    step = 2.0 ** (shift - 23)                                          # relative to the depth, at most
    for a, b in ranges[ranges[:, 1] > ranges[:, 0]]:
        assert np.array_equal(np.sort(vals[a:b]), ref["sorted_vals"][a:b].astype(np.int64))
        d = depth[vals[a:b]]
        assert float(np.max(np.maximum.accumulate(d) / d)) <= (1.0 + step) * (1.0 + 1e-6) if step < 1.0 else True
    diff = np.abs(fb.image.cpu().numpy() - ref["image"])
    assert float((diff > 1e-5).mean()) < 1e-3 and float(diff.max()) <= 5e-2
