"""The second HYBRID inference kernel, which takes the tiles whose lists are longer than ``long_list_threshold``: a
workgroup of waves splits the list, the K-buffers and tails are merged, and pixels at which fragments of exactly equal
depth met are walked again in one piece.  The threshold is forced down so that small scenes go through it; the result
must stay within the rasterizer's 1e-4 of the CPU oracle (whose walk is the reference's single one,
R/include/hybrid_blend/kernels/inference.cuh:70-213) and close to this library's own single-wave kernel."""
import dataclasses

import numpy as np
import pytest
import torch

from htgs_amd.synthetic import make_scene
from htgs_amd.torch_bindings import FrameBuffers, RasterizerMode
from util import oracle_render

pytestmark = pytest.mark.gpu

TOL = 1e-4
NEVER = 2 ** 31 - 1
SECOND_LOOKS = []


def render(scene_gpu, K, threshold, to_chw=True, median=False, fast=False, in_parts=None, mode=RasterizerMode.HYBRID_BLEND, part_rows=None):
    fb = FrameBuffers(*scene_gpu.gaussians(), scene_gpu.settings(mode, K), to_chw, median, fast=fast, long_list_threshold=threshold)
    fb.front()
    fb.alloc_instances(fb.read_instance_count())
    fb.create_instances()
    fb.selector = fb.sort()
    fb.extract_ranges()
    ranges = fb.ranges.to(torch.int64)
    lengths = ranges[:, 1] - ranges[:, 0]
    long_tiles = int((lengths > (threshold if threshold else 8192)).sum())
    fb.blend()
    torch.cuda.synchronize()
    if in_parts is not None:                      # lists long enough to be walked in parts by several workgroups
        part = max(4 * threshold, (part_rows or 3 * K + 7) * 64)
        assert (int((lengths >= 2 * part).sum()) > 0) == in_parts, f"longest list {int(lengths.max())}, a part {part}"
    assert not bool(fb.long_tiles[:6].any())      # the blend stage leaves the list empty for its next call
    # tiles with pixels at which depths coincided: settled by a second look at those pixels / walked again in one piece
    # (of the latter, third number: after a second look for which the room did not do)
    SECOND_LOOKS.append((int(fb.long_tiles[6]), int(fb.long_tiles[7]) & 0xffff, int(fb.long_tiles[7]) >> 16))
    image, depth = fb.image.clone(), None if fast else fb.depth.clone()
    fb.image.zero_()
    fb.blend()                                    # again, without htgs_extract_ranges in between
    torch.cuda.synchronize()
    assert torch.equal(fb.image, image) and (fast or torch.equal(fb.depth, depth))
    return image.cpu().numpy(), None if fast else depth.cpu().numpy(), long_tiles


def with_coincident_copies(scene, copies):
    """Every Gaussian ``copies`` times at the same place with the same shape (so every fragment meets fragments of
    exactly its own depth at every pixel) but other colours and opacities."""
    g = torch.Generator().manual_seed(11)
    rep = lambda t: t.repeat(copies, *([1] * (t.dim() - 1))).contiguous()
    n = scene.positions.shape[0] * copies
    return dataclasses.replace(
        scene, name=scene.name + "-coincident", positions=rep(scene.positions), scales=rep(scene.scales), rotations=rep(scene.rotations),
        opacities=(rep(scene.opacities) + 0.5 * torch.randn(n, *scene.opacities.shape[1:], generator=g)).contiguous(),
        sh_0=(rep(scene.sh_0) + 0.3 * torch.randn(n, *scene.sh_0.shape[1:], generator=g)).contiguous(), sh_rest=rep(scene.sh_rest))


@pytest.mark.parametrize("config,n,K,threshold", [(0, 3000, 4, 64), (0, 3000, 1, 24), (1, 60_000, 16, 16), (2, 100_000, 32, 20),
                                                    (3, 150_000, 16, 1000)])
def test_long_tiles_against_oracle(cuda, config, n, K, threshold):
    print(f"case config={config} n={n} K={K} threshold={threshold}", flush=True)
    scene = make_scene(config, n)
    ref = oracle_render(scene, 0, K)
    image, depth, long_tiles = render(scene.to(cuda), K, threshold)
    single, single_depth, none = render(scene.to(cuda), K, NEVER)
    assert long_tiles > 0 and none == 0
    err = [float(np.abs(image - ref["image"]).max()), float(np.abs(depth - ref["depth"]).max()),
           float(np.abs(image - single).max()), float(np.abs(depth - single_depth).max())]
    print(f"  long tiles {long_tiles}; against the oracle {err[0]:.3g} / {err[1]:.3g}, against the single walk {err[2]:.3g} / {err[3]:.3g}", flush=True)
    assert max(err) <= TOL


@pytest.mark.parametrize("to_chw,median", [(False, False), (True, True), (False, True)])
def test_long_tiles_layout_and_median_depth(cuda, to_chw, median):
    print(f"case to_chw={to_chw} median={median}", flush=True)
    scene = make_scene(0, 3000)
    ref = oracle_render(scene, 0, 4, to_chw=to_chw, median=median)
    image, depth, long_tiles = render(scene.to(cuda), 4, 64, to_chw, median)
    assert long_tiles > 0 and image.shape == ref["image"].shape
    assert np.abs(image - ref["image"]).max() <= TOL
    assert np.abs(depth - ref["depth"]).max() <= TOL


def with_some_twins(scene, n_twins):
    """``n_twins`` of the Gaussians once more at the same place with the same shape but other colours and opacities: a few
    pixels per tile get two fragments of exactly equal depth."""
    g = torch.Generator().manual_seed(12)
    pick = torch.randperm(scene.positions.shape[0], generator=g)[:n_twins]
    both = lambda t: torch.cat([t, t[pick]]).contiguous()
    opacities, sh_0 = both(scene.opacities), both(scene.sh_0)
    opacities[-n_twins:] = (opacities[-n_twins:] * 0.7 + 0.1)
    sh_0[-n_twins:] += 0.3 * torch.randn(sh_0[-n_twins:].shape, generator=g)
    return dataclasses.replace(scene, name=scene.name + "-twins", positions=both(scene.positions), scales=both(scene.scales),
                               rotations=both(scene.rotations), opacities=opacities, sh_0=sh_0, sh_rest=both(scene.sh_rest))


@pytest.mark.parametrize("config,n,K,threshold,twins", [(0, 3000, 4, 24, 150), (3, 150_000, 16, 1000, 300), (3, 150_000, 4, 200, 300)])
def test_long_tiles_second_look_at_a_few_pixels(cuda, config, n, K, threshold, twins):
    """Few pixels of a tile with fragments of equal depth: every wave looks at them again, lanes = instances, and the
    insertion is replayed on the fragments that decide their cores."""
    print(f"case config={config} n={n} K={K} threshold={threshold} twins={twins}", flush=True)
    scene = with_some_twins(make_scene(config, n), twins)
    ref = oracle_render(scene, 0, K)
    image, depth, long_tiles = render(scene.to(cuda), K, threshold)
    second_looks, walked_again, _ = SECOND_LOOKS[-1]
    err_i, err_d = float(np.abs(image - ref["image"]).max()), float(np.abs(depth - ref["depth"]).max())
    print(f"  long tiles {long_tiles}, second looks {second_looks}, walked again {walked_again}; against the oracle {err_i:.3g} / {err_d:.3g}", flush=True)
    assert second_looks > 0
    assert err_i <= TOL and err_d <= TOL


@pytest.mark.parametrize("K", [4, 16])
def test_long_tiles_with_fragments_of_equal_depth(cuda, K):
    """Coincident Gaussians: which of two stored fragments of equal depth leaves the core depends on the order of arrival in
    the reference's insertion, so the merged cores are not enough and the pixels are walked again in list order."""
    print(f"case K={K} (coincident copies)", flush=True)
    scene = with_coincident_copies(make_scene(0, 1500), 6)
    ref = oracle_render(scene, 0, K)
    image, depth, long_tiles = render(scene.to(cuda), K, 64)
    assert long_tiles > 0 and SECOND_LOOKS[-1][1] > 0
    err_i, err_d = float(np.abs(image - ref["image"]).max()), float(np.abs(depth - ref["depth"]).max())
    print(f"  long tiles {long_tiles}; against the oracle {err_i:.3g} / {err_d:.3g}", flush=True)
    assert err_i <= TOL and err_d <= TOL


@pytest.mark.parametrize("n,K,threshold,copies", [(150_000, 4, 200, 1), (150_000, 1, 64, 1), (300_000, 16, 500, 1), (30_000, 4, 200, 5)])
def test_long_tiles_walked_in_parts(cuda, n, K, threshold, copies):
    """Lists of many times the threshold are entered in parts, each walked by a workgroup of its own; the one that
    finishes last merges what the parts left (in the tile's stretch of the spare value buffer) and ends the tile."""
    print(f"case n={n} K={K} threshold={threshold} copies={copies} (parts)", flush=True)
    scene = make_scene(3, n)
    if copies > 1:
        scene = with_coincident_copies(scene, copies)
    ref = oracle_render(scene, 0, K)
    image, depth, long_tiles = render(scene.to(cuda), K, threshold, in_parts=True)
    err_i, err_d = float(np.abs(image - ref["image"]).max()), float(np.abs(depth - ref["depth"]).max())
    print(f"  long tiles {long_tiles}; against the oracle {err_i:.3g} / {err_d:.3g}", flush=True)
    assert err_i <= TOL and err_d <= TOL
    if copies == 1:
        # the fast variant neither walks pixels with equal depths again nor promises which of two fragments of exactly equal
        # depth stays in front (its insertion is the stable one, the merge of the shares the reference's exchange walk):
        # the few pixels of this scene at which depths coincide may differ by what the core's gate is worth
        fast, _, _ = render(scene.to(cuda), K, threshold, fast=True)
        single, _, _ = render(scene.to(cuda), K, NEVER, fast=True)
        diff = np.abs(fast - single).max(axis=0)
        assert (diff > TOL).sum() <= 1e-5 * diff.size and diff.max() <= 5e-2


def test_long_tiles_with_depths_that_coincide_by_the_hundred(cuda):
    """A few pixels with so many fragments as deep as their core's last entry that these do not fit the room the second
    look has for them: the pixels are then walked again in one piece."""
    print("case a few tiny Gaussians 400 times each", flush=True)
    scene = make_scene(0, 3000)
    g = torch.Generator().manual_seed(13)
    pick = torch.randperm(3000, generator=g)[:6]
    often = lambda t: torch.cat([t, t[pick].repeat(400, *([1] * (t.dim() - 1)))]).contiguous()
    scales, sh_0 = often(scene.scales), often(scene.sh_0)
    scales[3000:] = 2e-4                                    # a pixel or two each
    sh_0[3000:] += 0.3 * torch.randn(sh_0[3000:].shape, generator=g)
    scene = dataclasses.replace(scene, name=scene.name + "-heaps", positions=often(scene.positions), scales=scales, rotations=often(scene.rotations),
                                opacities=often(scene.opacities), sh_0=sh_0, sh_rest=often(scene.sh_rest))
    ref = oracle_render(scene, 0, 4)
    image, depth, long_tiles = render(scene.to(cuda), 4, 64)
    print(f"  second looks {SECOND_LOOKS[-1][0]}, walked again {SECOND_LOOKS[-1][1]}, of these for want of room {SECOND_LOOKS[-1][2]}", flush=True)
    assert long_tiles > 0 and SECOND_LOOKS[-1][2] > 0
    err_i, err_d = float(np.abs(image - ref["image"]).max()), float(np.abs(depth - ref["depth"]).max())
    print(f"  long tiles {long_tiles}; against the oracle {err_i:.3g} / {err_d:.3g}", flush=True)
    assert err_i <= TOL and err_d <= TOL


def test_long_tiles_fast_variant(cuda):
    """The variant without depth and with the hardware's reciprocal / exponential: same fragments, same sums up to their order."""
    print("case fast", flush=True)
    scene = make_scene(1, 60_000).to(cuda)
    image, _, long_tiles = render(scene, 16, 16, fast=True)
    single, _, none = render(scene, 16, NEVER, fast=True)
    assert long_tiles > 0 and none == 0
    assert np.abs(image - single).max() <= TOL


@pytest.mark.parametrize("config,n,threshold,in_parts,to_chw", [(0, 3000, 24, False, True), (1, 60_000, 16, False, False), (3, 150_000, 500, True, True),
                                                                 (3, 150_000, 100, True, False)])
def test_long_tiles_oit(cuda, config, n, threshold, in_parts, to_chw):
    """OIT_BLEND: the sums of the waves' shares, and of the parts of a list, add up in list order."""
    print(f"case OIT config={config} n={n} threshold={threshold}", flush=True)
    oit = RasterizerMode.OIT_BLEND
    scene = make_scene(config, n)
    ref = oracle_render(scene, 3, 16, to_chw=to_chw)
    image, depth, long_tiles = render(scene.to(cuda), 16, threshold, to_chw=to_chw, in_parts=in_parts, mode=oit, part_rows=6)
    single, single_depth, none = render(scene.to(cuda), 16, NEVER, to_chw=to_chw, mode=oit)
    assert long_tiles > 0 and none == 0
    err = [float(np.abs(image - ref["image"]).max()), float(np.abs(depth - ref["depth"]).max()),
           float(np.abs(image - single).max()), float(np.abs(depth - single_depth).max())]
    print(f"  long tiles {long_tiles}; against the oracle {err[0]:.3g} / {err[1]:.3g}, against the single walk {err[2]:.3g} / {err[3]:.3g}", flush=True)
    assert max(err) <= TOL
    fast, _, _ = render(scene.to(cuda), 16, threshold, to_chw=to_chw, fast=True, mode=oit)
    single_fast, _, _ = render(scene.to(cuda), 16, NEVER, to_chw=to_chw, fast=True, mode=oit)
    assert np.abs(fast - single_fast).max() <= TOL


FIRST_K = RasterizerMode.ALPHA_BLEND_FIRST_K


@pytest.mark.parametrize("config,n,K,threshold,in_parts,median", [(0, 3000, 4, 24, None, False), (0, 3000, 1, 24, None, True), (1, 60_000, 16, 16, None, False),
                                                                   (2, 100_000, 32, 20, None, True), (3, 150_000, 4, 200, True, False),
                                                                   (3, 300_000, 16, 500, True, False)])
def test_long_tiles_first_k(cuda, config, n, K, threshold, in_parts, median):
    """ALPHA_BLEND_FIRST_K: the cores of the waves' shares, and of the parts of a list, merged in list order."""
    print(f"case FIRST_K config={config} n={n} K={K} threshold={threshold}", flush=True)
    scene = make_scene(config, n)
    ref = oracle_render(scene, 1, K, median=median)
    image, depth, long_tiles = render(scene.to(cuda), K, threshold, median=median, in_parts=in_parts, mode=FIRST_K, part_rows=3 * K + 1)
    single, single_depth, none = render(scene.to(cuda), K, NEVER, median=median, mode=FIRST_K)
    assert long_tiles > 0 and none == 0
    err = [float(np.abs(image - ref["image"]).max()), float(np.abs(depth - ref["depth"]).max()),
           float(np.abs(image - single).max()), float(np.abs(depth - single_depth).max())]
    print(f"  long tiles {long_tiles}; against the oracle {err[0]:.3g} / {err[1]:.3g}, against the single walk {err[2]:.3g} / {err[3]:.3g}", flush=True)
    assert max(err) <= TOL
    fast, _, _ = render(scene.to(cuda), K, threshold, fast=True, mode=FIRST_K)
    single_fast, _, _ = render(scene.to(cuda), K, NEVER, fast=True, mode=FIRST_K)
    assert np.abs(fast - single_fast).max() <= TOL


@pytest.mark.parametrize("config,n,K,threshold,twins,copies", [(0, 3000, 4, 24, 150, 1), (3, 150_000, 16, 1000, 300, 1), (0, 1500, 4, 64, 0, 6),
                                                                (0, 1500, 16, 64, 0, 6)])
def test_long_tiles_first_k_with_fragments_of_equal_depth(cuda, config, n, K, threshold, twins, copies):
    """A few twins: the pixels get a second look and the insertion is replayed; coincident copies of everything: the first
    wave walks the list again."""
    print(f"case FIRST_K config={config} n={n} K={K} threshold={threshold} twins={twins} copies={copies}", flush=True)
    scene = make_scene(config, n)
    scene = with_some_twins(scene, twins) if twins else with_coincident_copies(scene, copies)
    ref = oracle_render(scene, 1, K)
    image, depth, long_tiles = render(scene.to(cuda), K, threshold, mode=FIRST_K)
    second_looks, walked_again, _ = SECOND_LOOKS[-1]
    err_i, err_d = float(np.abs(image - ref["image"]).max()), float(np.abs(depth - ref["depth"]).max())
    print(f"  long tiles {long_tiles}, second looks {second_looks}, walked again {walked_again}; against the oracle {err_i:.3g} / {err_d:.3g}", flush=True)
    assert long_tiles > 0 and (second_looks > 0 if twins else walked_again > 0)
    assert err_i <= TOL and err_d <= TOL


@pytest.mark.parametrize("mode,K", [(0, 1), (1, 1), (3, 1), (0, 16)])
def test_long_tiles_on_a_grid_of_four_tiles(cuda, mode, K):
    """A 16x16 image: the parts that lists may be walked in beyond one per tile are held to the number of tiles, which
    here is four."""
    import dataclasses
    print(f"case mode={mode} K={K} (16x16 image)", flush=True)
    scene = make_scene(0, 300_000)
    positions = scene.positions.clone()
    positions[:, :2] -= 1.6                                 # (the cloud's centre projects to the image's corner, which is the new image)
    scene = dataclasses.replace(scene, positions=positions, width=16, height=16)
    m = RasterizerMode(mode)
    ref = oracle_render(scene, mode, K)
    image, depth, long_tiles = render(scene.to(cuda), K, 64, mode=m)
    single, single_depth, none = render(scene.to(cuda), K, NEVER, mode=m)
    assert long_tiles > 0 and none == 0
    err = [float(np.abs(image - ref["image"]).max()), float(np.abs(depth - ref["depth"]).max()),
           float(np.abs(image - single).max()), float(np.abs(depth - single_depth).max())]
    print(f"  long tiles {long_tiles}; against the oracle {err[0]:.3g} / {err[1]:.3g}, against the single walk {err[2]:.3g} / {err[3]:.3g}", flush=True)
    assert max(err) <= TOL
