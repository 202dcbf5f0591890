"""The CPU oracle against the independent float64 evaluator (oracle/bruteforce.py) at the cameras and sizes of the
benchmark scenes, not only on toy scenes: the 3 M Gaussian / 1920x1080 / focal 1500 frame in all four modes, the stress
scene with its near-plane Gaussians (1600x1066, focal 35) and the 1 M training frame (unclamped image of the training
forward pass).  The cancellation in VPMT1 - x VPMT4 (R/include/hybrid_blend/kernels/inference.cuh:137-141) grows with the
pixel coordinate, so this is where the float32 evaluation is furthest from the exact one.

The dense evaluator cannot visit every (pixel, Gaussian) pair of such a frame, so it runs on small pixel patches against
the Gaussians near the patch's ray (a Euclidean pre-selection, ``bruteforce.near_ray``).  Pixels within 1e-4 (relative)
of a decision threshold are left out, as in the other float64 comparisons."""
import numpy as np
import pytest
import torch

import oracle
from oracle import bruteforce as bf
from htgs_amd.synthetic import make_scene
from util import oracle_frame, oracle_render

_scenes = {}


def scene(config, n):
    if (config, n) not in _scenes:
        _scenes.clear()                                     # one big scene at a time
        _scenes[(config, n)] = make_scene(config, n)
    return _scenes[(config, n)]


def patch_origins(sc, n_patches, size, seed):
    g = torch.Generator().manual_seed(seed)
    out = []
    for _ in range(n_patches):                              # denser towards the image centre, where the scenes are
        x0 = int(torch.clamp(torch.randn((), generator=g) * sc.width / 7 + sc.width / 2, 0, sc.width - size))
        y0 = int(torch.clamp(torch.randn((), generator=g) * sc.height / 7 + sc.height / 2, 0, sc.height - size))
        out.append((x0, y0))
    return out


def compare_on_patches(sc, mode, K, image, depth, n_patches, size, clamp):
    worst_i = worst_d = 0.0
    compared = total = most = 0
    for (x0, y0) in patch_origins(sc, n_patches, size, 100 + mode):
        ys, xs = torch.meshgrid(torch.arange(y0, y0 + size), torch.arange(x0, x0 + size), indexing="ij")
        pixels = torch.stack([xs.reshape(-1), ys.reshape(-1)], 1)
        near = bf.near_ray(sc.positions, sc.scales, sc.M, sc.VPM, (x0 + size / 2 - 0.5, y0 + size / 2 - 0.5), 0.75 * size + 1)
        fr = bf.evaluate(*[t[near] for t in sc.gaussians()], sc.M, sc.VPM, sc.cam_position, mode, sc.active_sh_bases,
                         sc.width, sc.height, sc.near_plane, sc.far_plane, pixels=pixels)
        img, dep, _, margin = bf.render(fr, mode, K, False, clamp=clamp)
        keep = (margin.reshape(-1) > 1e-4).numpy()
        most = max(most, int((fr.alpha >= bf.MIN_ALPHA[mode]).sum(1).max()))
        total += keep.size
        compared += int(keep.sum())
        if keep.any():
            worst_i = max(worst_i, float(np.abs(image[:, y0:y0 + size, x0:x0 + size].reshape(3, -1) - img.reshape(3, -1).numpy())[:, keep].max()))
            if depth is not None:
                worst_d = max(worst_d, float(np.abs(depth[y0:y0 + size, x0:x0 + size].reshape(-1) - dep.reshape(-1).numpy())[keep].max()))
    return worst_i, worst_d, compared / total, most


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_headline_frame_3m_gaussians_1080p(mode):
    sc = scene(2, None)
    ref = oracle_render(sc, mode, 16)
    err_i, err_d, share, most = compare_on_patches(sc, mode, 16, ref["image"], ref["depth"], 10, 10, True)
    print(f"mode {mode}: image {err_i:.2e} depth {err_d:.2e}, {share:.3f} of the pixels compared, up to {most} fragments per pixel")
    assert share > 0.9 and most > 150
    assert err_i <= 5e-5 and err_d <= 1e-4                  # depths are around 12


def test_stress_scene_with_near_plane_gaussians():
    sc = scene(3, 600_000)
    ref = oracle_render(sc, 0, 16)
    # focal 35: a pixel subtends 1.6 degrees, so the patches are small and many
    err_i, err_d, share, most = compare_on_patches(sc, 0, 16, ref["image"], ref["depth"], 40, 4, True)
    print(f"image {err_i:.2e} depth {err_d:.2e}, {share:.3f} of the pixels compared, up to {most} fragments per pixel")
    assert share > 0.9 and most > 150
    assert err_i <= 5e-5 and err_d <= 1e-4


def test_training_frame_1m_gaussians_1080p():
    sc = scene(4, None)
    fwd = oracle.forward(oracle_frame(sc, 0, 16), *[t.numpy() for t in sc.gaussians()])
    err_i, _, share, most = compare_on_patches(sc, 0, 16, fwd["image"], None, 10, 10, False)
    print(f"image {err_i:.2e}, {share:.3f} of the pixels compared, up to {most} fragments per pixel")
    assert share > 0.9 and most > 50
    assert err_i <= 5e-5
