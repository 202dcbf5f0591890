"""Pins the oracle's training path (forward records + backward): gradients against torch.autograd through the
independent float64 evaluator (oracle/bruteforce.py), which knows nothing of the reference's hand-derived chain
rule; linearity in the upstream gradient; zero gradients for culled Gaussians; the densification side outputs
against their definition (R/include/hybrid_blend/kernels/backward.cuh:85-98,306)."""
import numpy as np
import pytest
import torch

import oracle
from oracle import bruteforce as bf
from test_oracle_pinning import small_scene
from util import oracle_frame

NAMES = ["positions", "scales", "rotations", "opacities", "sh_0", "sh_rest"]


def autograd_reference(sc, mode, K, grad_image):
    leaves = [t.double().clone().requires_grad_(True) for t in sc.gaussians()]
    frags = bf.evaluate(*leaves, sc.M, sc.VPM, sc.cam_position, mode, sc.active_sh_bases, sc.width, sc.height,
                        sc.near_plane, sc.far_plane)
    img, _, _, margin = bf.render(frags, mode, K, False, clamp=False)
    mask = (margin > 1e-4)
    (img * grad_image.double() * mask.double()).sum().backward()
    return img.detach(), mask, [l.grad for l in leaves]


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
@pytest.mark.parametrize("K,sh_degree", [(4, 2), (16, 3), (1, 0)])
def test_backward_matches_float64_autograd(mode, K, sh_degree):
    sc = small_scene(n=70, seed=31 + mode + K, sh_degree=sh_degree)
    arrays = [t.numpy() for t in sc.gaussians()]
    fwd = oracle.forward(oracle_frame(sc, mode, K), *arrays)
    gi = torch.randn(3, sc.height, sc.width, generator=torch.Generator().manual_seed(1))
    img, mask, want = autograd_reference(sc, mode, K, gi)
    assert mask.float().mean() > 0.97
    assert np.abs(fwd["image"] - img.numpy())[:, mask.numpy()].max() < 2e-5
    got = oracle.backward(fwd, (gi * mask.float()).numpy(), *arrays)
    for name, w in zip(NAMES, want):
        g = got[name]
        if w is None or g.size == 0:          # sh_rest of an SH-degree-0 scene has no elements
            continue
        w = w.numpy().reshape(g.shape)
        scale = max(np.abs(w).max(), 1e-12)
        assert np.abs(g - w).max() / scale < 2e-5, (name, np.abs(g - w).max(), scale)


def test_backward_is_linear_in_the_upstream_gradient_and_ignores_culled_gaussians():
    sc = small_scene(n=80, seed=5)
    sc.positions[:10] = sc.positions[:10] * 0 + torch.tensor([0.0, 0.0, -30.0])        # behind the camera
    arrays = [t.numpy() for t in sc.gaussians()]
    fwd = oracle.forward(oracle_frame(sc, 0, 4), *arrays)
    g = torch.Generator().manual_seed(2)
    a, b = torch.randn(3, sc.height, sc.width, generator=g).numpy(), torch.randn(3, sc.height, sc.width, generator=g).numpy()
    ga, gb, gab = (oracle.backward(fwd, x, *arrays) for x in (a, b, 2 * a - 3 * b))
    for name in NAMES:
        np.testing.assert_allclose(gab[name], 2 * ga[name] - 3 * gb[name], rtol=0, atol=2e-4 * max(1.0, np.abs(gab[name]).max()))
        assert (ga[name][:10] == 0).all()


def test_densification_side_outputs():
    sc = small_scene(n=60, seed=9)
    arrays = [t.numpy() for t in sc.gaussians()]
    fwd = oracle.forward(oracle_frame(sc, 0, 4), *arrays)
    gi = torch.randn(3, sc.height, sc.width, generator=torch.Generator().manual_seed(3)).numpy()
    n = 60
    vis = fwd["pre"]["n_touched"] > 0
    z = (sc.positions.numpy() @ sc.M.numpy()[2, :3] + sc.M.numpy()[2, 3])
    for rows, scaling in [(2, False), (3, False), (3, True)]:
        info = np.full((rows, n), 0.5, np.float32)
        grads = oracle.backward(fwd, gi, *arrays, densification_info=info, use_distance_scaling=scaling)
        zs = z * 0.5 if scaling else np.ones(n)
        np.testing.assert_allclose(info[0], 0.5 + vis, rtol=0, atol=0)
        np.testing.assert_allclose(info[1], 0.5 + vis * np.linalg.norm(grads["positions"] * zs[:, None], axis=1), rtol=1e-5, atol=1e-6)
        if rows == 3:
            assert (info[2][vis] >= 0.5).all() and (info[2][~vis] == 0.5).all()


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
@pytest.mark.parametrize("scaling", [False, True])
def test_third_densification_row_is_the_per_pixel_l1_norm_of_the_position_gradient(mode, scaling):
    """Row 2 of densification_info accumulates, per Gaussian, z_scale * sum over pixels of |dL_p/dposition|_1 with L_p
    the loss carried by pixel p alone (R/include/hybrid_blend/kernels/backward.cuh:292-306,95).  Pinned on a
    12-Gaussian SH-0 scene (no view-dependent colour) by one float64 autograd pass per pixel through the independent
    evaluator: a factor, a sign convention or a dropped component in the hand-derived chain fails this."""
    sc = small_scene(n=12, seed=77 + mode, sh_degree=0, width=32, height=24, focal=40.0, scale=(0.1, 0.4))
    arrays = [t.numpy() for t in sc.gaussians()]
    K = 4
    fwd = oracle.forward(oracle_frame(sc, mode, K), *arrays)
    gi = torch.randn(3, sc.height, sc.width, generator=torch.Generator().manual_seed(5))
    frags = bf.evaluate(*sc.gaussians(), sc.M, sc.VPM, sc.cam_position, mode, sc.active_sh_bases, sc.width, sc.height,
                        sc.near_plane, sc.far_plane)
    mask = (bf.render(frags, mode, K, False, clamp=False)[3] > 1e-4)
    assert mask.float().mean() > 0.97
    gi = gi * mask.float()
    want = bf.per_fragment_position_gradient_l1(*sc.gaussians(), sc.M, sc.VPM, sc.cam_position, mode, sc.active_sh_bases,
                                                sc.width, sc.height, sc.near_plane, sc.far_plane, K, gi).numpy()
    z = (sc.positions.double().numpy() @ sc.M.double().numpy()[2, :3] + float(sc.M[2, 3]))
    want = want * (0.5 * z if scaling else 1.0)
    info = np.zeros((3, 12), np.float32)
    oracle.backward(fwd, gi.numpy(), *arrays, densification_info=info, use_distance_scaling=scaling)
    assert np.abs(want).max() > 1.0 and (want > 0).sum() >= 8
    assert np.abs(info[2] - want).max() <= 1e-4 * np.abs(want).max(), (info[2], want)


def faint_tail_scene(K: int, seed: int):
    """K fairly opaque Gaussians over the middle of the image in front of six large ones whose alpha stays between
    1/255 and 1/100: the case in which the colour sums of the hybrid tail (all fragments added, the core's share
    subtracted at the end) cancel most."""
    sc = small_scene(n=K + 6, seed=seed, sh_degree=1, width=32, height=24, focal=40.0, scale=(0.35, 0.55), z_range=(2.2, 3.0))
    g = torch.Generator().manual_seed(seed + 1)
    z = sc.positions @ sc.M[2, :3] + sc.M[2, 3]
    centre = sc.cam_position[None, :] + z[:, None] * sc.M[2, :3][None, :]
    sc.positions[:K] = centre[:K] + 0.4 * (sc.positions[:K] - centre[:K])
    sc.opacities[:K] = 0.1 + 0.5 * torch.rand(K, 1, generator=g)
    sc.opacities[K:] = 0.0045 + 0.0045 * torch.rand(6, 1, generator=g)
    sc.scales[K:] *= 3.0
    sc.positions[K:] += (7.0 - z[K:, None]) * sc.M[2, :3][None, :]                    # the faint ones behind the core
    return sc


@pytest.mark.parametrize("K", [4, 16])
def test_hybrid_tail_with_a_strong_core_and_a_faint_tail(K):
    """Image and gradients of HYBRID_BLEND against the float64 evaluator where the tail's colour sums are the small
    difference of two large ones (every fragment's alpha * colour is added when it is evaluated and the K core entries'
    share is taken out after the walk; the reference, R/include/hybrid_blend/kernels/inference.cuh:158-170, only ever
    adds what is outside the core)."""
    sc = faint_tail_scene(K, 100 + K)
    arrays = [t.numpy() for t in sc.gaussians()]
    fwd = oracle.forward(oracle_frame(sc, 0, K), *arrays)
    tail = fwd["tail_info"].reshape(6, -1)
    alpha_sum = 1.0 / np.maximum(tail[3], 1e-30)
    in_core = (fwd["core_idx"].reshape(K, -1) != 0xffffffff).sum(0)
    faint = (tail[3] > 0) & (alpha_sum < 0.1) & (tail[5] > 0.01) & (in_core >= min(K, 3))
    assert faint.mean() > 0.15, "the scene is meant to have faint tails behind a partly transparent core"
    assert (tail[:3] >= 0).all()
    gi = torch.randn(3, sc.height, sc.width, generator=torch.Generator().manual_seed(1))
    img, mask, want = autograd_reference(sc, 0, K, gi)
    assert mask.float().mean() > 0.9
    assert np.abs(fwd["image"] - img.numpy())[:, mask.numpy()].max() < 2e-5
    got = oracle.backward(fwd, (gi * mask.float()).numpy(), *arrays)
    for name, w in zip(NAMES, want):
        g = got[name]
        w = w.numpy().reshape(g.shape)
        scale = max(np.abs(w).max(), 1e-12)
        assert np.abs(g - w).max() / scale < 5e-5, (name, np.abs(g - w).max(), scale)
