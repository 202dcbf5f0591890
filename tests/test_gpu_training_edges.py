"""Training path on awkward inputs, and the determinism of its gradients."""
import dataclasses

import numpy as np
import pytest
import torch

import oracle
from htgs_amd.synthetic import make_scene
from htgs_amd.torch_bindings import FrameBuffers, RasterizerMode, diff_rasterize
from util import oracle_frame
from test_gpu_edge_cases import resized
from test_gpu_training import NAMES, assert_grad_close

pytestmark = pytest.mark.gpu


def run_both(scene, mode, K, cuda, seed=3):
    arrays = [t.numpy() for t in scene.gaussians()]
    fwd = oracle.forward(oracle_frame(scene, mode, K), *arrays)
    grad_image = torch.randn(3, scene.height, scene.width, generator=torch.Generator().manual_seed(seed))
    want = oracle.backward(fwd, grad_image.numpy(), *arrays)
    sg = scene.to(cuda)
    fb = FrameBuffers(*sg.gaussians(), sg.settings(RasterizerMode(mode), K), True, False, train=True)
    image = fb.run_forward()
    grads = fb.run_backward(grad_image.to(cuda))
    torch.cuda.synchronize()
    return fwd, want, image, grads


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_nothing_to_draw(cuda, mode):
    """No Gaussians at all, and Gaussians that are all behind the camera: zero image, zero gradients of the right shapes."""
    scene = make_scene(0, 50)
    empty = dataclasses.replace(scene, positions=scene.positions[:0], scales=scene.scales[:0], rotations=scene.rotations[:0],
                                opacities=scene.opacities[:0], sh_0=scene.sh_0[:0], sh_rest=scene.sh_rest[:0])
    behind = dataclasses.replace(scene, positions=scene.positions * torch.tensor([1.0, 1.0, -1.0]))
    for sc in (empty, behind):
        print(f"case mode={mode} n={sc.positions.shape[0]}", flush=True)
        g = sc.to(cuda)
        leaves = [t.clone().requires_grad_(True) for t in g.gaussians()]
        info = torch.zeros(3, sc.positions.shape[0], device=cuda)
        image = diff_rasterize(*leaves, info, g.settings(RasterizerMode(mode), 4), True)
        assert float(image.detach().abs().max()) == 0.0
        (image * 2.0).sum().backward()
        for leaf in leaves:
            assert leaf.grad is not None and leaf.grad.shape == leaf.shape and float(leaf.grad.abs().sum()) == 0.0
        assert float(info.abs().sum()) == 0.0


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_ragged_image_and_full_grid_gaussian(cuda, mode):
    scene = resized(make_scene(0, 1500), 203, 117, 180.0)
    scene.scales[0] = torch.tensor([20.0, 20.0, 0.05])
    scene.positions[0] = torch.tensor([0.0, 0.0, 6.0])
    scene.rotations[0] = torch.tensor([1.0, 0.0, 0.0, 0.0])
    scene.opacities[0] = 0.5
    print(f"case mode={mode}", flush=True)
    fwd, want, image, grads = run_both(scene, mode, 8, cuda)
    assert np.abs(image.cpu().numpy() - fwd["image"]).max() <= 1e-4
    for name, got in zip(NAMES, grads):
        assert_grad_close(name, got.cpu().numpy(), want[name])


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_gradients_are_deterministic(cuda, mode):
    """Every mode writes one gradient row per (Gaussian, tile) instance and sums a Gaussian's rows in a fixed order:
    two runs give the same bits."""
    scene = make_scene(1, 40_000)
    print(f"case mode={mode}", flush=True)
    _, _, _, first = run_both(scene, mode, 16, cuda)
    _, _, _, second = run_both(scene, mode, 16, cuda)
    for name, a, b in zip(NAMES, first, second):
        assert torch.equal(a, b), name
