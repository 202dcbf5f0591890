"""The HIP path against the frozen known answers of tests/golden/small_scene.npz (float64, independent formulation;
see tests/golden/make_fixtures.py).  No CPU oracle is involved here: image and depth of rasterize() within the
contract's 1e-4 (depth, a few units large, 3e-4), gradients of diff_rasterize() and the densification statistics
within 1e-3 of the largest element, all four blend modes."""
import numpy as np
import pytest
import torch

from htgs_amd.torch_bindings import RasterizerMode, diff_rasterize, rasterize
from util import load_golden

pytestmark = pytest.mark.gpu

NAMES = ["positions", "scales", "rotations", "opacities", "sh_0", "sh_rest"]


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_rasterize_and_gradients_reproduce_the_frozen_answers(cuda, mode):
    sc, z = load_golden()
    K = int(z["K"])
    mask = z[f"mask_{mode}"]
    print(f"case mode={mode} K={K}", flush=True)
    sg = sc.to(cuda)
    settings = sg.settings(RasterizerMode(mode), K)
    image, depth = rasterize(*sg.gaussians(), settings, True, False)
    assert np.abs(image.cpu().numpy() - np.clip(z[f"image_{mode}"], 0.0, 1.0))[:, mask].max() <= 1e-4
    assert np.abs(depth.cpu().numpy()[0] - z[f"depth_{mode}"])[mask].max() <= 3e-4

    leaves = [t.clone().requires_grad_(True) for t in sg.gaussians()]
    info = torch.zeros((3, sc.positions.shape[0]), device=cuda)
    out = diff_rasterize(*leaves, info, settings, False)
    assert np.abs(out.detach().cpu().numpy() - z[f"image_{mode}"])[:, mask].max() <= 1e-4
    upstream = torch.from_numpy(z["grad_image"] * mask).to(cuda)
    (out * upstream).sum().backward()
    for name, leaf in zip(NAMES, leaves):
        want = z[f"grad_{name}_{mode}"].reshape(leaf.shape)
        scale = max(np.abs(want).max(), 1e-12)
        assert np.abs(leaf.grad.cpu().numpy() - want).max() / scale <= 1e-3, name
    # densification rows: visibility count, |dL/dposition|_2, and the sum over pixels of |dL_p/dposition|_1
    want_l1 = z[f"dens_l1_{mode}"]
    got = info.cpu().numpy()
    assert np.abs(got[2] - want_l1).max() / np.abs(want_l1).max() <= 1e-3
    want_l2 = np.linalg.norm(z[f"grad_positions_{mode}"], axis=1)
    assert np.abs(got[1] - want_l2).max() / np.abs(want_l2).max() <= 1e-3
