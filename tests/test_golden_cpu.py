"""The CPU oracle against the frozen known answers of tests/golden/small_scene.npz (float64, independent
formulation; see tests/golden/make_fixtures.py): image, depth and the six gradients, all four blend modes."""
import numpy as np
import pytest

import oracle
from util import load_golden, oracle_frame

NAMES = ["positions", "scales", "rotations", "opacities", "sh_0", "sh_rest"]


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_oracle_reproduces_the_frozen_float64_answers(mode):
    sc, z = load_golden()
    K = int(z["K"])
    arrays = [t.numpy() for t in sc.gaussians()]
    mask = z[f"mask_{mode}"]
    assert mask.mean() > 0.97
    out = oracle.render(oracle_frame(sc, mode, K), *arrays)
    assert np.abs(out["image"] - np.clip(z[f"image_{mode}"], 0.0, 1.0))[:, mask].max() < 2e-5
    assert np.abs(out["depth"] - z[f"depth_{mode}"])[mask].max() < 2e-4
    fwd = oracle.forward(oracle_frame(sc, mode, K), *arrays)
    assert np.abs(fwd["image"] - z[f"image_{mode}"])[:, mask].max() < 2e-5
    got = oracle.backward(fwd, z["grad_image"] * mask, *arrays)
    for name in NAMES:
        want = z[f"grad_{name}_{mode}"].reshape(got[name].shape)
        scale = max(np.abs(want).max(), 1e-12)
        assert np.abs(got[name] - want).max() / scale < 2e-5, (name, np.abs(got[name] - want).max(), scale)
    # third densification statistic: per Gaussian, the sum over the compared pixels of |dL_p/dposition|_1
    info = np.zeros((3, sc.positions.shape[0]), np.float32)
    oracle.backward(fwd, z["grad_image"] * mask, *arrays, densification_info=info, use_distance_scaling=False)
    want = z[f"dens_l1_{mode}"]
    assert np.abs(info[2] - want).max() / np.abs(want).max() < 1e-4, np.abs(info[2] - want).max()
