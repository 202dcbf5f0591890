"""GPU parity of update_max_weights: the maximum is formed with integer atomicMax on the bit patterns, so the HIP
result must equal the oracle's bit for bit, for every mode, on a fresh and on a pre-filled ``max_weights``."""
import numpy as np
import pytest
import torch

import oracle
from htgs_amd.synthetic import make_scene
from htgs_amd.torch_bindings import RasterizerMode, update_max_weights
from util import oracle_frame

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("config,n,K", [(0, 6000, 4), (1, 50_000, 16), (3, 10_000, 16)])
@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_max_weights_bit_exact(cuda, config, n, K, mode):
    print(f"case config={config} n={n} mode={mode} K={K}", flush=True)
    scene = make_scene(config, n)
    rng = np.random.default_rng(config)
    start = np.where(rng.random(n) < 0.1, rng.random(n) * 0.5, 0.0).astype(np.float32)
    want = start.copy()
    threshold = 0.01
    oracle.update_max_weights(oracle_frame(scene, mode, K), want, *[t.numpy() for t in scene.gaussians()[:4]], threshold)
    sg = scene.to(cuda)
    got = torch.from_numpy(start.copy()).to(cuda).reshape(n, 1)
    ret = update_max_weights(got, *sg.gaussians()[:4], sg.settings(RasterizerMode(mode), K, scale_modifier=1.7), threshold)
    assert ret is None
    torch.cuda.synchronize()
    np.testing.assert_array_equal(got.cpu().numpy().reshape(-1).view(np.uint32), want.view(np.uint32))
    assert (want > start).sum() > n // 50


def test_two_views_accumulate(cuda):
    scene = make_scene(0, 4000).to(cuda)
    mw = torch.zeros(4000, device=cuda)
    s = scene.settings(RasterizerMode.HYBRID_BLEND, 4)
    update_max_weights(mw, *scene.gaussians()[:4], s, 0.02)
    first = mw.clone()
    shifted = s._replace(VPM=s.VPM.clone())
    shifted.VPM[0, 3] += 40.0 * 4.0          # pan the principal point: another view of the same Gaussians
    update_max_weights(mw, *scene.gaussians()[:4], shifted, 0.02)
    assert bool((mw >= first).all()) and bool((mw > first).any())
    with pytest.raises(RuntimeError):
        update_max_weights(mw[:10], *scene.gaussians()[:4], s, 0.02)
