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


@pytest.mark.parametrize("threshold", [1e-4, 0.0])
@pytest.mark.parametrize("mode", [0, 3])
def test_weight_threshold_below_the_alpha_threshold(cuda, mode, threshold):
    """The tail's second walk has no alpha threshold (only the cut-off), so with a weight threshold under 1/255 a
    fragment too faint for the blend still raises its Gaussian's weight; faint Gaussians make that the common case."""
    print(f"case mode={mode} threshold={threshold}", flush=True)
    n = 20_000
    scene = make_scene(1, n)
    scene.opacities.mul_(torch.rand(n, 1, generator=torch.Generator().manual_seed(5)) ** 3)
    want = np.zeros(n, dtype=np.float32)
    oracle.update_max_weights(oracle_frame(scene, mode, 8), want, *[t.numpy() for t in scene.gaussians()[:4]], threshold)
    sg = scene.to(cuda)
    got = torch.zeros(n, 1, device=cuda)
    update_max_weights(got, *sg.gaussians()[:4], sg.settings(RasterizerMode(mode), 8), threshold)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(got.cpu().numpy().reshape(-1).view(np.uint32), want.view(np.uint32))
    assert ((want > 0) & (want < 1.0 / 255.0)).sum() > n // 100


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


@pytest.mark.parametrize("config,n,K,long_threshold", [(0, 6000, 4, 40), (1, 50_000, 16, 24), (3, 30_000, 8, 300), (3, 30_000, 1, 100)])
@pytest.mark.parametrize("mode", [0, 1, 3])
def test_max_weights_with_very_long_lists(cuda, config, n, K, mode, long_threshold):
    """Tiles whose lists exceed the threshold (forced down here) go to the kernels that share a list between waves and
    workgroups -- the core's weights from the merged K-buffers, the tail's from a second walk in parts -- and the result
    is the oracle's: bit for bit in ALPHA_BLEND_FIRST_K (the maximum does not depend on the order of arrival), to the rounding of
    the tail's sums -- which the shares of a list add up in another order -- in the modes with a tail."""
    from htgs_amd.torch_bindings.rasterization import run_max_weights
    print(f"case config={config} n={n} mode={mode} K={K} long_threshold={long_threshold}", flush=True)
    scene = make_scene(config, n)
    want = np.zeros(n, dtype=np.float32)
    threshold = 0.01
    oracle.update_max_weights(oracle_frame(scene, mode, K), want, *[t.numpy() for t in scene.gaussians()[:4]], threshold)
    sg = scene.to(cuda)
    got = torch.zeros(n, 1, device=cuda)
    fb = run_max_weights(got, *sg.gaussians()[:4], sg.settings(RasterizerMode(mode), K), threshold, long_list_threshold=long_threshold)
    torch.cuda.synchronize()
    lengths = (fb.ranges[:, 1] - fb.ranges[:, 0]).to(torch.int64)
    assert int((lengths > long_threshold).sum()) > 0 and not bool(fb.long_tiles[:6].any())
    if mode == 1:
        np.testing.assert_array_equal(got.cpu().numpy().reshape(-1).view(np.uint32), want.view(np.uint32))
    else:
        # (a weight within rounding of the threshold may fall on the other side of it: compared where both sides kept it)
        g = got.cpu().numpy().reshape(-1)
        both = (g > 0) & (want > 0)
        np.testing.assert_allclose(g[both], want[both], rtol=1e-5)
        assert (both != ((g > 0) | (want > 0))).sum() <= 2
