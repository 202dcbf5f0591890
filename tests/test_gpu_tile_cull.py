"""The blend kernels leave out, batch by batch and per 4x4 quadrant, the instances whose Gaussian provably reaches no pixel
there (8x8 tiles: four quadrants; the 16x16 tiles of ALPHA_BLEND_GLOBAL_ORDERING: sixteen).  The library's self-check
evaluates every instance at all pixels of its tile with the kernels' own cut-off and alpha tests
and compares with the verdict of the staging lane: an instance that reaches a pixel must never be left out (then
the walk over the kept instances gives the full walk's results bit for bit, which the parity tests confirm on the
images), and nearly every instance that reaches none should be."""
import dataclasses

import pytest
import torch

from htgs_amd import _native
from htgs_amd.synthetic import make_scene
from htgs_amd.torch_bindings import FrameBuffers, RasterizerMode

pytestmark = pytest.mark.gpu


def _cull_counts(scene, mode, K=16):
    fb = FrameBuffers(*scene.gaussians(), scene.settings(RasterizerMode(mode), K), True, False)
    fb.preprocess()
    fb.scan()
    fb.alloc_instances(fb.read_instance_count())
    fb.create_instances()
    fb.sort()
    fb.extract_ranges()
    counts = torch.zeros(4, dtype=torch.int64, device=scene.positions.device)
    _native.check(fb.lib.htgs_check_tile_cull(fb._ref, fb.selector, counts.data_ptr()))
    seen, empty, left_out, wrong = counts.cpu().tolist()
    assert seen == fb.n_instances
    return seen, empty, left_out, wrong


def _variants(scene):
    """The scene itself and versions of it that stress the bound: needles, specks between the pixel centres, faint and
    over-range opacities."""
    g = torch.Generator().manual_seed(11)
    n = scene.positions.shape[0]
    yield "plain", scene
    stretch = torch.ones(n, 3)
    stretch[torch.arange(n), torch.randint(0, 3, (n,), generator=g)] = 40.0
    yield "needles", dataclasses.replace(scene, scales=scene.scales * 0.1 * stretch)
    yield "specks", dataclasses.replace(scene, scales=scene.scales * 0.03)
    faint = scene.opacities * torch.rand(n, 1, generator=g) ** 4
    faint[::7] = 0.0
    faint[3::11] = 1.5
    yield "faint", dataclasses.replace(scene, opacities=faint)
    yield "large", dataclasses.replace(scene, scales=scene.scales * 6.0)


@pytest.mark.parametrize("config,n", [(0, 10_000), (1, 60_000), (3, 40_000)])
def test_no_instance_that_reaches_a_pixel_is_left_out(cuda, config, n):
    base = make_scene(config, n)
    for name, scene in _variants(base):
        scene = scene.to(cuda)
        for mode in (0, 1, 2, 3):
            print(f"case config={config} variant={name} mode={mode}", flush=True)
            seen, empty, left_out, wrong = _cull_counts(scene, mode)
            assert wrong == 0
            assert left_out <= empty
            if name == "plain" and config != 0:
                assert seen > 10_000 and empty > 0
                assert left_out >= (0.95 if mode == 2 else 0.98) * empty
