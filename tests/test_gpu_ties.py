"""The HIP kernels against the hand-computed pixels of tests/test_oracle_ties.py (no oracle in between): fragments of
exactly equal depth in HYBRID_BLEND's core must come out in the order of the reference's exchange walk
(R/include/hybrid_blend/kernels/inference.cuh:159-167) -- through the kernel with one wave per tile (threshold 0, the
default of 8192: the core as sorted keys, the pixel walked a second time; threshold 2^31 - 1: the exchange insertion
throughout), through the kernels that share a long list between waves (threshold forced down to 2 instances: the cores
are merged and the pixel gets the second look), and in the core indices the training pass records."""
import numpy as np
import pytest
import torch

from htgs_amd.torch_bindings import FrameBuffers, RasterizerMode
from test_oracle_ties import PX, THREE, TWO
from util import hybrid_pixel_by_hand, tie_scene, u32

pytestmark = pytest.mark.gpu

CASES = [(TWO, [4, 0, 2, 1], [3]), (THREE, [4, 0, 2, 3], [1])]


@pytest.mark.parametrize("case,core,tail", CASES)
@pytest.mark.parametrize("threshold", [0, 2, 2 ** 31 - 1])
def test_inference_pixel_with_equal_depths(cuda, case, core, tail, threshold):
    print(f"case depths={case['depths']} threshold={threshold}", flush=True)
    scene = tie_scene(**case).to(cuda)
    fb = FrameBuffers(*scene.gaussians(), scene.settings(RasterizerMode.HYBRID_BLEND, 4), True, False, long_list_threshold=threshold)
    image, depth = fb.run()
    torch.cuda.synchronize()
    want_rgb, want_depth = hybrid_pixel_by_hand(core, tail, case["depths"], case["opacities"], case["colours"])
    assert np.abs(image[:, PX, PX].cpu().numpy() - want_rgb).max() <= 2e-6
    assert abs(float(depth[PX, PX]) - want_depth) <= 1e-5 * want_depth


@pytest.mark.parametrize("case,core,tail", CASES)
@pytest.mark.parametrize("threshold", [0, 2])
def test_recorded_core_with_equal_depths(cuda, case, core, tail, threshold):
    print(f"case depths={case['depths']} threshold={threshold}", flush=True)
    scene = tie_scene(**case).to(cuda)
    fb = FrameBuffers(*scene.gaussians(), scene.settings(RasterizerMode.HYBRID_BLEND, 4), True, False, train=True, long_list_threshold=threshold)
    fb.run_forward()
    torch.cuda.synchronize()
    idx = u32(fb.records_in_image_order(fb.core_idx))[:, PX * scene.width + PX]
    assert idx.tolist() == core
