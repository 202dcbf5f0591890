"""Tiles with very long lists in the training pass.  The forward blend hands a tile whose list exceeds
``long_list_threshold`` to the kernels that share a list between sixteen waves (and, for lists of several times the
threshold, between workgroups), the backward blend cuts such a list into parts for different workgroups (every instance
writes a gradient row of its own).  The threshold is forced down so that small scenes go through these kernels; records
and gradients must stay within the training path's tolerances of the CPU oracle, whose walk is the reference's single
one (R/include/hybrid_blend/kernels/forward.cuh:78-235, backward.cuh:104-331 and the other modes' counterparts), and
the core's indices must be the oracle's bit for bit (fragments of equal depth included)."""
import numpy as np
import pytest
import torch

import oracle
from htgs_amd.synthetic import make_scene
from htgs_amd.torch_bindings import FrameBuffers, RasterizerMode
from test_gpu_long_tiles import with_coincident_copies
from test_gpu_training import NAMES, assert_grad_close
from util import oracle_frame, u32

pytestmark = pytest.mark.gpu

NEVER = 2 ** 31 - 1
CASES = [(0, 4000, 0, 4, 64, 1), (0, 4000, 1, 4, 24, 1), (0, 4000, 3, 4, 64, 1), (1, 30_000, 0, 16, 40, 1), (1, 30_000, 1, 16, 16, 1),
         (1, 30_000, 3, 16, 40, 1), (3, 60_000, 0, 4, 100, 1), (3, 60_000, 1, 8, 100, 1), (3, 60_000, 3, 1, 100, 1), (0, 1500, 0, 4, 64, 4),
         (0, 1500, 1, 4, 24, 4)]


def run(scene_gpu, mode, K, threshold, grad_image, rows=0):
    fb = FrameBuffers(*scene_gpu.gaussians(), scene_gpu.settings(RasterizerMode(mode), K), True, False, train=True, long_list_threshold=threshold)
    image = fb.run_forward()
    info = torch.full((rows, fb.n), 0.25, device=image.device) if rows else None
    grads = fb.run_backward(grad_image, info, rows == 3)
    torch.cuda.synchronize()
    ranges = fb.ranges.to(torch.int64)
    lengths = ranges[:, 1] - ranges[:, 0]
    assert not bool(fb.long_tiles[:6].any())      # forward and backward leave the list of long tiles empty
    return fb, image, grads, info, lengths


@pytest.mark.parametrize("config,n,mode,K,threshold,copies", CASES)
def test_long_lists_in_the_training_pass(cuda, config, n, mode, K, threshold, copies):
    print(f"case config={config} n={n} mode={mode} K={K} threshold={threshold} copies={copies}", flush=True)
    scene = make_scene(config, n)
    if copies > 1:
        scene = with_coincident_copies(scene, copies)          # every fragment meets fragments of exactly its own depth
    arrays = [t.numpy() for t in scene.gaussians()]
    fwd = oracle.forward(oracle_frame(scene, mode, K), *arrays)
    grad_image = torch.randn(3, scene.height, scene.width, generator=torch.Generator().manual_seed(7))
    want = oracle.backward(fwd, grad_image.numpy(), *arrays)
    sg = scene.to(cuda)
    fb, image, grads, _, lengths = run(sg, mode, K, threshold, grad_image.to(cuda))
    n_long = int((lengths > threshold).sum())
    print(f"  long tiles {n_long} of {lengths.numel()}, longest list {int(lengths.max())}", flush=True)
    assert n_long > 0
    assert np.abs(image.cpu().numpy() - fwd["image"]).max() <= 1e-4
    Keff = oracle.effective_k(K)
    if mode in (0, 1):
        np.testing.assert_array_equal(u32(fb.records_in_image_order(fb.core_idx)), fwd["core_idx"][:Keff])
        np.testing.assert_allclose(fb.records_in_image_order(fb.core_info).cpu().numpy(), fwd["core_info"][:Keff], rtol=1e-5, atol=1e-5)
    if mode in (0, 3):
        rows = 6 if mode == 0 else 5
        np.testing.assert_allclose(fb.records_in_image_order(fb.tail_info).cpu().numpy()[:rows], fwd["tail_info"][:rows], rtol=2e-5, atol=2e-6)
    for name, got in zip(NAMES, grads):
        assert_grad_close(name, got.cpu().numpy(), want[name])
    # against this library's own kernels with one wave (workgroup) per tile
    single_fb, single_image, single_grads, _, _ = run(sg, mode, K, NEVER, grad_image.to(cuda))
    assert float((image - single_image).abs().max()) <= 1e-5
    if mode in (0, 1):
        assert torch.equal(fb.records_in_image_order(fb.core_idx), single_fb.records_in_image_order(single_fb.core_idx))
    for name, got, single in zip(NAMES, grads, single_grads):
        assert_grad_close(name + " (against one workgroup per tile)", got.cpu().numpy(), single.cpu().numpy())


@pytest.mark.parametrize("mode", [0, 1, 3])
def test_long_lists_with_the_third_densification_row(cuda, mode):
    """The per-fragment |dL/dposition|_1 sums of the backward blend (densification row 2) when lists are cut into parts."""
    print(f"case mode={mode}", flush=True)
    scene = make_scene(0, 3000)
    arrays = [t.numpy() for t in scene.gaussians()]
    fwd = oracle.forward(oracle_frame(scene, mode, 4), *arrays)
    grad_image = torch.randn(3, scene.height, scene.width, generator=torch.Generator().manual_seed(11))
    info_ref = np.full((3, 3000), 0.25, np.float32)
    want = oracle.backward(fwd, grad_image.numpy(), *arrays, densification_info=info_ref, use_distance_scaling=True)
    fb, image, grads, info, lengths = run(scene.to(cuda), mode, 4, 24, grad_image.to(cuda), rows=3)
    assert int((lengths > 24).sum()) > 0
    for name, got in zip(NAMES, grads):
        assert_grad_close(name, got.cpu().numpy(), want[name])
    got_info = info.cpu().numpy()
    np.testing.assert_array_equal(got_info[0], info_ref[0])
    for r in (1, 2):
        np.testing.assert_allclose(got_info[r], info_ref[r], rtol=2e-3, atol=2e-4 * float(np.abs(info_ref[r]).max()))
