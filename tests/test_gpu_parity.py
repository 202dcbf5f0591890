"""GPU parity: every stage of the HIP path, called through the C ABI, against the CPU oracle on the same
seeded inputs.  Integer stages (tile counts, offsets, instance keys, sort order, ranges) must match bit for
bit; image and depth within 1e-4 max abs (the tolerance of the rasterizer's contract, fp32)."""
import numpy as np
import pytest
import torch

from htgs_amd.synthetic import make_scene
from util import gpu_stages, oracle_render

pytestmark = pytest.mark.gpu

TOL = 1e-4

CASES = [
    # (scene config, n override, mode, K)
    (0, None, 0, 4),
    (0, None, 1, 4),
    (0, None, 2, 4),
    (0, None, 3, 4),
    (1, 60_000, 0, 16),
    (1, 60_000, 1, 16),
    (1, 60_000, 2, 16),
    (1, 60_000, 3, 16),
    (2, 100_000, 0, 16),
    (2, 100_000, 2, 16),
    # the stress scene as specified (near-plane group with unmodified scales): ellipsoids that cross the near plane or
    # reach NDC z < -1 (R/include/kernel_utils.cuh:110-116) and rectangles of thousands of tiles
    (3, 150_000, 0, 16),
    (3, 150_000, 2, 16),
]


def check_against_oracle(got, ref):
    vis = ref["pre"]["n_touched"] > 0
    np.testing.assert_array_equal(got["n_touched"], ref["pre"]["n_touched"])
    np.testing.assert_array_equal(got["bounds"][vis], ref["pre"]["bounds"][vis])
    for name in ("VPMT1", "VPMT2", "VPMT4", "MT3", "rgba"):
        np.testing.assert_array_equal(got[name][vis].view(np.uint32), ref["pre"][name][vis].view(np.uint32), err_msg=name)
    np.testing.assert_array_equal(got["offsets"], ref["offsets"])
    assert got["n_instances"] == len(ref["keys"])
    np.testing.assert_array_equal(got["keys"], ref["keys"])
    np.testing.assert_array_equal(got["vals"], ref["vals"])
    np.testing.assert_array_equal(got["sorted_keys"], ref["sorted_keys"])
    np.testing.assert_array_equal(got["sorted_vals"], ref["sorted_vals"])
    np.testing.assert_array_equal(got["ranges"], ref["ranges"])
    assert np.isfinite(got["image"]).all() and np.isfinite(got["depth"]).all()
    assert np.abs(got["image"] - ref["image"]).max() <= TOL
    assert np.abs(got["depth"] - ref["depth"]).max() <= TOL


@pytest.mark.parametrize("config,n,mode,K", CASES)
def test_stages_match_oracle(cuda, config, n, mode, K):
    scene = make_scene(config, n)
    print(f"case config={config} n={n} mode={mode} K={K}", flush=True)
    ref = oracle_render(scene, mode, K)
    got = gpu_stages(scene.to(cuda), mode, K)
    check_against_oracle(got, ref)


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
@pytest.mark.parametrize("to_chw,median", [(False, False), (True, True), (False, True)])
def test_layout_and_median_depth(cuda, mode, to_chw, median):
    scene = make_scene(0, 3000)
    print(f"case mode={mode} to_chw={to_chw} median={median}", flush=True)
    ref = oracle_render(scene, mode, 4, to_chw=to_chw, median=median)
    got = gpu_stages(scene.to(cuda), mode, 4, to_chw=to_chw, median=median)
    assert got["image"].shape == ref["image"].shape
    assert np.abs(got["image"] - ref["image"]).max() <= TOL
    assert np.abs(got["depth"] - ref["depth"]).max() <= TOL


@pytest.mark.parametrize("K", [1, 2, 3, 8, 32, 50])
@pytest.mark.parametrize("mode", [0, 1])
def test_k_dispatch(cuda, mode, K):
    """K is rounded down to a power of two <= 32 (R/src/hybrid_blend/inference.cu:22-27)."""
    scene = make_scene(0, 4000)
    print(f"case mode={mode} K={K}", flush=True)
    ref = oracle_render(scene, mode, K)
    got = gpu_stages(scene.to(cuda), mode, K)
    assert np.abs(got["image"] - ref["image"]).max() <= TOL
    assert np.abs(got["depth"] - ref["depth"]).max() <= TOL


def test_refined_reciprocal_equals_division_on_the_whole_guarded_range(cuda):
    """The blend kernels replace 1 / |d|^2 by v_rcp_f32 plus one fused Newton step inside [2^-120, 2^121) and keep
    the IEEE division outside; the library compares the two on every float of that range on this device."""
    from htgs_amd import _native
    counts = torch.zeros(2, dtype=torch.int64, device=cuda)
    _native.check(_native.lib().htgs_check_reciprocal(counts.data_ptr(), torch.cuda.current_stream().cuda_stream))
    tested, wrong = counts.cpu().tolist()
    assert tested == 241 * 2 ** 23
    assert wrong == 0


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
@pytest.mark.parametrize("config,n", [(0, 5000), (1, 60_000)])
def test_fast_rasterize_against_the_oracle(cuda, config, n, mode):
    """``fast_rasterize`` (reference: torch_bindings/rasterization.py:166-186) against the CPU oracle's image, not
    against this library's own ``rasterize``.  It evaluates 1/x and 2^x with the hardware's one-ulp instructions, so a
    fragment within an ulp of an alpha threshold may be decided differently: 1/255 is worth 4e-3 of a colour, 1/20 (the
    gate of the sorted core) up to 5e-2.  Bound: fewer than 0.1 % of the pixels off by more than 1e-5, none by more
    than 5e-2, in both image layouts."""
    from htgs_amd.torch_bindings import fast_rasterize
    scene = make_scene(config, n)
    print(f"case config={config} n={n} mode={mode}", flush=True)
    sc = scene.to(cuda)
    s = sc.settings(mode, 16)
    for to_chw in (True, False):
        ref = oracle_render(scene, mode, 16, to_chw=to_chw)["image"]
        fast = fast_rasterize(*sc.gaussians(), s, to_chw)
        assert fast.shape == ref.shape and float(ref.max()) > 0.05
        diff = np.abs(fast.cpu().numpy() - ref)
        assert float((diff > 1e-5).mean()) < 1e-3
        assert float(diff.max()) <= 5e-2


def test_fast_rasterize_with_lists_up_to_the_packing_limit(cuda):
    """HYBRID_BLEND's fast kernel with one wave per tile packs a core entry's place in its tile's list into 13 bits of a
    key; on the stress scene dozens of tiles have lists of 4096 to 8192 instances (the longest this kernel walks), and
    longer ones go to the kernel for long lists, which keeps three registers a slot.  Same bounds as above."""
    from htgs_amd.torch_bindings import FrameBuffers
    from util import u32
    scene = make_scene(3, 200_000)
    print("case config=3 n=200000 mode=0 (fast, long lists)", flush=True)
    ref = oracle_render(scene, 0, 16)["image"]
    sc = scene.to(cuda)
    fb = FrameBuffers(*sc.gaussians(), sc.settings(0, 16), True, False, fast=True)
    fb.run()
    ranges = u32(fb.ranges).astype(np.int64)
    length = ranges[:, 1] - ranges[:, 0]
    assert int(((length > 4096) & (length <= 8192)).sum()) > 10 and int((length > 8192).sum()) > 5
    diff = np.abs(fb.image.cpu().numpy() - ref)
    assert float((diff > 1e-5).mean()) < 1e-3
    assert float(diff.max()) <= 5e-2


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_fast_rasterize_reproduces_the_frozen_float64_image(cuda, mode):
    """The same entry point against tests/golden/small_scene.npz (independent float64 evaluator, no CPU oracle in
    between): within the contract's 1e-4 on the pixels whose decisions are not within 1e-4 of a threshold."""
    from htgs_amd.torch_bindings import RasterizerMode, fast_rasterize
    from util import load_golden
    sc, z = load_golden()
    mask = z[f"mask_{mode}"]
    want = np.clip(z[f"image_{mode}"], 0.0, 1.0)
    sg = sc.to(cuda)
    settings = sg.settings(RasterizerMode(mode), int(z["K"]))
    chw = fast_rasterize(*sg.gaussians(), settings, True).cpu().numpy()
    hwc = fast_rasterize(*sg.gaussians(), settings, False).cpu().numpy()
    assert np.abs(chw - want)[:, mask].max() <= 1e-4
    assert np.array_equal(hwc, chw.transpose(1, 2, 0))
