"""GPU parity on the inputs that break rasterizers: nothing to draw, image sizes that are not multiples of the tile,
one Gaussian over the whole image, degenerate and non-finite parameters, every SH degree, 32-bit tile keys, a scale
modifier and a rotated camera.  Same bar as the other parity tests: integer stages bit for bit, image and depth
within 1e-4 of the CPU oracle."""
import dataclasses

import numpy as np
import pytest
import torch
from scipy.spatial.transform import Rotation

from htgs_amd.synthetic import Scene, make_scene, pinhole
from htgs_amd.torch_bindings import RasterizerMode, rasterize
from util import gpu_stages, oracle_render
from test_gpu_parity import check_against_oracle

pytestmark = pytest.mark.gpu

TOL = 1e-4


def resized(scene: Scene, width: int, height: int, focal: float, translation=(0.0, 0.0, 0.0), rotation=None) -> Scene:
    M, VPM, cam = pinhole(width, height, focal, focal, width / 2, height / 2, scene.near_plane, scene.far_plane,
                          translation=translation, rotation=rotation)
    return dataclasses.replace(scene, M=M, VPM=VPM, cam_position=cam, width=width, height=height)


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_no_gaussians_and_nothing_visible(cuda, mode):
    """N = 0, and N > 0 with every Gaussian behind the camera: zero instances, black image, zero depth."""
    scene = make_scene(0, 64)
    empty = dataclasses.replace(scene, positions=scene.positions[:0], scales=scene.scales[:0], rotations=scene.rotations[:0],
                                opacities=scene.opacities[:0], sh_0=scene.sh_0[:0], sh_rest=scene.sh_rest[:0])
    behind = dataclasses.replace(scene, positions=scene.positions * torch.tensor([1.0, 1.0, -1.0]))
    for sc in (empty, behind):
        print(f"case mode={mode} n={sc.positions.shape[0]}", flush=True)
        g = sc.to(cuda)
        image, depth = rasterize(*g.gaussians(), g.settings(RasterizerMode(mode), 4), True, False)
        assert image.shape == (3, sc.height, sc.width) and depth.shape == (1, sc.height, sc.width)
        assert float(image.abs().max()) == 0.0 and float(depth.abs().max()) == 0.0
    ref = oracle_render(behind, mode, 4)
    assert len(ref["keys"]) == 0 and not ref["image"].any()


@pytest.mark.parametrize("mode", [0, 2])
@pytest.mark.parametrize("width,height", [(250, 131), (1, 1), (17, 300)])
def test_image_sizes_that_are_not_multiples_of_the_tile(cuda, mode, width, height):
    scene = resized(make_scene(0, 4000), width, height, 200.0)
    print(f"case mode={mode} {width}x{height}", flush=True)
    check_against_oracle(gpu_stages(scene.to(cuda), mode, 4), oracle_render(scene, mode, 4))


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_one_gaussian_covering_every_tile(cuda, mode):
    """A Gaussian much larger than the view frustum, in front of a handful of small ones: its rectangle is the whole
    tile grid, so the duplication kernel writes thousands of instances for one primitive."""
    scene = make_scene(0, 40)
    scene.scales[0] = torch.tensor([30.0, 30.0, 0.05])
    scene.positions[0] = torch.tensor([0.0, 0.0, 6.0])
    scene.rotations[0] = torch.tensor([1.0, 0.0, 0.0, 0.0])
    scene.opacities[0] = 0.6
    print(f"case mode={mode}", flush=True)
    ref = oracle_render(scene, mode, 4)
    assert ref["pre"]["n_touched"][0] == 32 * 32 // (4 if mode == 2 else 1)
    check_against_oracle(gpu_stages(scene.to(cuda), mode, 4), ref)


@pytest.mark.parametrize("mode", [0, 2])
def test_degenerate_and_non_finite_parameters(cuda, mode):
    """Flat and needle Gaussians (zero scales), zero and full opacity, and parameters that are NaN or infinite: the
    per-Gaussian stage must make the oracle's decision for every one of them, and the image must stay finite."""
    scene = make_scene(0, 600)
    s, p, o, q = scene.scales, scene.positions, scene.opacities, scene.rotations
    s[0:20, 2] = 0.0                      # discs
    s[20:40, 1:] = 0.0                    # needles
    s[40:50] = 0.0                        # points
    o[50:60] = 0.0
    o[60:70] = 1.0
    o[70:80] = 1.0 / 255.0                # exactly at the visibility threshold
    p[80:85, 0] = float("nan")
    p[85:90, 2] = float("inf")
    s[90:95, 0] = float("nan")
    s[95:100, 1] = float("inf")
    q[100:105] = 0.0                      # zero quaternion
    q[105:110, 0] = float("nan")
    o[110:115] = float("nan")
    print(f"case mode={mode}", flush=True)
    ref = oracle_render(scene, mode, 4)
    got = gpu_stages(scene.to(cuda), mode, 4)
    np.testing.assert_array_equal(got["n_touched"], ref["pre"]["n_touched"])
    np.testing.assert_array_equal(got["sorted_vals"], ref["sorted_vals"])
    np.testing.assert_array_equal(got["ranges"], ref["ranges"])
    finite = np.isfinite(ref["image"]).all(0) & np.isfinite(ref["depth"])
    assert finite.mean() > 0.5
    assert np.abs(got["image"] - ref["image"])[:, finite].max() <= TOL
    assert np.abs(got["depth"] - ref["depth"])[finite].max() <= TOL
    # where the oracle's arithmetic yields NaN or infinity, the kernels yield the same class of value
    np.testing.assert_array_equal(np.isnan(got["image"]), np.isnan(ref["image"]))
    np.testing.assert_array_equal(np.isnan(got["depth"]), np.isnan(ref["depth"]))


@pytest.mark.parametrize("active,total", [(1, 0), (1, 15), (4, 3), (4, 15), (9, 8), (16, 15), (16, 20)])
def test_every_sh_degree_and_unused_coefficients(cuda, active, total):
    """active_sh_bases 1, 4, 9, 16 with sh_rest holding exactly, or more than, the coefficients they need."""
    scene = make_scene(1, 5000)
    g = torch.Generator().manual_seed(active * 100 + total)
    scene = dataclasses.replace(scene, sh_rest=(torch.randn(5000, total, 3, generator=g) * 0.2).contiguous(), active_sh_bases=active)
    scene = resized(scene, 320, 200, 250.0, translation=(0.0, 0.0, 12.0))
    print(f"case active={active} total={total}", flush=True)
    check_against_oracle(gpu_stages(scene.to(cuda), 0, 8), oracle_render(scene, 0, 8))


@pytest.mark.parametrize("mode", [0, 3])
def test_more_than_65536_tiles_uses_32_bit_keys(cuda, mode):
    """2200 x 2000 pixels = 275 x 250 tiles of 8 x 8 = 68750 tiles: the tile index needs 17 bits."""
    scene = resized(make_scene(1, 30_000), 2200, 2000, 1800.0, translation=(0.0, 0.0, 12.0))
    print(f"case mode={mode}", flush=True)
    got = gpu_stages(scene.to(cuda), mode, 16)
    assert got["fb"].key_bytes == 4
    check_against_oracle(got, oracle_render(scene, mode, 16))


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_scale_modifier_and_rotated_camera(cuda, mode):
    rot = Rotation.from_euler("xyz", [12.0, -20.0, 31.0], degrees=True).as_matrix()
    scene = resized(make_scene(1, 20_000), 400, 300, 350.0, translation=(0.5, -0.3, 11.0), rotation=rot)
    print(f"case mode={mode}", flush=True)
    ref = oracle_render(scene, mode, 16, scale_modifier=0.6)
    got = gpu_stages(scene.to(cuda), mode, 16, scale_modifier=0.6)
    check_against_oracle(got, ref)
    assert ref["image"].max() > 0.05


def test_scan_publishes_a_marker_when_the_instance_count_does_not_fit_32_bits(cuda):
    """Offsets are 32-bit (as in the reference); tile counts (each at most 2^20, the largest supported tile grid) that
    add up to more than 2^32 - 2 make the scan publish 0xffffffff, which the host refuses, instead of a wrapped total."""
    import ctypes
    from htgs_amd import _native
    from htgs_amd.torch_bindings.rasterization import checked_instance_count
    lib = _native.lib()
    for counts, want in (([0x7fffffff, 0x7fffffff, 0], 0xfffffffe), ([0x7fffffff, 0x7fffffff, 1], 0xffffffff),
                         ([1 << 20] * 5000, 0xffffffff), ([1 << 20] * 4095 + [(1 << 20) - 2], 0xfffffffe), ([3] * 5000, 15000)):
        n = len(counts)
        c = torch.tensor(counts, dtype=torch.int64).to(torch.int32).to(cuda)
        offsets = torch.empty(n, dtype=torch.int32, device=cuda)
        total = torch.zeros(1, dtype=torch.int32, device=cuda)
        tmp = torch.empty(lib.htgs_scan_tmp_words(n), dtype=torch.int32, device=cuda)
        f = _native.Frame()
        f.n_primitives, f.n_touched, f.offsets, f.n_instances_dev, f.scan_tmp = n, c.data_ptr(), offsets.data_ptr(), total.data_ptr(), tmp.data_ptr()
        f.stream = torch.cuda.current_stream(cuda).cuda_stream
        _native.check(lib.htgs_scan_offsets(ctypes.byref(f)))
        got = int(total.item()) & 0xffffffff
        assert got == want
        if want == 0xffffffff:
            with pytest.raises(RuntimeError, match="instances"):
                checked_instance_count(got)
        else:
            assert checked_instance_count(got) == want
