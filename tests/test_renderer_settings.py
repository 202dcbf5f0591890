"""extract_settings (the reference's Renderer.py:18-57): a pixel-space projection checked against the pinhole model
itself -- a point on the optical axis lands on the principal point minus half a pixel, the clipping planes map to
depth -1 and +1 -- and against the matrices the synthetic scenes use."""
import types
import warnings

import numpy as np
import torch
from scipy.spatial.transform import Rotation

from htgs_amd.renderer import extract_settings
from htgs_amd.synthetic import pinhole
from htgs_amd.torch_bindings import RasterizerMode


def make_view(rotation, translation):
    w2c = np.eye(4)
    w2c[:3, :3], w2c[:3, 3] = rotation, translation
    camera = types.SimpleNamespace(focal_x=410.0, focal_y=395.0, center_x=161.25, center_y=118.5, near_plane=0.3, far_plane=80.0,
                                   width=320, height=240, distortion=None)
    position = torch.tensor(-rotation.T @ np.asarray(translation), dtype=torch.float32)
    return types.SimpleNamespace(camera=camera, w2c_numpy=w2c, position=position)


def test_projection_of_known_points():
    R = Rotation.from_euler("xyz", [10.0, -25.0, 40.0], degrees=True).as_matrix()
    view = make_view(R, [0.2, -0.1, 0.5])
    s = extract_settings(view, 2, 16, 9, 0.8, device="cpu")
    assert s.mode is RasterizerMode.ALPHA_BLEND_GLOBAL_ORDERING and s.K == 16 and s.active_sh_bases == 9
    assert (s.width, s.height, s.scale_modifier) == (320, 240, 0.8)
    VPM, M = s.VPM.double().numpy(), s.M.double().numpy()
    cam = view.camera
    for x_cam, y_cam, z in [(0.0, 0.0, 2.0), (0.4, -0.3, 5.0), (-1.0, 0.7, 30.0)]:
        p_world = R.T @ (np.array([x_cam, y_cam, z]) - np.array([0.2, -0.1, 0.5]))
        h = VPM @ np.append(p_world, 1.0)
        np.testing.assert_allclose(h[0] / h[3], cam.focal_x * x_cam / z + cam.center_x - 0.5, atol=1e-3)
        np.testing.assert_allclose(h[1] / h[3], cam.focal_y * y_cam / z + cam.center_y - 0.5, atol=1e-3)
        np.testing.assert_allclose((M @ np.append(p_world, 1.0))[2], z, atol=1e-5)
    for z, want in [(cam.near_plane, -1.0), (cam.far_plane, 1.0)]:
        h = VPM @ np.append(R.T @ (np.array([0.0, 0.0, z]) - np.array([0.2, -0.1, 0.5])), 1.0)
        np.testing.assert_allclose(h[2] / h[3], want, atol=1e-4)
    np.testing.assert_allclose(s.cam_position.numpy(), -R.T @ np.array([0.2, -0.1, 0.5]), atol=1e-6)


def test_same_matrices_as_the_synthetic_scenes_and_mode_fallback():
    R = Rotation.from_euler("z", 30.0, degrees=True).as_matrix()
    view = make_view(R, [0.0, 0.3, 1.0])
    cam = view.camera
    M, VPM, position = pinhole(cam.width, cam.height, cam.focal_x, cam.focal_y, cam.center_x, cam.center_y, cam.near_plane,
                               cam.far_plane, translation=(0.0, 0.3, 1.0), rotation=R)
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        s = extract_settings(view, 7, 4, 1, 1.0, device="cpu")
    assert s.mode is RasterizerMode.HYBRID_BLEND and any("HYBRID_BLEND" in str(w.message) for w in caught)
    assert torch.allclose(s.M, M) and torch.allclose(s.VPM, VPM, atol=1e-5) and torch.allclose(s.cam_position, position, atol=1e-6)
