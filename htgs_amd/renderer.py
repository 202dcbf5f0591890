"""Camera -> RasterizerSettings, as the reference's renderer builds them (Renderer.py:18-57 of the reference):
``extract_settings(view, mode, K, active_sh_bases, scale_modifier)`` with the same arguments and the same
matrices, so that a renderer written against the reference can keep calling it.

``view`` is any object with the attributes the reference reads: ``view.camera`` (``focal_x``, ``focal_y``,
``center_x``, ``center_y``, ``near_plane``, ``far_plane``, ``width``, ``height``, ``distortion``), ``view.w2c_numpy``
(4x4 world -> camera) and ``view.position`` (camera centre, a device tensor).  The framework classes of the
reference's host application (cameras, views, logging) are not needed.
"""
from __future__ import annotations

import warnings

import numpy as np
import torch

from .torch_bindings import RasterizerMode, RasterizerSettings


def view_projection(camera) -> np.ndarray:
    """The 4x4 pixel-space projection of Renderer.py:38-43: pixel centres at integer coordinates (hence the half
    pixel taken off the principal point), depth mapped to [-1, 1] between the clipping planes."""
    near_plane, far_plane = camera.near_plane, camera.far_plane
    z_range = far_plane - near_plane
    return np.array([
        [camera.focal_x, 0.0, camera.center_x - 0.5, 0.0],
        [0.0, camera.focal_y, camera.center_y - 0.5, 0.0],
        [0.0, 0.0, (far_plane + near_plane) / z_range, -2.0 * far_plane * near_plane / z_range],
        [0.0, 0.0, 1.0, 0.0],
    ])


def extract_settings(view, mode: int, K: int, active_sh_bases: int, scale_modifier: float, device="cuda") -> RasterizerSettings:
    camera = view.camera
    if getattr(camera, "distortion", None) is not None:
        warnings.warn("the camera carries lens-distortion parameters; the rasterizer renders an undistorted pinhole image")
    try:
        rasterizer_mode = RasterizerMode(mode)
    except ValueError:
        warnings.warn(f"rasterizer mode {mode!r} does not exist (0-3); using HYBRID_BLEND")
        rasterizer_mode = RasterizerMode.HYBRID_BLEND
    M = np.asarray(view.w2c_numpy)
    VPM = view_projection(camera).astype(M.dtype) @ M
    return RasterizerSettings(
        M=torch.as_tensor(M, dtype=torch.float32, device=device),
        VPM=torch.as_tensor(VPM, dtype=torch.float32, device=device),
        cam_position=torch.as_tensor(view.position, dtype=torch.float32, device=device),
        mode=rasterizer_mode,
        K=K,
        active_sh_bases=active_sh_bases,
        width=camera.width,
        height=camera.height,
        near_plane=camera.near_plane,
        far_plane=camera.far_plane,
        scale_modifier=scale_modifier,
    )
