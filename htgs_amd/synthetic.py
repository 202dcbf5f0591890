"""Seeded synthetic scenes and pinhole cameras for tests and benchmarks.

The camera follows the reference's ``extract_settings`` (``Renderer.py:34-57``): ``VP`` maps camera space to
pixel coordinates with the half-pixel shift ``cx - 0.5`` and to NDC depth, ``VPM = VP @ M``.  Gaussian
parameters are *activated* as the reference's renderer passes them (``Model.py:51-59,76-79,162-176``):
scales after exp, opacities after sigmoid ``[N,1]``, unit quaternions ``(w,x,y,z)``, ``sh_0 [N,1,3]``,
``sh_rest [N,B-1,3]`` (``[N,0,3]`` for SH degree 0).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import numpy as np
import torch

from .torch_bindings.rasterization import RasterizerMode, RasterizerSettings

SH_C0 = 0.28209479177387814
# focal length (pixels) of the 6 M stress scene: the value at which a visible Gaussian of that scene covers 16 tiles of
# 8x8 pixels on average (the scene is specified by its distributions and by 8-20 tiles per Gaussian, not by a focal length)
CFG3_FOCAL = 35.0


@dataclass
class Scene:
    name: str
    positions: torch.Tensor
    scales: torch.Tensor
    rotations: torch.Tensor
    opacities: torch.Tensor
    sh_0: torch.Tensor
    sh_rest: torch.Tensor
    M: torch.Tensor
    VPM: torch.Tensor
    cam_position: torch.Tensor
    width: int
    height: int
    near_plane: float
    far_plane: float
    active_sh_bases: int
    K: int

    def gaussians(self):
        return self.positions, self.scales, self.rotations, self.opacities, self.sh_0, self.sh_rest

    def to(self, device) -> "Scene":
        moved = {k: (v.to(device) if isinstance(v, torch.Tensor) else v) for k, v in self.__dict__.items()}
        return Scene(**moved)

    def settings(self, mode=RasterizerMode.HYBRID_BLEND, K: Optional[int] = None, scale_modifier: float = 1.0) -> RasterizerSettings:
        mode = mode if isinstance(mode, RasterizerMode) else RasterizerMode(int(mode))
        return RasterizerSettings(self.M, self.VPM, self.cam_position, mode, self.K if K is None else K,
                                  self.active_sh_bases, self.width, self.height, self.near_plane, self.far_plane,
                                  scale_modifier)


def pinhole(width, height, fx, fy, cx, cy, near_plane, far_plane, translation=(0.0, 0.0, 0.0), rotation=None):
    """``(M, VPM, cam_position)`` as float32 tensors.  ``M`` is world -> camera with rotation ``rotation``
    (3x3, default identity) and translation ``translation``."""
    M = np.eye(4, dtype=np.float64)
    if rotation is not None:
        M[:3, :3] = np.asarray(rotation, dtype=np.float64)
    M[:3, 3] = np.asarray(translation, dtype=np.float64)
    z_range = far_plane - near_plane
    VP = np.array([
        [fx, 0.0, cx - 0.5, 0.0],
        [0.0, fy, cy - 0.5, 0.0],
        [0.0, 0.0, (far_plane + near_plane) / z_range, -2.0 * far_plane * near_plane / z_range],
        [0.0, 0.0, 1.0, 0.0],
    ], dtype=np.float64)
    VPM = VP @ M
    cam = -M[:3, :3].T @ M[:3, 3]
    return (torch.tensor(M, dtype=torch.float32), torch.tensor(VPM, dtype=torch.float32),
            torch.tensor(cam, dtype=torch.float32))


def _unit_quaternions(n, g):
    q = torch.randn(n, 4, generator=g)
    return q / q.norm(dim=1, keepdim=True).clamp_min(1e-12)


def _sh(n, degree, g):
    dc = torch.rand(n, 1, 3, generator=g)
    sh_0 = (dc - 0.5) / SH_C0
    n_rest = (degree + 1) ** 2 - 1
    sh_rest = torch.randn(n, n_rest, 3, generator=g) * 0.05 if n_rest else torch.zeros(n, 0, 3)
    return sh_0.contiguous(), sh_rest.contiguous()


def _cluster_scene(name, seed, n, width, height, focal, K, g=None):
    """The 1 M / 3 M scenes: means ~ N(0, 2^2 I) clipped to radius 10, cluster centre 12 units ahead."""
    g = g or torch.Generator().manual_seed(seed)
    pos = torch.randn(n, 3, generator=g) * 2.0
    r = pos.norm(dim=1, keepdim=True)
    pos = pos * torch.clamp(10.0 / r.clamp_min(1e-12), max=1.0)
    scales = torch.exp(torch.randn(n, 3, generator=g) * 0.7 - 4.5)
    rot = _unit_quaternions(n, g)
    opac = torch.sigmoid(torch.randn(n, 1, generator=g) * 1.5)
    sh_0, sh_rest = _sh(n, 3, g)
    M, VPM, cam = pinhole(width, height, focal, focal, width / 2, height / 2, 0.2, 1000.0, translation=(0.0, 0.0, 12.0))
    return Scene(name, pos.contiguous(), scales, rot, opac, sh_0, sh_rest, M, VPM, cam, width, height, 0.2, 1000.0, 16, K)


def make_scene(config: int, n: Optional[int] = None) -> Scene:
    """The five benchmark scenes (CPU tensors; ``.to('cuda')`` moves them).  ``n`` overrides the Gaussian count
    while keeping the distributions, which is how tests get oracle-sized versions of the big scenes."""
    if config == 0:
        n = n or 10_000
        g = torch.Generator().manual_seed(0)
        pos = torch.rand(n, 3, generator=g) * 2.0 - 1.0
        pos[:, 2] += 4.0
        scales = torch.exp(torch.randn(n, 3, generator=g) * 0.5 - 4.0)
        rot = _unit_quaternions(n, g)
        opac = torch.sigmoid(torch.randn(n, 1, generator=g))
        sh_0, sh_rest = _sh(n, 0, g)
        M, VPM, cam = pinhole(256, 256, 300.0, 300.0, 128.0, 128.0, 0.2, 1000.0)
        return Scene("cfg0-tiny", pos.contiguous(), scales, rot, opac, sh_0, sh_rest, M, VPM, cam, 256, 256, 0.2, 1000.0, 1, 4)
    if config == 1:
        return _cluster_scene("cfg1-1M-720p", 1, n or 1_000_000, 1280, 720, 1000.0, 16)
    if config == 2:
        return _cluster_scene("cfg2-3M-1080p", 2, n or 3_000_000, 1920, 1080, 1500.0, 16)
    if config == 3:
        n = n or 6_000_000
        g = torch.Generator().manual_seed(3)
        d = torch.randn(n, 3, generator=g)
        d = d / d.norm(dim=1, keepdim=True).clamp_min(1e-12)
        pos = d * (6.0 * torch.rand(n, 1, generator=g) ** (1.0 / 3.0))
        pos[:, 2] += 4.0
        near = torch.rand(n, generator=g) < 0.2
        z_near = 0.2 + 0.5 * torch.rand(n, generator=g)
        # Gaussians hugging the near plane, kept inside the frustum's footprint at that depth
        xy_near = (torch.rand(n, 2, generator=g) * 2.0 - 1.0) * 0.5
        pos[near, 2] = z_near[near]
        pos[near, :2] = xy_near[near]
        # log-scales ~ N(-3, 0.8) for every Gaussian, the near-plane group included: those are the ellipsoids that
        # cross the near plane, reach NDC z < -1 or cover the whole tile grid
        scales = torch.exp(torch.randn(n, 3, generator=g) * 0.8 - 3.0)
        rot = _unit_quaternions(n, g)
        opac = torch.sigmoid(torch.randn(n, 1, generator=g) * 1.5)
        sh_0, sh_rest = _sh(n, 3, g)
        M, VPM, cam = pinhole(1600, 1066, CFG3_FOCAL, CFG3_FOCAL, 800.0, 533.0, 0.2, 1000.0)
        return Scene("cfg3-6M-stress", pos.contiguous(), scales, rot, opac, sh_0, sh_rest, M, VPM, cam, 1600, 1066, 0.2, 1000.0, 16, 16)
    if config == 4:
        return _cluster_scene("cfg4-1M-1080p-train", 4, n or 1_000_000, 1920, 1080, 1500.0, 16)
    raise ValueError(f"unknown scene config {config}")
