"""TEST INFRASTRUCTURE -- not part of the product.

ctypes front end of ``htgs_oracle.c``, the plain-C restatement of the reference rasterizer.
Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this package; nothing under ``htgs_amd/`` does.

All arrays are numpy, float32 / uint32 / uint64, C-contiguous.  The staged functions mirror the
launch order of the reference driver (R/src/hybrid_blend/inference.cu:57-183 and its siblings):
preprocess -> inclusive scan -> create instances -> stable sort -> ranges -> blend.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from dataclasses import dataclass
from typing import Optional

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libhtgs_oracle.so")
_lib = None

MODE_HYBRID, MODE_FIRST_K, MODE_GLOBAL, MODE_OIT = 0, 1, 2, 3


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (see the Makefile next to this file)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return _LIB_PATH


class _Cam(ctypes.Structure):
    _fields_ = [
        ("M3", ctypes.c_float * 4),
        ("VPM", ctypes.c_float * 16),
        ("cam", ctypes.c_float * 3),
        ("near_plane", ctypes.c_float),
        ("far_plane", ctypes.c_float),
        ("scale_modifier", ctypes.c_float),
        ("width", ctypes.c_int),
        ("height", ctypes.c_int),
        ("tile_w", ctypes.c_int),
        ("tile_h", ctypes.c_int),
        ("mode", ctypes.c_int),
        ("K", ctypes.c_int),
        ("active_sh", ctypes.c_int),
        ("total_sh", ctypes.c_int),
    ]


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.o_logf.restype = ctypes.c_float
        _lib.o_logf.argtypes = [ctypes.c_float]
        _lib.o_expf.restype = ctypes.c_float
        _lib.o_expf.argtypes = [ctypes.c_float]
        _lib.o_exp2.restype = ctypes.c_float
        _lib.o_exp2.argtypes = [ctypes.c_float]
        _lib.oracle_inclusive_scan.restype = ctypes.c_uint32
        _lib.oracle_num_threads.restype = ctypes.c_int
    return _lib


def num_threads() -> int:
    return int(lib().oracle_num_threads())


def _p(a: Optional[np.ndarray]):
    if a is None:
        return ctypes.c_void_p(0)
    assert a.flags["C_CONTIGUOUS"], "oracle arrays must be contiguous"
    return ctypes.c_void_p(a.ctypes.data)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def default_tile(mode: int) -> int:
    """Tile edge of each mode: R/include/<mode>/config.h (16 only for global ordering)."""
    return 16 if mode == MODE_GLOBAL else 8


@dataclass
class Frame:
    """Camera and rasterizer parameters, the fields of the reference's RasterizerSettings
    (B/torch_bindings/rasterization.py:16-42) plus the tile edge."""
    M: np.ndarray
    VPM: np.ndarray
    cam_position: np.ndarray
    mode: int
    K: int
    active_sh_bases: int
    width: int
    height: int
    near_plane: float
    far_plane: float
    scale_modifier: float = 1.0
    tile: Optional[int] = None

    def tile_edge(self) -> int:
        return self.tile if self.tile else default_tile(self.mode)

    def grid(self):
        t = self.tile_edge()
        return (self.width + t - 1) // t, (self.height + t - 1) // t

    def c_struct(self, total_sh: int) -> _Cam:
        cam = _Cam()
        M = _f32(self.M).reshape(4, 4)
        cam.M3[:] = M[2].tolist()
        cam.VPM[:] = _f32(self.VPM).reshape(16).tolist()
        cam.cam[:] = _f32(self.cam_position).reshape(3).tolist()
        cam.near_plane = self.near_plane
        cam.far_plane = self.far_plane
        cam.scale_modifier = self.scale_modifier
        cam.width, cam.height = self.width, self.height
        cam.tile_w = cam.tile_h = self.tile_edge()
        cam.mode, cam.K = int(self.mode), int(self.K)
        cam.active_sh, cam.total_sh = int(self.active_sh_bases), int(total_sh)
        return cam


def logf(x: float) -> float:
    return float(lib().o_logf(x))


def expf(x: float) -> float:
    return float(lib().o_expf(x))


def exp2(t: float) -> float:
    return float(lib().o_exp2(t))


def fragment_forms(V1, V2, V4, MT3, opacity: float, tile_x0: int, tile_y0: int, tile: int, local_x: int, local_y: int) -> np.ndarray:
    """(num, den, depth, alpha) of one fragment in the reference's plane form, then in the tile-relative form the
    forward direction uses; no rejection tests are applied."""
    out = np.zeros(8, np.float32)
    lib().oracle_fragment_forms(_p(_f32(V1)), _p(_f32(V2)), _p(_f32(V4)), _p(_f32(MT3)), ctypes.c_float(opacity),
                                ctypes.c_int(tile_x0), ctypes.c_int(tile_y0), ctypes.c_int(tile), ctypes.c_int(tile),
                                ctypes.c_int(local_x), ctypes.c_int(local_y), _p(out))
    return out


def preprocess(frame: Frame, positions, scales, rotations, opacities, sh_0, sh_rest, train: bool = False) -> dict:
    positions, scales, rotations = _f32(positions), _f32(scales), _f32(rotations)
    opacities, sh_0, sh_rest = _f32(opacities).reshape(-1), _f32(sh_0), _f32(sh_rest)
    n = positions.shape[0]
    total_sh = sh_rest.shape[1] if sh_rest.ndim == 3 else 0
    out = {
        "n_touched": np.zeros(n, np.uint32),
        "bounds": np.zeros((n, 4), np.uint32),
        "VPMT1": np.zeros((n, 4), np.float32),
        "VPMT2": np.zeros((n, 4), np.float32),
        "VPMT4": np.zeros((n, 4), np.float32),
        "MT3": np.zeros((n, 4), np.float32),
        "rgba": np.zeros((n, 4), np.float32),
    }
    if train:
        out["clamp_info"] = np.zeros((3, n), np.uint8)
    cam = frame.c_struct(total_sh)
    lib().oracle_preprocess(
        ctypes.byref(cam), ctypes.c_int(n), _p(positions), _p(scales), _p(rotations), _p(opacities), _p(sh_0), _p(sh_rest),
        _p(out["n_touched"]), _p(out["bounds"]), _p(out["VPMT1"]), _p(out["VPMT2"]), _p(out["VPMT4"]), _p(out["MT3"]),
        _p(out["rgba"]), _p(out.get("clamp_info")))
    return out


def inclusive_scan(n_touched: np.ndarray) -> np.ndarray:
    out = np.zeros_like(n_touched)
    lib().oracle_inclusive_scan(ctypes.c_int(n_touched.shape[0]), _p(n_touched), _p(out))
    return out


def create_instances(frame: Frame, pre: dict, offsets: np.ndarray):
    n = offsets.shape[0]
    total = int(offsets[-1]) if n else 0
    keys = np.zeros(total, np.uint64)
    vals = np.zeros(total, np.uint32)
    depth_src = pre["MT3"] if frame.mode == MODE_GLOBAL else None
    lib().oracle_create_instances(ctypes.c_int(n), _p(pre["n_touched"]), _p(offsets), _p(pre["bounds"]), _p(depth_src),
                                  ctypes.c_uint32(frame.grid()[0]), _p(keys), _p(vals))
    return keys, vals


def end_bit(frame: Frame) -> int:
    """extract_end_bit(n_tiles - 1) (+32 for tile|depth keys): R/include/rasterization_utils.h:3-13,
    R/src/alpha_blend_global_ordering/inference.cu:45."""
    gw, gh = frame.grid()
    bits = int(gw * gh - 1).bit_length()
    return bits + 32 if frame.mode == MODE_GLOBAL else bits


def sort_pairs(keys: np.ndarray, vals: np.ndarray, n_bits: int):
    k, v = keys.copy(), vals.copy()
    tk, tv = np.empty_like(k), np.empty_like(v)
    lib().oracle_sort_pairs(ctypes.c_size_t(k.shape[0]), _p(k), _p(v), _p(tk), _p(tv), ctypes.c_int(n_bits))
    return k, v


def extract_ranges(frame: Frame, sorted_keys: np.ndarray) -> np.ndarray:
    gw, gh = frame.grid()
    ranges = np.zeros((gw * gh, 2), np.uint32)
    if sorted_keys.shape[0]:
        shift = 32 if frame.mode == MODE_GLOBAL else 0
        lib().oracle_extract_ranges(ctypes.c_size_t(sorted_keys.shape[0]), _p(sorted_keys), ctypes.c_int(shift), _p(ranges))
    return ranges


def blend(frame: Frame, pre: dict, ranges: np.ndarray, sorted_vals: np.ndarray, to_chw: bool, use_median_depth: bool):
    h, w = frame.height, frame.width
    image = np.zeros((3, h, w) if to_chw else (h, w, 3), np.float32)
    depth = np.zeros((h, w), np.float32)
    alpha = np.zeros((h, w), np.float32)
    cam = frame.c_struct(0)
    lib().oracle_blend(ctypes.byref(cam), _p(ranges), _p(sorted_vals), _p(pre["VPMT1"]), _p(pre["VPMT2"]), _p(pre["VPMT4"]),
                       _p(pre["MT3"]), _p(pre["rgba"]), ctypes.c_int(bool(to_chw)), ctypes.c_int(bool(use_median_depth)),
                       _p(image), _p(depth), _p(alpha))
    return image, depth, alpha


def blend_hybrid_literal(frame: Frame, pre: dict, ranges: np.ndarray, sorted_vals: np.ndarray, use_median_depth: bool = False, margin: float = 1e-3):
    """The HYBRID_BLEND inference image by the word-for-word fp32 restatement of the reference's blend kernel (plane form,
    libm expf, premultiplied core, tail fed by what leaves the core): ``(image [3,H,W], depth [H,W], flags [H,W])`` where
    a flag marks a pixel one of whose decisions fell within ``margin`` (relative) of its bound."""
    h, w = frame.height, frame.width
    image = np.zeros((3, h, w), np.float32)
    depth = np.zeros((h, w), np.float32)
    flags = np.zeros((h, w), np.uint8)
    cam = frame.c_struct(0)
    lib().oracle_blend_hybrid_literal(ctypes.byref(cam), _p(ranges), _p(sorted_vals), _p(pre["VPMT1"]), _p(pre["VPMT2"]), _p(pre["VPMT4"]),
                                      _p(pre["MT3"]), _p(pre["rgba"]), ctypes.c_int(bool(use_median_depth)), ctypes.c_float(margin),
                                      _p(image), _p(depth), _p(flags))
    return image, depth, flags


def render(frame: Frame, positions, scales, rotations, opacities, sh_0, sh_rest,
           to_chw: bool = True, use_median_depth: bool = False) -> dict:
    """Whole inference path; returns every intermediate so that tests can compare stage by stage."""
    pre = preprocess(frame, positions, scales, rotations, opacities, sh_0, sh_rest)
    offsets = inclusive_scan(pre["n_touched"])
    keys, vals = create_instances(frame, pre, offsets)
    skeys, svals = sort_pairs(keys, vals, end_bit(frame))
    ranges = extract_ranges(frame, skeys)
    image, depth, alpha = blend(frame, pre, ranges, svals, to_chw, use_median_depth)
    return {
        "pre": pre, "offsets": offsets, "keys": keys, "vals": vals, "sorted_keys": skeys, "sorted_vals": svals,
        "ranges": ranges, "image": image, "depth": depth, "alpha": alpha,
    }


# ---------------------------------------------------------------------------------------------------------
# training: forward with per-pixel records, backward
# ---------------------------------------------------------------------------------------------------------
def effective_k(K: int) -> int:
    return 32 if K >= 32 else 16 if K >= 16 else 8 if K >= 8 else 4 if K >= 4 else 2 if K >= 2 else 1


def forward(frame: Frame, positions, scales, rotations, opacities, sh_0, sh_rest) -> dict:
    """``_C.forward`` of the reference (R/src/rasterization_api.cu:37-176): scale_modifier is ignored (the
    training preprocess always uses 1, R/include/hybrid_blend/kernels/forward.cuh:10-76), the image is [3,H,W]
    and not clamped, and the per-pixel records needed by backward are returned."""
    import dataclasses
    frame = dataclasses.replace(frame, scale_modifier=1.0)
    pre = preprocess(frame, positions, scales, rotations, opacities, sh_0, sh_rest, train=True)
    offsets = inclusive_scan(pre["n_touched"])
    keys, vals = create_instances(frame, pre, offsets)
    skeys, svals = sort_pairs(keys, vals, end_bit(frame))
    ranges = extract_ranges(frame, skeys)
    h, w = frame.height, frame.width
    K = effective_k(frame.K)
    image = np.zeros((3, h, w), np.float32)
    core_idx = np.full((K, h * w), 0xFFFFFFFF, np.uint32)
    core_info = np.zeros((K, h * w, 4), np.float32)
    tail_info = np.zeros((6, h * w), np.float32)
    cam = frame.c_struct(0)
    lib().oracle_blend_forward(ctypes.byref(cam), _p(ranges), _p(svals), _p(pre["VPMT1"]), _p(pre["VPMT2"]), _p(pre["VPMT4"]),
                               _p(pre["MT3"]), _p(pre["rgba"]), _p(image), _p(core_idx), _p(core_info), _p(tail_info))
    return {"frame": frame, "pre": pre, "offsets": offsets, "sorted_keys": skeys, "sorted_vals": svals, "ranges": ranges,
            "image": image, "core_idx": core_idx, "core_info": core_info, "tail_info": tail_info}


def backward(fwd: dict, grad_image, positions, scales, rotations, opacities, sh_0, sh_rest,
             densification_info: Optional[np.ndarray] = None, use_distance_scaling: bool = False) -> dict:
    """``_C.backward`` of the reference (R/src/rasterization_api.cu:178-363): gradients w.r.t. positions, scales,
    rotations (no normalisation term), opacities, sh_0, sh_rest; ``densification_info`` ([2,N] or [3,N]) is updated
    in place."""
    frame: Frame = fwd["frame"]
    positions, scales, rotations = _f32(positions), _f32(scales), _f32(rotations)
    sh_rest = _f32(sh_rest)
    grad_image = _f32(grad_image)
    n = positions.shape[0]
    total_sh = sh_rest.shape[1]
    pre = fwd["pre"]
    g_pos = np.zeros((n, 3), np.float32)
    g_scale = np.zeros((n, 3), np.float32)
    g_rot = np.zeros((n, 4), np.float32)
    g_op = np.zeros((n, 1), np.float32)
    g_sh0 = np.zeros((n, 1, 3), np.float32)
    g_rest = np.zeros((n, total_sh, 3), np.float32)
    vpmt_mode = frame.mode in (MODE_HYBRID, MODE_OIT)
    g_vpmt = np.zeros((9, n), np.float32) if vpmt_mode else None
    helper = np.zeros(n, np.float32) if densification_info is not None and densification_info.shape[0] == 3 else None
    cam = frame.c_struct(total_sh)
    lib().oracle_blend_backward(
        ctypes.byref(cam), ctypes.c_int(n), _p(fwd["ranges"]), _p(fwd["sorted_vals"]), _p(pre["VPMT1"]), _p(pre["VPMT2"]),
        _p(pre["VPMT4"]), _p(pre["rgba"]), _p(scales), _p(rotations), _p(fwd["image"]), _p(fwd["core_idx"]), _p(fwd["core_info"]),
        _p(fwd["tail_info"]), _p(grad_image), _p(g_pos), _p(g_scale), _p(g_rot), _p(g_op), _p(g_sh0), _p(g_vpmt), _p(helper))
    grad_rgb = g_sh0.reshape(n, 3).copy()
    lib().oracle_preprocess_backward(
        ctypes.byref(cam), ctypes.c_int(n), _p(positions), _p(scales), _p(rotations), _p(sh_rest), _p(pre["n_touched"]),
        _p(pre["clamp_info"]), _p(g_vpmt), _p(helper), _p(g_pos), _p(g_scale), _p(g_rot), _p(g_sh0), _p(g_rest),
        _p(densification_info), ctypes.c_int(bool(use_distance_scaling)))
    return {"positions": g_pos, "scales": g_scale, "rotations": g_rot, "opacities": g_op, "sh_0": g_sh0, "sh_rest": g_rest,
            "grad_rgb": grad_rgb, "grad_VPMT": g_vpmt}


def update_max_weights(frame: Frame, max_weights: np.ndarray, positions, scales, rotations, opacities, weight_threshold: float) -> None:
    """``_C.update_max_weights`` of the reference (R/src/rasterization_api.cu:518-631): ``max_weights`` [N] float32 is
    raised in place to the largest blending weight each Gaussian reaches in this view.  The per-Gaussian stage
    ignores the scale modifier and needs no colours."""
    import dataclasses
    frame = dataclasses.replace(frame, scale_modifier=1.0, active_sh_bases=1)
    n = np.asarray(positions).shape[0]
    pre = preprocess(frame, positions, scales, rotations, opacities, np.zeros((n, 1, 3), np.float32), np.zeros((n, 0, 3), np.float32))
    offsets = inclusive_scan(pre["n_touched"])
    keys, vals = create_instances(frame, pre, offsets)
    skeys, svals = sort_pairs(keys, vals, end_bit(frame))
    ranges = extract_ranges(frame, skeys)
    assert max_weights.dtype == np.float32 and max_weights.flags["C_CONTIGUOUS"]
    cam = frame.c_struct(0)
    lib().oracle_update_max_weights(ctypes.byref(cam), _p(ranges), _p(svals), _p(pre["VPMT1"]), _p(pre["VPMT2"]), _p(pre["VPMT4"]),
                                    _p(pre["MT3"]), _p(pre["rgba"]), _p(max_weights), ctypes.c_float(weight_threshold))


def update_3d_filter(positions, w2c, filter_3d, visibility_mask, width, height, focal_x, focal_y, center_x, center_y,
                     near_plane, clipping_tolerance, distance2filter) -> None:
    """numpy float32 restatement of update_3d_filter (filter3d/src/filter3d_api.cu:6-47, filter3d_kernels.cu:6-35);
    ``filter_3d`` (float32 [N]) and ``visibility_mask`` (bool [N]) are updated in place.
    pinned by: points placed at known angles inside / outside a frustum (tests/test_oracle_pinning.py)."""
    f32 = np.float32
    p = _f32(positions)
    w = _f32(w2c).reshape(16)
    bounds_factor = f32(clipping_tolerance) + f32(0.5)
    wf, hf = f32(width), f32(height)
    max_x, max_y = bounds_factor * wf, bounds_factor * hf
    off_x, off_y = f32(center_x) - f32(0.5) * wf, f32(center_y) - f32(0.5) * hf
    left, right = (-max_x - off_x) / f32(focal_x), (max_x - off_x) / f32(focal_x)
    top, bottom = (-max_y - off_y) / f32(focal_y), (max_y - off_y) / f32(focal_y)
    px, py, pz = p[:, 0], p[:, 1], p[:, 2]
    z = (w[8] * px + w[9] * py + w[10] * pz) + w[11]
    x_clip = (w[0] * px + w[1] * py + w[2] * pz) + w[3]
    y_clip = (w[4] * px + w[5] * py + w[6] * pz) + w[7]
    inside = ~(z < f32(near_plane)) & ~((x_clip < left * z) | (x_clip > right * z)) & ~((y_clip < top * z) | (y_clip > bottom * z))
    cand = f32(distance2filter) * z
    update = inside & ~(filter_3d < cand)
    filter_3d[update] = cand[update]
    visibility_mask[update] = True
