"""ctypes binding of ``libhtgs_amd.so`` (declarations: ``include/htgs_amd.h``).

There is no CPU fallback: if the library has not been built, loading raises.
"""
from __future__ import annotations

import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libhtgs_amd.so")

PRIM_FLOATS = 20
PRIM_FLOATS_TRAIN = 32

c_float_p = ctypes.c_void_p


class Frame(ctypes.Structure):
    """``struct htgs_frame``."""
    _fields_ = [
        ("positions", ctypes.c_void_p),
        ("scales", ctypes.c_void_p),
        ("rotations", ctypes.c_void_p),
        ("opacities", ctypes.c_void_p),
        ("sh_0", ctypes.c_void_p),
        ("sh_rest", ctypes.c_void_p),
        ("M", ctypes.c_void_p),
        ("VPM", ctypes.c_void_p),
        ("cam_position", ctypes.c_void_p),
        ("n_primitives", ctypes.c_int32),
        ("total_sh_bases", ctypes.c_int32),
        ("active_sh_bases", ctypes.c_int32),
        ("mode", ctypes.c_int32),
        ("K", ctypes.c_int32),
        ("width", ctypes.c_int32),
        ("height", ctypes.c_int32),
        ("near_plane", ctypes.c_float),
        ("far_plane", ctypes.c_float),
        ("scale_modifier", ctypes.c_float),
        ("n_touched", ctypes.c_void_p),
        ("offsets", ctypes.c_void_p),
        ("bounds", ctypes.c_void_p),
        ("prim", ctypes.c_void_p),
        ("prim_floats", ctypes.c_int32),
        ("clamp_info", ctypes.c_void_p),
        ("scan_tmp", ctypes.c_void_p),
        ("n_instances_dev", ctypes.c_void_p),
        ("ranges", ctypes.c_void_p),
        ("long_tiles", ctypes.c_void_p),
        ("long_list_threshold", ctypes.c_int32),
        ("tile_order", ctypes.c_void_p),
        ("depth_order", ctypes.c_void_p),
        ("n_instances", ctypes.c_uint64),
        ("keys", ctypes.c_void_p * 2),
        ("vals", ctypes.c_void_p * 2),
        ("sort_tmp", ctypes.c_void_p),
        ("image", ctypes.c_void_p),
        ("depth", ctypes.c_void_p),
        ("to_chw", ctypes.c_int32),
        ("use_median_depth", ctypes.c_int32),
        ("fast_math", ctypes.c_int32),
        ("core_idx", ctypes.c_void_p),
        ("core_info", ctypes.c_void_p),
        ("tail_info", ctypes.c_void_p),
        ("grad_image", ctypes.c_void_p),
        ("grad_rows", ctypes.c_void_p),
        ("dens_helper", ctypes.c_void_p),
        ("grad_positions", ctypes.c_void_p),
        ("grad_scales", ctypes.c_void_p),
        ("grad_rotations", ctypes.c_void_p),
        ("grad_opacities", ctypes.c_void_p),
        ("grad_sh_0", ctypes.c_void_p),
        ("grad_sh_rest", ctypes.c_void_p),
        ("densification_info", ctypes.c_void_p),
        ("densification_rows", ctypes.c_int32),
        ("use_distance_scaling", ctypes.c_int32),
        ("pixel_scratch", ctypes.c_void_p),
        ("stream", ctypes.c_void_p),
    ]


# every symbol include/htgs_amd.h declares: name -> (restype, argtypes)
_FRAME_P = ctypes.POINTER(Frame)
SYMBOLS = {
    "htgs_last_error": (ctypes.c_char_p, []),
    "htgs_tile_size": (ctypes.c_int, [ctypes.c_int]),
    "htgs_effective_k": (ctypes.c_int, [ctypes.c_int]),
    "htgs_end_bit": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "htgs_key_bytes": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "htgs_sort_passes": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "htgs_frame_end_bit": (ctypes.c_int, [_FRAME_P]),
    "htgs_frame_key_bytes": (ctypes.c_int, [_FRAME_P]),
    "htgs_frame_sort_passes": (ctypes.c_int, [_FRAME_P]),
    "htgs_frame_depth_sort_passes": (ctypes.c_int, [_FRAME_P]),
    "htgs_depth_order_words": (ctypes.c_size_t, [ctypes.c_int]),
    "htgs_depth_order_result_word": (ctypes.c_size_t, [_FRAME_P]),
    "htgs_scan_tmp_words": (ctypes.c_size_t, [ctypes.c_int]),
    "htgs_sort_tmp_words": (ctypes.c_size_t, [ctypes.c_uint64]),
    "htgs_tile_order_words": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "htgs_preprocess": (ctypes.c_int, [_FRAME_P]),
    "htgs_scan_offsets": (ctypes.c_int, [_FRAME_P]),
    "htgs_scan_offsets_static": (ctypes.c_int, [_FRAME_P]),
    "htgs_scan_static_max_primitives": (ctypes.c_int, []),
    "htgs_create_instances": (ctypes.c_int, [_FRAME_P]),
    "htgs_sort_instances": (ctypes.c_int, [_FRAME_P, ctypes.POINTER(ctypes.c_int)]),
    "htgs_extract_ranges": (ctypes.c_int, [_FRAME_P, ctypes.c_int]),
    "htgs_blend": (ctypes.c_int, [_FRAME_P, ctypes.c_int]),
    "htgs_render_front": (ctypes.c_int, [_FRAME_P]),
    "htgs_render_back": (ctypes.c_int, [_FRAME_P]),
    "htgs_forward_front": (ctypes.c_int, [_FRAME_P]),
    "htgs_forward_back": (ctypes.c_int, [_FRAME_P, ctypes.POINTER(ctypes.c_int)]),
    "htgs_blend_forward": (ctypes.c_int, [_FRAME_P, ctypes.c_int]),
    "htgs_blend_backward": (ctypes.c_int, [_FRAME_P, ctypes.c_int]),
    "htgs_preprocess_backward": (ctypes.c_int, [_FRAME_P]),
    "htgs_backward": (ctypes.c_int, [_FRAME_P, ctypes.c_int]),
    "htgs_max_weights_front": (ctypes.c_int, [_FRAME_P]),
    "htgs_max_weights_back": (ctypes.c_int, [_FRAME_P, ctypes.c_void_p, ctypes.c_float]),
    "htgs_max_weights_blend": (ctypes.c_int, [_FRAME_P, ctypes.c_int, ctypes.c_void_p, ctypes.c_float]),
    "htgs_update_3d_filter": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                             ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_float,
                                             ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_void_p]),
    "htgs_check_reciprocal": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p]),
    "htgs_check_tile_cull": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]),
}

_lib = None


def lib() -> ctypes.CDLL:
    """The loaded library.  Raises if it has not been built (``python -m htgs_amd.build``)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"htgs_amd: native library {LIB_PATH} is missing; build it with `python -m htgs_amd.build` "
                "(there is no fallback path)")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SYMBOLS.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def check(status: int) -> None:
    """Non-zero status -> RuntimeError with the library's message (the reference throws std::runtime_error,
    R/src/rasterization_api.cu:171-172, which pybind turns into RuntimeError)."""
    if status != 0:
        raise RuntimeError(lib().htgs_last_error().decode())
