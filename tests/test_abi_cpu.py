"""CPU-side checks of the boundary: the shared library loads without a GPU and exports every symbol that
include/htgs_amd.h declares, the ctypes mirror of ``htgs_frame`` has the C layout, the pure helper functions
agree with the reference's definitions, and the Python operator validates its arguments like the reference
(RuntimeError on an unsupported mode, R/src/rasterization_api.cu:171-172)."""
import ctypes
import os
import re
import subprocess

import pytest
import torch

import oracle
from htgs_amd import _native
from htgs_amd.synthetic import make_scene
from htgs_amd.torch_bindings import RasterizerMode, RasterizerSettings, rasterize

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "htgs_amd.h")


def declared_functions(header=HEADER):
    text = open(header).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(htgs_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert len(names) >= 15
    handle = ctypes.CDLL(_native.LIB_PATH)
    for name in names:
        assert hasattr(handle, name), f"{name} is declared in include/htgs_amd.h but not exported"
    assert sorted(_native.SYMBOLS) == names, "htgs_amd/_native.py must bind exactly the declared entry points"
    _native.lib()


def test_calibration_copy_kernel_is_a_library_of_its_own():
    """The plain copy that calibrates the traffic counters is not part of the drop-in boundary: its own library, no
    declaration in include/, no symbol in the product."""
    from htgs_amd import diagnostics
    assert sorted(os.listdir(os.path.join(ROOT, "include"))) == ["htgs_amd.h"]
    product = ctypes.CDLL(_native.LIB_PATH)
    for name in diagnostics.SYMBOLS:
        assert hasattr(diagnostics.lib(), name)
        assert not hasattr(product, name)
    assert diagnostics.lib().htgs_diag_copy_bytes(None, None, 16, None) == 2
    assert diagnostics.lib().htgs_diag_copy_bytes(1, 1, 8, None) == 2          # not a multiple of 16


def test_frame_struct_layout_matches_the_header(tmp_path):
    fields = [name for name, _ in _native.Frame._fields_]
    src = tmp_path / "layout.c"
    prints = "\n".join(f'    printf("{f} %zu\\n", offsetof(htgs_frame, {f}));' for f in fields)
    src.write_text(f'#include <stdio.h>\n#include <stddef.h>\n#include "{HEADER}"\nint main(void) {{\n'
                   f'    printf("sizeof %zu\\n", sizeof(htgs_frame));\n{prints}\n    return 0;\n}}\n')
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c11", "-o", str(exe), str(src)], check=True)
    out = dict(line.split() for line in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines())
    assert int(out["sizeof"]) == ctypes.sizeof(_native.Frame)
    for f in fields:
        assert int(out[f]) == getattr(_native.Frame, f).offset, f


def test_helper_functions():
    lib = _native.lib()
    assert [lib.htgs_tile_size(m) for m in range(4)] == [8, 8, 16, 8]
    # K is rounded down to a power of two, at most 32 (R/src/hybrid_blend/inference.cu:22-27)
    assert [lib.htgs_effective_k(k) for k in (0, 1, 2, 3, 4, 7, 8, 15, 16, 31, 32, 33, 1000)] == [1, 1, 2, 2, 4, 4, 8, 8, 16, 16, 32, 32, 32]
    for (w, h) in [(256, 256), (1280, 720), (1920, 1080), (1600, 1066), (8, 8), (9, 8), (4096, 4096), (16, 16)]:
        for mode in range(4):
            tile = 16 if mode == 2 else 8
            n_tiles = -(-w // tile) * -(-h // tile)
            bits = (n_tiles - 1).bit_length()           # extract_end_bit, R/include/rasterization_utils.h:3-13
            assert lib.htgs_end_bit(mode, w, h) == bits + (32 if mode == 2 else 0)
            assert lib.htgs_key_bytes(mode, w, h) == (8 if mode == 2 else (2 if bits <= 16 else 4))
            fr = oracle.Frame(None, None, None, mode, 16, 16, w, h, 0.2, 1000.0)
            assert oracle.end_bit(fr) == lib.htgs_end_bit(mode, w, h)
    assert lib.htgs_scan_tmp_words(0) >= 1 and lib.htgs_scan_tmp_words(3_000_000) >= 3_000_000 // 2048
    assert lib.htgs_sort_tmp_words(0) >= 256 and lib.htgs_sort_tmp_words(20_000_000) >= 256 * (20_000_000 // 4096)
    assert lib.htgs_tile_order_words(0, 1920, 1080) == 32400 + 264 and lib.htgs_tile_order_words(2, 1920, 1080) == 8160 + 264
    assert lib.htgs_tile_order_words(0, 8, 8) == 1 + 264 and lib.htgs_tile_order_words(9, 8, 8) == 0


def test_key_widths_of_a_frame_with_depth_order():
    """GLOBAL_ORDERING with htgs_frame.depth_order: the instance keys hold the tile alone; the Gaussians' depth keys are
    taken relative to the near plane and are as wide as the far plane makes them.  (No pointer is followed.)"""
    lib = _native.lib()
    f = _native.Frame()
    f.width, f.height, f.n_primitives = 1920, 1080, 1001
    f.near_plane, f.far_plane = 0.2, 1000.0
    ref = ctypes.byref(f)
    for mode in range(4):
        f.mode = mode
        f.depth_order = None
        plain = (lib.htgs_frame_end_bit(ref), lib.htgs_frame_key_bytes(ref), lib.htgs_frame_sort_passes(ref))
        assert plain == (lib.htgs_end_bit(mode, 1920, 1080), lib.htgs_key_bytes(mode, 1920, 1080), lib.htgs_sort_passes(mode, 1920, 1080))
        f.depth_order = 256                                  # any address that is not NULL
        ordered = (lib.htgs_frame_end_bit(ref), lib.htgs_frame_key_bytes(ref), lib.htgs_frame_sort_passes(ref))
        assert ordered == ((13, 2, 2) if mode == 2 else plain)
    # bits(1000.0) - bits(0.2) + 1 = 0x062d3334 has 27 bits: three passes of 9-bit digits, the result in the second buffers
    f.mode = 2
    n4 = 1004
    assert lib.htgs_depth_order_result_word(ref) == 3 * n4
    f.near_plane = 0.0                                       # all 32 bits, four passes of 8: the first buffers
    assert lib.htgs_depth_order_result_word(ref) == 2 * n4
    f.near_plane, f.far_plane = 0.5, float("inf")
    assert lib.htgs_depth_order_result_word(ref) == 2 * n4
    f.near_plane, f.far_plane = 1.0, 1.5                     # 0x3fc00000 - 0x3f800000 + 1: 23 bits, three passes of 8
    assert lib.htgs_depth_order_result_word(ref) == 3 * n4
    assert lib.htgs_depth_order_words(1001) >= 8 * n4 - n4 and lib.htgs_depth_order_words(0) >= 256


def test_entry_points_reject_bad_frames_without_touching_the_gpu():
    lib = _native.lib()
    f = _native.Frame()
    f.mode = 7
    f.width = f.height = 64
    for fn in (lib.htgs_preprocess, lib.htgs_create_instances):
        assert fn(ctypes.byref(f)) == 1
        assert b"unsupported rasterizer mode" in lib.htgs_last_error()
    sel = ctypes.c_int(0)
    assert lib.htgs_sort_instances(ctypes.byref(f), ctypes.byref(sel)) == 1
    assert lib.htgs_blend(ctypes.byref(f), 0) == 1
    f.mode = 0
    f.n_primitives = 10            # but every pointer is null
    assert lib.htgs_preprocess(ctypes.byref(f)) == 2
    assert lib.htgs_preprocess(None) == 2
    f.n_primitives = -1
    assert lib.htgs_preprocess(ctypes.byref(f)) == 2


def test_training_entry_points_refuse_a_frame_with_depth_order():
    """htgs_frame.depth_order belongs to the inference entry points (the per-Gaussian backward finds a Gaussian's gradient
    rows through offsets[] in index order): every training entry point refuses such a frame before it launches anything."""
    lib = _native.lib()
    f = _native.Frame()
    f.mode, f.width, f.height, f.n_primitives, f.n_instances = 2, 64, 64, 10, 10
    f.prim_floats = _native.PRIM_FLOATS_TRAIN
    f.clamp_info = 256                                       # any address that is not NULL
    f.depth_order = 256
    ref, sel = ctypes.byref(f), ctypes.c_int(0)
    for status in (lib.htgs_forward_front(ref), lib.htgs_forward_back(ref, ctypes.byref(sel)), lib.htgs_blend_forward(ref, 0),
                   lib.htgs_blend_backward(ref, 0), lib.htgs_preprocess_backward(ref), lib.htgs_backward(ref, 0)):
        assert status == 2 and b"depth_order is for the inference entry points" in lib.htgs_last_error()
    f.mode = 0                                               # depth_order is ignored outside GLOBAL_ORDERING
    assert lib.htgs_blend_forward(ref, 0) == 2 and b"null pointer" in lib.htgs_last_error()


def test_record_size_is_checked_by_every_entry_point_that_reads_records():
    """Inference entry points read 80-byte records, the training ones 128-byte records (htgs_frame.prim_floats); a frame
    laid out for the other kind is refused before anything is launched."""
    lib = _native.lib()
    f = _native.Frame()
    f.mode, f.width, f.height, f.n_primitives, f.n_instances = 0, 64, 64, 10, 10
    assert _native.PRIM_FLOATS == 20 and _native.PRIM_FLOATS_TRAIN == 32
    f.prim_floats = _native.PRIM_FLOATS_TRAIN
    assert lib.htgs_blend(ctypes.byref(f), 0) == 2 and b"prim_floats" in lib.htgs_last_error()
    assert lib.htgs_max_weights_blend(ctypes.byref(f), 0, None, ctypes.c_float(0.0)) == 2 and b"prim_floats" in lib.htgs_last_error()
    counts = (ctypes.c_ulonglong * 4)()
    for value in (0, _native.PRIM_FLOATS):
        f.prim_floats = value
        assert lib.htgs_blend_forward(ctypes.byref(f), 0) == 2 and b"prim_floats" in lib.htgs_last_error()
        assert lib.htgs_blend_backward(ctypes.byref(f), 0) == 2 and b"prim_floats" in lib.htgs_last_error()
        assert lib.htgs_blend(ctypes.byref(f), 0) == 2 and b"null pointer" in lib.htgs_last_error()
    f.prim_floats = 24
    assert lib.htgs_preprocess(ctypes.byref(f)) == 2
    assert lib.htgs_create_instances(ctypes.byref(f)) == 2


def test_instance_counts_beyond_32_bit_offsets_are_refused():
    """Offsets into the instance list are 32-bit, as in the reference; 0xffffffff is what the scan publishes when the
    tile counts do not fit.  The host refuses it, and so do the entry points that take the count."""
    from htgs_amd.torch_bindings.rasterization import MAX_INSTANCES, checked_instance_count
    assert MAX_INSTANCES == 2 ** 32 - 2
    assert checked_instance_count(0) == 0 and checked_instance_count(MAX_INSTANCES) == MAX_INSTANCES
    for bad in (MAX_INSTANCES + 1, 2 ** 32, 2 ** 40, -1):
        with pytest.raises(RuntimeError, match="instances"):
            checked_instance_count(bad)
    lib = _native.lib()
    f = _native.Frame()
    f.mode, f.width, f.height, f.n_primitives = 0, 1920, 1080, 1
    sel = ctypes.c_int(0)
    for n in (2 ** 32 - 1, 2 ** 32, 2 ** 33 + 5):
        f.n_instances = n
        assert lib.htgs_create_instances(ctypes.byref(f)) == 2 and b"2^32-2 instances" in lib.htgs_last_error()
        assert lib.htgs_sort_instances(ctypes.byref(f), ctypes.byref(sel)) == 2 and b"2^32-2 instances" in lib.htgs_last_error()
    f.n_instances = 2 ** 32 - 2              # allowed: the next complaint is about the (null) buffers
    assert lib.htgs_create_instances(ctypes.byref(f)) == 2 and b"null pointer" in lib.htgs_last_error()


def test_self_check_entry_points_reject_bad_arguments():
    lib = _native.lib()
    f = _native.Frame()
    f.mode = 2
    f.width = f.height = 64
    assert lib.htgs_check_tile_cull(ctypes.byref(f), 0, None) == 2
    counts = (ctypes.c_ulonglong * 4)()
    assert lib.htgs_check_tile_cull(ctypes.byref(f), 0, counts) == 2               # no ranges
    assert b"null pointer" in lib.htgs_last_error()
    f.mode = 7
    assert lib.htgs_check_tile_cull(ctypes.byref(f), 0, counts) == 1
    assert b"unsupported rasterizer mode" in lib.htgs_last_error()
    assert lib.htgs_check_reciprocal(None, None) == 2


def test_python_api_surface_and_validation():
    import HTGSCudaBackend.torch_bindings as alias
    import htgs_amd
    # the reference's export list (HTGSCudaBackend/__init__.py, torch_bindings/__init__.py)
    for name in ("rasterize", "diff_rasterize", "fast_rasterize", "update_max_weights", "update_3d_filter",
                 "RasterizerSettings", "RasterizerMode"):
        assert getattr(alias, name) is getattr(htgs_amd, name)
    assert [m.value for m in RasterizerMode] == [0, 1, 2, 3]
    assert RasterizerSettings._fields == ("M", "VPM", "cam_position", "mode", "K", "active_sh_bases", "width", "height",
                                          "near_plane", "far_plane", "scale_modifier")
    sc = make_scene(0, 10)
    s = sc.settings(RasterizerMode.OIT_BLEND, 4)
    assert s.as_tuple()[3:] == (3, 4, 1, 256, 256, 0.2, 1000.0, 1.0)
    with pytest.raises(RuntimeError, match="GPU"):
        rasterize(*sc.gaussians(), s, True, False)          # CPU tensors: there is no CPU path
    bad = s._replace(mode=5)
    with pytest.raises(RuntimeError, match="unsupported rasterizer mode"):
        rasterize(*sc.gaussians(), bad, True, False)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_native, "_lib", None)
    monkeypatch.setattr(_native, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no fallback"):
        _native.lib()


def test_bench_refuses_more_than_one_gpu():
    """One frame is rendered on one GPU; asking bench.py for more must end with a message, not with a wrong figure."""
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 2
    assert "--gpus must be 1" in out.stderr and out.stdout.strip() == ""
