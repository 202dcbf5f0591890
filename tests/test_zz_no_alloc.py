"""The allocation-free scan entry point (``htgs_scan_offsets_static``) against ``htgs_scan_offsets``: same offsets and
the same instance count, bit for bit, on two calls in a row, the second on a smaller input (the entry point's
built-in scratch keeps the first call's contents)."""
import ctypes

import numpy as np
import pytest
import torch

from htgs_amd import _native

pytestmark = pytest.mark.gpu


def _scan(lib, entry, counts: torch.Tensor, with_workspace: bool, check_free: bool = True):
    n = counts.numel()
    dev = counts.device
    offsets = torch.full((max(n, 1),), -1, dtype=torch.int32, device=dev)
    total = torch.full((1,), -1, dtype=torch.int32, device=dev)
    tmp = torch.empty(lib.htgs_scan_tmp_words(n), dtype=torch.int32, device=dev) if with_workspace else None
    f = _native.Frame()
    f.n_primitives = n
    f.n_touched = counts.data_ptr() if n else 0
    f.offsets = offsets.data_ptr()
    f.n_instances_dev = total.data_ptr()
    f.scan_tmp = tmp.data_ptr() if tmp is not None else 0
    f.stream = torch.cuda.current_stream(dev).cuda_stream
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(dev)[0]            # hipMemGetInfo: the device's free memory, not torch's cache
    _native.check(entry(ctypes.byref(f)))
    torch.cuda.synchronize()
    if not with_workspace and check_free:
        assert torch.cuda.mem_get_info(dev)[0] == free_before, "htgs_scan_offsets_static changed the device's free memory"
    return offsets[:n].cpu().numpy().view(np.uint32), int(total.item()) & 0xffffffff


def test_static_scan_matches_the_workspace_scan_twice_in_a_row(cuda):
    lib = _native.lib()
    g = torch.Generator().manual_seed(7)
    # (the first call on a device looks up the address of the built-in scratch and may load the library's code: one
    # warm-up call, as a caller would make before graph capture; from then on the device's free memory must not move)
    _scan(lib, lib.htgs_scan_offsets_static, torch.ones(10, dtype=torch.int32, device=cuda), False, check_free=False)
    for n in (3_000_001, 70_001, 2048, 1, 0):          # the second and later calls are smaller than the first
        counts = torch.randint(0, 40, (n,), generator=g, dtype=torch.int32).to(cuda)
        want, want_total = _scan(lib, lib.htgs_scan_offsets, counts, True)
        got, got_total = _scan(lib, lib.htgs_scan_offsets_static, counts, False)
        ref = np.cumsum(counts.cpu().numpy().astype(np.uint64)).astype(np.uint32)
        assert np.array_equal(want, ref) and np.array_equal(got, want), n
        assert got_total == want_total == (int(ref[-1]) if n else 0), n


def test_static_scan_rejects_sizes_beyond_its_scratch(cuda):
    lib = _native.lib()
    f = _native.Frame()
    f.n_primitives = lib.htgs_scan_static_max_primitives() + 1
    one = torch.zeros(1, dtype=torch.int32, device=cuda)
    f.n_touched = f.offsets = f.n_instances_dev = one.data_ptr()
    assert lib.htgs_scan_offsets_static(ctypes.byref(f)) == 2
    assert b"exceed" in lib.htgs_last_error()


def test_static_scan_of_a_frame_with_depth_order(cuda):
    """GLOBAL_ORDERING with htgs_frame.depth_order: the scan stage first sorts the Gaussians by depth on the caller's
    scratch and scans the counts in that order; through the allocation-free entry point the offsets, the instance count and
    the depth order must be those of htgs_scan_offsets, and the device's free memory must not move."""
    from htgs_amd.synthetic import make_scene
    from htgs_amd.torch_bindings import FrameBuffers, RasterizerMode
    lib = _native.lib()
    scene = make_scene(1, 150_000).to(cuda)
    settings = scene.settings(RasterizerMode.ALPHA_BLEND_GLOBAL_ORDERING, 16)
    frames = [FrameBuffers(*scene.gaussians(), settings, True, False) for _ in range(2)]
    for fb in frames:
        assert fb.depth_order is not None
        fb.preprocess()
    frames[0].scan()
    _scan(lib, lib.htgs_scan_offsets_static, torch.ones(10, dtype=torch.int32, device=cuda), False, check_free=False)
    frames[1].frame.scan_tmp = 0
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(cuda)[0]
    _native.check(lib.htgs_scan_offsets_static(frames[1]._ref))
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(cuda)[0] == free_before
    assert torch.equal(frames[0].offsets, frames[1].offsets)
    assert frames[0].read_instance_count() == frames[1].read_instance_count() > 0
    word = lib.htgs_depth_order_result_word(frames[0]._ref)
    assert torch.equal(frames[0].depth_order[word:word + scene.positions.shape[0]], frames[1].depth_order[word:word + scene.positions.shape[0]])
