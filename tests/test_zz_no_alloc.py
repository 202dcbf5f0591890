"""The allocation-free scan entry point (``htgs_scan_offsets_static``) against ``htgs_scan_offsets``: same offsets and
the same instance count, bit for bit, on two calls in a row, the second on a smaller input (the entry point's
built-in scratch keeps the first call's contents)."""
import ctypes

import numpy as np
import pytest
import torch

from htgs_amd import _native

pytestmark = pytest.mark.gpu


def _scan(lib, entry, counts: torch.Tensor, with_workspace: bool):
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
    _native.check(entry(ctypes.byref(f)))
    torch.cuda.synchronize()
    return offsets[:n].cpu().numpy().view(np.uint32), int(total.item()) & 0xffffffff


def test_static_scan_matches_the_workspace_scan_twice_in_a_row(cuda):
    lib = _native.lib()
    g = torch.Generator().manual_seed(7)
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
