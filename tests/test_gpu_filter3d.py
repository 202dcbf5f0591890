"""GPU parity of update_3d_filter against the numpy restatement: element-wise float32, bit for bit."""
import numpy as np
import pytest
import torch

import oracle
from htgs_amd.torch_bindings import update_3d_filter
from scipy.spatial.transform import Rotation

pytestmark = pytest.mark.gpu


def test_update_3d_filter_bit_exact_over_several_views(cuda):
    rng = np.random.default_rng(0)
    n = 200_000
    pts = (rng.normal(size=(n, 3)) * 3.0).astype(np.float32)
    filt = np.full(n, 1e6, np.float32)
    vis = np.zeros(n, bool)
    d_filt = torch.from_numpy(filt.copy()).to(cuda)
    d_vis = torch.zeros(n, dtype=torch.bool, device=cuda)
    d_pts = torch.from_numpy(pts).to(cuda)
    for view in range(4):
        w2c = np.eye(4, dtype=np.float32)
        w2c[:3, :3] = Rotation.from_euler("xyz", [10.0 * view, -25.0 * view, 5.0], degrees=True).as_matrix().astype(np.float32)
        w2c[:3, 3] = [0.1 * view, -0.2, 4.0 + view]
        args = (640, 480, 500.0 + 10 * view, 480.0, 322.5, 238.0, 0.2, 0.15, 0.004)
        oracle.update_3d_filter(pts, w2c, filt, vis, *args)
        assert update_3d_filter(d_pts, torch.from_numpy(w2c).to(cuda), d_filt, d_vis, *args) is None
    torch.cuda.synchronize()
    np.testing.assert_array_equal(d_filt.cpu().numpy().view(np.uint32), filt.view(np.uint32))
    np.testing.assert_array_equal(d_vis.cpu().numpy(), vis)
    assert 0.05 < vis.mean() < 0.95
