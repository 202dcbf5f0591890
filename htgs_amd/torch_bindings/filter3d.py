"""3-D filter update of Mip-Splatting, same signature as the reference's
``HTGSCudaBackend/HTGSCudaBackend/torch_bindings/filter3d.py:5-34``."""
import torch

from .. import _native


def update_3d_filter(
    positions: torch.Tensor,
    w2c: torch.Tensor,
    filter_3d: torch.Tensor,
    visibility_mask: torch.Tensor,
    width: int,
    height: int,
    focal_x: float,
    focal_y: float,
    center_x: float,
    center_y: float,
    near_plane: float,
    clipping_tolerance: float,
    distance2filter: float,
) -> None:
    """In place: ``filter_3d[i] = min(filter_3d[i], distance2filter * depth_i)`` and ``visibility_mask[i] = True`` for
    every point inside the view's frustum dilated by ``clipping_tolerance`` (fraction of the image size)."""
    n = positions.shape[0]
    for name, t, dtype, numel in (("positions", positions, torch.float32, 3 * n), ("w2c", w2c, torch.float32, 16),
                                  ("filter_3d", filter_3d, torch.float32, n), ("visibility_mask", visibility_mask, torch.bool, n)):
        if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == dtype and t.is_contiguous() and t.numel() == numel):
            raise RuntimeError(f"{name} must be a contiguous {dtype} GPU tensor with {numel} elements")
    _native.check(_native.lib().htgs_update_3d_filter(
        positions.data_ptr(), w2c.data_ptr(), filter_3d.data_ptr(), visibility_mask.data_ptr(), n, int(width), int(height),
        float(focal_x), float(focal_y), float(center_x), float(center_y), float(near_plane), float(clipping_tolerance),
        float(distance2filter), torch.cuda.current_stream(positions.device).cuda_stream))
