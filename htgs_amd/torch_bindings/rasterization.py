"""Operator API of the rasterizer on PyTorch-ROCm.

Same names, argument order, shapes and error behaviour as the reference's
``HTGSCudaBackend/HTGSCudaBackend/torch_bindings/rasterization.py`` (``RasterizerMode`` :9-13,
``RasterizerSettings`` :16-42, ``rasterize`` :140-163), implemented on the C ABI of ``libhtgs_amd.so``:
torch only owns the device memory and the stream, every kernel is hand-written HIP.
"""
from __future__ import annotations

import ctypes
import threading
from enum import Enum
from typing import NamedTuple, Optional

import torch

from .. import _native


class RasterizerMode(Enum):
    HYBRID_BLEND = 0
    ALPHA_BLEND_FIRST_K = 1
    ALPHA_BLEND_GLOBAL_ORDERING = 2
    OIT_BLEND = 3


class RasterizerSettings(NamedTuple):
    M: torch.Tensor  # [4,4] world -> camera
    VPM: torch.Tensor  # [4,4] world -> screen (pixel coordinates with the half-pixel shift, NDC depth)
    cam_position: torch.Tensor  # [3] world space
    mode: RasterizerMode
    K: int  # core size of HYBRID_BLEND / ALPHA_BLEND_FIRST_K
    active_sh_bases: int
    width: int
    height: int
    near_plane: float
    far_plane: float
    scale_modifier: float

    def as_tuple(self) -> tuple:
        return (self.M, self.VPM, self.cam_position, self.mode.value, self.K, self.active_sh_bases,
                self.width, self.height, self.near_plane, self.far_plane, self.scale_modifier)


def _mode_value(mode) -> int:
    return int(mode.value) if isinstance(mode, Enum) else int(mode)


def _dev_f32(t: torch.Tensor, name: str, device: Optional[torch.device] = None) -> torch.Tensor:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU (got {t.device})")
    if t.dtype != torch.float32:
        raise RuntimeError(f"{name} must be float32 (got {t.dtype})")
    if device is not None and t.device != device:
        raise RuntimeError(f"{name} is on {t.device}, expected {device}")
    return t.contiguous()


def _ptr(t: Optional[torch.Tensor]) -> int:
    return 0 if t is None or t.numel() == 0 else t.data_ptr()


MAX_INSTANCES = 0xfffffffe


def checked_instance_count(published: int) -> int:
    """The instance count the scan published.  Offsets into the instance list are 32-bit, as in the reference
    (R/include/hybrid_blend/buffer_utils.h:22-54); the scan publishes 0xffffffff for a frame whose tile counts add up
    to more than ``MAX_INSTANCES``, and such a frame is refused instead of being rendered from wrapped offsets."""
    if published < 0 or published > MAX_INSTANCES:
        raise RuntimeError(f"the frame needs more than {MAX_INSTANCES} (tile, Gaussian) instances; offsets are 32-bit -- "
                           "render fewer Gaussians per call or a smaller image")
    return published


class ScratchPool:
    """Grow-only device scratch that inference frames on one (device, stream, host thread) reuse, so that a steady
    stream of ``rasterize`` calls allocates nothing but its outputs.  A frame is issued front to back by one thread and
    ordered by the stream, which is what makes the reuse safe; frames issued on another stream or by another thread
    get another pool.  Training frames do not use it (their scratch has to survive until backward).

    The pools are bounded: the pool of a thread that has ended is dropped the next time a pool is looked up, and with
    ``ScratchPool.max_bytes`` set the pools used least recently are dropped (never the one being asked for) until the
    others fit under it.  Dropping a pool only releases the references; torch's stream-ordered allocator keeps the memory
    valid for work already queued."""

    _pools: dict = {}
    _lock = threading.Lock()
    _tick = 0
    max_bytes: Optional[int] = None       # cap on the bytes held by all pools together (None: no cap)

    def __init__(self):
        self.buffers: dict = {}
        self.last_used = 0

    def nbytes(self) -> int:
        return sum(b.numel() * b.element_size() for b in self.buffers.values())

    @staticmethod
    def _stream_id(device: torch.device) -> int:
        return torch.cuda.current_stream(device).cuda_stream if device.type == "cuda" else 0

    @classmethod
    def current(cls, device: torch.device) -> "ScratchPool":
        key = (device.type, device.index, cls._stream_id(device), threading.get_ident())
        with cls._lock:
            pool = cls._pools.get(key)
            if pool is None:
                pool = cls._pools[key] = ScratchPool()
                alive = {t.ident for t in threading.enumerate()}
                for other in [k for k in cls._pools if k[3] not in alive]:
                    del cls._pools[other]
            cls._tick += 1
            pool.last_used = cls._tick
            if cls.max_bytes is not None:
                others = sorted((k for k in cls._pools if k != key), key=lambda k: cls._pools[k].last_used)
                held = sum(p.nbytes() for p in cls._pools.values())
                for k in others:
                    if held <= cls.max_bytes:
                        break
                    held -= cls._pools[k].nbytes()
                    del cls._pools[k]
        return pool

    @classmethod
    def clear(cls):
        with cls._lock:
            cls._pools.clear()

    @classmethod
    def total_bytes(cls) -> int:
        with cls._lock:
            return sum(p.nbytes() for p in cls._pools.values())

    def get(self, name: str, numel: int, dtype: torch.dtype, device: torch.device, headroom: float = 0.0) -> torch.Tensor:
        buf = self.buffers.get(name)
        if buf is None or buf.dtype != dtype or buf.numel() < numel or buf.device != device:
            buf = torch.empty(max(int(numel * (1.0 + headroom)), 1), dtype=dtype, device=device)
            self.buffers[name] = buf
        return buf


class FrameBuffers:
    """One frame on the C ABI: validated inputs, caller-owned scratch, outputs.

    Scratch mirrors the reference's PerPrimitive / PerTile / PerInstance blobs
    (R/include/hybrid_blend/buffer_utils.h:22-94) as individual torch tensors.  The methods map one to
    one onto the entry points of ``include/htgs_amd.h`` so that tests and the benchmark can run and time
    single stages; ``rasterize`` runs ``front`` / ``back``.
    """

    def __init__(self, positions, scales, rotations, opacities, sh_0, sh_rest, settings: RasterizerSettings,
                 to_chw: bool = True, use_median_depth: bool = False, train: bool = False,
                 pool: Optional[ScratchPool] = None, fast: bool = False, long_list_threshold: int = 0, order_tiles: bool = True,
                 order_gaussians: bool = True):
        mode = _mode_value(settings.mode)
        if mode not in (0, 1, 2, 3):
            raise RuntimeError("unsupported rasterizer mode")
        self.lib = _native.lib()
        positions = _dev_f32(positions, "positions")
        dev = positions.device
        self.device = dev
        self.positions = positions
        self.scales = _dev_f32(scales, "scales", dev)
        self.rotations = _dev_f32(rotations, "rotations", dev)
        self.opacities = _dev_f32(opacities, "opacities", dev)
        # sh_0 / sh_rest may be None for the passes that compute no colour (update_max_weights)
        self.sh_0 = _dev_f32(sh_0, "sh_0", dev) if sh_0 is not None else None
        self.sh_rest = _dev_f32(sh_rest, "sh_rest", dev) if sh_rest is not None else torch.empty((positions.shape[0], 0, 3), dtype=torch.float32, device=dev)
        self.M = _dev_f32(settings.M, "settings.M", dev)
        self.VPM = _dev_f32(settings.VPM, "settings.VPM", dev)
        self.cam_position = _dev_f32(settings.cam_position, "settings.cam_position", dev)
        n = positions.shape[0]
        if positions.shape != (n, 3) or self.scales.shape != (n, 3) or self.rotations.shape != (n, 4) \
                or self.opacities.numel() != n or (self.sh_0 is not None and self.sh_0.numel() != 3 * n) or self.sh_rest.dim() != 3 \
                or self.sh_rest.shape[0] != n or self.sh_rest.shape[2] != 3:
            raise RuntimeError("inconsistent Gaussian tensor shapes")
        if self.M.numel() != 16 or self.VPM.numel() != 16 or self.cam_position.numel() != 3:
            raise RuntimeError("settings.M / VPM must be 4x4 and cam_position must have 3 elements")
        self.n = n
        self.mode = mode
        self.width, self.height = int(settings.width), int(settings.height)
        self.tile = self.lib.htgs_tile_size(mode)
        self.grid_w = (self.width + self.tile - 1) // self.tile
        self.grid_h = (self.height + self.tile - 1) // self.tile
        self.n_tiles = self.grid_w * self.grid_h
        self.to_chw = bool(to_chw)

        self.pool = pool
        self.n_touched = self._scratch("n_touched", n, torch.int32)[:n]
        self.offsets = self._scratch("offsets", n, torch.int32)[:n]
        self.bounds = self._scratch("bounds", 4 * n, torch.int16)[:4 * n].view(n, 4)
        # (training frames use 128-byte records: the backward pass finds the slot of an instance's gradient row in them)
        self.prim_floats = _native.PRIM_FLOATS_TRAIN if train else _native.PRIM_FLOATS
        self.prim = self._scratch("prim", self.prim_floats * n, torch.float32)[:self.prim_floats * n].view(n, self.prim_floats)
        self.clamp_info = torch.empty((3, n), dtype=torch.uint8, device=dev) if train else None
        self.scan_tmp = self._scratch("scan_tmp", self.lib.htgs_scan_tmp_words(n), torch.int32)
        self.n_instances_dev = self._scratch("n_instances_dev", 1, torch.int32)    # written by the scan
        self.ranges = self._scratch("ranges", 2 * self.n_tiles, torch.int32)[:2 * self.n_tiles].view(self.n_tiles, 2)
        # the modes that walk all of a list (every one but GLOBAL_ORDERING): the list of tiles with very long instance
        # lists, which several waves or workgroups walk together (inference, training forward and backward, max weights)
        self.long_tiles = self._scratch("long_tiles", 3 * self.n_tiles + 8, torch.int32) if mode != 2 else None
        # the tiles in the order the blend kernels take them (longest lists first), written with the ranges
        self.tile_order = (self._scratch("tile_order", self.lib.htgs_tile_order_words(mode, self.width, self.height), torch.int32)
                           if order_tiles else None)
        # GLOBAL_ORDERING inference: the Gaussians sorted by depth before the instances are made, whose keys then hold the
        # tile alone (two sort passes over 2-byte keys instead of five over 8-byte keys, the same sorted list).  The
        # image-only fast path of the two modes with a sorted core: the same with coarse depth keys (one pass), so that a
        # tile's fragments arrive roughly front to back and few of them have to be inserted in front of others
        self.depth_order = (self._scratch("depth_order", self.lib.htgs_depth_order_words(n), torch.int32)
                            if order_gaussians and not train and (mode == 2 or (fast and mode in (0, 1))) else None)
        self.image = torch.empty((3, self.height, self.width) if to_chw else (self.height, self.width, 3),
                                 dtype=torch.float32, device=dev)
        # the image-only fast path (``fast_rasterize``) writes no depth map
        self.depth = None if fast else torch.empty((self.height, self.width), dtype=torch.float32, device=dev)
        self.keys = [None, None]
        self.vals = [None, None]
        self.sort_tmp = None
        self.n_instances = 0
        self.selector = 0

        f = _native.Frame()
        f.positions, f.scales, f.rotations = _ptr(self.positions), _ptr(self.scales), _ptr(self.rotations)
        f.opacities, f.sh_0, f.sh_rest = _ptr(self.opacities), _ptr(self.sh_0), _ptr(self.sh_rest)
        f.M, f.VPM, f.cam_position = _ptr(self.M), _ptr(self.VPM), _ptr(self.cam_position)
        f.n_primitives = n
        f.total_sh_bases = int(self.sh_rest.shape[1])
        f.active_sh_bases = int(settings.active_sh_bases)
        f.mode, f.K = mode, int(settings.K)
        f.width, f.height = self.width, self.height
        f.near_plane, f.far_plane = float(settings.near_plane), float(settings.far_plane)
        f.scale_modifier = float(settings.scale_modifier)
        f.n_touched, f.offsets, f.bounds, f.prim = _ptr(self.n_touched), _ptr(self.offsets), _ptr(self.bounds), _ptr(self.prim)
        f.prim_floats = self.prim_floats
        f.clamp_info = _ptr(self.clamp_info)
        f.scan_tmp, f.n_instances_dev = _ptr(self.scan_tmp), _ptr(self.n_instances_dev)
        f.ranges = _ptr(self.ranges)
        f.long_tiles = _ptr(self.long_tiles)
        f.tile_order = _ptr(self.tile_order)
        f.depth_order = _ptr(self.depth_order)
        f.long_list_threshold = int(long_list_threshold)      # 0: the library's default
        f.image, f.depth = _ptr(self.image), _ptr(self.depth)
        f.to_chw, f.use_median_depth, f.fast_math = int(bool(to_chw)), int(bool(use_median_depth)), int(bool(fast))
        f.stream = torch.cuda.current_stream(dev).cuda_stream
        self.frame = f
        self._ref = ctypes.byref(f)
        self.key_bytes = self.lib.htgs_frame_key_bytes(self._ref)
        self.end_bit = self.lib.htgs_frame_end_bit(self._ref)
        self.sort_passes = self.lib.htgs_frame_sort_passes(self._ref)

    def _scratch(self, name: str, numel: int, dtype: torch.dtype, headroom: float = 0.0) -> torch.Tensor:
        """A buffer of at least ``numel`` elements: from the pool if the frame has one, else freshly allocated."""
        if self.pool is not None:
            return self.pool.get(name, numel, dtype, self.device, headroom)
        return torch.empty(max(int(numel), 1), dtype=dtype, device=self.device)

    # ---- stages -----------------------------------------------------------------------------
    def preprocess(self):
        _native.check(self.lib.htgs_preprocess(self._ref))

    def scan(self):
        _native.check(self.lib.htgs_scan_offsets(self._ref))

    def front(self):
        _native.check(self.lib.htgs_render_front(self._ref))

    def read_instance_count(self) -> int:
        """The frame's only host/device synchronisation (the reference's cudaMemcpy at
        R/src/hybrid_blend/inference.cu:118-119)."""
        return checked_instance_count(int(self.n_instances_dev.item()) & 0xffffffff) if self.n > 0 else 0

    def alloc_instances(self, n_instances: int):
        dev = self.device
        self.n_instances = int(n_instances)
        key_dtype = {2: torch.int16, 4: torch.int32, 8: torch.int64}[self.key_bytes]
        m = max(self.n_instances, 1)
        # pooled frames keep 1/8 headroom so that a slowly changing instance count does not reallocate every frame
        self.keys = [self._scratch(f"keys{i}_{self.key_bytes}", m, key_dtype, 0.125) for i in range(2)]
        self.vals = [self._scratch(f"vals{i}", m, torch.int32, 0.125) for i in range(2)]
        self.sort_tmp = self._scratch("sort_tmp", self.lib.htgs_sort_tmp_words(self.n_instances), torch.int32, 0.125)
        f = self.frame
        f.n_instances = self.n_instances
        f.keys[0], f.keys[1] = _ptr(self.keys[0]), _ptr(self.keys[1])
        f.vals[0], f.vals[1] = _ptr(self.vals[0]), _ptr(self.vals[1])
        f.sort_tmp = _ptr(self.sort_tmp)

    def create_instances(self):
        _native.check(self.lib.htgs_create_instances(self._ref))

    def sort(self) -> int:
        sel = ctypes.c_int(0)
        _native.check(self.lib.htgs_sort_instances(self._ref, ctypes.byref(sel)))
        self.selector = sel.value
        return self.selector

    def extract_ranges(self):
        _native.check(self.lib.htgs_extract_ranges(self._ref, self.selector))

    def blend(self):
        _native.check(self.lib.htgs_blend(self._ref, self.selector))

    def back(self):
        _native.check(self.lib.htgs_render_back(self._ref))
        self.selector = self.sort_passes & 1 if self.n_instances > 0 else 0

    def run(self):
        self.front()
        self.alloc_instances(self.read_instance_count())
        self.back()
        return self.image, self.depth

    # ---- training ---------------------------------------------------------------------------
    def alloc_pixel_records(self):
        """PerPixelBuffers of the reference (R/include/hybrid_blend/buffer_utils.h:96-108); here a plane holds the pixels
        tile by tile (64 per 8x8 tile, row-major inside the tile), see ``records_in_image_order``."""
        dev, P = self.device, 64 * self.n_tiles
        K = self.lib.htgs_effective_k(self.frame.K)
        if self.mode in (0, 1):
            self.core_idx = torch.empty((K, P), dtype=torch.int32, device=dev)
            self.core_info = torch.empty((K, P, 4), dtype=torch.float32, device=dev)
            self.frame.core_idx, self.frame.core_info = _ptr(self.core_idx), _ptr(self.core_info)
        if self.mode in (0, 3):
            self.tail_info = torch.empty((6, P), dtype=torch.float32, device=dev)
            self.frame.tail_info = _ptr(self.tail_info)

    def records_in_image_order(self, records: torch.Tensor) -> torch.Tensor:
        """``core_idx`` / ``tail_info`` (``[planes, 64 * n_tiles]``) or ``core_info`` (``[planes, 64 * n_tiles, 4]``) as
        ``[planes, H * W(, 4)]``, the layout of the reference's per-pixel buffers."""
        planes, tail = records.shape[0], records.shape[2:]
        t = records.reshape(planes, self.grid_h, self.grid_w, 8, 8, *tail)
        t = t.permute(0, 1, 3, 2, 4, *range(5, 5 + len(tail))).reshape(planes, 8 * self.grid_h, 8 * self.grid_w, *tail)
        return t[:, :self.height, :self.width].reshape(planes, self.height * self.width, *tail)

    def forward_front(self):
        _native.check(self.lib.htgs_forward_front(self._ref))

    def forward_back(self):
        sel = ctypes.c_int(0)
        _native.check(self.lib.htgs_forward_back(self._ref, ctypes.byref(sel)))
        self.selector = sel.value

    def blend_forward(self):
        _native.check(self.lib.htgs_blend_forward(self._ref, self.selector))

    def run_forward(self):
        """``_C.forward`` of the reference: unclamped [3,H,W] image; the frame keeps what backward needs."""
        assert self.clamp_info is not None and self.to_chw, "training frames are built with train=True, to_chw=True"
        self.forward_front()
        self.alloc_instances(self.read_instance_count())
        self.alloc_pixel_records()
        self.forward_back()
        return self.image

    def run_backward(self, grad_image: torch.Tensor, densification_info: Optional[torch.Tensor] = None,
                     use_distance_scaling: bool = False):
        """``_C.backward`` of the reference: the six gradients; ``densification_info`` is updated in place."""
        dev, n = self.device, self.n
        grad_image = _dev_f32(grad_image, "grad_image", dev)
        if tuple(grad_image.shape) != (3, self.height, self.width):
            raise RuntimeError("grad_image must be [3,H,W]")
        total_sh = int(self.sh_rest.shape[1])
        f32 = dict(dtype=torch.float32, device=dev)
        # one row per instance, every one written by the blend kernels: no initialisation needed
        self.grad_rows = torch.empty((max(self.n_instances, 1), 16), **f32)
        grads = [torch.empty((n, 3), **f32), torch.empty((n, 3), **f32), torch.empty((n, 4), **f32), torch.empty((n, 1), **f32),
                 torch.empty((n, 1, 3), **f32), torch.empty((n, total_sh, 3), **f32)]
        f = self.frame
        f.stream = torch.cuda.current_stream(dev).cuda_stream
        f.grad_image, f.grad_rows = _ptr(grad_image), _ptr(self.grad_rows)
        (f.grad_positions, f.grad_scales, f.grad_rotations, f.grad_opacities, f.grad_sh_0, f.grad_sh_rest) = [_ptr(g) for g in grads]
        rows = 0
        helper = None
        if densification_info is not None and densification_info.numel() > 0:
            rows = int(densification_info.shape[0])
            if rows not in (2, 3) or densification_info.numel() != rows * n or not densification_info.is_contiguous() \
                    or densification_info.dtype != torch.float32 or densification_info.device != dev:
                raise RuntimeError("densification_info must be a contiguous float32 [2,N] or [3,N] tensor on the GPU")
            f.densification_info = densification_info.data_ptr()
            if rows == 3:
                helper = torch.empty(max(self.n_instances, 1), **f32)
        else:
            f.densification_info = 0
        f.densification_rows = rows
        f.dens_helper = _ptr(helper)
        f.use_distance_scaling = int(bool(use_distance_scaling))
        self.grads = grads           # keeps the bound outputs alive for blend_backward / preprocess_backward
        _native.check(self.lib.htgs_backward(self._ref, self.selector))
        return grads

    def blend_backward(self):
        """The blend half of the last ``run_backward`` again, into the same buffers (per-stage timing)."""
        _native.check(self.lib.htgs_blend_backward(self._ref, self.selector))

    def preprocess_backward(self):
        """The per-Gaussian half of the last ``run_backward`` again (densification_info is accumulated once more)."""
        _native.check(self.lib.htgs_preprocess_backward(self._ref))


class _Rasterize(torch.autograd.Function):
    """Differentiable render (reference: rasterization.py:45-113).  The frame object saved on ``ctx`` owns the
    scratch that the reference returns to Python as four byte blobs and keeps in ``ctx.save_for_backward``
    (:71-82); like those it lives as long as ``ctx``, so ``backward(retain_graph=True)`` can run again."""

    @staticmethod
    def forward(ctx, positions, scales, rotations, opacities, sh_0, sh_rest, densification_info, rasterizer_settings,
                use_distance_scaling):
        fb = FrameBuffers(positions, scales, rotations, opacities, sh_0, sh_rest, rasterizer_settings, True, False, train=True)
        image = fb.run_forward()
        ctx.fb = fb
        ctx.save_for_backward(positions, scales, rotations, opacities, sh_0, sh_rest)
        ctx.densification_info = densification_info
        ctx.mark_non_differentiable(densification_info)
        ctx.use_distance_scaling = use_distance_scaling
        return image

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_image):
        _ = ctx.saved_tensors      # raises if an input was modified in place since forward
        grads = ctx.fb.run_backward(grad_image, ctx.densification_info, ctx.use_distance_scaling)
        return (*grads, None, None, None)


def diff_rasterize(
    positions: torch.Tensor,
    scales: torch.Tensor,
    rotations: torch.Tensor,
    opacities: torch.Tensor,
    sh_0: torch.Tensor,
    sh_rest: torch.Tensor,
    densification_info: torch.Tensor,
    settings: RasterizerSettings,
    use_distance_scaling: bool,
) -> torch.Tensor:
    """Training render: unclamped image ``[3,H,W]``, differentiable w.r.t. the six Gaussian tensors;
    ``densification_info`` ([0], [2,N] or [3,N]) is updated in place during backward (reference:
    rasterization.py:116-137).  ``settings.scale_modifier`` is ignored, as in the reference."""
    return _Rasterize.apply(positions, scales, rotations, opacities, sh_0, sh_rest, densification_info, settings,
                            use_distance_scaling)


def update_max_weights(
    max_weights: torch.Tensor,
    positions: torch.Tensor,
    scales: torch.Tensor,
    rotations: torch.Tensor,
    opacities: torch.Tensor,
    settings: RasterizerSettings,
    weight_threshold: float,
) -> None:
    """Raises ``max_weights`` ([N] or [N,1] float32, in place) to the largest blending weight each Gaussian reaches in
    this view; weights below ``weight_threshold`` are ignored (reference: rasterization.py:189-206)."""
    run_max_weights(max_weights, positions, scales, rotations, opacities, settings, weight_threshold)


def run_max_weights(max_weights, positions, scales, rotations, opacities, settings, weight_threshold, long_list_threshold: int = 0) -> FrameBuffers:
    """``update_max_weights`` with the length beyond which a tile's list is shared between waves and workgroups made
    explicit (0: the library's default); returns the frame."""
    n = positions.shape[0]
    if not (isinstance(max_weights, torch.Tensor) and max_weights.is_cuda and max_weights.dtype == torch.float32
            and max_weights.is_contiguous() and max_weights.numel() == n):
        raise RuntimeError("max_weights must be a contiguous float32 GPU tensor with one element per Gaussian")
    with torch.no_grad():
        fb = FrameBuffers(positions, scales, rotations, opacities, None, None, settings, True, False,
                          pool=ScratchPool.current(positions.device), long_list_threshold=long_list_threshold)
        if fb.mode in (0, 3):
            # the tail weights of the tiles with very long lists, kept between the pass's two walks
            fb.pixel_scratch = fb._scratch("pixel_scratch", 64 * fb.n_tiles, torch.float32)
            fb.frame.pixel_scratch = _ptr(fb.pixel_scratch)
        _native.check(fb.lib.htgs_max_weights_front(fb._ref))
        fb.alloc_instances(fb.read_instance_count())
        _native.check(fb.lib.htgs_max_weights_back(fb._ref, max_weights.data_ptr(), float(weight_threshold)))
    return fb


def rasterize(
    positions: torch.Tensor,
    scales: torch.Tensor,
    rotations: torch.Tensor,
    opacities: torch.Tensor,
    sh_0: torch.Tensor,
    sh_rest: torch.Tensor,
    settings: RasterizerSettings,
    to_chw: bool,
    use_median_depth: bool,
) -> tuple[torch.Tensor, torch.Tensor]:
    """Inference render: ``(image, depth)`` with ``image`` ``[3,H,W]`` (``to_chw``) or ``[H,W,3]`` clamped to
    [0,1] and ``depth`` ``[1,H,W]`` / ``[H,W,1]`` (reference: rasterization.py:140-163).

    HYBRID_BLEND and ALPHA_BLEND_FIRST_K hold a pixel's K nearest fragments as sorted 64-bit keys, in which alpha is a
    fraction of 19 to 23 bits (image within 1e-6, depth within 1e-5 of the same walk with alphas kept as floats; every
    test of a fragment is taken on the float).  ``FrameBuffers(..., long_list_threshold=8193).run()`` is that other
    walk: any threshold above 8192 selects it, a tenth slower in the blend stage."""
    with torch.no_grad():
        pool = ScratchPool.current(positions.device) if isinstance(positions, torch.Tensor) and positions.is_cuda else None
        image, depth = FrameBuffers(positions, scales, rotations, opacities, sh_0, sh_rest, settings,
                                    to_chw, use_median_depth, pool=pool).run()
    depth = depth.unsqueeze(0) if to_chw else depth.unsqueeze(-1)
    return image, depth


def fast_rasterize(
    positions: torch.Tensor,
    scales: torch.Tensor,
    rotations: torch.Tensor,
    opacities: torch.Tensor,
    sh_0: torch.Tensor,
    sh_rest: torch.Tensor,
    settings: RasterizerSettings,
    to_chw: bool,
) -> torch.Tensor:
    """The reference's benchmark entry (rasterization.py:166-186): image only, reduced accuracy.  There it is a
    fast-math build of the inference kernels with a half-precision core; here the same pipeline runs blend kernels that
    take the hardware's reciprocal and 2^x (one ulp each) instead of the exactly reproducible routines and skip the
    depth map.  The image agrees with ``rasterize`` to rounding, except at the few pixels where a fragment sits
    within an ulp of an alpha threshold."""
    with torch.no_grad():
        pool = ScratchPool.current(positions.device) if isinstance(positions, torch.Tensor) and positions.is_cuda else None
        image, _ = FrameBuffers(positions, scales, rotations, opacities, sh_0, sh_rest, settings, to_chw, False, pool=pool, fast=True).run()
    return image
