"""Helpers shared by the tests: oracle frames from synthetic scenes, GPU stage runner."""
import numpy as np
import torch

import oracle
from htgs_amd.synthetic import Scene
from htgs_amd.torch_bindings import FrameBuffers, RasterizerMode


def oracle_frame(scene: Scene, mode: int, K=None, scale_modifier: float = 1.0, tile=None) -> oracle.Frame:
    return oracle.Frame(scene.M.cpu().numpy(), scene.VPM.cpu().numpy(), scene.cam_position.cpu().numpy(), int(mode),
                        scene.K if K is None else K, scene.active_sh_bases, scene.width, scene.height,
                        scene.near_plane, scene.far_plane, scale_modifier, tile)


def oracle_render(scene: Scene, mode: int, K=None, to_chw=True, median=False, scale_modifier=1.0) -> dict:
    fr = oracle_frame(scene, mode, K, scale_modifier)
    return oracle.render(fr, *[t.cpu().numpy() for t in scene.gaussians()], to_chw=to_chw, use_median_depth=median)


def u32(t: torch.Tensor) -> np.ndarray:
    """int32 / int16 / int64 tensor holding unsigned data -> unsigned numpy array"""
    a = t.detach().cpu().numpy()
    return a.view({2: np.uint16, 4: np.uint32, 8: np.uint64}[a.dtype.itemsize])


def gpu_stages(scene_gpu: Scene, mode: int, K=None, to_chw=True, median=False, scale_modifier=1.0, order_gaussians=False) -> dict:
    """Runs the frame stage by stage through the C ABI and returns every intermediate as numpy.  (GLOBAL_ORDERING with the
    reference's tile | depth keys unless ``order_gaussians``, so that offsets and keys compare with the oracle's.)"""
    settings = scene_gpu.settings(RasterizerMode(int(mode)), K, scale_modifier)
    fb = FrameBuffers(*scene_gpu.gaussians(), settings, to_chw, median, order_gaussians=order_gaussians)
    fb.n_touched.fill_(-1)
    fb.bounds.zero_()
    fb.prim.zero_()
    fb.preprocess()
    fb.scan()
    n_inst = fb.read_instance_count()
    fb.alloc_instances(n_inst)
    fb.create_instances()
    keys0 = u32(fb.keys[0])[:n_inst].astype(np.uint64)
    vals0 = u32(fb.vals[0])[:n_inst].copy()
    sel = fb.sort()
    fb.extract_ranges()
    fb.blend()
    torch.cuda.synchronize()
    prim = fb.prim.cpu().numpy()
    return {
        "fb": fb, "n_instances": n_inst,
        "n_touched": u32(fb.n_touched), "offsets": u32(fb.offsets), "bounds": u32(fb.bounds).astype(np.uint32),
        "VPMT1": prim[:, 0:4], "VPMT2": prim[:, 4:8], "VPMT4": prim[:, 8:12], "MT3": prim[:, 12:16], "rgba": prim[:, 16:20],
        "keys": keys0, "vals": vals0,
        "sorted_keys": u32(fb.keys[sel])[:n_inst].astype(np.uint64), "sorted_vals": u32(fb.vals[sel])[:n_inst].copy(),
        "ranges": u32(fb.ranges), "image": fb.image.cpu().numpy(), "depth": fb.depth.cpu().numpy(),
    }


def load_golden(name: str = "small_scene"):
    """The frozen known-answer fixture tests/golden/<name>.npz (written by tests/golden/make_fixtures.py from the
    float64 evaluator): the scene and the arrays of expected outputs."""
    import os
    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", name + ".npz"))
    t = lambda k: torch.from_numpy(z[k].copy())
    width, height = (int(v) for v in z["size"])
    scene = Scene(name, t("positions"), t("scales"), t("rotations"), t("opacities"), t("sh_0"), t("sh_rest"), t("M"), t("VPM"),
                  t("cam_position"), width, height, float(z["planes"][0]), float(z["planes"][1]), int(z["active_sh_bases"]), int(z["K"]))
    return scene, z


def tie_scene(depths, opacities, colours):
    """Isotropic Gaussians on the optical axis of a 64x64 pinhole camera whose principal point maps to pixel (32, 32):
    at that pixel the ray passes through every centre, so fragment k has alpha = opacities[k] and depth = depths[k]
    exactly (|m|^2 = 0, exp(0) = 1, the point of maximum contribution is the centre), in list order = index order.
    Gaussians given the same depth are coincident (same shape): their fragments have bit-identical depths at every
    pixel.  SH degree 0 with the given colours."""
    from htgs_amd.synthetic import SH_C0, pinhole
    n = len(depths)
    pos = torch.zeros(n, 3)
    pos[:, 2] = torch.tensor(depths, dtype=torch.float32)
    scales = torch.full((n, 3), 0.05) * pos[:, 2:3]              # the same angular size
    rot = torch.zeros(n, 4)
    rot[:, 0] = 1.0
    opac = torch.tensor(opacities, dtype=torch.float32).reshape(n, 1)
    sh_0 = ((torch.tensor(colours, dtype=torch.float32) - 0.5) / SH_C0).reshape(n, 1, 3)
    M, VPM, cam = pinhole(64, 64, 100.0, 100.0, 32.5, 32.5, 0.1, 100.0)
    return Scene("ties", pos, scales.contiguous(), rot, opac, sh_0.contiguous(), torch.zeros(n, 0, 3), M, VPM, cam, 64, 64, 0.1, 100.0, 1, 4)


def hybrid_pixel_by_hand(order, tail, depths, opacities, colours):
    """HYBRID_BLEND's pixel in float64 from its definition, for a core given as a list of fragment numbers in the order
    they are blended and the fragments in the tail: (rgb, depth) (R/include/hybrid_blend/kernels/inference.cuh:172-200)."""
    a, c, d = np.asarray(opacities, np.float64), np.asarray(colours, np.float64), np.asarray(depths, np.float64)
    rgb, depth, T = np.zeros(3), 0.0, 1.0
    for k in order:
        rgb += T * a[k] * c[k]
        depth += T * a[k] * d[k]
        T *= 1.0 - a[k]
    total_alpha = 1.0 - T
    if tail:
        alpha_sum = sum(a[k] for k in tail)
        T_tail = np.prod([1.0 - a[k] for k in tail])
        w = T * (1.0 - T_tail) / alpha_sum
        rgb += w * sum(a[k] * c[k] for k in tail)
        depth += w * sum(a[k] * d[k] for k in tail)
        total_alpha += T * (1.0 - T_tail)
    return np.clip(rgb, 0.0, 1.0), depth / total_alpha
