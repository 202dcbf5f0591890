"""TEST INFRASTRUCTURE -- not part of the product.

Independent float64 evaluator of what the rasterizer is *supposed* to compute, used to pin the C oracle
(``htgs_oracle.c``).  It shares no formula with the oracle's per-pixel code: instead of intersecting two planes
in the Gaussian's local frame (R/include/hybrid_blend/kernels/inference.cuh:137-155) it uses the textbook
closed form for the maximum of a 3-D Gaussian along a ray,

    t* = r^T S^-1 (mu - o) / (r^T S^-1 r),   G = exp(-1/2 min_t (o + t r - mu)^T S^-1 (o + t r - mu)),

with S = R diag(s^2) R^T, evaluates every Gaussian at every pixel (no tiles, no bounding boxes, no sorting of
instances) and composites with the *definition* of each blend mode (reference README.md:17-20 and the
constants of R/include/<mode>/config.h).  Written in torch so that autograd provides reference gradients.

Everything is dense [pixels, Gaussians]; meant for a few hundred Gaussians and a few thousand pixels (or, with an
explicit pixel list and a pre-selected subset of the Gaussians, for patches of a large frame).
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch

F64 = torch.float64

MIN_ALPHA = {0: 1.0 / 255.0, 1: 1.0 / 20.0, 2: 1.0 / 255.0, 3: 1.0 / 255.0}
MIN_ALPHA_CORE = 1.0 / 20.0
T_THRESHOLD = 1e-4


def quat_to_rot(q: torch.Tensor) -> torch.Tensor:
    """Rotation matrix of the quaternion (w, x, y, z) -- textbook formula, not normalised."""
    w, x, y, z = q.unbind(-1)
    return torch.stack([
        1 - 2 * (y * y + z * z), 2 * (x * y - w * z), 2 * (x * z + w * y),
        2 * (x * y + w * z), 1 - 2 * (x * x + z * z), 2 * (y * z - w * x),
        2 * (x * z - w * y), 2 * (y * z + w * x), 1 - 2 * (x * x + y * y)], dim=-1).reshape(*q.shape[:-1], 3, 3)


def sh_basis(dirs: torch.Tensor) -> torch.Tensor:
    """Real spherical harmonics Y_l^m(dirs), l <= 3, as [..., 16] in the order l=0; l=1: m=-1,0,1; l=2: m=-2..2;
    l=3: m=-3..3, with the Condon-Shortley phase folded into the sign convention used by 3-D Gaussian splatting
    (Y_1^{-1} = -c y, Y_1^0 = c z, Y_1^1 = -c x, ...).  Cartesian closed forms."""
    x, y, z = dirs.unbind(-1)
    s = math.sqrt
    pi = math.pi
    return torch.stack([
        torch.full_like(x, 0.5 * s(1 / pi)),
        -s(3 / (4 * pi)) * y, s(3 / (4 * pi)) * z, -s(3 / (4 * pi)) * x,
        0.5 * s(15 / pi) * x * y, -0.5 * s(15 / pi) * y * z, 0.25 * s(5 / pi) * (3 * z * z - 1),
        -0.5 * s(15 / pi) * x * z, 0.25 * s(15 / pi) * (x * x - y * y),
        -0.25 * s(35 / (2 * pi)) * y * (3 * x * x - y * y), 0.5 * s(105 / pi) * x * y * z,
        -0.25 * s(21 / (2 * pi)) * y * (5 * z * z - 1), 0.25 * s(7 / pi) * z * (5 * z * z - 3),
        -0.25 * s(21 / (2 * pi)) * x * (5 * z * z - 1), 0.25 * s(105 / pi) * z * (x * x - y * y),
        -0.25 * s(35 / (2 * pi)) * x * (x * x - 3 * y * y)], dim=-1)


def sh_colour(positions, sh_0, sh_rest, cam_position, active_sh_bases: int) -> torch.Tensor:
    """max(0, 0.5 + sum_k Y_k(dir) c_k) with dir = normalised(position - camera)."""
    d = positions - cam_position
    d = d / d.norm(dim=-1, keepdim=True)
    Y = sh_basis(d)
    rgb = 0.5 + Y[:, 0:1] * sh_0.reshape(-1, 3)
    n_rest = {1: 0, 4: 3, 9: 8, 16: 15}[int(active_sh_bases)]
    if n_rest:
        rgb = rgb + (Y[:, 1:1 + n_rest, None] * sh_rest[:, :n_rest, :]).sum(dim=1)
    return rgb.clamp_min(0.0)


@dataclass
class Fragments:
    alpha: torch.Tensor      # [P, G]  min(opacity * G, 1), 0 for culled Gaussians
    depth: torch.Tensor      # [P, G]  camera-space z of the point of maximum contribution on the ray
    z_centre: torch.Tensor   # [G]
    rgb: torch.Tensor        # [G, 3]
    visible: torch.Tensor    # [G] bool
    height: int
    width: int
    maha2: torch.Tensor = None   # [P, G] squared Mahalanobis distance of the ray from the centre


def evaluate(positions, scales, rotations, opacities, sh_0, sh_rest, M, VPM, cam_position, mode: int, active_sh_bases: int,
             width: int, height: int, near_plane: float, far_plane: float, scale_modifier: float = 1.0,
             pixels: torch.Tensor = None) -> Fragments:
    """Every Gaussian at every pixel of the width x height image, or, with ``pixels`` ([P,2] integer (x, y)), at those
    pixels only (the result then describes a 1 x P image)."""
    positions, scales, rotations = positions.to(F64), scales.to(F64), rotations.to(F64)
    opacities = opacities.to(F64).reshape(-1)
    sh_0, sh_rest = sh_0.to(F64), sh_rest.to(F64)
    M, VPM, cam_position = M.to(F64).reshape(4, 4), VPM.to(F64).reshape(4, 4), cam_position.to(F64).reshape(3)
    VP = VPM @ torch.linalg.inv(M)                       # intrinsics with the half-pixel shift (Renderer.py:38-44)
    fx, fy, cxs, cys = VP[0, 0], VP[1, 1], VP[0, 2], VP[1, 2]
    Rc, tc = M[:3, :3], M[:3, 3]
    if pixels is None:
        ys, xs = torch.meshgrid(torch.arange(height, dtype=F64), torch.arange(width, dtype=F64), indexing="ij")
    else:
        xs, ys = pixels[:, 0].to(F64).reshape(1, -1), pixels[:, 1].to(F64).reshape(1, -1)
        height, width = 1, xs.shape[1]
    dir_c = torch.stack([(xs - cxs) / fx, (ys - cys) / fy, torch.ones_like(xs)], dim=-1).reshape(-1, 3)   # [P,3]
    origin = -Rc.T @ tc
    dir_w = dir_c @ Rc                                    # rows: Rc^T dir_c

    R = quat_to_rot(rotations)
    s = scales * scale_modifier
    # S = (R diag(s)) (R diag(s))^T.  Inverted numerically rather than as R diag(1/s^2) R^T so that derivatives
    # with respect to the quaternion are those of the matrix formula even off the unit sphere.
    Sigma = R @ torch.diag_embed(s * s) @ R.transpose(-1, -2)                 # [G,3,3]
    Sinv = torch.linalg.inv(Sigma)
    delta = positions - origin                                                # [G,3]
    Sd = torch.einsum("gij,gj->gi", Sinv, delta)                              # S^-1 (mu - o)
    rSr = torch.einsum("pi,gij,pj->pg", dir_w, Sinv, dir_w)
    rSd = dir_w @ Sd.T                                                        # [P,G]
    dSd = (delta * Sd).sum(-1)                                                # [G]
    t_star = rSd / rSr
    maha2 = (dSd[None, :] - rSd * rSd / rSr).clamp_min(0.0)
    G = torch.exp(-0.5 * maha2)
    alpha = (opacities[None, :] * G).clamp_max(1.0)
    # camera z of o + t* r: the ray direction has camera z = 1 and the origin has camera z = 0
    depth = t_star

    # culling (R/include/kernel_utils.cuh:89-90 and :104-116): centre outside [near, far], or the level set
    # alpha = min_alpha of the Gaussian (an ellipsoid of "radius" rho) reaching outside [near, far]
    z_centre = positions @ Rc[2] + tc[2]
    rho = 2.0 * torch.log(opacities / MIN_ALPHA[mode])
    sigma_z2 = torch.einsum("i,gij,j->g", Rc[2], Sigma, Rc[2])
    r_z = torch.sqrt((rho * sigma_z2).clamp_min(0.0))
    visible = (z_centre >= near_plane) & (z_centre <= far_plane) & (z_centre - r_z >= near_plane) & (z_centre + r_z <= far_plane)
    alpha = alpha * visible[None, :].to(F64)
    rgb = sh_colour(positions, sh_0, sh_rest, cam_position, active_sh_bases)
    return Fragments(alpha, depth, z_centre, rgb, visible, height, width, maha2)


def _composite_sorted(alpha_s, rgb_s, depth_s, valid_s):
    """Front-to-back alpha blending of fragments already in order along dim 1, stopping (per pixel) before the
    first fragment whose incoming transmittance is below 1e-4.  Returns rgb, sum w*depth, final T and the
    per-fragment incoming transmittance."""
    a = alpha_s * valid_s
    T_in = torch.cumprod(torch.cat([torch.ones_like(a[:, :1]), 1.0 - a[:, :-1]], dim=1), dim=1)
    # a dead fragment kills everything behind it
    live = torch.cumprod(((T_in >= T_THRESHOLD)).to(F64), dim=1) * valid_s
    w = T_in * a * live
    rgb = (w[..., None] * rgb_s).sum(1)
    dsum = (w * depth_s).sum(1)
    T_final = torch.prod(1.0 - a * live, dim=1)
    return rgb, dsum, T_final, T_in, live


def render(fr: Fragments, mode: int, K: int, use_median_depth: bool = False, clamp: bool = True):
    """Image [3,H,W], depth [H,W], alpha [H,W] and a per-pixel ``margin`` [H,W]: the smallest relative distance
    of any quantity from a threshold that decides its fate (pixels with a tiny margin may legitimately differ
    between float32 and float64 and are excluded by the tests)."""
    alpha, depth, rgb = fr.alpha, fr.depth, fr.rgb
    P, Gn = alpha.shape
    min_alpha = MIN_ALPHA[mode]
    accepted = alpha >= min_alpha
    margin = ((alpha / min_alpha - 1.0).abs() + (~fr.visible)[None, :].to(F64) * 1e9).min(dim=1).values
    big = torch.finfo(F64).max

    if mode in (0, 1):
        eligible = accepted & (alpha >= MIN_ALPHA_CORE) if mode == 0 else accepted
        if mode == 0:
            margin = torch.minimum(margin, ((alpha / MIN_ALPHA_CORE - 1.0).abs() + (~fr.visible)[None, :].to(F64) * 1e9).min(dim=1).values)
        key = torch.where(eligible, depth, torch.full_like(depth, big))
        k_eff = min(K, Gn)
        vals, idx = torch.topk(key, k_eff + 1 if Gn > k_eff else k_eff, dim=1, largest=False)
        if Gn > k_eff:   # gap between the last core fragment and the first one left out
            gap = ((vals[:, k_eff] - vals[:, k_eff - 1]).abs() / vals[:, k_eff - 1].abs().clamp_min(1e-30))
            both = vals[:, k_eff] < big
            margin = torch.minimum(margin, torch.where(both, gap, torch.full_like(gap, 1e9)))
            vals, idx = vals[:, :k_eff], idx[:, :k_eff]
        valid = (vals < big).to(F64)
        a_s = torch.gather(alpha, 1, idx)
        d_s = torch.gather(depth, 1, idx)
        c_s = rgb[idx]
        col, dsum, T, T_in, live = _composite_sorted(a_s, c_s, d_s, valid)
        margin = torch.minimum(margin, ((T_in / T_THRESHOLD - 1.0).abs() + (1 - valid) * 1e9).min(dim=1).values)
        in_core = torch.zeros_like(alpha, dtype=torch.bool)
        in_core.scatter_(1, idx, valid > 0)
        if use_median_depth:
            before_half = (T_in > 0.5) & (live > 0)
            margin = torch.minimum(margin, ((T_in - 0.5).abs() + (1 - valid) * 1e9).min(dim=1).values)
            last = before_half.to(F64).cumsum(1).argmax(1, keepdim=True)
            med = torch.where(before_half.any(1), torch.gather(d_s, 1, last).squeeze(1), torch.zeros(P, dtype=F64))
        if mode == 0:
            tail = accepted & ~in_core
            ta = alpha * tail
            sum_a = ta.sum(1)
            sum_ac = ta @ rgb
            sum_ad = (ta * depth).sum(1)
            T_tail = torch.prod(1.0 - ta, dim=1)
            use_tail = (T >= T_THRESHOLD) & (sum_a >= MIN_ALPHA[0])
            margin = torch.minimum(margin, (T / T_THRESHOLD - 1.0).abs())
            margin = torch.minimum(margin, torch.where(sum_a > 0, (sum_a / MIN_ALPHA[0] - 1.0).abs(), torch.full_like(sum_a, 1e9)))
            w_tail = torch.where(use_tail, T * (1.0 - T_tail), torch.zeros_like(T))
            inv = torch.where(use_tail, 1.0 / sum_a.clamp_min(1e-300), torch.zeros_like(T))
            col = col + (w_tail * inv)[:, None] * sum_ac
            dsum = dsum + w_tail * inv * sum_ad
            total_alpha = (1.0 - T) + w_tail
        else:
            total_alpha = 1.0 - T
        dep = torch.where(total_alpha > 0, dsum / total_alpha.clamp_min(1e-300), torch.zeros_like(dsum))
        if use_median_depth:
            dep = med
    elif mode == 2:
        order = torch.argsort(fr.z_centre, stable=True)
        a_s = alpha[:, order]
        valid = accepted[:, order].to(F64)
        # fragments that are not accepted are simply absent: compact them to the back per pixel
        rank = torch.argsort((1 - valid), dim=1, stable=True)
        a_s = torch.gather(a_s, 1, rank)
        valid = torch.gather(valid, 1, rank)
        g_s = order[rank]
        c_s = rgb[g_s]
        z_s = fr.z_centre[g_s]
        a = a_s * valid
        T_in = torch.cumprod(torch.cat([torch.ones_like(a[:, :1]), 1.0 - a[:, :-1]], dim=1), dim=1)
        live = torch.cumprod((T_in >= T_THRESHOLD).to(F64), dim=1) * valid
        margin = torch.minimum(margin, ((T_in / T_THRESHOLD - 1.0).abs() + (1 - valid) * 1e9).min(dim=1).values)
        w = T_in * a * live
        col = (w[..., None] * c_s).sum(1)
        T = torch.prod(1.0 - a * live, dim=1)
        total_alpha = 1.0 - T
        if use_median_depth:
            before_half = (T_in > 0.5) & (live > 0)
            margin = torch.minimum(margin, ((T_in - 0.5).abs() + (1 - valid) * 1e9).min(dim=1).values)
            last = before_half.to(F64).cumsum(1).argmax(1, keepdim=True)
            dep = torch.where(before_half.any(1), torch.gather(z_s, 1, last).squeeze(1), torch.zeros(P, dtype=F64))
        else:
            dep = torch.where(T < 1.0, (w * z_s).sum(1) / total_alpha.clamp_min(1e-300), torch.zeros_like(T))
    else:
        a = alpha * accepted
        sum_a = a.sum(1)
        T = torch.prod(1.0 - a, dim=1)
        ok = sum_a >= MIN_ALPHA[3]
        margin = torch.minimum(margin, torch.where(sum_a > 0, (sum_a / MIN_ALPHA[3] - 1.0).abs(), torch.full_like(sum_a, 1e9)))
        scale = torch.where(ok, (1.0 - T) / sum_a.clamp_min(1e-300), torch.zeros_like(T))
        col = scale[:, None] * (a @ rgb)
        dep = torch.where(ok, (a * depth).sum(1) / sum_a.clamp_min(1e-300), torch.zeros_like(T))
        total_alpha = torch.where(ok, 1.0 - T, torch.zeros_like(T))

    if clamp:
        col = col.clamp(0.0, 1.0)
    H, W = fr.height, fr.width
    return col.T.reshape(3, H, W), dep.reshape(H, W), total_alpha.reshape(H, W), margin.reshape(H, W)


CUTOFF_SQ = {0: 11.0825270903, 1: 5.99146454711, 2: 11.0825270903, 3: 11.0825270903}


def max_weights(fr: Fragments, mode: int, K: int, weight_threshold: float):
    """Largest blending weight of every Gaussian over all pixels, by the definition of each mode (the quantity the
    reference's update_max_weights accumulates).  Returns the maxima [G] and, per Gaussian, the largest weight it
    would have had without the threshold (to let callers skip Gaussians that sit on the threshold)."""
    alpha, depth = fr.alpha, fr.depth
    P, Gn = alpha.shape
    accepted = alpha >= MIN_ALPHA[mode]
    big = torch.finfo(F64).max
    W = torch.zeros_like(alpha)
    if mode == 2:
        order = torch.argsort(fr.z_centre, stable=True)
        a = (alpha * accepted)[:, order]
        T_in = torch.cumprod(torch.cat([torch.ones_like(a[:, :1]), 1.0 - a[:, :-1]], dim=1), dim=1)
        live = torch.cumprod((T_in >= T_THRESHOLD).to(F64), dim=1)
        W[:, order] = T_in * a * live
    else:
        T_core = torch.ones(P, dtype=F64)
        in_core = torch.zeros_like(alpha, dtype=torch.bool)
        if mode in (0, 1):
            eligible = accepted & (alpha >= MIN_ALPHA_CORE) if mode == 0 else accepted
            key = torch.where(eligible, depth, torch.full_like(depth, big))
            k_eff = min(K, Gn)
            vals, idx = torch.topk(key, k_eff, dim=1, largest=False)
            valid = (vals < big).to(F64)
            a_s = torch.gather(alpha, 1, idx) * valid
            T_in = torch.cumprod(torch.cat([torch.ones_like(a_s[:, :1]), 1.0 - a_s[:, :-1]], dim=1), dim=1)
            T_in = torch.where(T_in >= T_THRESHOLD, T_in, torch.zeros_like(T_in))     # transmittance is zeroed below 1e-4
            w_core = T_in * a_s
            W.scatter_(1, idx, w_core)
            T_after = T_in[:, -1] * (1.0 - a_s[:, -1])
            T_core = torch.where(T_after >= T_THRESHOLD, T_after, torch.zeros_like(T_after))
            in_core.scatter_(1, idx, valid > 0)
        if mode in (0, 3):
            tail = accepted & ~in_core
            ta = alpha * tail
            sum_a = ta.sum(1)
            T_tail = torch.prod(1.0 - ta, dim=1)
            tail_weight = torch.where(sum_a >= weight_threshold, T_core * (1.0 - T_tail) / sum_a.clamp_min(1e-300), torch.zeros_like(sum_a))
            tail_weight = torch.where(tail_weight >= weight_threshold, tail_weight, torch.zeros_like(tail_weight))
            inside_cutoff = (fr.maha2 <= CUTOFF_SQ[mode]) & fr.visible[None, :]
            W = torch.maximum(W, alpha * tail_weight[:, None] * inside_cutoff)
    raw = W.max(dim=0).values
    return torch.where(raw >= weight_threshold, raw, torch.zeros_like(raw)), raw


def per_fragment_position_gradient_l1(positions, scales, rotations, opacities, sh_0, sh_rest, M, VPM, cam_position, mode: int,
                                      active_sh_bases: int, width: int, height: int, near_plane: float, far_plane: float,
                                      K: int, grad_image: torch.Tensor) -> torch.Tensor:
    """Third densification statistic by its definition (R/include/hybrid_blend/kernels/backward.cuh:292-306): for every
    Gaussian g the sum over pixels p of  | d L_p / d position_g |_1 , where L_p = sum_c grad_image[c,p] image[c,p] is the
    loss carried by pixel p alone and the derivative is the geometric one (through the fragment's alpha; the colour's
    view dependence is added elsewhere and is not part of it).  One autograd pass per pixel through the float64
    evaluator; nothing of the reference's hand-derived chain is used.  Returns [G] (no distance scaling)."""
    pos = positions.to(F64).clone().requires_grad_(True)
    fr = evaluate(pos, scales, rotations, opacities, sh_0, sh_rest, M, VPM, cam_position, mode, active_sh_bases, width, height,
                  near_plane, far_plane)
    fr.rgb = fr.rgb.detach()
    image, _, _, _ = render(fr, mode, K, False, clamp=False)
    per_pixel = (image * grad_image.to(F64)).sum(0).reshape(-1)            # L_p, [P]
    out = torch.zeros(pos.shape[0], dtype=F64)
    for p in torch.nonzero(per_pixel.detach() != 0).reshape(-1).tolist():
        (g,) = torch.autograd.grad(per_pixel[p], pos, retain_graph=True)
        out += g.abs().sum(1)
    return out


def near_ray(positions, scales, M, VPM, centre_xy, radius_px: float, cutoff: float = 3.4, slack: float = 1.5) -> torch.Tensor:
    """Indices of the Gaussians that can reach a pixel within ``radius_px`` of the pixel ``centre_xy``: those whose centre
    lies within  cutoff * largest scale + slack * (distance along the ray) * radius_px / focal  of the ray through
    ``centre_xy`` (Euclidean distance in float64; sqrt(2 ln 255) = 3.33 standard deviations is the farthest a fragment is
    accepted).  A generous, formula-free pre-selection so that the dense evaluator can be run on patches of frames with
    millions of Gaussians; leaving out a Gaussian that contributes shows up as a mismatch, not as a silent pass."""
    positions, scales = positions.to(F64), scales.to(F64)
    M, VPM = M.to(F64).reshape(4, 4), VPM.to(F64).reshape(4, 4)
    VP = VPM @ torch.linalg.inv(M)
    fx, fy, cxs, cys = VP[0, 0], VP[1, 1], VP[0, 2], VP[1, 2]
    Rc, tc = M[:3, :3], M[:3, 3]
    d = torch.stack([(centre_xy[0] - cxs) / fx, (centre_xy[1] - cys) / fy, torch.ones((), dtype=F64)])
    norm = d.norm()
    d = (Rc.T @ d) / norm
    delta = positions - (-Rc.T @ tc)
    t = delta @ d
    dist = (delta - t[:, None] * d[None, :]).norm(dim=1)
    # a pixel radius_px away sees the ray tilted by at most radius_px / (focal * |d|) ... times |d|^2 off axis: use the
    # looser radius_px * |d| / focal
    reach = cutoff * scales.max(dim=1).values + slack * t.abs() * radius_px * norm / torch.minimum(fx, fy)
    return torch.nonzero(dist <= reach).reshape(-1)
