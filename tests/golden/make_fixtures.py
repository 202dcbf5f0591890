"""Writes tests/golden/small_scene.npz: known answers for a 140-Gaussian scene, from the independent float64
evaluator (oracle/bruteforce.py: textbook ray / Gaussian maximum, dense compositing by the definition of each blend
mode, gradients by torch.autograd).  The fixture holds the inputs, and per blend mode the image, the depth, the
pixels whose accept / reject decisions are not within 1e-4 of a threshold (only those are compared), the six
gradients of sum(image * grad_image) over those pixels, and the third densification statistic (per Gaussian, the sum
over those pixels of the 1-norm of the pixel's own position gradient).

The reference ships no test vectors; these are this repository's own, frozen so that a change of the CPU checker and
of the kernels in the same direction still has something to answer to.  Run from the repository root:

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))                       # tests/
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))      # repository root

from oracle import bruteforce as bf                            # noqa: E402
from test_oracle_pinning import small_scene                    # noqa: E402

K = 8
NAMES = ["positions", "scales", "rotations", "opacities", "sh_0", "sh_rest"]


def main():
    sc = small_scene(n=140, seed=2024, sh_degree=3)
    grad_image = torch.randn(3, sc.height, sc.width, generator=torch.Generator().manual_seed(7))
    out = {name: t.numpy() for name, t in zip(NAMES, sc.gaussians())}
    out.update(M=sc.M.numpy(), VPM=sc.VPM.numpy(), cam_position=sc.cam_position.numpy(),
               size=np.array([sc.width, sc.height]), planes=np.array([sc.near_plane, sc.far_plane], np.float32),
               active_sh_bases=np.array(sc.active_sh_bases), K=np.array(K), grad_image=grad_image.numpy())
    for mode in range(4):
        leaves = [t.double().clone().requires_grad_(True) for t in sc.gaussians()]
        frags = bf.evaluate(*leaves, sc.M, sc.VPM, sc.cam_position, mode, sc.active_sh_bases, sc.width, sc.height,
                            sc.near_plane, sc.far_plane)
        image, depth, _, margin = bf.render(frags, mode, K, False, clamp=False)
        mask = margin > 1e-4
        (image * grad_image.double() * mask.double()).sum().backward()
        out[f"image_{mode}"] = image.detach().numpy().astype(np.float32)
        out[f"depth_{mode}"] = depth.detach().numpy().astype(np.float32)
        out[f"mask_{mode}"] = mask.numpy()
        for name, leaf in zip(NAMES, leaves):
            out[f"grad_{name}_{mode}"] = leaf.grad.numpy().astype(np.float32)
        # third densification statistic (sum over pixels of |dL_p / dposition|_1), same upstream gradient and mask
        out[f"dens_l1_{mode}"] = bf.per_fragment_position_gradient_l1(
            *sc.gaussians(), sc.M, sc.VPM, sc.cam_position, mode, sc.active_sh_bases, sc.width, sc.height, sc.near_plane,
            sc.far_plane, K, grad_image.double() * mask.double()).numpy().astype(np.float32)
        print(f"mode {mode}: {float(mask.double().mean()):.3f} of the pixels compared, image max {float(image.detach().max()):.3f}")
    np.savez_compressed(os.path.join(HERE, "small_scene.npz"), **out)


if __name__ == "__main__":
    main()
