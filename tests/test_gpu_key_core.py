"""The kernels of HYBRID_BLEND and ALPHA_BLEND_FIRST_K with one wave per tile keep the K nearest fragments as sorted 64-bit keys (depth above alpha as a
fraction of 19 to 23 bits above the place in the list) when the frame has the list for long tiles and no list of the launch
is longer than 8192; pixels at which fragments of exactly equal depth met where they decide the core are walked again with the
reference's exchange insertion (R/include/hybrid_blend/kernels/inference.cuh:159-167,
R/include/alpha_blend_first_k/kernels/inference.cuh:155-163).  Without that list -- or with a
threshold above 8192 -- the same kernel keeps (depth, alpha, index) triples and inserts by exchange throughout.  The two
must agree to the rounding of the alphas (2^-20 each), and both with the CPU oracle to the rasterizer's 1e-4."""
import numpy as np
import pytest

from htgs_amd.synthetic import make_scene
from htgs_amd.torch_bindings import RasterizerMode
from test_gpu_long_tiles import NEVER, render, with_coincident_copies
from util import oracle_render

pytestmark = pytest.mark.gpu

TOL = 1e-4
BETWEEN = 1e-5          # image: sixteen alphas off by 2^-20 at worst, far less on average


@pytest.mark.parametrize("config,n,K", [(0, 3000, 4), (0, 3000, 1), (0, 3000, 2), (1, 60_000, 16), (2, 100_000, 32), (2, 100_000, 8), (3, 8_000, 16)])
def test_keys_against_the_exchange_walk_and_the_oracle(cuda, config, n, K):
    print(f"case config={config} n={n} K={K}", flush=True)
    scene = make_scene(config, n)
    ref = oracle_render(scene, 0, K)
    keyed, keyed_depth, long_tiles = render(scene.to(cuda), K, 0)
    assert long_tiles == 0                                     # every tile is the keyed kernel's
    exchanged, exchanged_depth, _ = render(scene.to(cuda), K, NEVER)
    between = float(np.abs(keyed - exchanged).max())
    scale = max(1.0, float(np.abs(ref["depth"]).max()))
    print(f"  keys against exchange: image {between:.3g}, depth {float(np.abs(keyed_depth - exchanged_depth).max()):.3g} (depths up to {scale:.3g})", flush=True)
    assert between <= BETWEEN
    assert float(np.abs(keyed_depth - exchanged_depth).max()) <= BETWEEN * scale
    assert float(np.abs(keyed - ref["image"]).max()) <= TOL and float(np.abs(keyed_depth - ref["depth"]).max()) <= TOL
    assert float(np.abs(exchanged - ref["image"]).max()) <= TOL and float(np.abs(exchanged_depth - ref["depth"]).max()) <= TOL


@pytest.mark.parametrize("config,n,K,copies", [(0, 1500, 4, 3), (1, 20_000, 16, 2), (0, 1500, 1, 2), (0, 1500, 32, 2), (1, 20_000, 8, 3), (0, 1500, 2, 3)])
def test_keys_where_every_fragment_meets_its_own_depth(cuda, config, n, K, copies):
    """Coincident copies of every Gaussian: every pixel with two fragments in its core is walked a second time."""
    print(f"case config={config} n={n} K={K} copies={copies}", flush=True)
    scene = with_coincident_copies(make_scene(config, n), copies)
    ref = oracle_render(scene, 0, K)
    keyed, keyed_depth, long_tiles = render(scene.to(cuda), K, 0)
    assert long_tiles == 0
    exchanged, exchanged_depth, _ = render(scene.to(cuda), K, NEVER)
    scale = max(1.0, float(np.abs(ref["depth"]).max()))
    assert float(np.abs(keyed - exchanged).max()) <= BETWEEN and float(np.abs(keyed_depth - exchanged_depth).max()) <= BETWEEN * scale
    # (the second walk is the exchange walk over the instances that reach the pixel: most pixels come out bit for bit)
    same = float((keyed == exchanged).all(axis=0).mean())
    print(f"  pixels equal bit for bit: {same:.3f}", flush=True)
    assert same >= 0.5
    assert float(np.abs(keyed - ref["image"]).max()) <= TOL and float(np.abs(keyed_depth - ref["depth"]).max()) <= TOL


@pytest.mark.parametrize("to_chw,median", [(False, False), (True, True)])
def test_keys_with_the_other_output_layouts(cuda, to_chw, median):
    scene = make_scene(0, 3000)
    keyed, keyed_depth, _ = render(scene.to(cuda), 4, 0, to_chw=to_chw, median=median)
    exchanged, exchanged_depth, _ = render(scene.to(cuda), 4, NEVER, to_chw=to_chw, median=median)
    assert float(np.abs(keyed - exchanged).max()) <= BETWEEN
    # (the median depth is one fragment's depth: the same fragment unless two transmittances straddle 1/2 within the alphas' rounding)
    assert float((np.abs(keyed_depth - exchanged_depth) > 1e-5 * max(1.0, float(np.abs(exchanged_depth).max()))).mean()) <= (1e-3 if median else 0.0)


FIRST_K = RasterizerMode.ALPHA_BLEND_FIRST_K


@pytest.mark.parametrize("config,n,K,copies", [(0, 3000, 4, 1), (0, 3000, 1, 1), (1, 60_000, 16, 1), (2, 100_000, 32, 1), (3, 8_000, 16, 1),
                                                 (0, 1500, 4, 3), (1, 20_000, 16, 2), (0, 1500, 32, 2), (1, 20_000, 8, 3)])
def test_first_k_keys_against_the_exchange_walk_and_the_oracle(cuda, config, n, K, copies):
    """ALPHA_BLEND_FIRST_K has no tail that takes what leaves the core: which of two fragments of equal depth holds the
    K-th place decides the pixel, so the second walk is what keeps the keyed kernel on the reference's result."""
    print(f"case config={config} n={n} K={K} copies={copies}", flush=True)
    scene = make_scene(config, n)
    if copies > 1: scene = with_coincident_copies(scene, copies)
    ref = oracle_render(scene, 1, K)
    keyed, keyed_depth, _ = render(scene.to(cuda), K, 0, mode=FIRST_K)
    exchanged, exchanged_depth, _ = render(scene.to(cuda), K, NEVER, mode=FIRST_K)
    scale = max(1.0, float(np.abs(ref["depth"]).max()))
    between = float(np.abs(keyed - exchanged).max())
    print(f"  keys against exchange: image {between:.3g}, depth {float(np.abs(keyed_depth - exchanged_depth).max()):.3g} (depths up to {scale:.3g})", flush=True)
    assert between <= BETWEEN and float(np.abs(keyed_depth - exchanged_depth).max()) <= BETWEEN * scale
    assert float(np.abs(keyed - ref["image"]).max()) <= TOL and float(np.abs(keyed_depth - ref["depth"]).max()) <= TOL


@pytest.mark.parametrize("config,n,K,mode", [(0, 3000, 4, 0), (1, 60_000, 16, 0), (1, 60_000, 16, 1)])
def test_a_threshold_above_8192_keeps_the_alphas_as_floats(cuda, config, n, K, mode):
    """``long_list_threshold = 8193`` selects the walk with (depth, alpha, index) triples, whose image and depth equal the
    CPU oracle's bit for bit (both implement one rounding convention)."""
    scene = make_scene(config, n)
    ref = oracle_render(scene, mode, K)
    image, depth, long_tiles = render(scene.to(cuda), K, 8193, mode=RasterizerMode(mode))
    assert long_tiles == 0
    assert np.array_equal(image, ref["image"]) and np.array_equal(depth, ref["depth"])


def test_fast_path_holds_a_fully_opaque_fragment(cuda):
    """alpha = 1 is the largest fraction a key can hold (fragments are held to it): an opaque Gaussian in front of another
    hides it at the pixel through both centres, on both paths."""
    from htgs_amd.torch_bindings import fast_rasterize, rasterize
    from test_oracle_ties import PX
    from util import tie_scene
    scene = tie_scene([2.0, 3.0], [1.0, 0.8], [[0.2, 0.5, 0.8], [0.9, 0.1, 0.1]]).to(cuda)
    settings = scene.settings(RasterizerMode.HYBRID_BLEND, 4)
    fast = fast_rasterize(*scene.gaussians(), settings, True)
    image, _ = rasterize(*scene.gaussians(), settings, True, False)
    want = np.array([0.2, 0.5, 0.8])
    assert np.abs(image[:, PX, PX].cpu().numpy() - want).max() <= 1e-6
    assert np.abs(fast[:, PX, PX].cpu().numpy() - want).max() <= 1e-5
