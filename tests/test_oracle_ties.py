"""Fragments of exactly equal depth in HYBRID_BLEND's sorted core, pinned by hand.

The reference inserts a fragment by walking the slots front to back and exchanging whenever the carried depth is
strictly smaller (R/include/hybrid_blend/kernels/inference.cuh:159-167).  When the walk passes over two stored entries of
equal depth, the displaced first one does not exchange with the second (2 < 2 is false), so it hops over it: the pair
swaps places, and at the end of the core the *first* of a run of equal entries is the one that leaves.  "Keep the K
nearest by (depth, index)" -- what a sort, or a merge of partial cores, would give -- differs there.  The scenes below put
Gaussians on the optical axis so that at the centre pixel every fragment's alpha and depth are known exactly; the
expected pixel is computed in float64 from the core the exchange walk must produce, worked out by hand, and the other
candidate order is shown to give a clearly different pixel, so that the test can tell them apart."""
import numpy as np

from util import hybrid_pixel_by_hand, oracle_render, tie_scene

PX = 32


def exchange_walk(fragments, K):
    """The reference's insertion on (depth, number) pairs in list order: the core and what left it (or never entered)."""
    core, tail = [(np.inf, None)] * K, []
    for depth, k in fragments:
        carried = (depth, k)
        if depth < core[K - 1][0]:
            for i in range(K):
                if carried[0] < core[i][0]:
                    carried, core[i] = core[i], carried
        if carried[1] is not None:
            tail.append(carried[1])
    return [k for _, k in core if k is not None], tail


def check(depths, opacities, colours, expected_core, expected_tail, other_core, other_tail):
    # the hand-worked core is what the exchange walk gives (a second statement of the walk, on integers, to guard the hand work)
    assert exchange_walk(list(zip(depths, range(len(depths)))), 4) == (expected_core, expected_tail)
    scene = tie_scene(depths, opacities, colours)
    ref = oracle_render(scene, 0, 4)
    want_rgb, want_depth = hybrid_pixel_by_hand(expected_core, expected_tail, depths, opacities, colours)
    other_rgb, _ = hybrid_pixel_by_hand(other_core, other_tail, depths, opacities, colours)
    assert np.abs(want_rgb - other_rgb).max() > 1e-2                     # the two candidate orders are far apart
    got = ref["image"][:, PX, PX]
    assert np.abs(got - want_rgb).max() <= 2e-6, (got, want_rgb, other_rgb)
    assert abs(ref["depth"][PX, PX] - want_depth) <= 1e-5 * want_depth
    return scene, want_rgb, want_depth


# fragment:        0 (A)            1 (B)            2 (C)            3 (E)            4 (D, arrives last, nearest)
TWO = dict(depths=[1.0, 2.0, 2.0, 3.0, 0.5], opacities=[0.3, 0.6, 0.5, 0.4, 0.2],
           colours=[[0.9, 0.1, 0.1], [0.1, 0.9, 0.1], [0.1, 0.1, 0.9], [0.8, 0.8, 0.1], [0.5, 0.5, 0.5]])
# A, B, C, F all but A at depth 2, then D: the first of the three equal entries is the one that leaves
THREE = dict(depths=[1.0, 2.0, 2.0, 2.0, 0.5], opacities=[0.3, 0.6, 0.5, 0.4, 0.2],
             colours=[[0.9, 0.1, 0.1], [0.1, 0.9, 0.1], [0.1, 0.1, 0.9], [0.8, 0.8, 0.1], [0.5, 0.5, 0.5]])


def test_two_equal_depths_swap_places_when_a_nearer_fragment_arrives():
    """Core after A, B, C, E: [A, B, C, E].  D (0.5) enters: slot 0 takes D and A is carried; slot 1 takes A, B is carried;
    slot 2 holds C at B's depth: no exchange; slot 3 (E, deeper) takes B, E leaves.  Core [D, A, C, B]: B and C have
    swapped; by (depth, index) it would be [D, A, B, C]."""
    check(**TWO, expected_core=[4, 0, 2, 1], expected_tail=[3], other_core=[4, 0, 1, 2], other_tail=[3])


def test_the_first_of_three_equal_depths_leaves_the_core():
    """Core after A, B, C, F: [A, B, C, F] with B, C, F at one depth.  D enters: A moves to slot 1, B is carried past C and F
    (no exchange with an equal depth) and leaves.  Core [D, A, C, F], tail B; by (depth, index) F would leave."""
    check(**THREE, expected_core=[4, 0, 2, 3], expected_tail=[1], other_core=[4, 0, 1, 2], other_tail=[3])
