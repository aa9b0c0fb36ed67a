"""Pins the oracle's R-MAT generator by the law it must follow: at every level the (source bit, destination bit)
pair of an edge is (0,0), (0,1), (1,0), (1,1) with probabilities a, b, c, d = 0.57, 0.19, 0.19, 0.05.  Every
benchmark configuration is defined through this generator."""
import numpy as np

from helpers import chi_square_p

A, B, C, D = 0.57, 0.19, 0.19, 0.05


def edges(orc, scale, ef, seed):
    xadj, adjncy = orc.rmat_csr(scale, ef, seed)
    src = np.repeat(np.arange(len(xadj) - 1, dtype=np.uint32), np.diff(xadj.astype(np.int64)))
    return xadj, src, adjncy


def test_quadrant_law_at_every_level(orc):
    scale = 13
    xadj, src, dst = edges(orc, scale, 64, 8)
    for lvl in range(scale):  # level 0 is the most significant bit
        sh = scale - 1 - lvl
        quad = ((src >> sh) & 1) * 2 + ((dst >> sh) & 1)  # 0: (0,0)  1: (0,1)  2: (1,0)  3: (1,1)
        counts = np.bincount(quad, minlength=4)
        assert chi_square_p(counts, [A, B, C, D]) > 0.001, (lvl, counts / counts.sum())
    # a swap of b and c cannot be seen (b = c), but a swap of the source
    # and destination thresholds with a or d would shift these by > 0.1
    top = np.bincount(((src >> (scale - 1)) & 1) * 2 + ((dst >> (scale - 1)) & 1), minlength=4) / len(src)
    assert np.allclose(top, [A, B, C, D], atol=0.01)


def test_levels_are_independent(orc):
    # joint law of the first two levels = product law (16 cells): consecutive 16-bit lanes of one Philox call do
    # not leak into each other
    scale = 12
    xadj, src, dst = edges(orc, scale, 32, 11)
    q0 = ((src >> 11) & 1) * 2 + ((dst >> 11) & 1)
    q1 = ((src >> 10) & 1) * 2 + ((dst >> 10) & 1)
    counts = np.bincount(q0 * 4 + q1, minlength=16)
    law = np.outer([A, B, C, D], [A, B, C, D]).ravel()
    assert chi_square_p(counts, law) > 0.001
    # and levels that come from different Philox calls (level 7 is the last of call 0, level 8 the first of call 1)
    q7 = ((src >> 4) & 1) * 2 + ((dst >> 4) & 1)
    q8 = ((src >> 3) & 1) * 2 + ((dst >> 3) & 1)
    assert chi_square_p(np.bincount(q7 * 4 + q8, minlength=16), law) > 0.001


def test_skew_is_on_both_sides_and_sources_follow_a_plus_b(orc):
    scale, ef = 14, 16
    xadj, src, dst = edges(orc, scale, ef, 3)
    V, E = 1 << scale, ef << scale
    deg = np.diff(xadj.astype(np.int64))
    assert deg.sum() == E
    # out-degree of a vertex with k one-bits is Binomial(E, (a+b)^(scale-k) (c+d)^k): vertex 0 is the hub
    exp0 = E * (A + B) ** scale
    assert abs(deg[0] - exp0) < 6 * np.sqrt(exp0)
    ones = np.array([bin(v).count("1") for v in range(V)])
    for k in (1, 2, 3):
        m = deg[ones == k].mean()
        want = E * (A + B) ** (scale - k) * (C + D) ** k
        assert abs(m - want) < 0.05 * want
    # in-degree of vertex 0 follows (a+c)^scale, the same number: the marginals are symmetric, the joint is not
    indeg0 = int((dst == 0).sum())
    assert abs(indeg0 - E * (A + C) ** scale) < 6 * np.sqrt(exp0)
    # self-pairing: P(src bit == dst bit) = a + d per level
    same = ((src ^ dst) == 0).sum()
    assert abs(same - E * (A + D) ** scale) < 6 * np.sqrt(E * (A + D) ** scale) + 3
    # rows are sorted by destination, duplicates kept
    for v in (0, 1, 5, V - 1):
        r = dst[xadj[v]:xadj[v + 1]]
        assert np.all(r[1:] >= r[:-1])
