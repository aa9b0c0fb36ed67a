"""Shared builders for test inputs (host side, numpy)."""
import numpy as np


def graph_from_degrees(degs, rng, dist="lognormal", V=None):
    """CSR whose row i has degs[i] sorted random neighbours, plus weights of the given family."""
    degs = np.asarray(degs, np.int64)
    n = len(degs)
    V = V or max(n, 2)
    xadj = np.zeros(V + 1, np.uint32)
    xadj[1:n + 1] = np.cumsum(degs)
    xadj[n + 1:] = xadj[n]
    E = int(xadj[-1])
    adjncy = rng.integers(0, V, E, dtype=np.uint32)
    for v in range(n):  # rows sorted by neighbour id, as the CSR contract asks
        adjncy[xadj[v]:xadj[v + 1]].sort()
    return xadj, adjncy, weights(E, rng, dist)


def weights(E, rng, dist):
    if dist == "uniform":
        w = rng.uniform(1, 100, E)
    elif dist == "unit":
        w = 1.0 - rng.random(E)
    elif dist == "lognormal":
        w = rng.lognormal(0, 1, E)
    elif dist == "lognormal2":
        w = rng.lognormal(0, 2, E)
    elif dist == "equal":
        w = np.full(E, 3.0)
    elif dist == "nearequal":
        w = 1.0 + rng.integers(-3, 4, E) * 2.0 ** -23
    elif dist == "sparse":  # many exact zeros, a few negatives and NaN
        w = rng.lognormal(0, 1, E)
        w[rng.random(E) < 0.5] = 0.0
        w[rng.random(E) < 0.02] = -1.0
        w[rng.random(E) < 0.01] = np.nan
    else:
        raise ValueError(dist)
    return w.astype(np.float32)


def chi_square_p(counts, probs):
    """p-value of Pearson's chi-square for observed counts against probabilities (cells with expectation >= 5)."""
    from scipy import stats
    counts = np.asarray(counts, np.float64)
    probs = np.asarray(probs, np.float64)
    n = counts.sum()
    exp = probs * n
    big = exp >= 5
    if big.sum() < 2:
        return 1.0
    obs = np.append(counts[big], counts[~big].sum())
    ex = np.append(exp[big], exp[~big].sum())
    if ex[-1] == 0:
        obs, ex = obs[:-1], ex[:-1]
    chi2 = ((obs - ex) ** 2 / ex).sum()
    return float(stats.chi2.sf(chi2, len(ex) - 1))
