"""Pins the oracle's alias-table builder without retyping its formula:
closed forms, the reconstruction invariant, and textbook Vose as a second opinion."""
import numpy as np
import pytest

TOL = 1e-6  # relative, per entry: the bar for every alias table in this repository


def target(w):
    w = np.asarray(w, np.float64)
    return w / w.sum()


def rel_err(q, t):
    m = t > 0
    assert np.all(q[~m] == 0)
    return np.max(np.abs(q[m] - t[m]) / t[m]) if m.any() else 0.0


def test_degree_one(orc):
    prob, alias, valid = orc.alias_build_row([3.5])
    assert valid == 1 and prob[0] == 1.0 and alias[0] == 0


def test_equal_weights(orc):
    for d in (2, 3, 7, 64, 65, 1000):
        prob, alias, valid = orc.alias_build_row(np.full(d, 2.25, np.float32))
        assert valid == 1
        # every column keeps its own mass: either prob 1 or alias to itself
        q = orc.reconstruct_row(prob, alias)
        assert np.allclose(q, 1.0 / d, rtol=TOL, atol=0)
        assert np.all((prob == 1.0) | (alias == np.arange(d)))


def test_two_weights(orc):
    a, b = 1.0, 3.0
    prob, alias, valid = orc.alias_build_row([a, b])
    assert valid == 1
    assert abs(prob[0] - 2 * a / (a + b)) < 1e-7 and alias[0] == 1
    assert prob[1] == 1.0
    prob, alias, _ = orc.alias_build_row([b, a])  # transposed operand
    assert abs(prob[1] - 2 * a / (a + b)) < 1e-7 and alias[1] == 0 and prob[0] == 1.0


def test_reference_toy_row(orc):
    # the 40-item row of the reference's test/tmp.cu:30-52: 35 x 0.5 and 5 x 2.0
    w = np.array([0.5] * 35 + [2.0] * 5, np.float32)
    prob, alias, valid = orc.alias_build_row(w)
    assert valid == 1
    scaled = w * 40 / w.sum()
    assert abs(scaled[0] - 0.72727) < 1e-4 and abs(scaled[-1] - 2.90909) < 1e-4
    assert np.allclose(prob[:35], scaled[0], rtol=1e-6)
    assert np.all(alias[:35] >= 35)  # every small is topped up by a large
    donors = np.bincount(alias[:35], minlength=40)[35:]
    assert donors.sum() == 35 and donors.max() <= 8 and donors.min() >= 6  # each large serves about 7 smalls
    assert rel_err(orc.reconstruct_row(prob, alias), target(w)) < TOL


def test_zero_rows(orc):
    prob, alias, valid = orc.alias_build_row(np.zeros(5, np.float32))
    assert valid == 0 and np.all(prob == 0) and np.all(alias == orc.INVALID)
    prob, alias, valid = orc.alias_build_row(np.array([], np.float32))
    assert valid == 0
    # zeros, negatives and NaN inside a live row get probability exactly 0
    w = np.array([0.0, 2.0, -1.0, np.nan, 6.0], np.float32)
    prob, alias, valid = orc.alias_build_row(w)
    q = orc.reconstruct_row(prob, alias)
    assert valid == 1 and q[0] == 0 and q[2] == 0 and q[3] == 0
    assert abs(q[1] - 0.25) < 1e-7 and abs(q[4] - 0.75) < 1e-7


@pytest.mark.parametrize("dist", ["uniform", "unit", "lognormal1", "lognormal2", "onehot", "nearequal", "geometric"])
@pytest.mark.parametrize("d", [2, 3, 5, 8, 17, 63, 64, 65, 257, 4099, 70001])
def test_invariant_random_rows(orc, dist, d):
    rng = np.random.default_rng(d * 131 + len(dist))
    if dist == "uniform":
        w = rng.uniform(1, 100, d)
    elif dist == "unit":
        w = 1.0 - rng.random(d)
    elif dist == "lognormal1":
        w = rng.lognormal(0, 1, d)
    elif dist == "lognormal2":
        w = rng.lognormal(0, 2, d)
    elif dist == "onehot":
        w = np.full(d, 1e-3)
        w[rng.integers(d)] = 1e4
    elif dist == "nearequal":
        w = 1.0 + rng.integers(-3, 4, d) * 2.0 ** -23
    else:
        w = 0.5 ** (np.arange(d) % 40)
    w = w.astype(np.float32)
    prob, alias, valid = orc.alias_build_row(w)
    assert valid == 1
    assert np.all((prob >= 0) & (prob <= 1)) and np.all(alias < d)
    assert rel_err(orc.reconstruct_row(prob, alias), target(w)) < TOL


def test_matches_textbook_vose_distribution(orc):
    rng = np.random.default_rng(7)
    for _ in range(300):
        d = int(rng.integers(1, 65))
        w = rng.lognormal(0, 1.5, d).astype(np.float32)
        prob, alias, valid = orc.alias_build_row(w)
        vprob, valias, ok = orc.vose_row(w)
        assert valid == 1 and ok == 1
        q = orc.reconstruct_row(prob, alias)
        vq = np.zeros(d)
        for i in range(d):  # same definition, written out here in fp64
            vq[i] += vprob[i]
            vq[valias[i]] += 1.0 - vprob[i]
        vq /= d
        assert np.allclose(q, vq, rtol=TOL, atol=0)
        assert np.allclose(vq, target(w), rtol=1e-9, atol=0)


def test_brute_force_sampling_of_a_table(orc):
    # enumerate every (column, accept/reject) outcome of a small table exactly
    w = np.array([4, 1, 1, 2, 8, 0.5], np.float32)
    prob, alias, _ = orc.alias_build_row(w)
    mass = np.zeros(6)
    for col in range(6):
        mass[col] += float(prob[col]) / 6
        mass[alias[col]] += (1 - float(prob[col])) / 6
    assert np.allclose(mass, target(w), rtol=TOL)


def test_build_all_on_rmat(orc):
    # config 1 of the baseline: scale 16, edge factor 16, U[1,100) weights, seed 42
    xadj, adjncy = orc.rmat_csr(16, 16, 42)
    w = orc.gen_weights(orc.W_UNIFORM, 42, len(adjncy), 1.0, 100.0)
    prob, alias, valid = orc.alias_build(xadj, w)
    st = orc.alias_check(xadj, w, prob, alias, valid)
    assert st["bad_valid"] == 0 and st["bad_range"] == 0 and st["bad_invalid"] == 0
    assert st["max_rel_err"] < TOL
    deg = np.diff(xadj.astype(np.int64))
    assert np.array_equal(valid != 0, deg > 0)
    # the thread count must not change a single bit
    prob1, alias1, valid1 = orc.alias_build(xadj, w, nthreads=1)
    assert np.array_equal(prob, prob1) and np.array_equal(alias, alias1) and np.array_equal(valid, valid1)


def test_check_detects_a_wrong_table(orc):
    xadj, adjncy = orc.rmat_csr(10, 8, 3)
    w = orc.gen_weights(orc.W_UNIFORM, 3, len(adjncy), 1.0, 100.0)
    prob, alias, valid = orc.alias_build(xadj, w)
    v = int(np.argmax(np.diff(xadj.astype(np.int64))))
    bad = prob.copy()
    bad[xadj[v]] = max(0.0, bad[xadj[v]] - 1e-3)
    assert orc.alias_check(xadj, w, bad, alias, valid)["max_rel_err"] > TOL
    bad_alias = alias.copy()
    bad_alias[xadj[v] + 1] = (bad_alias[xadj[v] + 1] + 1) % (xadj[v + 1] - xadj[v])
    assert orc.alias_check(xadj, w, prob, bad_alias, valid)["max_rel_err"] > TOL


def test_special_weight_values(orc):
    # NaN, infinities, negatives and -0 count as zero; values above 2^32 as 2^32; weights below 2^-64 add nothing
    # to the exact sum, so a row made only of them is invalid
    w = np.array([np.nan, np.inf, -np.inf, -1.0, -0.0, 0.0, 1e-45, 2.0 ** -64, 3e-19, 2.0 ** 32, 2.0 ** 33, 3e38,
                  1.0, 7.5], np.float32)
    with np.errstate(all="ignore"):
        prob, alias, valid = orc.alias_build_row(w)
        clamped = np.where(np.isnan(w) | (w <= 0), 0.0, np.minimum(w.astype(np.float64), 2.0 ** 32))
    assert valid == 1
    q = orc.reconstruct_row(prob, alias)
    t = clamped / clamped.sum()
    big = t > 1e-20
    assert np.allclose(q[big], t[big], rtol=1e-6, atol=0) and np.all(q[~big] < 1e-20)
    # the four entries clamped to 2^32 (inf, 2^32, 2^33, 3e38) get equal shares
    assert np.allclose(q[[1, 9, 10, 11]], q[1], rtol=1e-6, atol=0)
    for tiny in ([1e-30, 1e-25], [1e-45], [2.0 ** -65, 0.0, -2.0]):
        p2, a2, v2 = orc.alias_build_row(np.array(tiny, np.float32))
        assert v2 == 0 and np.all(p2 == 0) and np.all(a2 == orc.INVALID)
    p3, a3, v3 = orc.alias_build_row(np.array([2.0 ** -64, 2.0 ** -64], np.float32))
    assert v3 == 1 and np.allclose(orc.reconstruct_row(p3, a3), [0.5, 0.5])
