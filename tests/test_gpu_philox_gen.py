"""Device Philox and the device-side synthetic input generators against the oracle."""
import numpy as np
import pytest

from test_oracle_philox import KAT

pytestmark = pytest.mark.gpu


def test_device_philox_known_answers():
    from skywalker_amd import capi
    ctr = np.array([k[0] for k in KAT], np.uint32)
    key = np.array([k[1] for k in KAT], np.uint32)
    out = capi.philox_selftest(ctr, key)
    assert out.tolist() == [k[2] for k in KAT]


def test_device_philox_matches_oracle(orc):
    from skywalker_amd import capi
    rng = np.random.default_rng(0)
    ctr = rng.integers(0, 2**32, (1000, 4), dtype=np.uint32)
    key = rng.integers(0, 2**32, (1000, 2), dtype=np.uint32)
    out = capi.philox_selftest(ctr, key)
    for i in range(0, 1000, 37):
        assert np.array_equal(out[i], orc.philox(ctr[i], key[i]))


@pytest.mark.parametrize("scale,ef,seed", [(10, 8, 3), (16, 16, 42), (18, 7, 5)])
def test_rmat_topology_and_uniform_weights(orc, scale, ef, seed):
    from skywalker_amd import capi
    print("rmat", scale, ef, seed, flush=True)
    g = capi.Graph.rmat(scale, ef, seed, capi.W_UNIFORM, 1.0, 100.0, seed)
    xadj, adjncy, w = g.download()
    md = g.max_degree
    g.free()
    oxadj, oadj = orc.rmat_csr(scale, ef, seed)
    assert np.array_equal(xadj, oxadj) and np.array_equal(adjncy, oadj)
    assert np.array_equal(w, orc.gen_weights(orc.W_UNIFORM, seed, len(oadj), 1.0, 100.0))
    assert md == int(np.diff(oxadj.astype(np.int64)).max())
    assert w.min() >= 1.0 and w.max() < 100.0
    # rows sorted by neighbour id
    deg = np.diff(xadj.astype(np.int64))
    inner = np.ones(len(adjncy), bool)
    inner[xadj[:-1][deg > 0]] = False
    assert np.all(adjncy[1:][inner[1:]] >= adjncy[:-1][inner[1:]])


def test_unit_and_lognormal_weights(orc):
    from skywalker_amd import capi
    g = capi.Graph.rmat(12, 8, 1, capi.W_UNIT, 0.0, 0.0, 1)
    _, adjncy, w = g.download()
    g.free()
    assert np.array_equal(w, orc.gen_weights(orc.W_UNIT, 1, len(adjncy)))
    assert w.min() > 0 and w.max() <= 1.0
    g = capi.Graph.rmat(12, 8, 1, capi.W_LOGNORMAL, 0.0, 2.0, 77)
    _, adjncy, w = g.download()
    g.free()
    ow = orc.gen_weights(orc.W_LOGNORMAL, 77, len(adjncy), 0.0, 2.0)
    # libm of host and device differ in the last bits: compare to 1e-4 relative, and the law's moments
    assert np.allclose(w, ow, rtol=1e-4)
    lw = np.log(w.astype(np.float64))
    assert abs(lw.mean()) < 0.05 and abs(lw.std() - 2.0) < 0.05


def test_seeds(orc):
    from skywalker_amd import capi
    g = capi.Graph.rmat(10, 4, 1, capi.W_UNIT, 0, 0, 1)
    s = g.gen_seeds(99, 5000).to_host()
    g.free()
    assert np.array_equal(s, orc.gen_seeds(99, 1 << 10, 5000))
    assert s.max() < (1 << 10)


def test_graph_from_degrees(orc):
    # rows of chosen lengths, neighbours and weights drawn on the device: the build of such a graph = the oracle's on
    # the arrays it downloads, and the generator repeats itself for the same seeds
    from skywalker_amd import capi
    rng = np.random.default_rng(3)
    degs = np.concatenate([rng.integers(0, 40, 3000), rng.integers(100, 3000, 60), [9000, 70000]])
    rng.shuffle(degs)
    xadj = np.zeros(len(degs) + 1, np.uint32)
    xadj[1:] = np.cumsum(degs)
    g = capi.Graph.from_degrees(xadj, 11, capi.W_LOGNORMAL, 0.0, 2.0, 12)
    assert g.V == len(degs) and g.E == int(xadj[-1]) and g.max_degree == 70000
    hx, hadj, hw = g.download()
    assert np.array_equal(hx, xadj) and hadj.max() < g.V and len(np.unique(hadj)) > g.V // 2
    assert np.allclose(hw, orc.gen_weights(orc.W_LOGNORMAL, 12, g.E, 0.0, 2.0), rtol=1e-4)  # device expf, logf, cosf
    g.build_tables()
    prob, alias, valid = g.tables()
    oprob, oalias, ovalid = orc.alias_build(hx, hw)
    assert np.array_equal(prob, oprob) and np.array_equal(alias, oalias) and np.array_equal(valid, ovalid)
    g2 = capi.Graph.from_degrees(xadj, 11, capi.W_LOGNORMAL, 0.0, 2.0, 12)
    assert np.array_equal(g2.download()[1], hadj)
    g.free()
    g2.free()
