"""Walks on the GPU against the oracle: bit-exact paths for the same Philox stream and tables."""
import numpy as np
import pytest

from helpers import chi_square_p, graph_from_degrees

pytestmark = pytest.mark.gpu


def run_offline(orc, xadj, adjncy, w, seeds, length, stop, seed):
    from skywalker_amd import capi
    g = capi.Graph.upload(xadj, adjncy, w)
    g.build_tables()
    prob, alias, valid = g.tables()
    paths_d, len_d, sampled, sec = g.walk_offline(seeds, length, stop, seed)
    paths, lengths = paths_d.to_host((len(seeds), length + 1)), len_d.to_host()
    g.free()
    opaths, olengths, osampled = orc.walk_offline(xadj, adjncy, prob, alias, seeds, length, stop, seed)
    return (paths, lengths, sampled), (opaths, olengths, osampled), (prob, alias, valid)


def test_config1_deepwalk_bit_exact(orc):
    xadj, adjncy = orc.rmat_csr(16, 16, 42)
    w = orc.gen_weights(orc.W_UNIFORM, 42, len(adjncy), 1.0, 100.0)
    seeds = orc.gen_seeds(42, 1 << 16, 4096)
    got, want, _ = run_offline(orc, xadj, adjncy, w, seeds, 80, 0.0, 42)
    assert np.array_equal(got[1], want[1])
    assert np.array_equal(got[0], want[0])
    assert got[2] == want[2] == int(want[1].sum())


def test_ppr_bit_exact_and_length_law(orc):
    # every vertex has out-edges so only the stop test ends a walk
    rng = np.random.default_rng(4)
    V = 2000
    xadj, adjncy, w = graph_from_degrees(rng.integers(1, 40, V), rng, "lognormal", V=V)
    seeds = rng.integers(0, V, 60000, dtype=np.uint32)
    tp, L = 0.15, 100
    got, want, _ = run_offline(orc, xadj, adjncy, w, seeds, L, tp, 7)
    assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1]) and got[2] == want[2]
    lengths = got[1].astype(np.float64)
    mean = (1 - (1 - tp) ** L) / tp - 1 + (1 - tp) ** L  # E[min(G, L)] with G ~ Geometric(tp) counting failures
    assert abs(lengths.mean() - mean) < 4 * np.sqrt((1 - tp) / tp**2 / len(seeds))
    k = np.arange(0, 30)
    cnt = np.array([(lengths == x).sum() for x in k])
    pk = tp * (1 - tp) ** k
    assert chi_square_p(np.append(cnt, len(seeds) - cnt.sum()), np.append(pk, 1 - pk.sum())) > 0.01


def test_dead_ends_and_zero_weight_rows(orc):
    # path graph 0 -> 1 -> 2 -> 3 (3 has no out-edge); vertex 4 has one zero-weight edge; 5 loops on itself
    xadj = np.array([0, 1, 2, 3, 3, 4, 5], np.uint32)
    adjncy = np.array([1, 2, 3, 0, 5], np.uint32)
    w = np.array([1, 1, 1, 0, 2], np.float32)
    seeds = np.array([0, 1, 2, 3, 4, 5], np.uint32)
    got, want, _ = run_offline(orc, xadj, adjncy, w, seeds, 6, 0.0, 1)
    assert got[1].tolist() == [3, 2, 1, 0, 0, 6]
    assert got[0][0, :4].tolist() == [0, 1, 2, 3] and np.all(got[0][0, 4:] == 0xFFFFFFFF)
    assert np.all(got[0][5] == 5)
    assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])


def test_next_hop_frequencies_chi_square(orc):
    # star: hub 0 with 50 weighted spokes; one step from the hub must follow w / sum(w)
    rng = np.random.default_rng(8)
    d = 50
    xadj = np.zeros(d + 2, np.uint32)
    xadj[1:] = d
    adjncy = np.arange(1, d + 1, dtype=np.uint32)
    w = rng.lognormal(0, 1, d).astype(np.float32)
    N = 200000
    seeds = np.zeros(N, np.uint32)
    got, want, _ = run_offline(orc, xadj, adjncy, w, seeds, 1, 0.0, 3)
    assert np.array_equal(got[0], want[0])
    counts = np.bincount(got[0][:, 1], minlength=d + 1)[1:]
    assert chi_square_p(counts, w.astype(np.float64) / w.astype(np.float64).sum()) > 0.01


def test_walk_does_not_depend_on_batch_composition(orc):
    # walker i's path is a function of (seed, i, start vertex) only
    from skywalker_amd import capi
    xadj, adjncy = orc.rmat_csr(12, 8, 5)
    w = orc.gen_weights(orc.W_UNIT, 5, len(adjncy))
    g = capi.Graph.upload(xadj, adjncy, w)
    g.build_tables()
    seeds = orc.gen_seeds(1, 1 << 12, 3000)
    full = g.walk_offline(seeds, 20, 0.0, 9)[0].to_host((3000, 21))
    part = g.walk_offline(seeds[:1000], 20, 0.0, 9)[0].to_host((1000, 21))
    g.free()
    assert np.array_equal(full[:1000], part)


@pytest.mark.parametrize("mode", [0, 1, -1, 2])
def test_online_static_walk_equals_offline_and_oracle(orc, mode):
    # mode 0: rows built step by step as walkers reach them; 1: every row first; -1: the library chooses;
    # 2: step by step with the host waiting for the size of every step's row list (option online_device_sized 0)
    from skywalker_amd import capi
    if mode == 2:
        capi.set_option("online_device_sized", 0)
        mode = 0
    xadj, adjncy = orc.rmat_csr(13, 8, 6)
    w = orc.gen_weights(orc.W_UNIFORM, 6, len(adjncy), 1.0, 100.0)
    seeds = orc.gen_seeds(3, 1 << 13, 2000)
    g = capi.Graph.upload(xadj, adjncy, w)
    capi.set_option("online_full_build", mode)
    try:
        p_on, l_on, s_on, _ = g.walk_online(capi.BIAS_STATIC, 1.0, 1.0, seeds, 30, 0.1, 5)
    finally:
        capi.set_option("online_full_build", -1)
        capi.set_option("online_device_sized", 1)
    on = (p_on.to_host((2000, 31)), l_on.to_host())
    g.build_tables()
    p_off, l_off, s_off, _ = g.walk_offline(seeds, 30, 0.1, 5)
    off = (p_off.to_host((2000, 31)), l_off.to_host())
    g.free()
    assert np.array_equal(on[0], off[0]) and np.array_equal(on[1], off[1]) and s_on == s_off
    opaths, olengths, osampled = orc.walk_online(xadj, adjncy, w, 0, 1.0, 1.0, seeds, 30, 0.1, 5)
    assert np.array_equal(on[0], opaths) and np.array_equal(on[1], olengths) and s_on == osampled


@pytest.mark.parametrize("scale,ef,stop", [(11, 8, 0.0), (13, 16, 0.05)])
def test_node2vec_bit_exact(orc, scale, ef, stop):
    from skywalker_amd import capi
    xadj, adjncy = orc.rmat_csr(scale, ef, 31)
    w = orc.gen_weights(orc.W_UNIFORM, 31, len(adjncy), 1.0, 100.0)
    seeds = orc.gen_seeds(2, 1 << scale, 1500)
    g = capi.Graph.upload(xadj, adjncy, w)
    paths, lengths, sampled, _ = g.walk_online(capi.BIAS_NODE2VEC, 2.0, 0.5, seeds, 20, stop, 13)
    got = (paths.to_host((1500, 21)), lengths.to_host())
    g.free()
    opaths, olengths, osampled = orc.walk_online(xadj, adjncy, w, 1, 2.0, 0.5, seeds, 20, stop, 13)
    assert np.array_equal(got[1], olengths)
    assert np.array_equal(got[0], opaths)
    assert sampled == osampled


def test_node2vec_hub_rows_beyond_the_weight_cache(orc):
    # a hub of degree 6000 (more than the kernel keeps in LDS) reached from and returning to small rows
    from skywalker_amd import capi
    rng = np.random.default_rng(12)
    V = 6001
    hub = np.arange(1, V, dtype=np.uint32)
    xadj = np.zeros(V + 1, np.uint32)
    xadj[1] = V - 1
    spokes = []
    for v in range(1, V):
        nb = sorted({0, int(rng.integers(1, V)), int(rng.integers(1, V))} - {v})
        spokes.append(nb)
        xadj[v + 1] = xadj[v] + len(nb)
    adjncy = np.concatenate([hub] + [np.array(s, np.uint32) for s in spokes])
    w = rng.lognormal(0, 1, len(adjncy)).astype(np.float32)
    seeds = rng.integers(0, V, 600, dtype=np.uint32)
    g = capi.Graph.upload(xadj, adjncy, w)
    paths, lengths, sampled, _ = g.walk_online(capi.BIAS_NODE2VEC, 2.0, 0.5, seeds, 12, 0.0, 4)
    got = (paths.to_host((600, 13)), lengths.to_host())
    g.free()
    opaths, olengths, osampled = orc.walk_online(xadj, adjncy, w, 1, 2.0, 0.5, seeds, 12, 0.0, 4)
    assert np.array_equal(got[0], opaths) and np.array_equal(got[1], olengths) and sampled == osampled


@pytest.mark.parametrize("scale,ef,stop,p,q", [(11, 8, 0.0, 2.0, 0.5), (13, 16, 0.05, 0.25, 4.0), (12, 8, 0.0, 1.0, 1.0)])
def test_node2vec_rejection_bit_exact(orc, scale, ef, stop, p, q):
    from skywalker_amd import capi
    xadj, adjncy = orc.rmat_csr(scale, ef, 33)
    w = orc.gen_weights(orc.W_LOGNORMAL, 33, len(adjncy), 0.0, 1.0)
    seeds = orc.gen_seeds(3, 1 << scale, 5000)
    g = capi.Graph.upload(xadj, adjncy, w)
    # no tables yet: the call builds the first-order tables itself
    paths, lengths, sampled, _ = g.walk_online(capi.BIAS_NODE2VEC_REJECT, p, q, seeds, 40, stop, 17)
    got = (paths.to_host((5000, 41)), lengths.to_host())
    prob, alias, valid = g.tables()
    g.free()
    oprob, oalias, ovalid = orc.alias_build(xadj, w)
    assert np.array_equal(prob.view(np.uint32), oprob.view(np.uint32)) and np.array_equal(alias, oalias)
    opaths, olengths, osampled = orc.walk_node2vec_reject(xadj, adjncy, oprob, oalias, p, q, seeds, 40, stop, 17)
    assert np.array_equal(got[1], olengths)
    assert np.array_equal(got[0], opaths)
    assert sampled == osampled


def test_read_once_gathers_give_the_same_paths(orc):
    from skywalker_amd import capi
    xadj, adjncy = orc.rmat_csr(12, 16, 36)
    w = orc.gen_weights(orc.W_LOGNORMAL, 36, len(adjncy), 0.0, 1.0)
    seeds = orc.gen_seeds(9, 1 << 12, 3000)
    g = capi.Graph.upload(xadj, adjncy, w)
    g.build_tables()
    prob, alias, _ = g.tables()
    want = orc.walk_offline(xadj, adjncy, prob, alias, seeds, 30, 0.02, 21)
    try:
        for mode in (0, 1):
            for indexed in (False, True):
                capi.set_option("walk_read_once", mode)
                g.build_tables()
                if indexed:
                    g.build_walk_index()
                paths, lengths, sampled, _ = g.walk_offline(seeds, 30, 0.02, 21)
                assert np.array_equal(paths.to_host((3000, 31)), want[0]) and np.array_equal(lengths.to_host(), want[1])
                assert sampled == want[2]
        with pytest.raises(capi.SkyError):
            capi.set_option("walk_read_once", 2)
    finally:
        capi.set_option("walk_read_once", -1)
        g.free()


def test_node2vec_rejection_one_walker_per_lane_for_large_batches(orc):
    # up to 262,144 walkers take 8 lanes each (they search the previous row together); larger batches one lane each
    from skywalker_amd import capi
    xadj, adjncy = orc.rmat_csr(12, 16, 35)
    w = orc.gen_weights(orc.W_LOGNORMAL, 35, len(adjncy), 0.0, 1.0)
    seeds = orc.gen_seeds(8, 1 << 12, 300000)
    g = capi.Graph.upload(xadj, adjncy, w)
    g.build_tables()
    paths, lengths, sampled, _ = g.walk_online(capi.BIAS_NODE2VEC_REJECT, 2.0, 0.5, seeds, 10, 0.0, 19)
    big = (paths.to_host((300000, 11)), lengths.to_host())
    small, _, _, _ = g.walk_online(capi.BIAS_NODE2VEC_REJECT, 2.0, 0.5, seeds[:70000], 10, 0.0, 19)
    small = small.to_host((70000, 11))
    prob, alias, valid = g.tables()
    g.free()
    opaths, olengths, osampled = orc.walk_node2vec_reject(xadj, adjncy, prob, alias, 2.0, 0.5, seeds, 10, 0.0, 19)
    assert np.array_equal(big[0], opaths) and np.array_equal(big[1], olengths) and sampled == osampled
    assert np.array_equal(small, opaths[:70000])


def test_node2vec_rejection_second_step_law(orc):
    # exact second-order law on a small graph, sampled on the device
    from skywalker_amd import capi
    edges = [(0, 1), (0, 2), (1, 2), (2, 3), (2, 4)]
    wts = [1.0, 2.0, 3.0, 4.0, 5.0]
    src = [a for a, b in edges] + [b for a, b in edges]
    dst = [b for a, b in edges] + [a for a, b in edges]
    ww = wts + wts
    order = np.lexsort((dst, src))
    adjncy = np.array(dst, np.uint32)[order]
    w = np.array(ww, np.float32)[order]
    xadj = np.zeros(6, np.uint32)
    np.add.at(xadj, np.array(src)[order] + 1, 1)
    xadj = np.cumsum(xadj).astype(np.uint32)
    p, q, N = 2.0, 0.5, 400000
    g = capi.Graph.upload(xadj, adjncy, w)
    paths, lengths, sampled, _ = g.walk_online(capi.BIAS_NODE2VEC_REJECT, p, q, np.zeros(N, np.uint32), 2, 0.0, 9)
    paths = paths.to_host((N, 3))
    g.free()
    sel = paths[:, 1] == 2
    second = np.bincount(paths[sel, 2], minlength=5)
    law = np.array([2.0 / p, 3.0, 0.0, 4.0 / q, 5.0 / q])
    law /= law.sum()
    assert second[2] == 0 and sampled == 2 * N
    assert chi_square_p(second[[0, 1, 3, 4]], law[[0, 1, 3, 4]]) > 0.01


def test_start_vertices_that_do_not_exist_never_move(orc):
    # same rule as the oracle's, in every walk kernel: the seed is recorded, the length is 0
    from skywalker_amd import capi
    xadj, adjncy = orc.rmat_csr(10, 8, 3)
    V = len(xadj) - 1
    w = orc.gen_weights(orc.W_UNIFORM, 3, len(adjncy), 1.0, 10.0)
    seeds = orc.gen_seeds(2, V, 300)
    seeds[::7] = V
    seeds[3::11] = 0xFFFFFFFF
    seeds[5] = V + 1

    def host(r, length):
        out = (r[0].to_host((len(seeds), length + 1)), r[1].to_host(), r[2])
        r[0].free()
        r[1].free()
        return out

    g = capi.Graph.upload(xadj, adjncy, w)
    capi.set_option("online_full_build", 0)
    try:
        lazy = host(g.walk_online(capi.BIAS_STATIC, 1.0, 1.0, seeds, 12, 0.05, 9), 12)
    finally:
        capi.set_option("online_full_build", -1)
    n2v = host(g.walk_online(capi.BIAS_NODE2VEC, 2.0, 0.5, seeds, 12, 0.05, 9), 12)
    g.build_tables()
    prob, alias, _ = g.tables()
    off = host(g.walk_offline(seeds, 12, 0.05, 9), 12)
    rej = host(g.walk_online(capi.BIAS_NODE2VEC_REJECT, 2.0, 0.5, seeds, 12, 0.05, 9), 12)
    g.free()
    want = orc.walk_offline(xadj, adjncy, prob, alias, seeds, 12, 0.05, 9)
    for got in (off, lazy):
        assert np.array_equal(got[1], want[1]) and np.array_equal(got[0], want[0]) and got[2] == want[2]
    want = orc.walk_online(xadj, adjncy, w, 1, 2.0, 0.5, seeds, 12, 0.05, 9)
    assert np.array_equal(n2v[1], want[1]) and np.array_equal(n2v[0], want[0]) and n2v[2] == want[2]
    want = orc.walk_node2vec_reject(xadj, adjncy, prob, alias, 2.0, 0.5, seeds, 12, 0.05, 9)
    assert np.array_equal(rej[1], want[1]) and np.array_equal(rej[0], want[0]) and rej[2] == want[2]
    assert np.all(off[1][seeds >= V] == 0)


@pytest.mark.parametrize("every", [0, 1, 7, 16])
@pytest.mark.parametrize("indexed", [False, True])
def test_walk_index_and_walker_lists_give_the_same_paths(orc, indexed, every):
    # the 16-byte walk index and the hand-over of live walkers between launches change how a walk is run, not what
    # it finds: DeepWalk and PPR paths, lengths and counts equal the oracle's
    from skywalker_amd import capi
    xadj, adjncy = orc.rmat_csr(14, 8, 17)
    w = orc.gen_weights(orc.W_LOGNORMAL, 17, len(adjncy), 0.0, 2.0)
    w[xadj[5]:xadj[6]] = 0.0  # a row without weight: walkers that reach it stop there
    V = len(xadj) - 1
    seeds = orc.gen_seeds(4, V, 20011)
    seeds[3] = V + 7
    g = capi.Graph.upload(xadj, adjncy, w)
    g.build_tables()
    prob, alias, _ = g.tables()
    if indexed:
        g.build_walk_index()
    capi.set_option("walk_compact_every", every)
    try:
        for length, stop, seed in ((80, 0.0, 5), (100, 0.15, 6), (3, 0.0, 7)):
            paths, lengths, sampled, _ = g.walk_offline(seeds, length, stop, seed)
            opaths, olengths, osampled = orc.walk_offline(xadj, adjncy, prob, alias, seeds, length, stop, seed)
            assert np.array_equal(lengths.to_host(), olengths)
            assert np.array_equal(paths.to_host((len(seeds), length + 1)), opaths)
            assert sampled == osampled
    finally:
        capi.set_option("walk_compact_every", 0)
    g.free()


def test_walk_index_goes_stale_when_tables_change(orc):
    # the index is a copy of table entries: a rebuild with other weights must not be walked with the old copy
    from skywalker_amd import capi
    xadj, adjncy = orc.rmat_csr(12, 8, 19)
    w1 = orc.gen_weights(orc.W_UNIFORM, 19, len(adjncy), 1.0, 100.0)
    w2 = orc.gen_weights(orc.W_LOGNORMAL, 20, len(adjncy), 0.0, 2.0)
    seeds = orc.gen_seeds(5, len(xadj) - 1, 3000)
    g = capi.Graph.upload(xadj, adjncy, w1)
    g.build_tables()
    g.build_walk_index()
    p2, a2, v2 = orc.alias_build(xadj, w2)
    g.upload_tables(p2, a2, v2)
    paths, lengths, sampled, _ = g.walk_offline(seeds, 30, 0.0, 2)
    opaths, olengths, osampled = orc.walk_offline(xadj, adjncy, p2, a2, seeds, 30, 0.0, 2)
    assert np.array_equal(paths.to_host((3000, 31)), opaths) and sampled == osampled
    g.build_walk_index()
    paths, lengths, sampled, _ = g.walk_offline(seeds, 30, 0.0, 2)
    assert np.array_equal(paths.to_host((3000, 31)), opaths) and sampled == osampled
    g.free()
