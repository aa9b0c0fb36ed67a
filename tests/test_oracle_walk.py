"""Pins the oracle's walk / PPR / node2vec / k-hop samplers by what the mathematics fixes:
closed forms on tiny graphs, chi-square against the exact transition laws, and the output layout."""
import numpy as np

from helpers import chi_square_p, graph_from_degrees


def undirected(edges, V, weights=None):
    """Sorted CSR of an undirected graph given as a list of (u, v)."""
    rows = [[] for _ in range(V)]
    for idx, (u, v) in enumerate(edges):
        w = 1.0 if weights is None else weights[idx]
        rows[u].append((v, w))
        rows[v].append((u, w))
    xadj, adj, wgt = [0], [], []
    for r in rows:
        r.sort()
        adj += [a for a, _ in r]
        wgt += [b for _, b in r]
        xadj.append(len(adj))
    return np.array(xadj, np.uint32), np.array(adj, np.uint32), np.array(wgt, np.float32)


def test_path_graph_and_dead_end(orc):
    xadj = np.array([0, 1, 2, 3, 3], np.uint32)
    adjncy = np.array([1, 2, 3], np.uint32)
    w = np.ones(3, np.float32)
    prob, alias, valid = orc.alias_build(xadj, w)
    paths, lengths, sampled = orc.walk_offline(xadj, adjncy, prob, alias, np.array([0, 2, 3], np.uint32), 5, 0.0, 1)
    assert lengths.tolist() == [3, 1, 0] and sampled == 4
    assert paths[0, :4].tolist() == [0, 1, 2, 3] and np.all(paths[0, 4:] == orc.FILL)
    assert paths[2, 0] == 3 and np.all(paths[2, 1:] == orc.FILL)


def test_star_next_hop_law(orc):
    rng = np.random.default_rng(1)
    d = 37
    xadj = np.zeros(d + 2, np.uint32)
    xadj[1:] = d
    adjncy = np.arange(1, d + 1, dtype=np.uint32)
    w = rng.lognormal(0, 1.2, d).astype(np.float32)
    prob, alias, valid = orc.alias_build(xadj, w)
    N = 300000
    paths, lengths, _ = orc.walk_offline(xadj, adjncy, prob, alias, np.zeros(N, np.uint32), 1, 0.0, 11)
    assert np.all(lengths == 1)
    counts = np.bincount(paths[:, 1], minlength=d + 1)[1:]
    assert chi_square_p(counts, w.astype(np.float64) / w.sum(dtype=np.float64)) > 0.01
    # a second seed gives a different stream (the key is used)
    paths2, _, _ = orc.walk_offline(xadj, adjncy, prob, alias, np.zeros(N, np.uint32), 1, 0.0, 12)
    assert not np.array_equal(paths, paths2)


def test_complete_graph_uniform_law(orc):
    V = 12
    edges = [(u, v) for u in range(V) for v in range(u + 1, V)]
    xadj, adjncy, w = undirected(edges, V)
    prob, alias, valid = orc.alias_build(xadj, w)
    N = 120000
    paths, lengths, sampled = orc.walk_offline(xadj, adjncy, prob, alias, np.zeros(N, np.uint32), 3, 0.0, 5)
    assert sampled == 3 * N
    # after 3 steps from 0 on K12: P(back at 0) = (1 - (-1/11)^3)/12 ... use the exact Markov chain instead
    P = (np.ones((V, V)) - np.eye(V)) / (V - 1)
    law = np.linalg.matrix_power(P, 3)[0]
    assert chi_square_p(np.bincount(paths[:, 3], minlength=V), law) > 0.01


def test_ppr_length_law(orc):
    rng = np.random.default_rng(3)
    V = 300
    xadj, adjncy, w = graph_from_degrees(rng.integers(2, 9, V), rng, "uniform", V=V)
    prob, alias, valid = orc.alias_build(xadj, w)
    N, tp, L = 200000, 0.15, 100
    _, lengths, sampled = orc.walk_offline(xadj, adjncy, prob, alias, rng.integers(0, V, N, dtype=np.uint32), L, tp, 2)
    assert sampled == int(lengths.sum())
    k = np.arange(0, 40)
    cnt = np.array([(lengths == x).sum() for x in k])
    pk = tp * (1 - tp) ** k  # stop test comes before the step: length k = k survivals then a stop
    assert chi_square_p(np.append(cnt, N - cnt.sum()), np.append(pk, 1 - pk.sum())) > 0.01
    assert lengths.max() <= L


def test_online_static_equals_offline(orc):
    xadj, adjncy = orc.rmat_csr(10, 8, 4)
    w = orc.gen_weights(orc.W_UNIFORM, 4, len(adjncy), 1.0, 100.0)
    prob, alias, valid = orc.alias_build(xadj, w)
    seeds = orc.gen_seeds(1, 1 << 10, 500)
    a = orc.walk_offline(xadj, adjncy, prob, alias, seeds, 25, 0.05, 9)
    b = orc.walk_online(xadj, adjncy, w, 0, 1.0, 1.0, seeds, 25, 0.05, 9)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1]) and a[2] == b[2]


def test_node2vec_second_order_factors_brute_force(orc):
    # triangle 0-1-2 with a tail 2-3 and a second tail 2-4; walk 0 -> 2 -> ?
    edges = [(0, 1), (0, 2), (1, 2), (2, 3), (2, 4)]
    wts = [1.0, 2.0, 3.0, 4.0, 5.0]
    xadj, adjncy, w = undirected(edges, 5, wts)
    p, q = 2.0, 0.5
    N = 400000
    paths, lengths, _ = orc.walk_online(xadj, adjncy, w, 1, p, q, np.zeros(N, np.uint32), 2, 0.0, 77)
    assert np.all(lengths == 2)
    # first step has no previous vertex: plain weights of row 0 = {1: 1.0, 2: 2.0}
    first = np.bincount(paths[:, 1], minlength=5)
    assert chi_square_p(first[[1, 2]], np.array([1.0, 2.0]) / 3.0) > 0.01
    # second step from cur=2 with prev=0: row of 2 = {0: 2.0, 1: 3.0, 3: 4.0, 4: 5.0}
    #   0 is the previous vertex -> /p ; 1 is adjacent to 0 -> x1 ; 3 and 4 are not -> /q
    sel = paths[:, 1] == 2
    second = np.bincount(paths[sel, 2], minlength=5)
    law = np.array([2.0 / p, 3.0, 0.0, 4.0 / q, 5.0 / q])
    law /= law.sum()
    assert second[2] == 0
    assert chi_square_p(second[[0, 1, 3, 4]], law[[0, 1, 3, 4]]) > 0.01
    # from cur=1 with prev=0: row of 1 = {0: 1.0, 2: 3.0}; 0 -> /p, 2 adjacent to 0 -> x1
    sel = paths[:, 1] == 1
    second = np.bincount(paths[sel, 2], minlength=5)
    law = np.array([1.0 / p, 0, 3.0, 0, 0])
    law /= law.sum()
    assert chi_square_p(second[[0, 2]], law[[0, 2]]) > 0.01


def test_node2vec_p_q_one_is_first_order(orc):
    xadj, adjncy = orc.rmat_csr(9, 8, 2)
    w = orc.gen_weights(orc.W_UNIFORM, 2, len(adjncy), 1.0, 100.0)
    seeds = orc.gen_seeds(5, 1 << 9, 300)
    a = orc.walk_online(xadj, adjncy, w, 1, 1.0, 1.0, seeds, 20, 0.0, 3)
    b = orc.walk_online(xadj, adjncy, w, 0, 1.0, 1.0, seeds, 20, 0.0, 3)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])


def test_node2vec_rejection_brute_force_law(orc):
    # same graph and laws as the table-per-step test above, sampled by rejection on the first-order tables
    edges = [(0, 1), (0, 2), (1, 2), (2, 3), (2, 4)]
    wts = [1.0, 2.0, 3.0, 4.0, 5.0]
    xadj, adjncy, w = undirected(edges, 5, wts)
    prob, alias, valid = orc.alias_build(xadj, w)
    for p, q in [(2.0, 0.5), (0.25, 4.0)]:
        N = 400000
        paths, lengths, sampled = orc.walk_node2vec_reject(xadj, adjncy, prob, alias, p, q, np.zeros(N, np.uint32), 2,
                                                           0.0, 78)
        assert np.all(lengths == 2) and sampled == 2 * N
        first = np.bincount(paths[:, 1], minlength=5)
        assert chi_square_p(first[[1, 2]], np.array([1.0, 2.0]) / 3.0) > 0.01
        sel = paths[:, 1] == 2
        second = np.bincount(paths[sel, 2], minlength=5)
        law = np.array([2.0 / p, 3.0, 0.0, 4.0 / q, 5.0 / q])
        law /= law.sum()
        assert second[2] == 0
        assert chi_square_p(second[[0, 1, 3, 4]], law[[0, 1, 3, 4]]) > 0.01
        sel = paths[:, 1] == 1
        second = np.bincount(paths[sel, 2], minlength=5)
        law = np.array([1.0 / p, 0, 3.0, 0, 0])
        law /= law.sum()
        assert chi_square_p(second[[0, 2]], law[[0, 2]]) > 0.01


def test_node2vec_rejection_p_q_one_is_first_order(orc):
    # f == fmax == 1 for every candidate: trial 0 is always kept, so the walk is the offline walk
    xadj, adjncy = orc.rmat_csr(9, 8, 2)
    w = orc.gen_weights(orc.W_UNIFORM, 2, len(adjncy), 1.0, 100.0)
    prob, alias, valid = orc.alias_build(xadj, w)
    seeds = orc.gen_seeds(5, 1 << 9, 300)
    a = orc.walk_node2vec_reject(xadj, adjncy, prob, alias, 1.0, 1.0, seeds, 20, 0.1, 3)
    b = orc.walk_offline(xadj, adjncy, prob, alias, seeds, 20, 0.1, 3)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1]) and a[2] == b[2]


def test_node2vec_rejection_and_table_agree_in_law(orc):
    # third vertex of walks from one seed on a random graph: both node2vec samplers, one chi-square each
    # against the exact two-step law computed from the weights
    rng = np.random.default_rng(21)
    V = 40
    xadj, adjncy, w = graph_from_degrees(rng.integers(3, 9, V), rng, "lognormal", V=V)
    # node2vec needs rows sorted by neighbour id and an undirected membership relation is not required
    for v in range(V):
        o = np.argsort(adjncy[xadj[v]:xadj[v + 1]], kind="stable")
        adjncy[xadj[v]:xadj[v + 1]] = adjncy[xadj[v]:xadj[v + 1]][o]
        w[xadj[v]:xadj[v + 1]] = w[xadj[v]:xadj[v + 1]][o]
    p, q = 2.0, 0.5
    law = np.zeros(V)
    row0 = slice(xadj[0], xadj[1])
    w0 = np.zeros(V)
    np.add.at(w0, adjncy[row0], w[row0].astype(np.float64))
    w0 /= w0.sum()
    nb0 = set(adjncy[row0].tolist())
    for v in range(V):
        if w0[v] == 0:
            continue
        sec = np.zeros(V)
        for e in range(xadj[v], xadj[v + 1]):
            x = int(adjncy[e])
            f = 1 / p if x == 0 else (1.0 if x in nb0 else 1 / q)
            sec[x] += float(w[e]) * f
        law += w0[v] * sec / sec.sum()
    N = 300000
    prob, alias, valid = orc.alias_build(xadj, w)
    seeds = np.zeros(N, np.uint32)
    a, la, _ = orc.walk_node2vec_reject(xadj, adjncy, prob, alias, p, q, seeds, 2, 0.0, 5)
    b, lb, _ = orc.walk_online(xadj, adjncy, w, 1, p, q, seeds, 2, 0.0, 5)
    assert np.all(la == 2) and np.all(lb == 2)
    keep = law > 0
    for paths in (a, b):
        cnt = np.bincount(paths[:, 2], minlength=V)
        assert cnt[~keep].sum() == 0
        assert chi_square_p(cnt[keep], law[keep]) > 0.01


def test_sample_layout_and_counts(orc):
    assert orc.sample_layout([1, 25, 10])[:2] == (276, 26)
    assert orc.sample_layout([1, 25, 10])[2] == [0, 1, 26]
    rng = np.random.default_rng(4)
    V = 200
    xadj, adjncy, w = graph_from_degrees(rng.integers(30, 50, V), rng, "uniform", V=V)
    prob, alias, valid = orc.alias_build(xadj, w)
    seeds = rng.integers(0, V, 100, dtype=np.uint32)
    data, sl, sampled = orc.sample_offline(xadj, adjncy, prob, alias, seeds, [1, 25, 10], 8)
    assert sampled == 100 * (25 + 250) and np.all(sl[:, 0] == 25) and np.all(sl[:, 1:] == 10)
    assert np.array_equal(data[:, 0], seeds) and not np.any(data == orc.FILL)
    # every hop-1 vertex is a neighbour of the seed; every hop-2 vertex a neighbour of its parent slot
    for s in range(0, 100, 17):
        nb = set(adjncy[xadj[seeds[s]]:xadj[seeds[s] + 1]].tolist())
        assert set(data[s, 1:26].tolist()) <= nb
        for j in range(25):
            par = data[s, 1 + j]
            nb2 = set(adjncy[xadj[par]:xadj[par + 1]].tolist())
            assert set(data[s, 26 + 10 * j:36 + 10 * j].tolist()) <= nb2


def test_sample_small_degrees_copy_all(orc):
    # degree <= fanout: every neighbour is copied in order and the count is the degree
    xadj = np.array([0, 3, 4, 4, 6], np.uint32)
    adjncy = np.array([1, 2, 3, 0, 0, 1], np.uint32)
    w = np.ones(6, np.float32)
    prob, alias, valid = orc.alias_build(xadj, w)
    data, sl, sampled = orc.sample_offline(xadj, adjncy, prob, alias, np.array([0], np.uint32), [1, 4, 2], 1)
    assert sl[0].tolist() == [3, 1, 0, 2, 0]  # hop-1 count, then children counts of slots 0..3
    assert data[0, 1:4].tolist() == [1, 2, 3] and data[0, 4] == orc.FILL
    assert data[0, 5] == 0 and data[0, 6] == orc.FILL          # child of slot 0 (vertex 1)
    assert data[0, 7] == orc.FILL and data[0, 8] == orc.FILL   # vertex 2 has no out-edge
    assert data[0, 9:11].tolist() == [0, 1]                    # vertex 3
    assert sampled == 6


def test_sample_draw_law_and_online_equals_offline(orc):
    rng = np.random.default_rng(5)
    d = 30
    xadj = np.zeros(d + 2, np.uint32)
    xadj[1:] = d
    adjncy = np.arange(1, d + 1, dtype=np.uint32)
    w = rng.lognormal(0, 1, d).astype(np.float32)
    prob, alias, valid = orc.alias_build(xadj, w)
    N = 30000
    data, sl, sampled = orc.sample_offline(xadj, adjncy, prob, alias, np.zeros(N, np.uint32), [1, 8], 3)
    assert sampled == 8 * N
    assert chi_square_p(np.bincount(data[:, 1:].ravel(), minlength=d + 1)[1:],
                        w.astype(np.float64) / w.sum(dtype=np.float64)) > 0.01
    d2, sl2, s2 = orc.sample_online(xadj, adjncy, w, np.zeros(N, np.uint32), [1, 8], 3)
    assert np.array_equal(data, d2) and np.array_equal(sl, sl2) and sampled == s2


def distinct_law(p, k, rounds=11):
    """Exact law of the ordered list of distinct slots that k draws leave: draw i tries up to `rounds` times and
    keeps the first slot not taken yet; a draw whose tries all hit taken slots leaves nothing."""
    dist = {(): 1.0}
    for _ in range(k):
        nxt = {}
        for taken, pr in dist.items():
            m = sum(p[c] for c in taken)
            tries = sum(m ** t for t in range(rounds))  # a free slot c is kept with probability p[c] * sum_t m^t
            nxt[taken] = nxt.get(taken, 0.0) + pr * m ** rounds
            for c in range(len(p)):
                if c not in taken:
                    nxt[taken + (c,)] = nxt.get(taken + (c,), 0.0) + pr * p[c] * tries
        dist = nxt
    return dist


def test_distinct_sampling_law_brute_force(orc):
    # a row of five slots, one of which holds 70 % of the weight, so that tries do run out now and then
    w = np.array([70.0, 12.0, 9.0, 6.0, 3.0], np.float32)
    d, k = len(w), 3
    xadj = np.zeros(d + 2, np.uint32)
    xadj[1:] = d
    adjncy = np.arange(1, d + 1, dtype=np.uint32)
    prob, alias, _ = orc.alias_build(xadj, w)
    N = 200000
    data, sl, sampled = orc.sample_offline(xadj, adjncy, prob, alias, np.zeros(N, np.uint32), [1, k], 9, distinct=True)
    assert sampled == int(sl.sum()) and sl.max() <= k
    law = distinct_law((w.astype(np.float64) / w.sum(dtype=np.float64)).tolist(), k)
    assert abs(sum(law.values()) - 1.0) < 1e-12
    keys = sorted(law)
    index = {key: i for i, key in enumerate(keys)}
    counts = np.zeros(len(keys))
    for row, n in zip(data, sl[:, 0]):
        got = tuple(int(x) - 1 for x in row[1:1 + n])
        assert len(set(got)) == len(got) and np.all(row[1 + n:] == orc.FILL)
        counts[index[got]] += 1
    expect = np.array([law[key] for key in keys])
    rare = expect * N < 5  # pooled: too few expected for a chi-square cell of their own
    c = np.append(counts[~rare], counts[rare].sum())
    e = np.append(expect[~rare], expect[rare].sum())
    assert chi_square_p(c[e > 0], e[e > 0]) > 0.01
    assert (sl[:, 0] < k).mean() > 0.001  # the case of a draw that leaves nothing is in the sample
    # same tables rebuilt on the way: same result
    d2, sl2, s2 = orc.sample_online(xadj, adjncy, w, np.zeros(N, np.uint32), [1, k], 9, distinct=True)
    assert np.array_equal(data, d2) and np.array_equal(sl, sl2) and sampled == s2
    # the first child is the first draw of the rule with replacement (try 0 uses the same random numbers)
    d3, _, _ = orc.sample_offline(xadj, adjncy, prob, alias, np.zeros(N, np.uint32), [1, k], 9)
    assert np.array_equal(data[:, 1], d3[:, 1])


def test_distinct_sampling_counts_and_limits(orc):
    rng = np.random.default_rng(12)
    V = 300
    xadj, adjncy, w = graph_from_degrees(rng.integers(0, 60, V), rng, "lognormal", V=V)
    prob, alias, valid = orc.alias_build(xadj, w)
    seeds = rng.integers(0, V, 500, dtype=np.uint32)
    data, sl, sampled = orc.sample_offline(xadj, adjncy, prob, alias, seeds, [1, 25, 10], 2, distinct=True)
    deg = np.diff(xadj)
    assert sampled == int(sl.sum())
    for s in range(len(seeds)):
        n = sl[s, 0]
        if deg[seeds[s]] <= 25:
            assert n == deg[seeds[s]] * valid[seeds[s]]
        else:
            assert 1 <= n <= 25
        for j in range(n):
            par = data[s, 1 + j]
            m = sl[s, 1 + j]
            assert m == deg[par] * valid[par] if deg[par] <= 10 else 1 <= m <= 10
    import pytest
    with pytest.raises(ValueError):
        orc.sample_offline(xadj, adjncy, prob, alias, seeds, [1, 65], 2, distinct=True)


def test_start_vertices_that_do_not_exist_never_move(orc):
    # every walk and the sampler record such a seed and stop there: length 0, no children
    xadj, adjncy = orc.rmat_csr(8, 8, 3)
    V = len(xadj) - 1
    w = orc.gen_weights(orc.W_UNIFORM, 3, len(adjncy), 1.0, 10.0)
    prob, alias, _ = orc.alias_build(xadj, w)
    seeds = np.array([5, V, 7, 0xFFFFFFFF, V + 1000, 9], np.uint32)
    bad = seeds >= V
    runs = [orc.walk_offline(xadj, adjncy, prob, alias, seeds, 6, 0.0, 1),
            orc.walk_online(xadj, adjncy, w, 0, 1.0, 1.0, seeds, 6, 0.0, 1),
            orc.walk_online(xadj, adjncy, w, 1, 2.0, 0.5, seeds, 6, 0.0, 1),
            orc.walk_node2vec_reject(xadj, adjncy, prob, alias, 2.0, 0.5, seeds, 6, 0.0, 1)]
    for paths, lengths, sampled in runs:
        assert np.array_equal(paths[:, 0], seeds)
        assert np.all(lengths[bad] == 0) and np.all(paths[bad, 1:] == orc.FILL)
        assert sampled == int(lengths.sum())
    good = runs[0]
    ref = orc.walk_offline(xadj, adjncy, prob, alias, seeds[~bad], 6, 0.0, 1)
    assert np.array_equal(good[1][~bad] > 0, ref[1] > 0)  # the others walk as usual (walker ids differ, so not the same paths)
    for data, sl, sampled in (orc.sample_offline(xadj, adjncy, prob, alias, seeds, [1, 3, 2], 1),
                              orc.sample_online(xadj, adjncy, w, seeds, [1, 3, 2], 1)):
        assert np.array_equal(data[:, 0], seeds)
        assert np.all(data[bad, 1:] == orc.FILL) and np.all(sl[bad] == 0)
        assert sampled == int(sl.sum())
