"""k-hop neighbour sampling on the GPU against the oracle: bit-exact blocks and counts."""
import numpy as np
import pytest

from helpers import chi_square_p, graph_from_degrees

pytestmark = pytest.mark.gpu


def test_layout_closed_form():
    from skywalker_amd import capi
    assert capi.sample_layout([1, 25, 10]) == (276, 26)
    assert capi.sample_layout([1, 2, 2]) == (7, 3)
    assert capi.sample_layout([1, 20, 20]) == (421, 21)


@pytest.mark.parametrize("device_sized", [1, 0])
@pytest.mark.parametrize("fanout", [[1, 25, 10], [1, 3, 2, 2], [1, 5]])
def test_offline_and_online_match_oracle(orc, fanout, device_sized):
    # device_sized 1 (the default): the size of every frontier stays on the device and the host never waits inside
    # the call; 0: the host reads it before it launches the build of the frontier's rows
    from skywalker_amd import capi
    xadj, adjncy = orc.rmat_csr(13, 8, 21)
    w = orc.gen_weights(orc.W_LOGNORMAL, 21, len(adjncy), 0.0, 1.0)
    seeds = orc.gen_seeds(4, 1 << 13, 1500)
    lps, slen = capi.sample_layout(fanout)
    g = capi.Graph.upload(xadj, adjncy, w)
    capi.set_option("online_device_sized", device_sized)
    try:
        d_on, sl_on, s_on, _ = g.sample_online(seeds, fanout, 17)
    finally:
        capi.set_option("online_device_sized", 1)
    on = (d_on.to_host((1500, lps)), sl_on.to_host((1500, slen)))
    g.build_tables()
    prob, alias, valid = g.tables()
    d_off, sl_off, s_off, _ = g.sample_offline(seeds, fanout, 17)
    off = (d_off.to_host((1500, lps)), sl_off.to_host((1500, slen)))
    g.free()
    odata, osl, osampled = orc.sample_offline(xadj, adjncy, prob, alias, seeds, fanout, 17)
    assert np.array_equal(off[1], osl) and np.array_equal(off[0], odata) and s_off == osampled
    assert np.array_equal(on[0], off[0]) and np.array_equal(on[1], off[1]) and s_on == s_off
    o2data, o2sl, o2sampled = orc.sample_online(xadj, adjncy, w, seeds, fanout, 17)
    assert np.array_equal(on[0], o2data) and np.array_equal(on[1], o2sl) and s_on == o2sampled
    assert osampled == int(osl.sum())


@pytest.mark.parametrize("fanout", [[1, 25, 10], [1, 3, 2, 2], [1, 64]])
def test_distinct_children_match_oracle(orc, fanout):
    # option sample_distinct: the reference's online rule (no slot of a row twice, at most 11 tries per draw)
    from skywalker_amd import capi
    xadj, adjncy = orc.rmat_csr(13, 8, 22)
    w = orc.gen_weights(orc.W_LOGNORMAL, 22, len(adjncy), 0.0, 2.0)  # skewed rows: tries do run out
    seeds = orc.gen_seeds(5, 1 << 13, 1500)
    lps, slen = capi.sample_layout(fanout)
    g = capi.Graph.upload(xadj, adjncy, w)
    capi.set_option("sample_distinct", 1)
    try:
        d_on, sl_on, s_on, _ = g.sample_online(seeds, fanout, 23)
        on = (d_on.to_host((1500, lps)), sl_on.to_host((1500, slen)))
        g.build_tables()
        d_off, sl_off, s_off, _ = g.sample_offline(seeds, fanout, 23)
        off = (d_off.to_host((1500, lps)), sl_off.to_host((1500, slen)))
        with pytest.raises(capi.SkyError):
            g.sample_offline(seeds, [1, 65], 23)
    finally:
        capi.set_option("sample_distinct", 0)
    prob, alias, valid = g.tables()
    g.free()
    odata, osl, osampled = orc.sample_offline(xadj, adjncy, prob, alias, seeds, fanout, 23, distinct=True)
    assert np.array_equal(off[1], osl) and np.array_equal(off[0], odata) and s_off == osampled
    assert np.array_equal(on[0], off[0]) and np.array_equal(on[1], off[1]) and s_on == s_off
    assert osampled == int(osl.sum())
    if fanout[1] >= 25:
        deg = np.diff(xadj)
        big = deg[seeds] > fanout[1]
        assert (osl[big, 0] < fanout[1]).any()  # a parent that ended with fewer children than its fanout is among the cases


def test_online_sampling_with_short_rows_built_in_vertex_order(orc):
    # option small_in_place = 1 on a list of frontier vertices (by default only builds of 2^25 rows and more use it)
    from skywalker_amd import capi
    xadj, adjncy = orc.rmat_csr(13, 8, 24)
    w = orc.gen_weights(orc.W_LOGNORMAL, 24, len(adjncy), 0.0, 1.0)
    seeds = orc.gen_seeds(6, 1 << 13, 1200)
    fanout = [1, 6, 4, 3]
    lps, slen = capi.sample_layout(fanout)
    g = capi.Graph.upload(xadj, adjncy, w)
    capi.set_option("small_in_place", 1)
    try:
        d_on, sl_on, s_on, _ = g.sample_online(seeds, fanout, 29)
        with pytest.raises(capi.SkyError):
            capi.set_option("small_in_place", 2)
    finally:
        capi.set_option("small_in_place", -1)
    got = (d_on.to_host((1200, lps)), sl_on.to_host((1200, slen)))
    g.free()
    odata, osl, osampled = orc.sample_online(xadj, adjncy, w, seeds, fanout, 29)
    assert np.array_equal(got[0], odata) and np.array_equal(got[1], osl) and s_on == osampled


def test_exact_count_when_every_degree_exceeds_fanout(orc):
    from skywalker_amd import capi
    rng = np.random.default_rng(6)
    V = 500
    xadj, adjncy, w = graph_from_degrees(rng.integers(30, 60, V), rng, "uniform", V=V)
    g = capi.Graph.upload(xadj, adjncy, w)
    g.build_tables()
    seeds = rng.integers(0, V, 300, dtype=np.uint32)
    data, sl, sampled, _ = g.sample_offline(seeds, [1, 25, 10], 3)
    g.free()
    assert sampled == 300 * (25 + 250)
    assert not np.any(data.to_host() == 0xFFFFFFFF)


def test_per_parent_draw_frequencies(orc):
    from skywalker_amd import capi
    rng = np.random.default_rng(9)
    d = 40
    xadj = np.zeros(d + 2, np.uint32)
    xadj[1:] = d
    adjncy = np.arange(1, d + 1, dtype=np.uint32)
    w = rng.lognormal(0, 1, d).astype(np.float32)
    g = capi.Graph.upload(xadj, adjncy, w)
    g.build_tables()
    N = 20000
    data, sl, sampled, _ = g.sample_offline(np.zeros(N, np.uint32), [1, 10], 5)
    g.free()
    draws = data.to_host((N, 11))[:, 1:].ravel()
    assert sampled == N * 10
    assert chi_square_p(np.bincount(draws, minlength=d + 1)[1:], w.astype(np.float64) / w.sum(dtype=np.float64)) > 0.01


def test_seeds_that_do_not_exist_have_no_children(orc):
    from skywalker_amd import capi
    xadj, adjncy = orc.rmat_csr(10, 8, 5)
    V = len(xadj) - 1
    w = orc.gen_weights(orc.W_UNIFORM, 5, len(adjncy), 1.0, 10.0)
    seeds = orc.gen_seeds(6, V, 200)
    seeds[::5] = V
    seeds[1] = 0xFFFFFFFF
    fanout = [1, 4, 3]
    lps, slen = capi.sample_layout(fanout)
    g = capi.Graph.upload(xadj, adjncy, w)
    d_on, sl_on, s_on, _ = g.sample_online(seeds, fanout, 3)
    on = (d_on.to_host((200, lps)), sl_on.to_host((200, slen)))
    g.build_tables()
    d_off, sl_off, s_off, _ = g.sample_offline(seeds, fanout, 3)
    off = (d_off.to_host((200, lps)), sl_off.to_host((200, slen)))
    g.free()
    odata, osl, osampled = orc.sample_online(xadj, adjncy, w, seeds, fanout, 3)
    for got, s in ((on, s_on), (off, s_off)):
        assert np.array_equal(got[0], odata) and np.array_equal(got[1], osl) and s == osampled
    assert np.all(osl[seeds >= V] == 0)


def test_online_sampling_builds_rows_of_every_class_without_waiting(orc):
    # frontiers whose rows fall into every degree class up to the streaming kernel's, their sizes known to the
    # device alone; a second call on the same graph finds the class census in place
    from helpers import graph_from_degrees
    from skywalker_amd import capi
    rng = np.random.default_rng(77)
    degs = [0, 1, 2, 3, 8, 9, 16, 17, 32, 33, 64, 65, 128, 129, 160, 161, 192, 193, 253, 254, 509, 510, 1021, 1022]
    degs += [512 * nw - 3 for nw in range(3, 11)] + [5118, 6500, 8190, 9000, 25000, 70000, 300000]
    degs += list(rng.integers(0, 300, 600))
    rng.shuffle(degs)
    xadj, adjncy, w = graph_from_degrees(degs, rng, "lognormal")
    V = len(xadj) - 1
    fanout = [1, 4, 3]
    lps, slen = capi.sample_layout(fanout)
    g = capi.Graph.upload(xadj, adjncy, w)
    for rep, n in enumerate((V, 50)):
        seeds = np.arange(n, dtype=np.uint32) if rep == 0 else rng.integers(0, V, n).astype(np.uint32)
        d_on, sl_on, s_on, _ = g.sample_online(seeds, fanout, 31 + rep)
        odata, osl, osampled = orc.sample_online(xadj, adjncy, w, seeds, fanout, 31 + rep)
        assert np.array_equal(d_on.to_host((n, lps)), odata) and np.array_equal(sl_on.to_host((n, slen)), osl)
        assert s_on == osampled
    g.free()


def test_sampling_hop_by_hop_with_the_callers_weights(orc):
    # sky_sample_session_*: the frontier of every hop is handed out, the rows are built from the weights the caller
    # gives for that hop.  With the graph's own weights the result is sky_sample_online's; with other weights it is
    # the oracle's online sample on a graph that carries those
    from skywalker_amd import capi
    xadj, adjncy = orc.rmat_csr(12, 8, 23)
    w = orc.gen_weights(orc.W_LOGNORMAL, 23, len(adjncy), 0.0, 1.0)
    w2 = orc.gen_weights(orc.W_UNIFORM, 29, len(adjncy), 1.0, 100.0)
    seeds = orc.gen_seeds(6, 1 << 12, 900)
    fanout = [1, 6, 4]
    lps, slen = capi.sample_layout(fanout)
    g = capi.Graph.upload(xadj, adjncy, w)
    d0, s0, n0, _ = g.sample_online(seeds, fanout, 31)
    want = (d0.to_host((900, lps)), s0.to_host((900, slen)), n0)
    d1, s1, n1, _ = g.sample_session(seeds, fanout, 31)
    assert np.array_equal(d1.to_host((900, lps)), want[0]) and np.array_equal(s1.to_host((900, slen)), want[1]) and n1 == n0
    import ctypes
    E = len(w2)
    w2_d = capi.DeviceArray.from_host(w2)
    # the same weights in memory that ends with the last of them (the allocation holds 4 * (E + 8) + 16 bytes): the
    # library copies such an array before its kernels read whole vectors from it
    room = capi.DeviceArray(E + 8, np.float32)

    class Exact:
        ptr = ctypes.c_void_p(room.ptr.value + 32)
    capi._ck(capi.lib().sky_memcpy_h2d(Exact.ptr, capi._p(w2), E * 4))
    odata, osl, osampled = orc.sample_online(xadj, adjncy, w2, seeds, fanout, 31)
    for arr in (w2_d, Exact):
        uppers = []
        d2, s2, n2, _ = g.sample_session(seeds, fanout, 31, lambda hop, upper: (uppers.append(upper), arr)[1])
        got = (d2.to_host((900, lps)), s2.to_host((900, slen)))
        assert uppers[0] == 900 and 0 < uppers[1] <= 900 * 6
        assert np.array_equal(got[1], osl) and np.array_equal(got[0], odata) and n2 == osampled
    g.free()
