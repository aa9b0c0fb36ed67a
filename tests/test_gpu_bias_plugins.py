"""The bias operator (include/skywalker_bias.h): each shipped plug-in library against the oracle run on the weights
the operator stands for."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def degree_weights(xadj, adjncy):
    deg = np.diff(xadj.astype(np.int64))
    return deg[adjncy].astype(np.float32)


def test_degree_plugin_tables_and_walks(orc):
    # src/api/bias_degree.cu:12-16: an edge weighs as much as its end vertex has out-edges (0 for a dead end)
    from skywalker_amd import capi
    xadj, adjncy = orc.rmat_csr(13, 8, 41)
    w = orc.gen_weights(orc.W_UNIFORM, 41, len(adjncy), 1.0, 100.0)  # ignored by the operator
    wd = degree_weights(xadj, adjncy)
    assert (wd == 0).any() and wd.max() > 500
    plug = capi.BiasPlugin("degree")
    assert plug.name == "degree"
    g = capi.Graph.upload(xadj, adjncy, w)
    plug.build_all(g)
    prob, alias, valid = g.tables()
    oprob, oalias, ovalid = orc.alias_build(xadj, wd)
    assert np.array_equal(prob.view(np.uint32), oprob.view(np.uint32)) and np.array_equal(alias, oalias)
    assert np.array_equal(valid, ovalid)
    # the graph's own weights are untouched
    assert np.array_equal(g.download()[2], w)
    seeds = orc.gen_seeds(2, len(xadj) - 1, 1500)
    # offline walk on the operator's tables, and the online walk that evaluates the operator at every step
    paths, lengths, sampled, _ = g.walk_offline(seeds, 25, 0.05, 3)
    opaths, olengths, osampled = orc.walk_offline(xadj, adjncy, oprob, oalias, seeds, 25, 0.05, 3)
    assert np.array_equal(paths.to_host((1500, 26)), opaths) and sampled == osampled
    paths, lengths, sampled, _ = plug.walk_online(g, 1.0, 1.0, seeds, 25, 0.05, 3)
    assert np.array_equal(lengths.to_host(), olengths)
    assert np.array_equal(paths.to_host((1500, 26)), opaths) and sampled == osampled
    g.free()


@pytest.mark.parametrize("p,q,stop", [(2.0, 0.5, 0.0), (0.25, 4.0, 0.05)])
def test_node2vec_plugin_equals_the_built_in_bias(orc, p, q, stop):
    # src/api/bias_node2vec.cu:15-27 through the operator = SKY_BIAS_NODE2VEC = the oracle's table per step
    from skywalker_amd import capi
    xadj, adjncy = orc.rmat_csr(12, 8, 43)
    w = orc.gen_weights(orc.W_LOGNORMAL, 43, len(adjncy), 0.0, 1.0)
    seeds = orc.gen_seeds(3, len(xadj) - 1, 1200)
    seeds[7] = len(xadj) + 3  # a start vertex that does not exist
    plug = capi.BiasPlugin("node2vec")
    g = capi.Graph.upload(xadj, adjncy, w)
    paths, lengths, sampled, _ = plug.walk_online(g, p, q, seeds, 20, stop, 11)
    got = (paths.to_host((1200, 21)), lengths.to_host(), sampled)
    ref = g.walk_online(capi.BIAS_NODE2VEC, p, q, seeds, 20, stop, 11)
    g.free()
    opaths, olengths, osampled = orc.walk_online(xadj, adjncy, w, 1, p, q, seeds, 20, stop, 11)
    assert np.array_equal(got[1], olengths) and np.array_equal(got[0], opaths) and got[2] == osampled
    assert np.array_equal(ref[0].to_host((1200, 21)), opaths)


def test_static_plugin_is_the_edge_weight(orc):
    from skywalker_amd import capi
    xadj, adjncy = orc.rmat_csr(12, 8, 45)
    w = orc.gen_weights(orc.W_UNIFORM, 45, len(adjncy), 1.0, 100.0)
    w[xadj[9]:xadj[10]] = 0.0
    seeds = orc.gen_seeds(4, len(xadj) - 1, 1000)
    plug = capi.BiasPlugin("static")
    g = capi.Graph.upload(xadj, adjncy, w)
    plug.build_all(g)
    prob, alias, valid = g.tables()
    oprob, oalias, ovalid = orc.alias_build(xadj, w)
    assert np.array_equal(prob.view(np.uint32), oprob.view(np.uint32)) and np.array_equal(alias, oalias)
    assert np.array_equal(valid, ovalid)
    paths, lengths, sampled, _ = plug.walk_online(g, 1.0, 1.0, seeds, 30, 0.1, 5)
    opaths, olengths, osampled = orc.walk_online(xadj, adjncy, w, 0, 1.0, 1.0, seeds, 30, 0.1, 5)
    assert np.array_equal(paths.to_host((1000, 31)), opaths) and np.array_equal(lengths.to_host(), olengths)
    assert sampled == osampled
    g.free()


@pytest.mark.parametrize("device_sized", [1, 0])
def test_degree_plugin_online_sampling(orc, device_sized):
    # the operator inside online k-hop sampling: hop by hop, evaluated for the distinct frontier rows alone, their
    # tables built from those weights = the oracle's online sampler on the weights the operator stands for
    from skywalker_amd import capi
    xadj, adjncy = orc.rmat_csr(13, 8, 47)
    w = orc.gen_weights(orc.W_UNIFORM, 47, len(adjncy), 1.0, 100.0)  # ignored by the operator
    wd = degree_weights(xadj, adjncy)
    seeds = orc.gen_seeds(5, len(xadj) - 1, 1200)
    fanout = [1, 6, 4]
    lps, slen = capi.sample_layout(fanout)
    plug = capi.BiasPlugin("degree")
    g = capi.Graph.upload(xadj, adjncy, w)
    capi.set_option("online_device_sized", device_sized)
    try:
        data, sl, sampled, _ = plug.sample_online(g, 1.0, 1.0, seeds, fanout, 13)
    finally:
        capi.set_option("online_device_sized", 1)
    odata, osl, osampled = orc.sample_online(xadj, adjncy, wd, seeds, fanout, 13)
    assert np.array_equal(sl.to_host((1200, slen)), osl) and np.array_equal(data.to_host((1200, lps)), odata)
    assert sampled == osampled
    # and it differs from sampling on the graph's own weights, which stay as they are
    d2, _, _, _ = g.sample_online(seeds, fanout, 13)
    assert not np.array_equal(d2.to_host((1200, lps)), odata)
    assert np.array_equal(g.download()[2], w)
    g.free()


def test_static_plugin_online_sampling_equals_the_built_in(orc):
    from skywalker_amd import capi
    xadj, adjncy = orc.rmat_csr(12, 8, 48)
    w = orc.gen_weights(orc.W_LOGNORMAL, 48, len(adjncy), 0.0, 1.0)
    seeds = orc.gen_seeds(6, len(xadj) - 1, 800)
    fanout = [1, 5, 3]
    lps, slen = capi.sample_layout(fanout)
    plug = capi.BiasPlugin("static")
    g = capi.Graph.upload(xadj, adjncy, w)
    data, sl, sampled, _ = plug.sample_online(g, 1.0, 1.0, seeds, fanout, 14)
    ref = g.sample_online(seeds, fanout, 14)
    g.free()
    assert np.array_equal(data.to_host(), ref[0].to_host()) and np.array_equal(sl.to_host(), ref[1].to_host())
    assert sampled == ref[2]
