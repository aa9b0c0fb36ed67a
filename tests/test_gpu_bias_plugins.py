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
