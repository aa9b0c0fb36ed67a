"""The fixtures of tests/golden (written by tests/golden/make_golden.py) against the oracle, and on a GPU box
against the HIP path: the same bits as on the day they were written."""
import json
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
SCALE, EF, SEED, N, LEN, P, Q, FANOUT = 8, 8, 7, 64, 10, 2.0, 0.5, [1, 4, 3]


def load(name):
    with np.load(os.path.join(GOLDEN, name), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def bits(a):
    return np.ascontiguousarray(a).view(np.uint8)


def same(a, b):
    return a.shape == b.shape and np.array_equal(bits(a), bits(b))


def test_philox_known_answers(orc):
    with open(os.path.join(GOLDEN, "philox_kat.json")) as f:
        kat = json.load(f)
    assert len(kat) == 3
    for k in kat:
        assert orc.philox(k["ctr"], k["key"]).tolist() == k["out"]


def test_toy_row_of_the_reference(orc):
    # 35 x 0.5 and 5 x 2.0 (test/tmp.cu:30-52): scaled weights 0.7273 and 2.9091
    z = load("toy_row.npz")
    prob, alias, valid = orc.alias_build_row(z["w"])
    assert valid and same(prob, z["prob"]) and same(alias, z["alias"])
    assert np.allclose(z["prob"][:35], 40 * 0.5 / 27.5, rtol=1e-6)
    q = orc.reconstruct_row(z["prob"], z["alias"])
    assert np.allclose(q, z["w"] / z["w"].sum(), rtol=1e-6)


def test_small_graph_oracle_reproduces_the_fixture(orc):
    z = load("rmat_s8.npz")
    xadj, adjncy = orc.rmat_csr(SCALE, EF, SEED)
    assert same(xadj, z["xadj"]) and same(adjncy, z["adjncy"])
    w = orc.gen_weights(orc.W_LOGNORMAL, SEED, len(adjncy), 0.0, 1.0)
    w[xadj[3]:xadj[4]] = 0.0
    assert same(w, z["w"])
    prob, alias, valid = orc.alias_build(xadj, w)
    assert same(prob, z["prob"]) and same(alias, z["alias"]) and same(valid, z["valid"])
    assert valid[3] == 0 or xadj[4] == xadj[3]
    seeds = z["seeds"]
    got = orc.walk_offline(xadj, adjncy, prob, alias, seeds, LEN, 0.0, SEED)
    assert same(got[0], z["dw_paths"]) and same(got[1], z["dw_lengths"])
    got = orc.walk_offline(xadj, adjncy, prob, alias, seeds, LEN, 0.15, SEED)
    assert same(got[0], z["ppr_paths"]) and same(got[1], z["ppr_lengths"])
    got = orc.walk_online(xadj, adjncy, w, 1, P, Q, seeds, LEN, 0.0, SEED)
    assert same(got[0], z["n2v_paths"]) and same(got[1], z["n2v_lengths"])
    got = orc.walk_node2vec_reject(xadj, adjncy, prob, alias, P, Q, seeds, LEN, 0.0, SEED)
    assert same(got[0], z["rej_paths"]) and same(got[1], z["rej_lengths"])
    got = orc.sample_offline(xadj, adjncy, prob, alias, seeds, FANOUT, SEED)
    assert same(got[0], z["sample_data"]) and same(got[1], z["sample_lengths"])
    assert z["dw_lengths"][5] == 0  # the start vertex that does not exist


@pytest.mark.gpu
def test_small_graph_gpu_reproduces_the_fixture():
    from skywalker_amd import capi
    z = load("rmat_s8.npz")
    seeds = z["seeds"]
    lps, slen = capi.sample_layout(FANOUT)

    def host(r):
        out = (r[0].to_host((N, LEN + 1)), r[1].to_host())
        r[0].free()
        r[1].free()
        return out

    g = capi.Graph.upload(z["xadj"], z["adjncy"], z["w"])
    capi.set_option("online_full_build", 0)
    try:
        lazy = host(g.walk_online(capi.BIAS_STATIC, 1.0, 1.0, seeds, LEN, 0.0, SEED))
    finally:
        capi.set_option("online_full_build", -1)
    n2v = host(g.walk_online(capi.BIAS_NODE2VEC, P, Q, seeds, LEN, 0.0, SEED))
    r = g.sample_online(seeds, FANOUT, SEED)
    s_on = (r[0].to_host((N, lps)), r[1].to_host((N, slen)))
    g.build_tables()
    prob, alias, valid = g.tables()
    assert same(prob, z["prob"]) and same(alias, z["alias"]) and same(valid, z["valid"])
    dw = host(g.walk_offline(seeds, LEN, 0.0, SEED))
    ppr = host(g.walk_offline(seeds, LEN, 0.15, SEED))
    rej = host(g.walk_online(capi.BIAS_NODE2VEC_REJECT, P, Q, seeds, LEN, 0.0, SEED))
    r = g.sample_offline(seeds, FANOUT, SEED)
    s_off = (r[0].to_host((N, lps)), r[1].to_host((N, slen)))
    g.free()
    for got, name in ((dw, "dw"), (lazy, "dw"), (ppr, "ppr"), (n2v, "n2v"), (rej, "rej")):
        assert same(got[0], z[name + "_paths"]) and same(got[1], z[name + "_lengths"]), name
    for got in (s_off, s_on):
        assert same(got[0], z["sample_data"]) and same(got[1], z["sample_lengths"])
