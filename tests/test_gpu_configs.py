"""The benchmark configurations 2, 3 and 4 at their full sizes on the GPU against the oracle on the host
(configuration 1 is test_config1_deepwalk_bit_exact, configuration 5 is test_gpu_fullsize.py).  Graphs come from
the device generator and are downloaded, as the log-normal weights are not bit-portable between libm and the GPU."""
import time

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def same_tables(got, want):
    return (np.array_equal(got[0].view(np.uint32), want[0].view(np.uint32)) and np.array_equal(got[1], want[1]) and
            np.array_equal(got[2], want[2]))


def test_config2_scale20_unit_weights_build_and_deepwalk(orc):
    # R-MAT scale 20, edge factor 16, weights U(0,1], 40,000 start vertices, length 80, Philox seed 1
    from skywalker_amd import capi
    g = capi.Graph.rmat(20, 16, 1, capi.W_UNIT, 0.0, 0.0, 1)
    assert g.V == 1 << 20 and g.E == 16 << 20
    xadj, adjncy, w = g.download()
    oxadj, oadjncy = orc.rmat_csr(20, 16, 1)
    assert np.array_equal(xadj, oxadj) and np.array_equal(adjncy, oadjncy)
    assert np.array_equal(w, orc.gen_weights(orc.W_UNIT, 1, g.E))
    assert w.min() > 0.0 and w.max() <= 1.0
    g.build_tables()
    tables = g.tables()
    assert same_tables(tables, orc.alias_build(xadj, w))
    st = orc.alias_check(xadj, w, *tables)
    assert st["max_rel_err"] < 1e-6 and st["bad_valid"] == 0 and st["bad_range"] == 0 and st["bad_invalid"] == 0
    N, L = 40000, 80
    seeds_d = g.gen_seeds(1, N)
    seeds = seeds_d.to_host()
    assert np.array_equal(seeds, orc.gen_seeds(1, g.V, N))
    paths, lengths, sampled, _ = g.walk_offline(seeds_d, L, 0.0, 1)
    opaths, olengths, osampled = orc.walk_offline(xadj, adjncy, tables[0], tables[1], seeds, L, 0.0, 1)
    assert np.array_equal(lengths.to_host(), olengths) and np.array_equal(paths.to_host((N, L + 1)), opaths)
    assert sampled == osampled == int(olengths.sum())
    g.free()


def test_config3_scale22_online_two_hop_sampling(orc):
    # R-MAT scale 22, edge factor 32, log-normal(0, 1) weights; fanout 25 then 10 from 40,000 seeds, tables built
    # on the fly for the frontier only
    from skywalker_amd import capi
    t0 = time.time()
    g = capi.Graph.rmat(22, 32, 3, capi.W_LOGNORMAL, 0.0, 1.0, 3)
    assert g.V == 1 << 22 and g.E == 32 << 22
    xadj, adjncy, w = g.download()
    N, fan = 40000, [1, 25, 10]
    seeds_d = g.gen_seeds(3, N)
    seeds = seeds_d.to_host()
    data, sl, sampled, _ = g.sample_online(seeds_d, fan, 3)
    lps, slen = capi.sample_layout(fan)
    assert (lps, slen) == (276, 26)
    data, sl = data.to_host((N, lps)), sl.to_host((N, slen))
    say("config 3: GPU sampled %d edges (%.1f s)" % (sampled, time.time() - t0))
    odata, osl, osampled = orc.sample_online(xadj, adjncy, w, seeds, fan, 3)
    say("config 3: oracle done (%.1f s)" % (time.time() - t0))
    assert sampled == osampled == int(osl.sum())
    assert np.array_equal(sl, osl)
    assert np.array_equal(data, odata)
    # the rows the call built on the way are rows of the offline table
    g.build_tables()
    off, osl2, osampled2, _ = g.sample_offline(seeds_d, fan, 3)
    assert osampled2 == sampled and np.array_equal(off.to_host((N, lps)), data)
    g.free()


def test_config4_scale24_online_node2vec(orc):
    # R-MAT scale 24, edge factor 16, weights U[1,100); p = 2, q = 0.5, 40,000 walkers of length 80 by rejection on
    # first-order tables the call builds itself; the table-per-step method on the first 2,000 walkers
    from skywalker_amd import capi
    t0 = time.time()
    g = capi.Graph.rmat(24, 16, 4, capi.W_UNIFORM, 1.0, 100.0, 4)
    assert g.V == 1 << 24 and g.E == 16 << 24
    xadj, adjncy, w = g.download()
    N, L, p, q = 40000, 80, 2.0, 0.5
    seeds_d = g.gen_seeds(4, N)
    seeds = seeds_d.to_host()
    few = 2000
    tp, tl, tsampled, _ = g.walk_online(capi.BIAS_NODE2VEC, p, q, seeds[:few], L, 0.0, 4)
    tp, tl = tp.to_host((few, L + 1)), tl.to_host()
    say("config 4: table per step on the GPU, %d steps (%.1f s)" % (tsampled, time.time() - t0))
    paths, lengths, sampled, _ = g.walk_online(capi.BIAS_NODE2VEC_REJECT, p, q, seeds_d, L, 0.0, 4)
    paths, lengths = paths.to_host((N, L + 1)), lengths.to_host()
    tables = g.tables()
    say("config 4: rejection on the GPU, %d steps (%.1f s)" % (sampled, time.time() - t0))
    otables = orc.alias_build(xadj, w)
    assert same_tables(tables, otables)
    opaths, olengths, osampled = orc.walk_node2vec_reject(xadj, adjncy, otables[0], otables[1], p, q, seeds, L, 0.0, 4)
    assert sampled == osampled == int(olengths.sum())
    assert np.array_equal(lengths, olengths) and np.array_equal(paths, opaths)
    say("config 4: rejection identical (%.1f s)" % (time.time() - t0))
    del otables, tables
    opaths, olengths, osampled = orc.walk_online(xadj, adjncy, w, 1, p, q, seeds[:few], L, 0.0, 4)
    say("config 4: oracle table per step done (%.1f s)" % (time.time() - t0))
    assert tsampled == osampled and np.array_equal(tl, olengths) and np.array_equal(tp, opaths)
    g.free()
