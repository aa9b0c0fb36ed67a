"""The largest configuration (R-MAT scale 26, edge factor 28, lognormal(0, 2) weights; 1.88 G edges) on the GPU
against the oracle on the host: tables bit for bit and through the reconstruction invariant, 1 M DeepWalk and
PPR walkers bit for bit.  About 45 GB of host memory and a minute of host time."""
import time

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

SCALE, EF, SEED = 26, 28, 5


def say(*a):
    print(*a, flush=True)


def test_scale26_tables_and_walks_match_the_oracle(orc):
    from skywalker_amd import capi
    t0 = time.time()
    g = capi.Graph.rmat(SCALE, EF, SEED, capi.W_LOGNORMAL, 0.0, 2.0, SEED)
    assert g.V == 1 << SCALE and g.E == EF << SCALE
    sec = g.build_tables()
    say("generated and built: V %d E %d, build %.2f ms (%.1f s so far)" % (g.V, g.E, sec * 1e3, time.time() - t0))
    xadj, adjncy, w = g.download()
    prob, alias, valid = g.tables()
    say("downloaded (%.1f s)" % (time.time() - t0))

    # size-independent property: every row's table reproduces its normalised weights
    st = orc.alias_check(xadj, w, prob, alias, valid)
    say("reconstruction:", st, "(%.1f s)" % (time.time() - t0))
    assert st["bad_valid"] == 0 and st["bad_range"] == 0 and st["bad_invalid"] == 0
    assert st["max_rel_err"] < 1e-6  # the tolerance the tables are specified to

    # and the same bits as the oracle's sequential sweep
    oprob, oalias, ovalid = orc.alias_build(xadj, w)
    say("oracle build done (%.1f s)" % (time.time() - t0))
    assert np.array_equal(valid, ovalid)
    step = 1 << 27
    for lo in range(0, g.E, step):
        hi = min(g.E, lo + step)
        assert np.array_equal(prob[lo:hi].view(np.uint32), oprob[lo:hi].view(np.uint32)), "prob differs in [%d, %d)" % (lo, hi)
        assert np.array_equal(alias[lo:hi], oalias[lo:hi]), "alias differs in [%d, %d)" % (lo, hi)
    del oprob, oalias, w
    say("tables identical (%.1f s)" % (time.time() - t0))

    # 1 M walkers: DeepWalk of length 80, and PPR with stop probability 0.15 and at most 100 steps
    N = 1_000_000
    seeds_d = g.gen_seeds(SEED, N)
    seeds = seeds_d.to_host()
    assert np.array_equal(seeds, orc.gen_seeds(SEED, g.V, N))
    for length, stop in ((80, 0.0), (100, 0.15)):
        paths_d, lengths_d, sampled, _ = g.walk_offline(seeds_d, length, stop, SEED)
        paths, lengths = paths_d.to_host((N, length + 1)), lengths_d.to_host()
        paths_d.free()
        lengths_d.free()
        opaths, olengths, osampled = orc.walk_offline(xadj, adjncy, prob, alias, seeds, length, stop, SEED)
        assert sampled == osampled == int(lengths.sum())
        assert np.array_equal(lengths, olengths)
        assert np.array_equal(paths, opaths)
        say("walk length %d stop %.2f: %d steps identical (%.1f s)" % (length, stop, sampled, time.time() - t0))
    g.free()
