"""The allocation-free walk entry point against sky_walk_offline: same paths, lengths and count."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_noalloc_walk_equals_walk_offline_twice_in_a_row(orc):
    from skywalker_amd import capi
    xadj, adjncy = orc.rmat_csr(14, 16, 5)
    w = orc.gen_weights(orc.W_LOGNORMAL, 5, len(adjncy), 0.0, 1.0)
    g = capi.Graph.upload(xadj, adjncy, w)
    g.build_tables()
    V = len(xadj) - 1
    # the second call is smaller than the first: stale per-workgroup counts of the first call must not be added
    for N, length, stop, seed in ((70001, 40, 0.0, 11), (999, 25, 0.15, 12)):
        seeds = g.gen_seeds(seed, N)
        want_paths, want_len, want_sampled, _ = g.walk_offline(seeds, length, stop, seed)
        paths = capi.DeviceArray(N * (length + 1), np.uint32, fill=capi.FILL)
        lengths = capi.DeviceArray(N, np.uint32, fill=0)
        sampled = capi.DeviceArray(1, np.uint64)
        g.walk_offline_noalloc(seeds, length, stop, seed, paths, lengths, sampled)
        capi.synchronize()
        assert np.array_equal(paths.to_host(), want_paths.to_host())
        assert np.array_equal(lengths.to_host(), want_len.to_host())
        assert int(sampled.to_host()[0]) == want_sampled == int(want_len.to_host().sum())
        opaths, olen, osampled = orc.walk_offline(xadj, adjncy, *g.tables()[:2], seeds.to_host(), length, stop, seed)
        assert np.array_equal(paths.to_host((N, length + 1)), opaths) and osampled == want_sampled
    g.free()


def test_noalloc_walk_leaves_device_memory_as_it_found_it(orc):
    # a graph whose pooled buffers are still empty: a call that allocated a counter, a list or an event pool would
    # show up as a change of the free device memory the runtime reports
    from skywalker_amd import capi
    xadj, adjncy = orc.rmat_csr(12, 8, 6)
    w = orc.gen_weights(orc.W_UNIFORM, 6, len(adjncy), 1.0, 100.0)
    g = capi.Graph.upload(xadj, adjncy, w)
    g.build_tables()
    N, length = 300001, 20  # outputs of 25 MB: far above the granularity of the report
    seeds = g.gen_seeds(3, N)
    paths = capi.DeviceArray(N * (length + 1), np.uint32, fill=capi.FILL)
    lengths = capi.DeviceArray(N, np.uint32, fill=0)
    sampled = capi.DeviceArray(1, np.uint64)
    g.walk_offline_noalloc(seeds, length, 0.0, 3, paths, lengths, sampled)  # first call on this device: looks up the array
    capi.synchronize()
    free0, _ = capi.mem_info()
    for _ in range(3):
        g.walk_offline_noalloc(seeds, length, 0.0, 3, paths, lengths, sampled)
    free1, _ = capi.mem_info()
    capi.synchronize()
    free2, _ = capi.mem_info()
    assert free0 == free1 == free2
    opaths, olen, osampled = orc.walk_offline(xadj, adjncy, *g.tables()[:2], seeds.to_host(), length, 0.0, 3)
    assert np.array_equal(paths.to_host((N, length + 1)), opaths) and int(sampled.to_host()[0]) == osampled
    g.free()


def test_noalloc_walk_rejects_batches_beyond_its_scratch(orc):
    from skywalker_amd import capi
    xadj = np.array([0, 1, 2], np.uint32)
    g = capi.Graph.upload(xadj, np.array([1, 0], np.uint32), np.ones(2, np.float32))
    g.build_tables()
    N = 4194304 + 1
    seeds = capi.DeviceArray(N, np.uint32, fill=0)
    paths = capi.DeviceArray(N * 2, np.uint32)
    lengths = capi.DeviceArray(N, np.uint32)
    with pytest.raises(capi.SkyError) as e:
        g.walk_offline_noalloc(seeds, 1, 0.0, 1, paths, lengths, None)
    assert e.value.code == -5 and "4194304" in str(e.value)
    g.free()
