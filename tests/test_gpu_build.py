"""Offline alias build on the GPU (through the C-ABI) against the CPU oracle: bit-exact tables,
and the reconstruction invariant on every row."""
import numpy as np
import pytest

from helpers import graph_from_degrees

pytestmark = pytest.mark.gpu
TOL = 1e-6

# degrees that straddle every dispatch class boundary of the build
EDGE_DEGREES = [0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 16, 17, 22, 23, 24, 25, 28, 29, 30, 32, 33, 46, 47, 48,
                49, 60, 61, 62, 63, 64, 65, 66, 67, 68, 94, 95, 96, 97, 124, 125, 126, 127, 190, 191, 192, 193, 253, 254, 255, 256, 257, 380, 381, 382, 383, 509, 510, 511, 764, 765, 766, 767, 1021,
                1022, 1023, 1024, 1025, 4093, 4094, 4095, 4096, 4097, 5116, 5117, 5118, 5119, 5120, 5121, 8189, 8190, 8191, 8192, 8193, 16380, 16381, 16382, 16383, 20000, 70001, 128, 129, 130, 144, 145, 159, 160, 161, 162, 34, 35, 36, 45]


def build_and_compare(orc, xadj, adjncy, w, label):
    from skywalker_amd import capi
    print("case", label, "V", len(xadj) - 1, "E", len(w), flush=True)
    oprob, oalias, ovalid = orc.alias_build(xadj, w)
    deg = np.diff(xadj)
    # rows of 8190..524287 entries: once through their own kernel, once (the default for so few of them)
    # through the tile-parallel path
    routes = (0, 4000000) if ((deg >= 8190) & (deg <= 524287)).any() else (4000000,)
    # rows of at most 32 entries: by degree class (the default below 2^25 rows), and by the kernel that walks the
    # vertices in order
    for stream_min_edges, small_in_place in [(r, 0) for r in routes] + [(routes[0], 1)]:
        g = capi.Graph.upload(xadj, adjncy, w)
        # knobs of this graph alone: nothing to restore, whatever happens below
        g.set_option("stream_min_edges", stream_min_edges)
        g.set_option("stream_wide_min_edges", stream_min_edges)  # 0: also the rows above 65533 entries are streamed
        g.set_option("small_in_place", small_in_place)
        g.build_tables()
        prob, alias, valid = g.tables()
        g.free()
        st = orc.alias_check(xadj, w, prob, alias, valid)
        assert st["bad_valid"] == 0 and st["bad_range"] == 0 and st["bad_invalid"] == 0, st
        assert st["max_rel_err"] < TOL, st
        bad = np.flatnonzero((prob != oprob) | (alias != oalias))
        if len(bad):
            v = int(np.searchsorted(xadj, bad[0], side="right") - 1)
            raise AssertionError("%s (stream_min_edges %d, small_in_place %d): %d entries differ from the oracle, first "
                                 "at slot %d (vertex %d, degree %d)" % (label, stream_min_edges, small_in_place, len(bad),
                                                                        bad[0], v, xadj[v + 1] - xadj[v]))
        assert np.array_equal(valid, ovalid)


@pytest.mark.parametrize("dist", ["lognormal", "uniform", "unit", "lognormal2", "equal", "nearequal", "sparse"])
def test_every_degree_class(orc, dist):
    rng = np.random.default_rng(11)
    degs = EDGE_DEGREES + list(rng.integers(1, 300, 400)) + list(rng.integers(300, 6000, 30))
    rng.shuffle(degs)
    xadj, adjncy, w = graph_from_degrees(degs, rng, dist, V=len(degs) + 7)
    build_and_compare(orc, xadj, adjncy, w, "classes/" + dist)


def test_class_kernels_over_side_streams_give_the_same_table(orc):
    # a build of 2 M .. 1 G entries spreads its class kernels over side streams; option build_streams = 0 keeps
    # them on the graph's stream
    from skywalker_amd import capi
    rng = np.random.default_rng(21)
    degs = EDGE_DEGREES[:60] + list(rng.integers(1, 300, 3000)) + list(rng.integers(300, 9000, 400)) + [30_000, 70_000, 600_000]
    rng.shuffle(degs)
    xadj, adjncy, w = graph_from_degrees(degs, rng, "lognormal")
    assert 2_000_000 <= len(w) < (1 << 30)
    for on in (0, 1):
        capi.set_option("build_streams", on)
        try:
            for rep in range(2):  # twice: the second build finds the side streams and their events in place
                build_and_compare(orc, xadj, adjncy, w, "side streams %d" % on)
        finally:
            capi.set_option("build_streams", 1)


def test_unaligned_row_starts(orc):
    # rows of every residue mod 4 in front of each LDS-class row
    rng = np.random.default_rng(5)
    degs = []
    for d in (70, 254, 700, 1021, 3000, 4093, 5117, 5118, 8000, 8189, 9000):
        for pad in (1, 2, 3, 5):
            degs += [pad, d]
    xadj, adjncy, w = graph_from_degrees(degs, rng, "lognormal")
    build_and_compare(orc, xadj, adjncy, w, "unaligned")


def test_all_zero_and_empty_rows(orc):
    rng = np.random.default_rng(2)
    degs = [0, 5, 0, 40, 100, 1, 2, 3000, 9000, 0]
    xadj, adjncy, w = graph_from_degrees(degs, rng, "uniform")
    for v in (1, 3, 4, 5, 6, 7, 8):
        if v % 2 == 1 or v == 8:
            w[xadj[v]:xadj[v + 1]] = 0.0
    build_and_compare(orc, xadj, adjncy, w, "zero rows")


def test_hub_row(orc):
    rng = np.random.default_rng(3)
    xadj, adjncy, w = graph_from_degrees([1_200_000, 3, 90_000], rng, "lognormal2", V=4096)
    build_and_compare(orc, xadj, adjncy, w, "hub")


def test_config1_rmat_s16(orc):
    xadj, adjncy = orc.rmat_csr(16, 16, 42)
    w = orc.gen_weights(orc.W_UNIFORM, 42, len(adjncy), 1.0, 100.0)
    build_and_compare(orc, xadj, adjncy, w, "config1")


def test_rebuild_is_idempotent(orc):
    from skywalker_amd import capi
    xadj, adjncy = orc.rmat_csr(12, 8, 9)
    w = orc.gen_weights(orc.W_UNIT, 9, len(adjncy))
    g = capi.Graph.upload(xadj, adjncy, w)
    g.build_tables()
    a = g.tables()
    g.build_tables()
    b = g.tables()
    g.free()
    for x, y in zip(a, b):
        assert np.array_equal(x, y)


@pytest.mark.parametrize("exact", [True, False])
def test_build_from_a_callers_weight_array(orc, exact):
    # sky_alias_build_from_weights with weights other than the graph's own: in device memory that ends with the
    # last of its E floats (E a multiple of 1024, ending in a short row whose 16-byte loads reach past the last
    # weight: the library copies such an array into a padded one), and in an array from sky_device_malloc, which
    # adds 16 bytes to every allocation (read where it lies)
    from skywalker_amd import capi
    import ctypes
    rng = np.random.default_rng(41)
    degs = list(rng.integers(1, 200, 300)) + [3000, 9000, 70, 33, 17]
    fill = (-sum(degs) - 5) % 1024
    degs += [fill, 5]
    xadj, adjncy, w = graph_from_degrees(degs, rng, "uniform")
    E = len(w)
    assert E % 1024 == 0 and xadj[-1] == E and xadj[len(degs)] - xadj[len(degs) - 1] == 5
    other = rng.lognormal(0, 2, E).astype(np.float32)
    g = capi.Graph.upload(xadj, adjncy, w)
    # the allocation holds 4 * (E + 8) + 16 bytes: 32 bytes in, exactly E floats are left
    dev = capi.DeviceArray(E + 8 if exact else E, np.float32)

    class View:
        ptr = ctypes.c_void_p(dev.ptr.value + 32) if exact else dev.ptr
    capi._ck(capi.lib().sky_memcpy_h2d(View.ptr, capi._p(other), E * 4))
    for rep in range(2):  # the second call finds the padded copy in place
        g.build_tables_from_weights(View)
        prob, alias, valid = g.tables()
        oprob, oalias, ovalid = orc.alias_build(xadj, other)
        assert np.array_equal(prob, oprob) and np.array_equal(alias, oalias) and np.array_equal(valid, ovalid)
    assert np.array_equal(g.download()[2], w)  # the graph's own weights are left as they are
    g.build_tables()
    prob, alias, valid = g.tables()
    oprob, oalias, ovalid = orc.alias_build(xadj, w)
    assert np.array_equal(prob, oprob) and np.array_equal(alias, oalias) and np.array_equal(valid, ovalid)
    dev.free()
    g.free()


def test_bad_arguments_are_reported(orc):
    from skywalker_amd import capi
    xadj = np.array([0, 2, 1], np.uint32)  # not monotone
    with pytest.raises(capi.SkyError):
        capi.Graph.upload(xadj, np.zeros(1, np.uint32), np.ones(1, np.float32))
    xadj = np.array([0, 1], np.uint32)
    with pytest.raises(capi.SkyError):
        capi.Graph.upload(xadj, np.array([5], np.uint32), np.ones(1, np.float32))  # neighbour out of range
    g = capi.Graph.upload(np.array([0, 1, 1], np.uint32), np.array([1], np.uint32), np.ones(1, np.float32))
    with pytest.raises(capi.SkyError):
        g.walk_offline(np.array([0], np.uint32), 4, 0.0, 1)  # tables not built
    g.free()


@pytest.mark.parametrize("dist", ["lognormal2", "nearequal", "sparse", "fewlights", "fewheavies"])
def test_rows_built_tile_by_tile(orc, dist):
    # rows beyond one workgroup's LDS: 8 to 320 tiles, starts of every alignment
    from helpers import weights
    rng = np.random.default_rng(21)
    degs = [4094, 4097, 7, 5121, 8190, 1, 8193, 2, 12288, 3, 12289, 40000, 5, 100001, 330000]
    xadj, adjncy, w = graph_from_degrees(degs, rng, "lognormal", V=4096)
    if dist == "fewlights":      # almost every entry barely heavy, 1 % very light: a light tile spans many partners
        w = np.where(rng.random(len(w)) < 0.01, 0.01, 1.01).astype(np.float32)
    elif dist == "fewheavies":   # 0.1 % of the entries carry almost all the mass
        w = np.where(rng.random(len(w)) < 0.001, 1000.0, 0.5).astype(np.float32)
    else:
        w = weights(len(w), rng, dist)
    build_and_compare(orc, xadj, adjncy, w, "tiled/" + dist)


def test_streaming_kernel_for_rows_with_too_many_tiles(orc):
    from skywalker_amd import capi
    rng = np.random.default_rng(22)
    xadj, adjncy, w = graph_from_degrees([4100, 9000, 20000, 3, 70000], rng, "lognormal2", V=4096)
    capi.set_option("tiled_max_tiles", 10)  # up to 9000 (9 tiles) stays tile-parallel, the other two are streamed
    try:
        build_and_compare(orc, xadj, adjncy, w, "streaming")
    finally:
        capi.set_option("tiled_max_tiles", 1 << 22)


def test_search_variant_of_the_row_kernels_gives_the_same_table(orc):
    # "row_merge" = 0 selects the kernels that do one binary search per entry (rows of 62..4093 entries) and
    # sends rows of 4094..5117 entries down the tile-parallel path (longer ones stream or go tile by tile anyway)
    from skywalker_amd import capi
    rng = np.random.default_rng(23)
    degs = [70, 126, 254, 300, 509, 510, 1021, 1500, 2046, 3000, 4093, 4094, 5000, 8189, 8190, 3, 0, 1]
    xadj, adjncy, w = graph_from_degrees(degs, rng, "lognormal", V=8192)
    capi.set_option("row_merge", 0)
    try:
        build_and_compare(orc, xadj, adjncy, w, "row_merge=0")
    finally:
        capi.set_option("row_merge", 1)
    build_and_compare(orc, xadj, adjncy, w, "row_merge=1")


@pytest.mark.parametrize("dist", ["lognormal2", "uniform", "nearequal", "sparse", "fewlights", "fewheavies"])
def test_rows_streamed_by_one_workgroup(orc, dist):
    # rows of 5118..8189 entries are held by one workgroup, its heavies listed in LDS (5632 at a time), rows of
    # 8190..524287 entries stream through one with a window of 5080 heavies ("fewlights" has rows with several lists
    # or windows, "uniform" too among the streamed ones, "nearequal" rows without a heavy); 524288 is the first degree
    # of the tile-parallel class
    from helpers import weights
    rng = np.random.default_rng(31)
    degs = [5118, 5119, 6000, 8189, 8190, 8191, 7, 8193, 12288, 2, 12289, 16381, 16382, 16385, 1, 30000, 65533, 65534, 0, 9001, 150001, 524287, 524288]
    xadj, adjncy, w = graph_from_degrees(degs, rng, "lognormal", V=4096)
    if dist == "fewlights":
        w = np.where(rng.random(len(w)) < 0.01, 0.01, 1.01).astype(np.float32)
    elif dist == "fewheavies":
        w = np.where(rng.random(len(w)) < 0.001, 1000.0, 0.5).astype(np.float32)
    else:
        w = weights(len(w), rng, dist)
    build_and_compare(orc, xadj, adjncy, w, "stream/" + dist)


def test_special_weight_values_in_every_kind_of_row(orc):
    # NaN, infinities, negatives, -0, denormals, values at and beyond the 2^32 clamp, and values whose
    # contribution to the exact sum is only a few units of 2^-64: same bits as the oracle in every class
    rng = np.random.default_rng(41)
    degs = [1, 2, 3, 5, 9, 20, 40, 100, 150, 200, 400, 700, 1500, 3000, 5000, 6000, 8189, 9000, 20000, 70000]
    xadj, adjncy, w = graph_from_degrees(degs, rng, "lognormal", V=4096)
    special = np.array([np.nan, np.inf, -np.inf, -1.0, -0.0, 0.0, 1e-45, 1e-40, 2.0 ** -64, 2.0 ** -63, 3e-19,
                        2.0 ** 32, 2.0 ** 32 * 1.5, 3e38, 2.0 ** -20, 1.0, 123456.789], np.float32)
    pick = rng.random(len(w)) < 0.3
    w[pick] = special[rng.integers(0, len(special), pick.sum())]
    with np.errstate(all="ignore"):
        build_and_compare(orc, xadj, adjncy, w, "special values")
    # rows made of nothing but contributions that vanish: invalid rows in every class
    w2 = np.where(rng.random(len(w)) < 0.5, np.float32(1e-30), np.float32(-3.0)).astype(np.float32)
    build_and_compare(orc, xadj, adjncy, w2, "all-vanishing rows")


def test_build_profile_is_opt_in(orc):
    # without the option one bracket spans the build; with it every launched class has its own entry
    from skywalker_amd import capi
    g = capi.Graph.rmat(14, 16, 3, capi.W_UNIFORM, 1.0, 100.0, 3)
    sec = g.build_tables()
    prof = g.build_profile()
    assert [p[0] for p in prof] == ["build"] and prof[0][2] == g.E
    assert abs(prof[0][1] * 1e-3 - sec) < 1e-6
    before = g.tables()
    capi.set_option("build_profile", 1)
    try:
        sec = g.build_tables()
    finally:
        capi.set_option("build_profile", 0)
    prof = g.build_profile()
    assert prof[0][0] == "bin" and len(prof) > 3
    assert abs(sum(p[1] for p in prof) * 1e-3 - sec) < 1e-5  # the brackets tile the build
    after = g.tables()
    g.free()
    for a, b in zip(before, after):
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8))


def test_degenerate_inputs(orc):
    # a graph without edges, a graph without vertices, no walkers, zero steps: every entry point returns
    # cleanly and the counts are zero
    from skywalker_amd import capi
    for V in (0, 1, 300):
        xadj = np.zeros(V + 1, np.uint32)
        g = capi.Graph.upload(xadj, np.zeros(0, np.uint32), np.zeros(0, np.float32))
        assert g.V == V and g.E == 0
        g.build_tables()
        prob, alias, valid = g.tables()
        assert len(prob) == 0 and len(alias) == 0 and len(valid) == V and not valid.any()
        seeds = np.arange(min(V, 5), dtype=np.uint32)
        for length in (0, 4):
            p, l, sampled, _ = g.walk_offline(seeds, length, 0.0, 1)
            assert sampled == 0 and not l.to_host().any()
            assert np.array_equal(p.to_host((len(seeds), length + 1))[:, 0], seeds)
            p, l, sampled, _ = g.walk_online(capi.BIAS_STATIC, 1.0, 1.0, seeds, length, 0.0, 1)
            assert sampled == 0 and not l.to_host().any()
            p, l, sampled, _ = g.walk_online(capi.BIAS_NODE2VEC_REJECT, 2.0, 0.5, seeds, length, 0.0, 1)
            assert sampled == 0 and not l.to_host().any()
        d, sl, sampled, _ = g.sample_offline(seeds, [1, 3, 2], 1)
        assert sampled == 0 and not sl.to_host().any()
        d, sl, sampled, _ = g.sample_online(seeds, [1, 3, 2], 1)
        assert sampled == 0 and not sl.to_host().any()
        g.free()
    # an ordinary graph, no walkers
    xadj, adjncy = orc.rmat_csr(8, 4, 1)
    g = capi.Graph.upload(xadj, adjncy, None)  # unit weights
    g.build_tables()
    none = np.zeros(0, np.uint32)
    assert g.walk_offline(none, 5, 0.0, 1)[2] == 0
    assert g.walk_online(capi.BIAS_NODE2VEC, 2.0, 0.5, none, 5, 0.0, 1)[2] == 0
    assert g.sample_offline(none, [1, 2], 1)[2] == 0
    g.free()


@pytest.mark.parametrize("seed", range(8))
def test_random_mixtures_of_every_class(orc, seed):
    # both ends of every degree class plus random rows of every size, a different weight law per seed,
    # special values sprinkled into some
    from helpers import weights
    rng = np.random.default_rng(1000 + seed)
    ends = [0, 1, 2, 3, 5, 6, 8, 9, 13, 14, 16, 17, 29, 30, 32, 33, 61, 62, 64, 65, 125, 126, 128, 129, 191, 192, 193, 253, 254,
            381, 382, 509, 510, 765, 766, 5117, 5118, 8189, 8190, 16381, 16382, 24576, 24577, 65533, 65534]
    for nw in range(2, 11):
        ends += [512 * (nw - 1) - 2, 512 * nw - 3]
    degs = ends + list(rng.integers(0, 70, 3000)) + list(rng.integers(60, 600, 600)) + \
        list(rng.integers(500, 8300, 260)) + list(rng.integers(8000, 66000, 12)) + list(rng.integers(66000, 400000, 2))
    degs = np.array(degs)
    rng.shuffle(degs)
    xadj = np.zeros(len(degs) + 1, np.uint32)
    xadj[1:] = np.cumsum(degs)
    E = int(xadj[-1])
    adjncy = rng.integers(0, len(degs), E).astype(np.uint32)
    dist = ["lognormal", "uniform", "lognormal2", "nearequal", "sparse", "unit", "equal"][seed % 7]
    w = weights(E, rng, dist)
    if seed % 3 == 0:
        pick = rng.random(E) < 0.001
        special = np.array([0.0, -1.0, np.inf, np.nan, 1e-30, 2.0 ** -64, 2.0 ** 32, 1e38], np.float32)
        w[pick] = special[rng.integers(0, len(special), pick.sum())]
    with np.errstate(all="ignore"):
        build_and_compare(orc, xadj, adjncy, w, "mixture %d/%s" % (seed, dist))


def test_two_graphs_hold_different_settings(orc):
    # a knob set on one graph (sky_graph_set_option) leaves the other graph and the process-wide value alone
    from skywalker_amd import capi
    rng = np.random.default_rng(51)
    xadj, adjncy, w = graph_from_degrees(list(rng.integers(1, 200, 500)) + [300, 2000], rng, "lognormal")
    a = capi.Graph.upload(xadj, adjncy, w)
    b = capi.Graph.upload(xadj, adjncy, w)
    a.set_option("build_profile", 1)
    a.build_tables()
    b.build_tables()
    assert len(a.build_profile()) > 3 and [p[0] for p in b.build_profile()] == ["build"]
    c = capi.Graph.upload(xadj, adjncy, w)
    c.build_tables()
    assert [p[0] for p in c.build_profile()] == ["build"]  # the process-wide value did not move
    a.set_option("build_profile", None)
    a.build_tables()
    assert [p[0] for p in a.build_profile()] == ["build"]
    with pytest.raises(capi.SkyError):
        a.set_option("no_such_knob", 1)
    with pytest.raises(capi.SkyError):
        a.set_option("small_in_place", 7)
    want = a.tables()[0]
    for g in (a, b, c):
        assert np.array_equal(g.tables()[0], want)
        g.free()


def test_device_addresses_of_the_resident_arrays(orc):
    # sky_graph_device_ptrs: what lies at the addresses is what sky_graph_download and sky_alias_download give
    from skywalker_amd import capi
    import ctypes
    xadj, adjncy = orc.rmat_csr(10, 8, 5)
    w = orc.gen_weights(orc.W_UNIFORM, 5, len(adjncy), 1.0, 100.0)
    g = capi.Graph.upload(xadj, adjncy, w)
    g.build_tables()
    prob, alias, valid = g.tables()
    px, pa, pw, pt, pv = g.device_ptrs()
    assert px and pa and pw and pt and pv

    def read(addr, count, dtype):
        out = np.empty(count, dtype)
        capi._ck(capi.lib().sky_memcpy_d2h(capi._p(out), ctypes.c_void_p(addr), ctypes.c_size_t(out.nbytes)))
        return out
    assert np.array_equal(read(px, len(xadj), np.uint32), xadj)
    assert np.array_equal(read(pa, len(adjncy), np.uint32), adjncy)
    assert np.array_equal(read(pw, len(w), np.float32), w)
    entries = read(pt, 2 * len(w), np.uint32).reshape(-1, 2)  # {float prob; uint32 alias} per slot
    assert np.array_equal(entries[:, 0].view(np.float32), prob) and np.array_equal(entries[:, 1], alias)
    assert np.array_equal(read(pv, len(xadj) - 1, np.int8), valid)
    g.free()
