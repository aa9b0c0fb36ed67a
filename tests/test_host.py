"""Host-side logic of the drop-in surface: the gflags-compatible parser and the Galois .gr reader
(CPU only), and the `skywalker` command line end to end (GPU)."""
import os
import re
import struct
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "skywalker_amd", "host")


def write_gr(path, xadj, adjncy, weights_u32=None):
    """Galois .gr v1: header, V row-end offsets (u64), E destinations (u32), pad, E weights (u32)."""
    V, E = len(xadj) - 1, len(adjncy)
    with open(path, "wb") as f:
        f.write(struct.pack("<4Q", 1, 0 if weights_u32 is None else 4, V, E))
        f.write(np.asarray(xadj[1:], np.uint64).tobytes())
        f.write(np.asarray(adjncy, np.uint32).tobytes())
        if weights_u32 is not None:
            if E % 2:
                f.write(b"\0\0\0\0")
            f.write(np.asarray(weights_u32, np.uint32).tobytes())


def run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=120)
    return r.returncode, r.stdout, r.stderr


def test_flag_forms():
    tool = os.path.join(HOST, "gr_tool")
    rc, out, _ = run([tool, "flags", "--input=/x/y.gr", "-n", "40000", "--tp", "0.15", "--ol=1", "--nobias", "-v"])
    assert rc == 0 and out.strip() == "input=/x/y.gr n=40000 tp=0.15 ol=1 bias=0 v=1"
    rc, out, _ = run([tool, "flags", "--ol", "--bias=false", "-n=7"])
    assert rc == 0 and "n=7" in out and "ol=1" in out and "bias=0" in out
    rc, _, err = run([tool, "flags", "--nosuchflag"])
    assert rc == 1 and "unknown command line flag" in err
    rc, _, err = run([tool, "flags", "-n", "abc"])
    assert rc == 1 and "illegal value" in err


@pytest.mark.parametrize("odd", [False, True])
def test_gr_reader_round_trip(tmp_path, orc, odd):
    xadj, adjncy = orc.rmat_csr(8, 5, 3)
    if odd:  # an odd edge count exercises the 4-byte pad in front of the weights
        adjncy = adjncy[:-1]
        xadj = np.minimum(xadj, len(adjncy)).astype(np.uint32)
    w = (np.arange(len(adjncy)) % 97 + 1).astype(np.uint32)
    p = str(tmp_path / "g.w.gr")
    write_gr(p, xadj, adjncy, w)
    rc, out, _ = run([os.path.join(HOST, "gr_tool"), "info", p])
    assert rc == 0
    V, E, md, sa, sw = out.split()[-5:]
    assert int(V) == len(xadj) - 1 and int(E) == len(adjncy)
    assert int(md) == int(np.diff(xadj.astype(np.int64)).max())
    assert int(sa) == int(adjncy.astype(np.int64).sum()) and float(sw) == float(w.sum())


@pytest.mark.gpu
def test_cli_offline_deepwalk_matches_oracle(tmp_path, orc):
    xadj, adjncy = orc.rmat_csr(12, 8, 11)
    w = (orc.gen_weights(orc.W_UNIFORM, 11, len(adjncy), 1.0, 100.0)).astype(np.uint32)
    p = str(tmp_path / "rmat12.w.gr")
    write_gr(p, xadj, adjncy, w)
    rc, out, err = run([os.path.join(HOST, "skywalker"), "--deepwalk", "--bias=1", "--ol=0", "--input", p, "-n", "600",
                        "--d", "20", "--printresult", "--seed", "5"])
    assert rc == 0, err
    lines = out.splitlines()
    assert lines[0] == "rmat12.w.gr"
    prob, alias, valid = orc.alias_build(xadj, w.astype(np.float32))
    seeds = np.arange(600, dtype=np.uint32)
    paths, lengths, sampled = orc.walk_offline(xadj, adjncy, prob, alias, seeds, 20, 0.0, 5)
    for j in range(3):
        i = lines.index("%drd path len %d " % (j, lengths[j]))
        got = [int(x) for x in lines[i + 1].split()]
        assert got == paths[j, :min(lengths[j], 21)].tolist()
    # last three lines: table ms, sample ms, MSEPS (src/main.cu:406-419)
    table_ms, sample_ms, mseps = (float(l.strip()) for l in lines[-3:])
    assert table_ms > 0 and sample_ms > 0
    assert abs(mseps - sampled / (sample_ms * 1e-3) / 1e6) <= 0.02 * mseps + 0.02


@pytest.mark.gpu
def test_cli_saved_tables_give_the_same_walks(tmp_path, orc):
    xadj, adjncy = orc.rmat_csr(11, 8, 5)
    w = (orc.gen_weights(orc.W_UNIFORM, 5, len(adjncy), 1.0, 100.0)).astype(np.uint32)
    p, t = str(tmp_path / "t.w.gr"), str(tmp_path / "t.tbl")
    write_gr(p, xadj, adjncy, w)
    common = [os.path.join(HOST, "skywalker"), "--deepwalk", "--bias=1", "--ol=0", "--input", p, "-n", "300", "--d", "10",
              "--printresult", "--seed", "6"]
    rc, out1, err = run(common + ["--savetable", t])
    assert rc == 0, err
    raw = open(t, "rb").read()
    V, E = len(xadj) - 1, len(adjncy)
    assert raw[:8] == b"SKYTBL02" and struct.unpack("<2Q", raw[8:24]) == (V, E) and len(raw) == 32 + 8 * E + V
    prob, alias, valid = orc.alias_build(xadj, w.astype(np.float32))
    assert np.array_equal(np.frombuffer(raw, np.float32, E, 32).view(np.uint32), prob.view(np.uint32))
    assert np.array_equal(np.frombuffer(raw, np.uint32, E, 32 + 4 * E), alias)
    rc, out2, err = run(common + ["--loadtable", t])
    assert rc == 0, err
    keep = lambda o: [l for l in o.splitlines() if l.strip()][:-3]  # everything but the timing lines
    assert keep(out1)[1:] == keep(out2)[1:] and len(keep(out1)) >= 7
    rc, _, err = run(common + ["--loadtable", p])  # not a table file
    assert rc != 0 and "cannot use table file" in err
    # a damaged file: one alias points outside its row.  The library refuses the arrays, nothing walks on them.
    row = int(np.argmax(np.diff(xadj.astype(np.int64)) >= 3))
    bad = bytearray(raw)
    struct.pack_into("<I", bad, 32 + 4 * E + 4 * int(xadj[row]), 0x7FFFFFFF)
    open(t + ".bad", "wb").write(bytes(bad))
    rc, _, err = run(common + ["--loadtable", t + ".bad"])
    assert rc != 0 and "cannot use table file" in err and "alias of slot %d" % xadj[row] in err
    # the tables of another graph with the same V and E (every R-MAT graph of one scale and edge factor has them)
    xadj2, adjncy2 = orc.rmat_csr(11, 8, 6)
    p2 = str(tmp_path / "t2.w.gr")
    write_gr(p2, xadj2, adjncy2, w)
    rc, _, err = run([common[0], "--deepwalk", "--bias=1", "--ol=0", "--input", p2, "-n", "10", "--d", "3",
                      "--loadtable", t])
    assert rc != 0 and "cannot use table file" in err


@pytest.mark.gpu
def test_alias_upload_checks_the_arrays(orc):
    from skywalker_amd import capi
    xadj = np.array([0, 3, 3, 5], np.uint32)
    adjncy = np.array([1, 2, 2, 0, 1], np.uint32)
    w = np.array([1, 2, 3, 0, 0], np.float32)
    g = capi.Graph.upload(xadj, adjncy, w)
    prob, alias, valid = orc.alias_build(xadj, w)
    assert valid.tolist() == [1, 0, 0] and alias[3] == capi.INVALID
    g.upload_tables(prob, alias, valid)  # the oracle's own table passes
    cases = []
    a = alias.copy(); a[1] = 3; cases.append((prob, a, valid, "alias of slot 1"))
    a = alias.copy(); a[3] = 0; cases.append((prob, a, valid, "alias of slot 3"))      # invalid row must hold SKY_INVALID
    a = alias.copy(); a[0] = capi.INVALID; cases.append((prob, a, valid, "alias of slot 0"))
    p = prob.copy(); p[2] = np.nan; cases.append((p, alias, valid, "prob of slot 2"))
    p = prob.copy(); p[0] = 1.5; cases.append((p, alias, valid, "prob of slot 0"))
    p = prob.copy(); p[0] = -0.25; cases.append((p, alias, valid, "prob of slot 0"))
    v = valid.copy(); v[1] = 1; cases.append((prob, alias, v, "no edge"))
    v = valid.copy(); v[0] = 2; cases.append((prob, alias, v, "neither 0 nor 1"))
    for pp, aa, vv, msg in cases:
        with pytest.raises(capi.SkyError) as e:
            g.upload_tables(pp, aa, vv)
        assert e.value.code == -1 and msg in str(e.value), (msg, str(e.value))
    got = g.tables()  # the graph still holds the last good tables
    assert np.array_equal(got[0], prob) and np.array_equal(got[1], alias) and np.array_equal(got[2], valid)
    g.free()


@pytest.mark.gpu
def test_cli_unbiased_walk_is_the_unit_weight_walk(tmp_path, orc):
    # --bias=0 ignores the weights of the file: uniform neighbour choice through the same tables
    xadj, adjncy = orc.rmat_csr(11, 8, 3)
    w = (orc.gen_weights(orc.W_UNIFORM, 3, len(adjncy), 1.0, 100.0)).astype(np.uint32)
    p = str(tmp_path / "u.w.gr")
    write_gr(p, xadj, adjncy, w)
    rc, out, err = run([os.path.join(HOST, "skywalker"), "--deepwalk", "--bias=0", "--ol=0", "--input", p, "-n", "500",
                        "--d", "12", "--printresult", "--seed", "4"])
    assert rc == 0, err
    lines = out.splitlines()
    prob, alias, valid = orc.alias_build(xadj, np.ones(len(adjncy), np.float32))
    paths, lengths, sampled = orc.walk_offline(xadj, adjncy, prob, alias, np.arange(500, dtype=np.uint32), 12, 0.0, 4)
    for j in range(3):
        i = lines.index("%drd path len %d " % (j, lengths[j]))
        assert [int(x) for x in lines[i + 1].split()] == paths[j, :min(lengths[j], 13)].tolist()


@pytest.mark.gpu
@pytest.mark.parametrize("table", [False, True])
def test_cli_node2vec_matches_oracle(tmp_path, orc, table):
    # --node2vec runs the rejection sampler on the first-order tables; --n2v_table the table per step
    xadj, adjncy = orc.rmat_csr(11, 8, 7)
    w = (orc.gen_weights(orc.W_UNIFORM, 7, len(adjncy), 1.0, 100.0)).astype(np.uint32)
    p = str(tmp_path / "n2v.w.gr")
    write_gr(p, xadj, adjncy, w)
    cmd = [os.path.join(HOST, "skywalker"), "--node2vec", "--bias=1", "--input", p, "-n", "400", "--d", "15", "--p", "2",
           "--q", "0.5", "--printresult", "--seed", "9"]
    rc, out, err = run(cmd + (["--n2v_table"] if table else []))
    assert rc == 0, err
    lines = out.splitlines()
    seeds = np.arange(400, dtype=np.uint32)
    wf = w.astype(np.float32)
    if table:
        paths, lengths, sampled = orc.walk_online(xadj, adjncy, wf, 1, 2.0, 0.5, seeds, 15, 0.0, 9)
    else:
        prob, alias, valid = orc.alias_build(xadj, wf)
        paths, lengths, sampled = orc.walk_node2vec_reject(xadj, adjncy, prob, alias, 2.0, 0.5, seeds, 15, 0.0, 9)
    for j in range(3):
        i = lines.index("%drd path len %d " % (j, lengths[j]))
        got = [int(x) for x in lines[i + 1].split()]
        assert got == paths[j, :min(lengths[j], 16)].tolist()
    sample_ms, mseps = (float(l.strip()) for l in lines[-2:])
    assert abs(mseps - sampled / (sample_ms * 1e-3) / 1e6) <= 0.02 * mseps + 0.02


@pytest.mark.gpu
def test_cli_online_sage_and_csv(tmp_path, orc):
    xadj, adjncy = orc.rmat_csr(11, 8, 2)
    w = (orc.gen_weights(orc.W_UNIFORM, 2, len(adjncy), 1.0, 100.0)).astype(np.uint32)
    p = str(tmp_path / "s.w.gr")
    write_gr(p, xadj, adjncy, w)
    rc, out, err = run([os.path.join(HOST, "skywalker"), "--sage", "--bias=1", "--ol=1", "--input", p, "-n", "300",
                        "--csv", "--printresult"])
    assert rc == 0, err
    data, sl, sampled = orc.sample_online(xadj, adjncy, w.astype(np.float32), np.arange(300, dtype=np.uint32),
                                          [1, 25, 10], 0)
    m = re.search(r"0th sample src: (\d+), 1-hop len: (\d+)", out)
    assert m and int(m.group(1)) == 0 and int(m.group(2)) == sl[0, 0]
    hop1 = [int(x) for x in out.split("1-hop : ")[1].splitlines()[0].split()]
    assert hop1 == data[0, 1:1 + sl[0, 0]].tolist()
    last = out.strip().splitlines()[-1]
    assert last.startswith("s.w.gr,") or re.match(r"^[\d.]+,\t[\d.]+,$", last)


@pytest.mark.gpu
@pytest.mark.parametrize("online", [0, 1])
def test_cli_unbiased_two_hop_sampling(tmp_path, orc, online):
    # --bias=0 --sage: the reference's unbiased k-hop sampler (src/unbiased_sample.cu:10-316) = unit weights here
    xadj, adjncy = orc.rmat_csr(11, 8, 21)
    w = (orc.gen_weights(orc.W_UNIFORM, 21, len(adjncy), 1.0, 100.0)).astype(np.uint32)
    p = str(tmp_path / "us.w.gr")
    write_gr(p, xadj, adjncy, w)
    rc, out, err = run([os.path.join(HOST, "skywalker"), "--sage", "--bias=0", "--ol=%d" % online, "--input", p, "-n", "300",
                        "--printresult", "--seed", "3"])
    assert rc == 0, err
    ones = np.ones(len(adjncy), np.float32)
    data, sl, sampled = orc.sample_online(xadj, adjncy, ones, np.arange(300, dtype=np.uint32), [1, 25, 10], 3)
    blocks = out.split("th sample src: ")[1:]
    assert len(blocks) == 4
    for j, blk in enumerate(blocks):
        m = re.match(r"(\d+), 1-hop len: (\d+)", blk)
        assert int(m.group(1)) == j and int(m.group(2)) == sl[j, 0]
        hop1 = [int(x) for x in blk.split("1-hop : ")[1].splitlines()[0].split()]
        assert hop1 == data[j, 1:1 + sl[j, 0]].tolist()
        for i in range(sl[j, 0]):
            line = blk.split("\t %d th 2-hop [%d]: " % (i, data[j, 1 + i]))[1].splitlines()[0]
            assert [int(x) for x in line.split()] == data[j, 26 + 10 * i:26 + 10 * i + min(sl[j, 1 + i], 30)].tolist()
    lines = [l for l in out.splitlines() if l.strip()]
    sample_ms, mseps = float(lines[-2]), float(lines[-1])  # no table line for an unbiased run (main.cu:406)
    assert abs(mseps - sampled / (sample_ms * 1e-3) / 1e6) <= 0.02 * mseps + 0.02


@pytest.mark.gpu
def test_cli_two_hop_sampling_without_replacement(tmp_path, orc):
    # --replace=0: every parent's children are distinct slots of its row, as in the reference's online sampler
    xadj, adjncy = orc.rmat_csr(11, 16, 25)
    w = (orc.gen_weights(orc.W_UNIFORM, 25, len(adjncy), 1.0, 100.0)).astype(np.uint32)
    p = str(tmp_path / "nr.w.gr")
    write_gr(p, xadj, adjncy, w)
    rc, out, err = run([os.path.join(HOST, "skywalker"), "--sage", "--bias=1", "--ol=1", "--replace=0", "--input", p, "-n", "300",
                        "--printresult", "--seed", "6"])
    assert rc == 0, err
    data, sl, sampled = orc.sample_online(xadj, adjncy, w.astype(np.float32), np.arange(300, dtype=np.uint32), [1, 25, 10], 6,
                                          distinct=True)
    blocks = out.split("th sample src: ")[1:]
    assert len(blocks) == 4
    for j, blk in enumerate(blocks):
        m = re.match(r"(\d+), 1-hop len: (\d+)", blk)
        assert int(m.group(1)) == j and int(m.group(2)) == sl[j, 0]
        hop1 = [int(x) for x in blk.split("1-hop : ")[1].splitlines()[0].split()]
        assert hop1 == data[j, 1:1 + sl[j, 0]].tolist()
    lines = [l for l in out.splitlines() if l.strip()]
    sample_ms, mseps = float(lines[-2]), float(lines[-1])
    assert abs(mseps - sampled / (sample_ms * 1e-3) / 1e6) <= 0.02 * mseps + 0.02
    rc, out, err = run([os.path.join(HOST, "skywalker"), "--replace=0", "--k", "70", "--d", "2", "--input", p, "-n", "10"])
    assert rc != 0 and "64" in err


@pytest.mark.gpu
@pytest.mark.parametrize("table", [False, True])
def test_cli_unbiased_node2vec(tmp_path, orc, table):
    # --bias=0 --node2vec: the reference's unbiased node2vec walker (src/unbiased_walk.cu:14-60) = unit weights here
    xadj, adjncy = orc.rmat_csr(11, 8, 23)
    w = (orc.gen_weights(orc.W_UNIFORM, 23, len(adjncy), 1.0, 100.0)).astype(np.uint32)
    p = str(tmp_path / "un.w.gr")
    write_gr(p, xadj, adjncy, w)
    rc, out, err = run([os.path.join(HOST, "skywalker"), "--node2vec", "--bias=0", "--input", p, "-n", "400", "--d", "15",
                        "--p", "0.5", "--q", "2", "--printresult", "--seed", "8"] + (["--n2v_table"] if table else []))
    assert rc == 0, err
    lines = out.splitlines()
    ones = np.ones(len(adjncy), np.float32)
    seeds = np.arange(400, dtype=np.uint32)
    if table:
        paths, lengths, sampled = orc.walk_online(xadj, adjncy, ones, 1, 0.5, 2.0, seeds, 15, 0.0, 8)
    else:
        prob, alias, valid = orc.alias_build(xadj, ones)
        paths, lengths, sampled = orc.walk_node2vec_reject(xadj, adjncy, prob, alias, 0.5, 2.0, seeds, 15, 0.0, 8)
    for j in range(3):
        i = lines.index("%drd path len %d " % (j, lengths[j]))
        assert [int(x) for x in lines[i + 1].split()] == paths[j, :min(lengths[j], 16)].tolist()
    sample_ms, mseps = (float(l.strip()) for l in lines[-2:])
    assert abs(mseps - sampled / (sample_ms * 1e-3) / 1e6) <= 0.02 * mseps + 0.02


@pytest.mark.parametrize("flags,msg", [(["--d", "-1"], "--d >= 1"), (["--d", "0"], "--d >= 1"), (["-n", "-5"], "-n >= 0"),
                                       (["--k", "0"], "--k >= 1"), (["--tp", "1.5"], "--tp"), (["--p", "0"], "--p > 0")])
def test_cli_rejects_bad_numbers(flags, msg):
    # checked before any file is opened or any device is touched
    rc, out, err = run([os.path.join(HOST, "skywalker"), "--input", "/nonexistent"] + flags)
    assert rc == 1 and msg in err


@pytest.mark.gpu
def test_cli_rejects_a_graph_without_vertices(tmp_path):
    p = str(tmp_path / "empty.gr")
    write_gr(p, np.zeros(1, np.uint32), np.zeros(0, np.uint32))
    rc, out, err = run([os.path.join(HOST, "skywalker"), "--deepwalk", "--input", p])
    assert rc == 1 and "no vertices" in err


@pytest.mark.gpu
def test_cli_rejects_multi_gpu(tmp_path):
    rc, out, err = run([os.path.join(HOST, "skywalker"), "--ngpu", "2", "--input", "/nonexistent"])
    assert rc == 1 and "one GPU" in err


@pytest.mark.gpu
def test_cli_degree_bias_plugin(tmp_path, orc):
    # --biasplugin: the operator library takes the place of the reference's link-time bias (src/api/bias_degree.cu)
    xadj, adjncy = orc.rmat_csr(11, 8, 27)
    p = str(tmp_path / "d.gr")
    write_gr(p, xadj, adjncy, np.ones(len(adjncy), np.uint32))
    deg = np.diff(xadj.astype(np.int64))
    wd = deg[adjncy].astype(np.float32)
    plug = os.path.join(ROOT, "skywalker_amd", "libskywalker_bias_degree.so")
    seeds = np.arange(300, dtype=np.uint32)
    for online in (0, 1):
        rc, out, err = run([os.path.join(HOST, "skywalker"), "--deepwalk", "--bias=1", "--ol=%d" % online, "--input", p,
                            "-n", "300", "--d", "12", "--printresult", "--seed", "6", "--biasplugin", plug])
        assert rc == 0, err
        lines = out.splitlines()
        prob, alias, valid = orc.alias_build(xadj, wd)
        paths, lengths, sampled = orc.walk_offline(xadj, adjncy, prob, alias, seeds, 12, 0.0, 6)
        for j in range(3):
            i = lines.index("%drd path len %d " % (j, lengths[j]))
            assert [int(x) for x in lines[i + 1].split()] == paths[j, :min(lengths[j], 13)].tolist()
    rc, out, err = run([os.path.join(HOST, "skywalker"), "--deepwalk", "--input", p, "--biasplugin", "/nonexistent.so"])
    assert rc == 1 and "cannot load bias plug-in" in err


def _walk_lines(out, lengths, paths, n, width):
    lines = out.splitlines()
    for j in range(n):
        i = lines.index("%drd path len %d " % (j, lengths[j]))
        assert [int(x) for x in lines[i + 1].split()] == paths[j, :min(lengths[j], width)].tolist()


@pytest.mark.gpu
def test_cli_degree_as_weight(tmp_path, orc):
    # --dw: every edge of a row weighs the row's out-degree (include/graph.cuh:299-310), whatever the file holds
    xadj, adjncy = orc.rmat_csr(11, 8, 31)
    stored = (orc.gen_weights(orc.W_UNIFORM, 31, len(adjncy), 1.0, 100.0)).astype(np.uint32)
    p = str(tmp_path / "rmat11.w.gr")
    write_gr(p, xadj, adjncy, stored)
    rc, out, err = run([os.path.join(HOST, "skywalker"), "--deepwalk", "--bias=1", "--ol=0", "--dw", "--input", p, "-n", "300",
                        "--d", "16", "--printresult", "--seed", "6"])
    assert rc == 0, err
    w = np.repeat(np.diff(xadj).astype(np.float32), np.diff(xadj))
    prob, alias, valid = orc.alias_build(xadj, w)
    assert (prob[alias != 0xFFFFFFFF] == 1.0).all()  # equal weights inside a row: every slot keeps its bucket
    paths, lengths, sampled = orc.walk_offline(xadj, adjncy, prob, alias, np.arange(300, dtype=np.uint32), 16, 0.0, 6)
    _walk_lines(out, lengths, paths, 3, 17)
    # and it is not the walk on the stored weights
    sprob, salias, _ = orc.alias_build(xadj, stored.astype(np.float32))
    spaths, _, _ = orc.walk_offline(xadj, adjncy, sprob, salias, np.arange(300, dtype=np.uint32), 16, 0.0, 6)
    assert not np.array_equal(spaths, paths)


@pytest.mark.gpu
@pytest.mark.parametrize("weighted_file", [True, False])
def test_cli_random_weights(tmp_path, orc, weighted_file):
    # --randomweight --weightrange=R: weight i = float(rand()) / float(RAND_MAX / R) after srand(0)
    # (include/graph.cuh:210-219), for a file with weights and for one without
    import ctypes
    xadj, adjncy = orc.rmat_csr(11, 8, 32)
    p = str(tmp_path / "rmat11.gr")
    write_gr(p, xadj, adjncy, np.ones(len(adjncy), np.uint32) if weighted_file else None)
    R = 7
    rc, out, err = run([os.path.join(HOST, "skywalker"), "--deepwalk", "--bias=1", "--ol=0", "--randomweight",
                        "--weightrange=%d" % R, "--input", p, "-n", "300", "--d", "16", "--printresult", "--seed", "8"])
    assert rc == 0, err
    assert "generating random weight" in out
    libc = ctypes.CDLL("libc.so.6")
    libc.srand(0)
    RAND_MAX = 2147483647
    w = (np.array([libc.rand() for _ in range(len(adjncy))], np.float32) / np.float32(RAND_MAX // R)).astype(np.float32)
    prob, alias, valid = orc.alias_build(xadj, w)
    paths, lengths, sampled = orc.walk_offline(xadj, adjncy, prob, alias, np.arange(300, dtype=np.uint32), 16, 0.0, 8)
    _walk_lines(out, lengths, paths, 3, 17)


@pytest.mark.gpu
def test_cli_degree_bias_plugin_in_online_sampling(tmp_path, orc):
    # --sage --ol=1 --biasplugin: the operator is asked for the weights of every frontier row the sampler builds
    # (include/alias_table_new.cuh:1090-1091 via src/online_sample_new.cu:3-70)
    xadj, adjncy = orc.rmat_csr(11, 8, 29)
    p = str(tmp_path / "ds.gr")
    write_gr(p, xadj, adjncy, np.ones(len(adjncy), np.uint32))
    deg = np.diff(xadj.astype(np.int64))
    wd = deg[adjncy].astype(np.float32)
    plug = os.path.join(ROOT, "skywalker_amd", "libskywalker_bias_degree.so")
    rc, out, err = run([os.path.join(HOST, "skywalker"), "--sage", "--bias=1", "--ol=1", "--input", p, "-n", "300",
                        "--printresult", "--seed", "4", "--biasplugin", plug])
    assert rc == 0, err
    data, sl, sampled = orc.sample_online(xadj, adjncy, wd, np.arange(300, dtype=np.uint32), [1, 25, 10], 4)
    blocks = out.split("th sample src: ")[1:]
    assert len(blocks) == 4
    for j, blk in enumerate(blocks):
        m = re.match(r"(\d+), 1-hop len: (\d+)", blk)
        assert int(m.group(1)) == j and int(m.group(2)) == sl[j, 0]
        hop1 = [int(x) for x in blk.split("1-hop : ")[1].splitlines()[0].split()]
        assert hop1 == data[j, 1:1 + sl[j, 0]].tolist()
        for i in range(sl[j, 0]):
            line = blk.split("\t %d th 2-hop [%d]: " % (i, data[j, 1 + i]))[1].splitlines()[0]
            assert [int(x) for x in line.split()] == data[j, 26 + 10 * i:26 + 10 * i + min(sl[j, 1 + i], 30)].tolist()
