"""ctypes binding of the CPU oracle (oracle/liboracle.so).  TEST INFRASTRUCTURE ONLY.

Loaded by tests/, the smoke test and the benchmark's cpu_baseline leg; never by
the product package.  Arrays are numpy, results are returned as new arrays.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
INVALID = 0xFFFFFFFF

_u32p = np.ctypeslib.ndpointer(np.uint32, flags="C_CONTIGUOUS")
_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_f64p = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")
_i8p = np.ctypeslib.ndpointer(np.int8, flags="C_CONTIGUOUS")


def build():
    """Compile the oracle with its Makefile (g++)."""
    subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        build()
    L = C.CDLL(_LIB_PATH)
    L.orc_philox4x32_10.argtypes = [_u32p, _u32p, _u32p]
    L.orc_rmat_csr.argtypes = [C.c_uint32, C.c_uint32, C.c_uint64, _u32p, _u32p]
    L.orc_gen_weights.argtypes = [C.c_int, C.c_uint64, C.c_uint64, C.c_float, C.c_float, _f32p]
    L.orc_gen_seeds.argtypes = [C.c_uint64, C.c_uint32, C.c_uint32, _u32p]
    L.orc_alias_build_row.argtypes = [_f32p, C.c_uint32, _f32p, _u32p]
    L.orc_alias_build.argtypes = [_u32p, _f32p, C.c_uint32, _f32p, _u32p, _i8p, C.c_int]
    L.orc_vose_row.argtypes = [_f32p, C.c_uint32, _f64p, _u32p]
    L.orc_alias_reconstruct_row.argtypes = [_f32p, _u32p, C.c_uint32, _f64p]
    L.orc_alias_reconstruct_row.restype = None
    L.orc_alias_check.argtypes = [_u32p, _f32p, _f32p, _u32p, _i8p, C.c_uint32, _f64p]
    L.orc_walk_offline.argtypes = [_u32p, C.c_uint32, _u32p, _f32p, _u32p, _u32p, C.c_uint32, C.c_uint32, C.c_float, C.c_uint64,
                                   _u32p, _u32p, C.POINTER(C.c_uint64)]
    L.orc_walk_online.argtypes = [_u32p, C.c_uint32, _u32p, _f32p, C.c_int, C.c_float, C.c_float, _u32p, C.c_uint32, C.c_uint32,
                                  C.c_float, C.c_uint64, _u32p, _u32p, C.POINTER(C.c_uint64)]
    L.orc_walk_node2vec_reject.argtypes = [_u32p, C.c_uint32, _u32p, _f32p, _u32p, C.c_float, C.c_float, _u32p, C.c_uint32, C.c_uint32,
                                           C.c_float, C.c_uint64, _u32p, _u32p, C.POINTER(C.c_uint64)]
    L.orc_sample_offline.argtypes = [_u32p, C.c_uint32, _u32p, _f32p, _u32p, _u32p, C.c_uint32, _u32p, C.c_uint32, C.c_uint64,
                                     _u32p, _u32p, C.POINTER(C.c_uint64)]
    L.orc_sample_online.argtypes = [_u32p, C.c_uint32, _u32p, _f32p, _u32p, C.c_uint32, _u32p, C.c_uint32, C.c_uint64, _u32p,
                                    _u32p, C.POINTER(C.c_uint64)]
    L.orc_sample_offline_distinct.argtypes = L.orc_sample_offline.argtypes
    L.orc_sample_online_distinct.argtypes = L.orc_sample_online.argtypes
    L.orc_num_threads.restype = C.c_int
    _lib = L
    return L


FILL = 0xFFFFFFFF  # value callers pre-fill output slots with; the kernels leave unreached slots untouched

W_UNIFORM, W_UNIT, W_LOGNORMAL = 0, 1, 2


def philox(ctr, key):
    out = np.zeros(4, np.uint32)
    lib().orc_philox4x32_10(np.asarray(ctr, np.uint32), np.asarray(key, np.uint32), out)
    return out


def rmat_csr(scale, edge_factor, seed):
    V, E = 1 << scale, edge_factor << scale
    xadj = np.zeros(V + 1, np.uint32)
    adjncy = np.zeros(E, np.uint32)
    rc = lib().orc_rmat_csr(scale, edge_factor, seed, xadj, adjncy)
    assert rc == 0
    return xadj, adjncy


def gen_weights(kind, seed, E, a=0.0, b=1.0):
    w = np.zeros(E, np.float32)
    lib().orc_gen_weights(kind, seed, E, a, b, w)
    return w


def gen_seeds(seed, V, N):
    s = np.zeros(N, np.uint32)
    lib().orc_gen_seeds(seed, V, N, s)
    return s


def alias_build_row(w):
    w = np.ascontiguousarray(w, np.float32)
    prob = np.zeros(len(w), np.float32)
    alias = np.zeros(len(w), np.uint32)
    valid = lib().orc_alias_build_row(w, len(w), prob, alias)
    return prob, alias, valid


def alias_build(xadj, w, nthreads=0):
    V, E = len(xadj) - 1, len(w)
    prob = np.zeros(E, np.float32)
    alias = np.zeros(E, np.uint32)
    valid = np.zeros(V, np.int8)
    lib().orc_alias_build(xadj, np.ascontiguousarray(w, np.float32), V, prob, alias, valid, nthreads)
    return prob, alias, valid


def vose_row(w):
    w = np.ascontiguousarray(w, np.float32)
    prob = np.zeros(len(w), np.float64)
    alias = np.zeros(len(w), np.uint32)
    ok = lib().orc_vose_row(w, len(w), prob, alias)
    return prob, alias, ok


def reconstruct_row(prob, alias):
    q = np.zeros(len(prob), np.float64)
    lib().orc_alias_reconstruct_row(np.ascontiguousarray(prob, np.float32), np.ascontiguousarray(alias, np.uint32),
                                    len(prob), q)
    return q


def alias_check(xadj, w, prob, alias, valid):
    """Returns dict(max_rel_err, bad_valid, bad_range, bad_invalid, worst_vertex)."""
    st = np.zeros(5, np.float64)
    lib().orc_alias_check(xadj, np.ascontiguousarray(w, np.float32), np.ascontiguousarray(prob, np.float32),
                          np.ascontiguousarray(alias, np.uint32), np.ascontiguousarray(valid, np.int8),
                          len(xadj) - 1, st)
    return dict(max_rel_err=st[0], bad_valid=int(st[1]), bad_range=int(st[2]), bad_invalid=int(st[3]),
                worst_vertex=int(st[4]))


def walk_offline(xadj, adjncy, prob, alias, seeds, length, stop_prob, seed):
    N = len(seeds)
    paths = np.full((N, length + 1), FILL, np.uint32)
    lengths = np.zeros(N, np.uint32)
    sampled = C.c_uint64(0)
    lib().orc_walk_offline(xadj, len(xadj) - 1, adjncy, prob, alias, np.ascontiguousarray(seeds, np.uint32), N, length, stop_prob,
                           seed, paths, lengths, C.byref(sampled))
    return paths, lengths, sampled.value


def walk_online(xadj, adjncy, w, bias_kind, p, q, seeds, length, stop_prob, seed):
    N = len(seeds)
    paths = np.full((N, length + 1), FILL, np.uint32)
    lengths = np.zeros(N, np.uint32)
    sampled = C.c_uint64(0)
    lib().orc_walk_online(xadj, len(xadj) - 1, adjncy, np.ascontiguousarray(w, np.float32), bias_kind, p, q,
                          np.ascontiguousarray(seeds, np.uint32), N, length, stop_prob, seed, paths, lengths,
                          C.byref(sampled))
    return paths, lengths, sampled.value


def walk_node2vec_reject(xadj, adjncy, prob, alias, p, q, seeds, length, stop_prob, seed):
    N = len(seeds)
    paths = np.full((N, length + 1), FILL, np.uint32)
    lengths = np.zeros(N, np.uint32)
    sampled = C.c_uint64(0)
    lib().orc_walk_node2vec_reject(xadj, len(xadj) - 1, adjncy, prob, alias, p, q, np.ascontiguousarray(seeds, np.uint32), N, length,
                                   stop_prob, seed, paths, lengths, C.byref(sampled))
    return paths, lengths, sampled.value


def sample_layout(fanout):
    """fanout = [1, k1, k2, ...] -> (length_per_sample, size_of_sample_lengths, offsets, length_offsets)."""
    width, lps, slen, offs, loffs = 1, 0, 0, [], []
    for h, k in enumerate(fanout):
        width *= k
        offs.append(lps)
        lps += width
        if h + 1 < len(fanout):
            loffs.append(slen)
            slen += width
    return lps, slen, offs, loffs


def sample_offline(xadj, adjncy, prob, alias, seeds, fanout, seed, distinct=False):
    """distinct: children of a parent are distinct slots of its row (the reference's online rule), at most 11 tries each."""
    N = len(seeds)
    fan = np.asarray(fanout, np.uint32)
    lps, slen, _, _ = sample_layout(list(fanout))
    data = np.full((N, lps), FILL, np.uint32)
    sl = np.zeros((N, slen), np.uint32)
    sampled = C.c_uint64(0)
    fn = lib().orc_sample_offline_distinct if distinct else lib().orc_sample_offline
    rc = fn(xadj, len(xadj) - 1, adjncy, prob, alias, np.ascontiguousarray(seeds, np.uint32), N, fan, len(fan),
            seed, data, sl, C.byref(sampled))
    if rc:
        raise ValueError("distinct sampling needs fanouts <= 64 and at most 256 hops")
    return data, sl, sampled.value


def sample_online(xadj, adjncy, w, seeds, fanout, seed, distinct=False):
    N = len(seeds)
    fan = np.asarray(fanout, np.uint32)
    lps, slen, _, _ = sample_layout(list(fanout))
    data = np.full((N, lps), FILL, np.uint32)
    sl = np.zeros((N, slen), np.uint32)
    sampled = C.c_uint64(0)
    fn = lib().orc_sample_online_distinct if distinct else lib().orc_sample_online
    rc = fn(xadj, len(xadj) - 1, adjncy, np.ascontiguousarray(w, np.float32),
            np.ascontiguousarray(seeds, np.uint32), N, fan, len(fan), seed, data, sl, C.byref(sampled))
    if rc:
        raise ValueError("distinct sampling needs fanouts <= 64 and at most 256 hops")
    return data, sl, sampled.value


def num_threads():
    return lib().orc_num_threads()
