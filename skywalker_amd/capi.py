"""ctypes view of libskywalker_hip.so: one Python function per C-ABI entry point.

This is plumbing for tests and the benchmark; the product is the shared library.
There is no CPU fallback: loading fails loudly when the library has not been built,
and every call fails loudly when no MI355X is visible.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libskywalker_hip.so")

INVALID = 0xFFFFFFFF
FILL = 0xFFFFFFFF
BIAS_STATIC, BIAS_NODE2VEC, BIAS_NODE2VEC_REJECT = 0, 1, 2
W_UNIFORM, W_UNIT, W_LOGNORMAL = 0, 1, 2

EXPORTS = [
    "sky_last_error", "sky_version", "sky_device_malloc", "sky_device_free", "sky_memcpy_h2d", "sky_memcpy_d2h",
    "sky_device_fill_u32", "sky_device_copy_u32", "sky_device_synchronize", "sky_device_mem_info", "sky_device_name", "sky_graph_upload",
    "sky_graph_generate_rmat", "sky_graph_generate_from_degrees", "sky_graph_info", "sky_graph_download", "sky_graph_device_ptrs", "sky_graph_free",
    "sky_alias_build_all", "sky_alias_build_from_weights", "sky_alias_download", "sky_alias_upload", "sky_gen_seeds", "sky_walk_offline",
    "sky_walk_offline_noalloc", "sky_walk_index_build",
    "sky_walk_online", "sky_sample_layout", "sky_sample_offline", "sky_sample_online", "sky_sample_session_begin", "sky_sample_session_frontier", "sky_sample_session_hop",
    "sky_sample_session_end", "sky_philox_selftest",
    "sky_last_build_profile", "sky_set_option", "sky_graph_set_option", "sky_graph_unset_option",
]


class SkyError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("libskywalker_hip error %d: %s" % (code, msg))
        self.code = code


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("%s is missing: run `python -c 'import __graft_entry__ as g; g.build()'` "
                              "(there is no CPU fallback)" % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        L.sky_last_error.restype = C.c_char_p
        L.sky_version.restype = C.c_char_p
        _lib = L
    return _lib


def _ck(rc):
    if rc != 0:
        raise SkyError(rc, lib().sky_last_error().decode())


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def device_name():
    buf = C.create_string_buffer(256)
    cu = C.c_int(0)
    _ck(lib().sky_device_name(buf, C.c_size_t(256), C.byref(cu)))
    return buf.value.decode(), cu.value


def synchronize():
    _ck(lib().sky_device_synchronize())


def mem_info():
    """(free, total) bytes of device memory as the HIP runtime reports them."""
    f, t = C.c_size_t(0), C.c_size_t(0)
    _ck(lib().sky_device_mem_info(C.byref(f), C.byref(t)))
    return f.value, t.value


class DeviceArray:
    """A device allocation of `count` elements of `dtype`, owned by this object."""

    def __init__(self, count, dtype, fill=None):
        self.count, self.dtype = int(count), np.dtype(dtype)
        self.ptr = C.c_void_p()
        _ck(lib().sky_device_malloc(C.c_size_t(self.nbytes), C.byref(self.ptr)))
        if fill is not None:
            assert self.dtype.itemsize == 4
            _ck(lib().sky_device_fill_u32(self.ptr, C.c_uint32(fill), C.c_size_t(self.count)))

    @property
    def nbytes(self):
        return self.count * self.dtype.itemsize

    @classmethod
    def from_host(cls, arr):
        arr = np.ascontiguousarray(arr)
        d = cls(arr.size, arr.dtype)
        _ck(lib().sky_memcpy_h2d(d.ptr, _p(arr), C.c_size_t(arr.nbytes)))
        return d

    def to_host(self, shape=None):
        out = np.empty(self.count, self.dtype)
        _ck(lib().sky_memcpy_d2h(_p(out), self.ptr, C.c_size_t(self.nbytes)))
        return out.reshape(shape) if shape is not None else out

    def free(self):
        if self.ptr:
            lib().sky_device_free(self.ptr)
            self.ptr = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def device_copy(dst, src, count):
    _ck(lib().sky_device_copy_u32(dst.ptr, src.ptr, C.c_size_t(count)))


def sample_layout(fanout):
    fan = np.asarray(fanout, np.uint32)
    lps, slen = C.c_uint64(0), C.c_uint64(0)
    _ck(lib().sky_sample_layout(_p(fan), C.c_uint32(len(fan)), C.byref(lps), C.byref(slen)))
    return lps.value, slen.value


class Graph:
    """Device-resident CSR plus its alias tables (a sky_graph handle)."""

    def __init__(self, handle):
        self.h = handle
        V, E, md = C.c_uint32(0), C.c_uint32(0), C.c_uint32(0)
        _ck(lib().sky_graph_info(self.h, C.byref(V), C.byref(E), C.byref(md)))
        self.V, self.E, self.max_degree = V.value, E.value, md.value

    @classmethod
    def upload(cls, xadj, adjncy, adjwgt):
        xadj = np.ascontiguousarray(xadj, np.uint32)
        adjncy = np.ascontiguousarray(adjncy, np.uint32)
        w = None if adjwgt is None else np.ascontiguousarray(adjwgt, np.float32)
        h = C.c_void_p()
        _ck(lib().sky_graph_upload(_p(xadj), _p(adjncy), _p(w), C.c_uint32(len(xadj) - 1), C.c_uint32(len(adjncy)),
                                   C.byref(h)))
        return cls(h)

    @classmethod
    def rmat(cls, scale, edge_factor, graph_seed, weight_kind, wa, wb, weight_seed):
        h = C.c_void_p()
        _ck(lib().sky_graph_generate_rmat(C.c_uint32(scale), C.c_uint32(edge_factor), C.c_uint64(graph_seed),
                                          C.c_int(weight_kind), C.c_float(wa), C.c_float(wb),
                                          C.c_uint64(weight_seed), C.byref(h)))
        return cls(h)

    @classmethod
    def from_degrees(cls, xadj, graph_seed, weight_kind, wa, wb, weight_seed):
        """Rows of the given lengths, neighbours uniform over the vertices, weights of the given law (device side)."""
        xadj = np.ascontiguousarray(xadj, np.uint32)
        h = C.c_void_p()
        _ck(lib().sky_graph_generate_from_degrees(_p(xadj), C.c_uint32(len(xadj) - 1), C.c_uint64(graph_seed),
                                                  C.c_int(weight_kind), C.c_float(wa), C.c_float(wb),
                                                  C.c_uint64(weight_seed), C.byref(h)))
        return cls(h)

    def download(self, weights=True):
        xadj = np.empty(self.V + 1, np.uint32)
        adjncy = np.empty(self.E, np.uint32)
        w = np.empty(self.E, np.float32) if weights else None
        _ck(lib().sky_graph_download(self.h, _p(xadj), _p(adjncy), _p(w)))
        return xadj, adjncy, w

    def download_xadj(self):
        xadj = np.empty(self.V + 1, np.uint32)
        _ck(lib().sky_graph_download(self.h, _p(xadj), None, None))
        return xadj

    def build_tables(self):
        """ConstructTable: returns the kernel-region seconds."""
        sec = C.c_double(0)
        _ck(lib().sky_alias_build_all(self.h, C.byref(sec)))
        return sec.value

    def build_tables_from_weights(self, weights):
        """Tables from a caller's device array of E floats (a DeviceArray) instead of the graph's own weights."""
        sec = C.c_double(0)
        _ck(lib().sky_alias_build_from_weights(self.h, weights.ptr, C.byref(sec)))
        return sec.value

    def build_profile(self):
        names = (C.c_char_p * 64)()
        ms = (C.c_float * 64)()
        edges = (C.c_uint64 * 64)()
        n = lib().sky_last_build_profile(self.h, names, ms, edges, 64)
        return [(names[i].decode(), float(ms[i]), int(edges[i])) for i in range(n)]

    def tables(self):
        prob = np.empty(self.E, np.float32)
        alias = np.empty(self.E, np.uint32)
        valid = np.empty(self.V, np.int8)
        _ck(lib().sky_alias_download(self.h, _p(prob), _p(alias), _p(valid)))
        return prob, alias, valid

    def upload_tables(self, prob, alias, valid):
        prob = np.ascontiguousarray(prob, np.float32)
        alias = np.ascontiguousarray(alias, np.uint32)
        valid = np.ascontiguousarray(valid, np.int8)
        _ck(lib().sky_alias_upload(self.h, _p(prob), _p(alias), _p(valid)))

    def gen_seeds(self, seed, N):
        d = DeviceArray(N, np.uint32)
        _ck(lib().sky_gen_seeds(C.c_uint64(seed), C.c_uint32(self.V), C.c_uint32(N), d.ptr))
        return d

    def _walk(self, fn, pre, seeds, length, stop_prob, seed, out=None):
        seeds_d = seeds if isinstance(seeds, DeviceArray) else DeviceArray.from_host(np.asarray(seeds, np.uint32))
        N = seeds_d.count
        if out is None:
            paths = DeviceArray(N * (length + 1), np.uint32, fill=FILL)
            lengths = DeviceArray(N, np.uint32, fill=0)
        else:
            paths, lengths = out
        sampled, sec = C.c_uint64(0), C.c_double(0)
        _ck(fn(self.h, *pre, seeds_d.ptr, C.c_uint32(N), C.c_uint32(length), C.c_float(stop_prob), C.c_uint64(seed),
               paths.ptr, lengths.ptr, C.byref(sampled), C.byref(sec)))
        return paths, lengths, sampled.value, sec.value

    def walk_offline(self, seeds, length, stop_prob, seed, out=None):
        """OfflineWalk: returns (paths DeviceArray, lengths DeviceArray, sampled, seconds)."""
        return self._walk(lib().sky_walk_offline, (), seeds, length, stop_prob, seed, out)

    def build_walk_index(self):
        """sky_walk_index_build: returns the kernel-region seconds."""
        sec = C.c_double(0)
        _ck(lib().sky_walk_index_build(self.h, C.byref(sec)))
        return sec.value

    def walk_offline_noalloc(self, seeds_d, length, stop_prob, seed, paths, lengths, sampled_d):
        """sky_walk_offline_noalloc: every buffer is the caller's; enqueues and returns (synchronize() before reading)."""
        _ck(lib().sky_walk_offline_noalloc(self.h, seeds_d.ptr, C.c_uint32(seeds_d.count), C.c_uint32(length),
                                           C.c_float(stop_prob), C.c_uint64(seed), paths.ptr, lengths.ptr,
                                           sampled_d.ptr if sampled_d is not None else None))

    def walk_online(self, bias_kind, p, q, seeds, length, stop_prob, seed, out=None):
        """OnlineWalkShMem."""
        return self._walk(lib().sky_walk_online, (C.c_int(bias_kind), C.c_float(p), C.c_float(q)), seeds, length,
                          stop_prob, seed, out)

    def _sample(self, fn, seeds, fanout, seed, out=None):
        seeds_d = seeds if isinstance(seeds, DeviceArray) else DeviceArray.from_host(np.asarray(seeds, np.uint32))
        N = seeds_d.count
        fan = np.asarray(fanout, np.uint32)
        lps, slen = sample_layout(fan)
        if out is None:
            data = DeviceArray(N * lps, np.uint32, fill=FILL)
            sl = DeviceArray(N * slen, np.uint32, fill=0)
        else:
            data, sl = out
        sampled, sec = C.c_uint64(0), C.c_double(0)
        _ck(fn(self.h, seeds_d.ptr, C.c_uint32(N), _p(fan), C.c_uint32(len(fan)), C.c_uint64(seed), data.ptr, sl.ptr,
               C.byref(sampled), C.byref(sec)))
        return data, sl, sampled.value, sec.value

    def sample_offline(self, seeds, fanout, seed, out=None):
        """OfflineSample."""
        return self._sample(lib().sky_sample_offline, seeds, fanout, seed, out)

    def sample_online(self, seeds, fanout, seed, out=None):
        """OnlineGBSampleNew."""
        return self._sample(lib().sky_sample_online, seeds, fanout, seed, out)

    def device_ptrs(self):
        """Device addresses of xadj, adjncy, adjwgt, table, valid (integers; 0 for an array that does not exist)."""
        ptrs = [C.c_void_p() for _ in range(5)]
        _ck(lib().sky_graph_device_ptrs(self.h, *[C.byref(p) for p in ptrs]))
        return tuple(p.value or 0 for p in ptrs)

    def sample_session(self, seeds, fanout, seed, weights_of_hop=None):
        """sky_sample_session_*: online k-hop sampling one hop at a time.  weights_of_hop(hop, frontier_upper) returns
        the DeviceArray of E weights (16 spare bytes, as DeviceArray gives them) from which that hop's frontier rows are
        built, or None for the graph's own."""
        seeds_d = seeds if isinstance(seeds, DeviceArray) else DeviceArray.from_host(np.asarray(seeds, np.uint32))
        N = seeds_d.count
        fan = np.asarray(fanout, np.uint32)
        lps, slen = sample_layout(fan)
        data = DeviceArray(N * lps, np.uint32, fill=FILL)
        sl = DeviceArray(N * slen, np.uint32, fill=0)
        sess = C.c_void_p()
        _ck(lib().sky_sample_session_begin(self.h, seeds_d.ptr, C.c_uint32(N), _p(fan), C.c_uint32(len(fan)),
                                           C.c_uint64(seed), data.ptr, sl.ptr, C.byref(sess)))
        try:
            for hop in range(len(fan) - 1):
                lst, cnt, upper = C.c_void_p(), C.c_void_p(), C.c_uint32(0)
                _ck(lib().sky_sample_session_frontier(sess, C.c_uint32(hop), C.byref(lst), C.byref(cnt), C.byref(upper)))
                w = weights_of_hop(hop, upper.value) if weights_of_hop else None
                _ck(lib().sky_sample_session_hop(sess, C.c_uint32(hop), w.ptr if w is not None else None))
        finally:
            sampled, sec = C.c_uint64(0), C.c_double(0)
            rc = lib().sky_sample_session_end(sess, C.byref(sampled), C.byref(sec))
        _ck(rc)
        return data, sl, sampled.value, sec.value

    def set_option(self, name, value):
        """A tuning knob for this graph alone (None: back to the process-wide value)."""
        if value is None:
            _ck(lib().sky_graph_unset_option(self.h, name.encode()))
        else:
            _ck(lib().sky_graph_set_option(self.h, name.encode(), C.c_long(value)))

    def free(self):
        if self.h:
            lib().sky_graph_free(self.h)
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class BiasPlugin:
    """A bias-operator library (include/skywalker_bias.h): libskywalker_bias_<name>.so next to the main library."""

    def __init__(self, name):
        path = os.path.join(HERE, "libskywalker_bias_%s.so" % name)
        if not os.path.exists(path):
            raise ImportError("%s is missing: run `python -c 'import __graft_entry__ as g; g.build()'`" % path)
        lib()  # the plug-in links against the main library
        self.lib = C.CDLL(path)
        self.lib.sky_bias_name.restype = C.c_char_p
        self.lib.sky_bias_last_error.restype = C.c_char_p
        self.name = self.lib.sky_bias_name().decode()

    def _ck(self, rc):
        if rc != 0:
            raise SkyError(rc, self.lib.sky_bias_last_error().decode() or lib().sky_last_error().decode())

    def build_all(self, g, p=1.0, q=1.0):
        sec = C.c_double(0)
        self._ck(self.lib.sky_bias_build_all(g.h, C.c_float(p), C.c_float(q), C.byref(sec)))
        return sec.value

    def walk_online(self, g, p, q, seeds, length, stop_prob, seed):
        seeds_d = seeds if isinstance(seeds, DeviceArray) else DeviceArray.from_host(np.asarray(seeds, np.uint32))
        N = seeds_d.count
        paths = DeviceArray(N * (length + 1), np.uint32, fill=FILL)
        lengths = DeviceArray(N, np.uint32, fill=0)
        sampled, sec = C.c_uint64(0), C.c_double(0)
        self._ck(self.lib.sky_bias_walk_online(g.h, C.c_float(p), C.c_float(q), seeds_d.ptr, C.c_uint32(N),
                                               C.c_uint32(length), C.c_float(stop_prob), C.c_uint64(seed), paths.ptr,
                                               lengths.ptr, C.byref(sampled), C.byref(sec)))
        return paths, lengths, sampled.value, sec.value

    def sample_online(self, g, p, q, seeds, fanout, seed):
        seeds_d = seeds if isinstance(seeds, DeviceArray) else DeviceArray.from_host(np.asarray(seeds, np.uint32))
        N = seeds_d.count
        fan = np.asarray(fanout, np.uint32)
        lps, slen = sample_layout(fan)
        data = DeviceArray(N * lps, np.uint32, fill=FILL)
        sl = DeviceArray(N * slen, np.uint32, fill=0)
        sampled, sec = C.c_uint64(0), C.c_double(0)
        self._ck(self.lib.sky_bias_sample_online(g.h, C.c_float(p), C.c_float(q), seeds_d.ptr, C.c_uint32(N), _p(fan),
                                                 C.c_uint32(len(fan)), C.c_uint64(seed), data.ptr, sl.ptr,
                                                 C.byref(sampled), C.byref(sec)))
        return data, sl, sampled.value, sec.value


def set_option(name, value):
    _ck(lib().sky_set_option(name.encode(), C.c_long(value)))


def philox_selftest(ctr, key):
    ctr = np.ascontiguousarray(ctr, np.uint32).reshape(-1, 4)
    key = np.ascontiguousarray(key, np.uint32).reshape(-1, 2)
    out = np.zeros_like(ctr)
    _ck(lib().sky_philox_selftest(_p(ctr), _p(key), C.c_uint32(len(ctr)), _p(out)))
    return out
