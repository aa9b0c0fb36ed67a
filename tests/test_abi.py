"""CPU-side checks of the drop-in boundary: the library loads and exports what the header declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "skywalker_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sky_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from skywalker_amd import capi
    lib = ctypes.CDLL(capi.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), "missing export " + n
    assert sorted(capi.EXPORTS) == [n for n in names]


def test_plugin_libraries_export_the_operator_entry_points():
    from skywalker_amd import build
    ctypes.CDLL(os.path.join(ROOT, "skywalker_amd", "libskywalker_hip.so"), mode=ctypes.RTLD_GLOBAL)
    text = open(os.path.join(ROOT, "include", "skywalker_bias.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    host = text[text.index('extern "C"'):]
    names = sorted(set(re.findall(r"\b(sky_bias_[a-z0-9_]+)\s*\(", host)))
    assert names == ["sky_bias_build_all", "sky_bias_last_error", "sky_bias_name", "sky_bias_sample_online",
                     "sky_bias_walk_online"]
    for plug in build.PLUGINS:
        lib = ctypes.CDLL(build.plugin_path(plug))
        for n in names:
            assert hasattr(lib, n), "%s: missing export %s" % (plug, n)
        lib.sky_bias_name.restype = ctypes.c_char_p
        assert lib.sky_bias_name().decode() == plug


def test_version_string():
    from skywalker_amd import capi
    assert b"gfx950" in capi.lib().sky_version()


def test_null_arguments_are_refused_without_touching_a_gpu():
    # every entry point that takes a handle checks it first: an error code and a message, no device call
    from skywalker_amd import capi
    lib = capi.lib()
    null = ctypes.c_void_p()
    out = ctypes.c_void_p()
    calls = [
        lambda: lib.sky_alias_build_all(null, None),
        lambda: lib.sky_alias_build_from_weights(null, None, None),
        lambda: lib.sky_walk_index_build(null, None),
        lambda: lib.sky_graph_info(null, None, None, None),
        lambda: lib.sky_graph_device_ptrs(null, None, None, None, None, None),
        lambda: lib.sky_graph_set_option(null, b"row_merge", ctypes.c_long(1)),
        lambda: lib.sky_graph_unset_option(null, b"row_merge"),
        lambda: lib.sky_sample_session_begin(null, None, ctypes.c_uint32(0), None, ctypes.c_uint32(0), ctypes.c_uint64(0),
                                             None, None, ctypes.byref(out)),
        lambda: lib.sky_sample_session_frontier(null, ctypes.c_uint32(0), None, None, None),
        lambda: lib.sky_sample_session_hop(null, ctypes.c_uint32(0), None),
        lambda: lib.sky_sample_session_end(null, None, None),
    ]
    for call in calls:
        assert call() == -1  # SKY_ERR_ARG
        assert lib.sky_last_error().decode()
    # a knob that does not exist, and a value outside a knob's range
    assert lib.sky_set_option(b"no_such_knob", ctypes.c_long(1)) != 0
    assert lib.sky_set_option(b"small_in_place", ctypes.c_long(7)) != 0
    assert "small_in_place" in lib.sky_last_error().decode()
