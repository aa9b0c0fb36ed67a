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
