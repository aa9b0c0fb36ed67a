"""Compiles libskywalker_hip.so (hand-written HIP for gfx950) in-tree with hipcc."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libskywalker_hip.so")
SOURCES = ["sky_capi.hip", "sky_build.hip", "sky_build_tiled.hip", "sky_build_stream.hip", "sky_walk.hip", "sky_online.hip", "sky_sample.hip", "sky_gen.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math",
    # packed fp32 instructions are kept out of every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _compile(src):
    obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, r.stdout, r.stderr))
    warn = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    return obj, warn


def build_library(verbose=False, jobs=6):
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(_compile, SOURCES))
    objs = [o for o, _ in results]
    if verbose:
        for _, w in results:
            if w:
                print(w, file=sys.stderr)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (r.stdout, r.stderr))
    return LIB


PLUGINS = ["static", "node2vec", "degree"]


def plugin_path(name):
    return os.path.join(HERE, "libskywalker_bias_%s.so" % name)


def build_plugins(names=PLUGINS):
    """One shared library per bias plug-in: the engine that calls the operator and the plug-in that defines it are
    compiled as relocatable device code and linked together, as the reference links one executable per plug-in."""
    pdir = os.path.join(HERE, "plugins")
    rdc = FLAGS + ["-fgpu-rdc"]

    def cc(src, obj):
        r = subprocess.run([HIPCC] + rdc + ["-c", src, "-o", obj], capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, r.stdout, r.stderr))
        return obj

    engine = cc(os.path.join(CSRC, "sky_bias_engine.hip"), os.path.join(CSRC, "sky_bias_engine.o"))
    out = []
    for name in names:
        obj = cc(os.path.join(pdir, "bias_%s.hip" % name), os.path.join(pdir, "bias_%s.o" % name))
        lib = plugin_path(name)
        cmd = [HIPCC, "--offload-arch=gfx950", "-fgpu-rdc", "--hip-link", "-shared", "-fPIC", "-o", lib, engine, obj,
               "-L" + HERE, "-lskywalker_hip", "-Wl,-rpath,$ORIGIN"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed for %s:\n%s\n%s" % (lib, r.stdout, r.stderr))
        out.append(lib)
    return out


if __name__ == "__main__":
    print(build_library(verbose=True))
    print(build_plugins())


def build_host():
    """Builds the C++ facade and the `skywalker` CLI on top of the C-ABI (skywalker_amd/host)."""
    host = os.path.join(HERE, "host")
    if os.path.exists(os.path.join(host, "Makefile")):
        subprocess.check_call(["make", "-C", host, "-B", "-j4"], stdout=subprocess.DEVNULL)
