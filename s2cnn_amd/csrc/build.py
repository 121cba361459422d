"""Ahead-of-time build of libs2cnn_hip.so for gfx950 with hipcc (no JIT, no torch headers).

    python -m s2cnn_amd.csrc.build [--probes] [--stale | source.hip ...]

Every source is compiled to an object of its own (in parallel), then linked.  Without arguments everything is
recompiled.  Naming sources (or --stale) rebuilds those objects; every other object is reused only if it is newer than
its source and than every header of this tree the source includes, directly or through other headers (otherwise it is
rebuilt too: a stale object never reaches the link).  `--probes` also builds the measurement library
libs2cnn_probe.so (csrc/probe/, include/s2cnn_hip_probe.h) that `bench.py --floor` loads; the package never does.
"""
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
SOURCES = ["so3_mm.hip", "so3_mm_real.hip", "so3_real_basis.hip", "so3_rft.hip", "so3_fft.hip", "s2_fft.hip", "s2_mm.hip",
           "s2_mm_real.hip", "so3_integrate.hip"]
PROBE_SOURCES = ["probe/so3_fft64_probe.hip"]
LIB = os.path.join(HERE, "libs2cnn_hip.so")
PROBE_LIB = os.path.join(HERE, "libs2cnn_probe.so")
OBJDIR = os.path.join(HERE, "build")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-I", os.path.join(ROOT, "include"), "-I", HERE]


def _obj(src):
    return os.path.join(OBJDIR, os.path.splitext(src)[0].replace("/", "_") + ".o")


def _dependencies(path, seen=None):
    """`path` and every header of this tree it includes with quotes, directly or through other headers."""
    seen = set() if seen is None else seen
    if path in seen:
        return seen
    seen.add(path)
    for name in re.findall(r'^\s*#\s*include\s+"([^"]+)"', open(path).read(), flags=re.M):
        for base in (os.path.dirname(path), HERE, os.path.join(ROOT, "include")):
            cand = os.path.normpath(os.path.join(base, name))
            if os.path.exists(cand):
                _dependencies(cand, seen)
                break
    return seen


def _stale(src):
    obj = _obj(src)
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    return any(t < os.path.getmtime(d) for d in _dependencies(os.path.join(HERE, src)))


def build(verbose=True, only=None, jobs=None, probes=False):
    """Compile and link.  only=None: every source is recompiled; only=[names]: those plus whatever is stale."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(OBJDIR, exist_ok=True)
    sources = SOURCES + (PROBE_SOURCES if probes else [])
    todo = [s for s in sources if only is None or s in only or _stale(s)]

    def compile_one(src):
        cmd = [hipcc] + FLAGS + ["-c", os.path.join(HERE, src), "-o", _obj(src)]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True)

    with ThreadPoolExecutor(max_workers=jobs or min(8, os.cpu_count() or 1)) as pool:
        list(pool.map(compile_one, todo))
    links = [(LIB, SOURCES)] + ([(PROBE_LIB, PROBE_SOURCES)] if probes else [])
    for lib, srcs in links:
        cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + [_obj(s) for s in srcs]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    argv = sys.argv[1:]
    named = [a for a in argv if not a.startswith("--")]
    build(only=named if (named or "--stale" in argv) else None, probes="--probes" in argv)
    sys.exit(0)
