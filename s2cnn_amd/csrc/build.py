"""Ahead-of-time build of libs2cnn_hip.so for gfx950 with hipcc (no JIT, no torch headers).

    python -m s2cnn_amd.csrc.build        # or: python s2cnn_amd/csrc/build.py

Every source is compiled to an object of its own (in parallel), then linked; `only` rebuilds a subset of the
objects and relinks with whatever objects are already there.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
SOURCES = ["so3_mm.hip", "so3_mm_real.hip", "so3_real_basis.hip", "so3_rft.hip", "so3_fft.hip", "s2_fft.hip", "s2_mm.hip",
           "s2_mm_real.hip", "so3_integrate.hip"]
LIB = os.path.join(HERE, "libs2cnn_hip.so")
OBJDIR = os.path.join(HERE, "build")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-I", os.path.join(ROOT, "include"), "-I", HERE]


def _obj(src):
    return os.path.join(OBJDIR, os.path.splitext(src)[0] + ".o")


def build(verbose=True, only=None, jobs=None):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(OBJDIR, exist_ok=True)
    todo = [s for s in SOURCES if only is None or s in only or not os.path.exists(_obj(s))]

    def compile_one(src):
        cmd = [hipcc] + FLAGS + ["-c", os.path.join(HERE, src), "-o", _obj(src)]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True)

    with ThreadPoolExecutor(max_workers=jobs or min(8, os.cpu_count() or 1)) as pool:
        list(pool.map(compile_one, todo))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + [_obj(s) for s in SOURCES]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    build(only=sys.argv[1:] or None)
    sys.exit(0)
