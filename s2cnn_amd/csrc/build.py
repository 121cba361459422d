"""Ahead-of-time build of libs2cnn_hip.so for gfx950 with hipcc (no JIT, no torch headers).

    python -m s2cnn_amd.csrc.build        # or: python s2cnn_amd/csrc/build.py
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
SOURCES = ["so3_mm.hip", "so3_mm_real.hip", "so3_real_basis.hip", "so3_rft.hip", "so3_fft.hip", "s2_fft.hip", "s2_mm.hip", "s2_mm_real.hip", "so3_integrate.hip"]
LIB = os.path.join(HERE, "libs2cnn_hip.so")


def build(verbose=True):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-I", os.path.join(ROOT, "include"), "-I", HERE,
           "-o", LIB] + [os.path.join(HERE, s) for s in SOURCES]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)
