"""Index arithmetic of the per-volume SO(3) kernels, checked on the CPU: tests/geometry_check.cpp includes the kernels'
headers, walks over every (round, thread) place of the 20^3, 32^3, 44^3 and 64^3 grids and checks that each item of the
half spectrum sits in exactly one place, that truncated spectra keep every item below their bandwidth, and that the slot
permutation of a line inverts.  Needs hipcc (the headers are HIP), no GPU."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_item_places_and_line_slots_of_the_per_volume_kernels(tmp_path):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    if not (os.path.exists(hipcc) or shutil.which(hipcc)):
        pytest.skip("hipcc not found")
    exe = str(tmp_path / "geometry_check")
    cmd = [hipcc, "--offload-arch=gfx950", "-std=c++17", "-O1", "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "s2cnn_amd", "csrc"),
           "-x", "hip", os.path.join(ROOT, "tests", "geometry_check.cpp"), "-o", exe]
    subprocess.run(cmd, check=True, capture_output=True)
    run = subprocess.run([exe], capture_output=True, text=True)
    print(run.stdout)
    assert run.returncode == 0, run.stdout
    for grid in ("20^3", "32^3", "44^3", "64^3"):
        assert any(line.startswith(grid) and line.rstrip().endswith("ok") for line in run.stdout.splitlines()), run.stdout
