"""The C-ABI library loads and exports every symbol include/s2cnn_hip.h declares; argument
checks that need no GPU (they return before any launch)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "s2cnn_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(s2cnn_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from s2cnn_amd import _hip
    lib = _hip.lib()
    names = _declared()
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(_hip.SIGNATURES) == names
    assert lib.s2cnn_abi_version() == 1


def test_measurement_entry_is_not_in_the_product_library():
    """Kernels with parts compiled out live in a library of their own (include/s2cnn_hip_probe.h) that only
    `bench.py --floor` loads: the drop-in boundary exports nothing of it."""
    from s2cnn_amd import _hip
    lib = _hip.lib()
    text = open(os.path.join(ROOT, "include", "s2cnn_hip_probe.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(s2cnn_[a-z0-9_]+)\s*\(", text)))
    assert names == ["s2cnn_so3_fft64_probe"]
    for n in names:
        assert not hasattr(lib, n) and n not in _hip.SIGNATURES
    if os.path.exists(_hip.PROBE_LIB_PATH):
        probe = _hip.probe_lib()
        fake, null = ctypes.c_void_p(0x1000), ctypes.c_void_p(0)
        assert probe.s2cnn_so3_fft64_probe(fake, fake, fake, fake, 1 << 30, 2, 1, 3, null) == -1     # there is no probe 3
        assert probe.s2cnn_so3_fft64_probe(fake, fake, fake, fake, 0, 2, 0, 1, null) == -2           # workspace too small


def test_argument_rejection_without_gpu():
    from s2cnn_amd import _hip
    lib = _hip.lib()
    null = ctypes.c_void_p(0)
    assert lib.s2cnn_so3_mm_fwd(null, null, null, 4, 2, 3, 5, null) == -1
    assert lib.s2cnn_s2_mm_fwd(null, null, null, 4, 2, 3, 5, null) == -1
    assert lib.s2cnn_so3_analysis(null, null, null, null, null, 0, 4, 4, 1, 0, null) == -1
    assert lib.s2cnn_so3_integrate(null, null, null, 4, 1, null) == -1
    fake = ctypes.c_void_p(0x1000)
    assert lib.s2cnn_so3_mm_fwd(fake, fake, fake, 0, 2, 3, 5, null) == -1          # nl < 1
    assert lib.s2cnn_so3_mm_fwd(ctypes.c_void_p(0x1004), fake, fake, 2, 2, 3, 5, null) == -3
    assert lib.s2cnn_so3_analysis(fake, fake, null, fake, null, 0, 4, 4, 1, 0, null) == -2  # no workspace
    assert lib.s2cnn_s2_analysis(fake, fake, fake, fake, 1 << 30, 4, 5, 1, 0, null) == -1  # b_out > b_in
    packed = lib.s2cnn_so3_packed_table_bytes(32, 32, 0)
    assert packed == 32 * 7 * 2 * 512 * 4 * 4                                        # one-kernel path: 32 beta pairs x 7 items x 2 x 512 threads x 4 degrees
    assert lib.s2cnn_so3_analysis_workspace(32, 32, 256, 0) == 256 * 28 * 512 * 16 + packed   # one record per volume (7 items x 4 float4 x 512 threads), no intermediate planes
    assert lib.s2cnn_so3_synthesis_workspace(40, 32, 256, 0) == 256 * 28 * 512 * 16 + packed
    packed16 = lib.s2cnn_so3_packed_table_bytes(16, 16, 0)
    assert packed16 == 16 * 2 * 2 * 256 * 4 * 4                                      # the 32^3 grid has the same path: 16 beta pairs x 2 items x 2 x 256 threads x 4 degrees
    assert lib.s2cnn_so3_packed_table_bytes(12, 16, 1) == packed16
    assert lib.s2cnn_so3_analysis_workspace(16, 16, 256, 0) == 256 * 8 * 256 * 16 + packed16    # records of 2 items x 4 float4 x 256 threads
    assert lib.s2cnn_so3_synthesis_workspace(20, 16, 256, 0) == 256 * 8 * 256 * 16 + packed16
    packed12 = lib.s2cnn_so3_packed_table_bytes(12, 12, 0)
    assert packed12 == 23 * 24 * 256 * 4                                            # small problems of the two-stage path: 16 x 16 table values per beta
    assert lib.s2cnn_so3_packed_table_bytes(12, 12, 1) == 23 * 12 * 16 * 32 * 4        # ... and a 16 x 32 tile per degree in the synthesis
    assert lib.s2cnn_so3_packed_table_bytes(22, 22, 0) == 22 * 3 * 2 * 512 * 4 * 4 == lib.s2cnn_so3_packed_table_bytes(7, 22, 1)     # and the 44^3 grid: 22 beta pairs x 3 items x 2 x 512 threads
    assert lib.s2cnn_so3_analysis_workspace(22, 7, 200, 0) == 200 * 12 * 512 * 16 + 22 * 3 * 2 * 512 * 4 * 4
    assert lib.s2cnn_so3_analysis_workspace(22, 7, 10, 0) == 10 * 4 * 12 * 512 * 16 + 22 * 3 * 2 * 512 * 4 * 4     # few volumes: four workgroups and records per volume
    assert lib.s2cnn_so3_analysis_workspace(16, 16, 100, 0) == 100 * 2 * 8 * 256 * 16 + packed16                    # two
    assert lib.s2cnn_so3_packed_table_bytes(20, 20, 0) == 39 * 40 * 1024 * 4 and lib.s2cnn_so3_packed_table_bytes(20, 20, 1) == 39 * 20 * 2048 * 4
    assert lib.s2cnn_so3_analysis_workspace(12, 12, 256, 0) == 256 * 24 * 23 * 12 * 8 + packed12
    assert lib.s2cnn_so3_relu_bits_bytes(32, 3) == 3 * 64 * 64 * 8 and lib.s2cnn_so3_relu_bits_bytes(16, 3) == 0     # bit masks: the 64^3 grid only
    assert lib.s2cnn_so3_analysis(ctypes.c_void_p(0x1008), fake, fake, fake, null, 0, 32, 32, 1, 0, null) == -3   # 64^3 real input: 16-byte alignment
    assert lib.s2cnn_so3_synthesis_workspace(4, 6, 3, 1) == 16 * 12 * 7 * 7 * 8      # batch padded to the z tile, no fast path
    # more than 32 frequencies / degrees or 64 betas: one packed table per part of the Wigner stage; none beyond 64 / 128
    assert lib.s2cnn_so3_packed_table_bytes(40, 40, 0) == 3 * 79 * 80 * 1024 * 4
    assert lib.s2cnn_so3_packed_table_bytes(32, 40, 1) == 2 * 63 * 32 * 2048 * 4
    assert lib.s2cnn_so3_packed_table_bytes(70, 70, 0) == 0 and lib.s2cnn_so3_packed_table_bytes(70, 70, 1) == 0
    assert lib.s2cnn_so3_pack_table(fake, fake, 70, 70, 0, null) == -1
    assert b"workspace" in lib.s2cnn_strerror(-2)
    # the normalisation inside the transforms: where the loads can do it, and what the entries refuse before any launch
    assert lib.s2cnn_so3_analysis_prologue_available(32, 32) == 1 and lib.s2cnn_so3_analysis_prologue_available(22, 7) == 1
    assert lib.s2cnn_so3_analysis_prologue_available(32, 40) == 0            # 64-point planes outside the per-volume kernels
    assert lib.s2cnn_so3_analysis_real_affine_relu(fake, fake, 3, fake, null, fake, fake, 1 << 30, 32, 40, 3, 0, null) == -1
    assert lib.s2cnn_so3_analysis_real_affine_relu(fake, fake, 3, fake, null, fake, fake, 1 << 30, 22, 22, 4, 0, null) == -1   # 4 volumes, 3 features
    assert lib.s2cnn_so3_analysis_real_bn_relu_grad(fake, null, fake, 3, fake, null, fake, fake, 1 << 30, 22, 22, 3, 0, null) == -1   # no second tensor
    assert lib.s2cnn_volume_moments(null, fake, 3, 8, null) == -1
    assert lib.s2cnn_bn_relu_grad_moments(fake, fake, fake, 2, fake, 3, 8, null) == -1                  # 3 volumes, 2 features
    assert lib.s2cnn_bn_forward_from_moments(fake, 2, 3, 1, 16.0, null, null, null, null, 1e-5, 0.1, 0, fake, fake, null) == -1   # evaluation mode without running statistics
    assert lib.s2cnn_bn_backward_from_moments(fake, 0, 3, 1, 16.0, fake, fake, 1, fake, fake, null) == -1
    # sums per plane out of the synthesis: where it stages whole planes, not on the 64^3 grid
    assert lib.s2cnn_so3_synthesis_moment_parts(20, 20) == 40 and lib.s2cnn_so3_synthesis_moment_parts(7, 20) == 40
    assert lib.s2cnn_so3_synthesis_moment_parts(12, 12) == 24 and lib.s2cnn_so3_synthesis_moment_parts(32, 32) == 0
    assert lib.s2cnn_so3_synthesis_moment_parts(16, 16) == 1 and lib.s2cnn_so3_synthesis_moment_parts(10, 16) == 1      # per volume on the 32^3 grid
    assert lib.s2cnn_so3_synthesis_moment_parts(22, 22) == 1 and lib.s2cnn_so3_synthesis_moment_parts(7, 22) == 1       # ... and on the 44^3 grid
    assert lib.s2cnn_so3_synthesis_real_moments(fake, fake, null, fake, fake, 1 << 30, 32, 32, 3, null, 1, fake, null, null, null) == -1
    assert lib.s2cnn_so3_synthesis_real_moments(fake, fake, null, fake, fake, 1 << 30, 22, 22, 4, null, 3, fake, fake, fake, null) == -1   # 4 volumes, 3 features
    assert lib.s2cnn_so3_synthesis_real_basis_moment_parts(32, 32, 0) == 1 and lib.s2cnn_so3_synthesis_real_basis_moment_parts(32, 32, 1) == 0
    assert lib.s2cnn_so3_synthesis_real_basis_moment_parts(22, 32, 1) == 1 and lib.s2cnn_so3_synthesis_real_basis_moment_parts(20, 20, 0) == 40
    assert lib.s2cnn_so3_synthesis_real_basis_moment_parts(22, 22, 0) == 1 and lib.s2cnn_so3_synthesis_real_basis_moment_parts(22, 22, 1) == 1
    assert lib.s2cnn_so3_synthesis_real_basis_moment_parts(70, 70, 0) == 0
    assert lib.s2cnn_so3_synthesis_real_basis_moments(fake, fake, null, fake, fake, 1 << 30, 70, 70, 3, null, 1, fake, null, null, null) == -1    # no tiled stage at this size
    assert lib.s2cnn_so3_synthesis_real_basis_moments(fake, fake, null, fake, fake, 1 << 30, 32, 32, 3, null, 1, null, null, null, null) == -1    # nowhere to write the sums
    assert lib.s2cnn_so3_synthesis_real_basis_moments(fake, fake, null, fake, fake, 1 << 30, 32, 32, 3, null, 3, fake, fake, fake, null) == -1    # all 32 degrees with a second tensor
    assert lib.s2cnn_so3_integrate_affine_relu(fake, fake, 2, fake, fake, 4, 3, null) == -1              # 3 volumes, 2 features
    # entry points of the real-basis path and the biased synthesis
    assert lib.s2cnn_s2_mm_real_fwd(null, null, null, 4, 2, 3, 5, null) == -1
    assert lib.s2cnn_s2_mm_real_gradx(fake, fake, fake, 4, 0, 3, 5, null) == -1                # empty batch
    assert lib.s2cnn_s2_mm_real_grady(ctypes.c_void_p(0x1002), fake, fake, 4, 2, 3, 5, null) == -3
    assert lib.s2cnn_so3_mm_real_fwd(null, null, null, 4, 2, 3, 5, null) == -1
    assert lib.s2cnn_so3_synthesis_real_bias(null, null, null, null, null, 0, 4, 4, 1, null, 1, null) == -1
    assert lib.s2cnn_so3_synthesis_real_bias(fake, fake, null, fake, fake, 1 << 30, 4, 4, 6, fake, 4, null) == -1   # 6 volumes, 4 features
    assert lib.s2cnn_so3_synthesis_real_basis(fake, fake, null, fake, fake, 1 << 30, 70, 70, 1, null, 1, null) == -1  # no direct kernel for this grid
    assert lib.s2cnn_so3_real_basis_transform_available(32, 22, 0) == 1 and lib.s2cnn_so3_real_basis_transform_available(22, 22, 0) == 1
    assert lib.s2cnn_so3_real_basis_transform_available(40, 36, 0) == 0          # a spectrum of more than 32 degrees: several parts
    assert lib.s2cnn_so3_real_basis_transform_available(22, 22, 1) == 1 and lib.s2cnn_so3_real_basis_transform_available(70, 70, 1) == 0
    assert lib.s2cnn_so3_rft_expand_real(null, null, null, 4, 3, 8, null) == -1
    # relu in the epilogue of the synthesis, its mask in the loads of the analysis
    assert lib.s2cnn_so3_synthesis_real_relu(null, null, null, null, null, 0, 4, 4, 1, null, 1, 0, null) == -1
    assert lib.s2cnn_so3_synthesis_real_relu(fake, fake, null, fake, fake, 1 << 30, 4, 4, 6, fake, 4, 0, null) == -1    # 6 volumes, 4 features
    assert lib.s2cnn_so3_synthesis_real_relu(fake, fake, null, fake, fake, 1 << 30, 70, 70, 1, null, 1, 1, null) == -1    # no real-basis kernel for this grid
    assert lib.s2cnn_so3_analysis_real_masked(fake, null, fake, null, fake, fake, 1 << 30, 4, 4, 1, 0, null) == -1      # no mask
    assert lib.s2cnn_so3_analysis_real_masked(fake, fake, fake, null, fake, fake, 1 << 30, 40, 36, 1, 1, null) == -1    # no real-basis kernel for this size
    assert lib.s2cnn_so3_analysis_real_masked(fake, fake, fake, null, fake, null, 0, 4, 4, 1, 0, null) == -2            # no workspace


def test_product_has_no_cpu_path():
    import torch
    import s2cnn_amd
    from s2cnn_amd.soft.so3_fft import so3_rfft
    with pytest.raises(RuntimeError, match="no CPU path"):
        so3_rfft(torch.zeros(4, 4, 4))
    with pytest.raises(RuntimeError, match="no CPU path"):
        s2cnn_amd.so3_mm(torch.zeros(1, 1, 1, 2), torch.zeros(1, 1, 1, 2))
    with pytest.raises(RuntimeError, match="no CPU path"):
        s2cnn_amd.so3_integrate(torch.zeros(2, 4, 4, 4))


def test_product_does_not_import_oracle():
    import subprocess
    import sys
    code = ("import sys; sys.path.insert(0, %r); import s2cnn_amd, s2cnn_amd.soft.so3_fft, s2cnn_amd.soft.s2_fft; "
            "assert not any(m == 'oracle' or m.startswith('oracle.') for m in sys.modules)" % ROOT)
    subprocess.run([sys.executable, "-c", code], check=True)
    for dirpath, _, files in os.walk(os.path.join(ROOT, "s2cnn_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                assert "oracle" not in open(os.path.join(dirpath, f)).read(), f
