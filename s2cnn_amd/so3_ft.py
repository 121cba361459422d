"""Spectrum of a kernel sampled on an arbitrary SO(3) grid (s2cnn/so3_ft.py).  In general one dense real GEMM with a
precomputed matrix of conjugated Wigner-D samples (torch.matmul -> hipBLASLt); grids with few distinct beta values go
through the factorised real-basis transform of s2cnn_amd.so3_real."""
from functools import lru_cache

import numpy as np
import torch

from . import wigner


@lru_cache(maxsize=32)
def _setup_so3_ft(b, grid, device):
    """F as a real [n_grid, nspec(b) * 2] matrix, (re, im) interleaved (s2cnn/so3_ft.py:28-62)."""
    F = wigner.so3_ft_matrix(b, grid)
    F = np.stack((F.real, F.imag), axis=-1).reshape(len(grid), -1)
    return torch.tensor(F.astype(np.float32), dtype=torch.float32, device=device)


def so3_rft(x, b, grid):
    """
    Real Fourier Transform
    :param x: [..., beta_alpha_gamma]
    :param b: output bandwidth signal
    :param grid: tuple of (beta, alpha, gamma) tuples
    :return: [l * m * n, ..., complex]
    """
    sz = x.size()
    if x.is_cuda and so3_rft.factorised:
        # The kernel is real, so its spectrum is that of a real signal: the real-basis transform (factorised over the
        # few distinct beta values of the grid, s2cnn_amd.so3_real) with its last pass written as complex pairs is the
        # same function
        from . import so3_real
        out = so3_real.so3_rft_complex(x, b, tuple(grid))
        if out is not None:
            return out
    F = _setup_so3_ft(b, grid, x.device)  # [beta_alpha_gamma, l * m * n * complex]
    assert x.size(-1) == F.size(0)
    # [spec*2, n_grid] @ [n_grid, rows] -> [spec, 2, rows] -> [spec, rows, 2]
    out = torch.matmul(F.t(), x.reshape(-1, sz[-1]).t())
    out = out.view(-1, 2, out.size(-1)).transpose(1, 2).contiguous()
    return out.view(-1, *sz[:-1], 2)


so3_rft.factorised = True   # False: always the dense product with the [len(grid), nspec * 2] matrix
