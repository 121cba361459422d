"""Spectrum of a kernel sampled on an arbitrary grid of the sphere: mirrors s2cnn/s2_ft.py of
the reference (one dense real GEMM with conjugated Wigner-D samples of the column n = 0)."""
from functools import lru_cache

import numpy as np
import torch

from . import wigner


@lru_cache(maxsize=32)
def _setup_s2_ft(b, grid, device):
    """F as a real [n_grid, b^2 * 2] matrix, (re, im) interleaved (s2cnn/s2_ft.py:28-60)."""
    F = wigner.s2_ft_matrix(b, grid)
    F = np.stack((F.real, F.imag), axis=-1).reshape(len(grid), -1)
    return torch.tensor(F.astype(np.float32), dtype=torch.float32, device=device)


def s2_rft(x, b, grid):
    """
    Real Fourier Transform
    :param x: [..., beta_alpha]
    :param b: output bandwidth signal
    :param grid: tuple of (beta, alpha) tuples
    :return: [l * m, ..., complex]
    """
    F = _setup_s2_ft(b, grid, x.device)  # [beta_alpha, l * m * complex]
    assert x.size(-1) == F.size(0)
    sz = x.size()
    out = torch.matmul(F.t(), x.reshape(-1, sz[-1]).t())
    out = out.view(-1, 2, out.size(-1)).transpose(1, 2).contiguous()
    return out.view(-1, *sz[:-1], 2)
