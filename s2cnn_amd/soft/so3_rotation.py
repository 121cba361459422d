"""Rotation of a signal on SO(3) in the spectral domain: mirrors s2cnn/soft/so3_rotation.py of the
reference (fft -> per-degree product with conj(U^l) -> ifft).  The transforms are the HIP kernels, and the
per-degree products are ONE call of the block product so3_mm with a single feature on either side:
with F' = conj(U) F per degree,  F'[m, n] = sum_p F[p, n] conj(U[m, p]) = so3_mm(F^T, U)[n, m]."""
from functools import lru_cache

import numpy as np
import torch

from .. import wigner
from ..so3_mm import so3_mm
from .so3_fft import SO3_fft_real, SO3_ifft_real


@lru_cache(maxsize=32)
def _setup_so3_rotation(b, alpha, beta, gamma, device):
    """U^l[m, n] = exp(i m alpha) d^l_mn(beta) exp(i n gamma) for l < b (s2cnn/soft/so3_rotation.py:52-72), laid out as
    the kernel operand of so3_mm, [l * m * n, 1, 1, complex], and the index map that transposes every (2l+1)^2 block."""
    Us = [wigner.wigner_D(l, alpha, beta, gamma)[0].astype(np.complex64).reshape(-1) for l in range(b)]
    U = torch.view_as_real(torch.tensor(np.concatenate(Us), device=device)).reshape(-1, 1, 1, 2).contiguous()
    perm, begin = [], 0
    for l in range(b):
        L = 2 * l + 1
        perm.append(begin + np.arange(L * L).reshape(L, L).T.reshape(-1))
        begin += L * L
    return U, torch.tensor(np.concatenate(perm), dtype=torch.long, device=device)


def so3_rotation(x, alpha, beta, gamma):
    '''
    :param x: [..., beta, alpha, gamma] (..., 2b, 2b, 2b)
    '''
    b = x.size()[-1] // 2
    x_size = x.size()
    U, transpose = _setup_so3_rotation(b, float(alpha), float(beta), float(gamma), x.device)

    x = SO3_fft_real.apply(x)  # [l * m * n, ..., complex]
    Fx = x.reshape(x.size(0), -1, 1, 2).index_select(0, transpose)  # [l * n * m, batch, 1, complex]
    Fz = so3_mm(Fx, U).index_select(0, transpose)  # [l * m * n, batch, 1, complex]
    z = SO3_ifft_real.apply(Fz.reshape(x.size()).contiguous())
    return z.contiguous().view(*x_size)
