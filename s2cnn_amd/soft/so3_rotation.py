"""Rotation of a signal on SO(3) in the spectral domain: mirrors s2cnn/soft/so3_rotation.py of the
reference (fft -> per-degree product with conj(U^l) -> ifft).  The transforms are the HIP kernels; the
per-degree products are small dense complex matrix products and stay library GEMMs (torch.matmul)."""
from functools import lru_cache

import numpy as np
import torch

from .. import wigner
from .so3_fft import SO3_fft_real, SO3_ifft_real


@lru_cache(maxsize=32)
def _setup_so3_rotation(b, alpha, beta, gamma, device):
    """U^l[m, n] = exp(i m alpha) d^l_mn(beta) exp(i n gamma) for l < b, as complex64 tensors
    (s2cnn/soft/so3_rotation.py:52-72)."""
    Us = [wigner.wigner_D(l, alpha, beta, gamma)[0] for l in range(b)]
    return [torch.tensor(U.astype(np.complex64), device=device) for U in Us]


def so3_rotation(x, alpha, beta, gamma):
    '''
    :param x: [..., beta, alpha, gamma] (..., 2b, 2b, 2b)
    '''
    b = x.size()[-1] // 2
    x_size = x.size()
    Us = _setup_so3_rotation(b, float(alpha), float(beta), float(gamma), x.device)

    x = SO3_fft_real.apply(x)  # [l * m * n, ..., complex]
    xc = torch.view_as_complex(x.reshape(x.size(0), -1, 2))  # [l * m * n, batch]

    Fz_list = []
    begin = 0
    for l in range(b):
        L = 2 * l + 1
        size = L ** 2
        Fx = xc[begin:begin + size].reshape(L, -1)  # [m, n * batch]
        Fz = torch.matmul(Us[l].conj(), Fx)  # [m, n * batch]  (complex_mm(U, Fx, conj_x=True) of the reference)
        Fz_list.append(Fz.reshape(size, -1))
        begin += size

    Fz = torch.view_as_real(torch.cat(Fz_list, 0))  # [l * m * n, batch, complex]
    z = SO3_ifft_real.apply(Fz.contiguous())
    return z.contiguous().view(*x_size)
