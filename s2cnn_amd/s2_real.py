"""S^2 spectral operands of the S^2 convolution for real signals, in the real basis.

The reference forms z[l,m,n] = x[l,m] conj(y[l,n]) on complex spectra (s2cnn/s2_mm.py, called from
s2cnn/soft/s2_conv.py:47-52).  The spectrum of a real signal on the sphere and the spectrum of a real kernel
(s2cnn/s2_ft.py:4-25) obey x[l,-m] = (-1)^m conj(x[l,m]); the basis change of s2cnn_amd.so3_real then maps them
to REAL vectors (row +m: sqrt2 Re x[l,m], row -m: sqrt2 Im x[l,m], row 0: x[l,0]) and their outer product to the
real-basis SO(3) spectrum, with half the bytes of the complex product.  No counterpart in the reference; the
layer's results are the same.
"""
from functools import lru_cache
import math

import numpy as np
import torch

from . import _hip, wigner


@lru_cache(maxsize=32)
def _real_rows(nl, device):
    """For every real row (l, r): the spectral row (l, |r|) it is read from, and its weights on the real and the
    imaginary part."""
    src = np.empty(nl * nl, dtype=np.int64)
    w = np.zeros((nl * nl, 2), dtype=np.float32)
    for l in range(nl):
        for r in range(-l, l + 1):
            o = l * l + l + r
            src[o] = l * l + l + abs(r)
            if r == 0:
                w[o, 0] = 1.0
            else:
                w[o, 0 if r > 0 else 1] = math.sqrt(2.0)
    return torch.tensor(src, device=device), torch.tensor(w, device=device)


def s2_spectrum_to_real(x):
    """[l * m, ..., complex] -> [l * m, ...]: Re(U x) per degree (exact for the spectrum of a real signal).
    Plain tensor operations (the S^2 spectra of the layer are small); autograd supplies the adjoint."""
    assert x.size(-1) == 2
    nl = round(x.size(0) ** 0.5)
    assert x.size(0) == nl * nl
    src, w = _real_rows(nl, x.device)
    w = w.reshape(nl * nl, *([1] * (x.dim() - 2)), 2)
    return (x.index_select(0, src) * w).sum(-1)


@lru_cache(maxsize=32)
def _setup_s2_ft_real(b, grid, device):
    F = wigner.s2_ft_matrix(b, grid)                       # [n_grid, b^2] complex
    out = np.empty(F.shape, dtype=np.float64)
    for l in range(b):
        for r in range(-l, l + 1):
            col = F[:, l * l + l + abs(r)]
            out[:, l * l + l + r] = col.real if r == 0 else math.sqrt(2.0) * (col.real if r > 0 else col.imag)
    return torch.tensor(out.astype(np.float32), dtype=torch.float32, device=device)


def s2_rft_real(x, b, grid):
    """
    s2_rft followed by s2_spectrum_to_real, as one real product with the transformed matrix
    :param x: [..., beta_alpha]
    :return: [l * m, ...]
    """
    F = _setup_s2_ft_real(b, tuple(grid), x.device)        # [beta_alpha, l * m]
    assert x.size(-1) == F.size(0)
    sz = x.size()
    out = torch.matmul(F.t(), x.reshape(-1, sz[-1]).t())
    return out.view(-1, *sz[:-1])


class _S2_mm_real(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, y):
        _hip.require_gpu_f32(x, y)
        assert x.dim() == 3 and y.dim() == 3
        nbatch, f_in, f_out = x.size(1), x.size(2), y.size(2)
        assert y.size(1) == f_in
        assert y.size(0) == x.size(0)
        nl = round(x.size(0) ** 0.5)
        assert x.size(0) == nl ** 2
        nspec = (4 * nl ** 2 - 1) * nl // 3
        x = x.contiguous()
        y = y.contiguous()
        ctx.save_for_backward(x, y)
        z = x.new_empty((nspec, nbatch, f_out))
        if nbatch > 0:
            _hip.call("s2cnn_s2_mm_real_fwd", _hip.ptr(x), _hip.ptr(y), _hip.ptr(z), nl, nbatch, f_in, f_out, _hip.stream_ptr())
        return z

    @staticmethod
    def backward(ctx, gz):
        x, y = ctx.saved_tensors
        nl = round(x.size(0) ** 0.5)
        nbatch, f_in, f_out = x.size(1), x.size(2), y.size(2)
        gz = gz.contiguous()
        gx = gy = None
        if ctx.needs_input_grad[0]:
            gx = gz.new_empty((nl ** 2, nbatch, f_in))
            if nbatch > 0:
                _hip.call("s2cnn_s2_mm_real_gradx", _hip.ptr(gz), _hip.ptr(y), _hip.ptr(gx), nl, nbatch, f_in, f_out, _hip.stream_ptr())
        if ctx.needs_input_grad[1]:
            gy = gz.new_empty((nl ** 2, f_in, f_out))
            if nbatch > 0:
                _hip.call("s2cnn_s2_mm_real_grady", _hip.ptr(gz), _hip.ptr(x), _hip.ptr(gy), nl, nbatch, f_in, f_out, _hip.stream_ptr())
            else:
                gy.zero_()
        return gx, gy


def s2_mm_real(x, y):
    '''
    :param x: [l * m,     batch,      feature_in ]  real-basis S^2 spectrum
    :param y: [l * m,     feature_in, feature_out]  real-basis S^2 spectrum
    :return:  [l * m * n, batch,      feature_out]  real-basis SO(3) spectrum of s2_mm of the complex spectra
    '''
    return _S2_mm_real.apply(x, y)
