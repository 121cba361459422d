"""SO(3) spectral products for real signals, in the real basis.

The reference multiplies complex spectra (s2cnn/so3_mm.py) although everything the convolution layer
(s2cnn/soft/so3_conv.py:36-56) feeds to the product - the spectrum of a real signal, the spectrum of
a real kernel (s2cnn/so3_ft.py:4-25) and every gradient between them - obeys
X[l,-m,-n] = (-1)^(m-n) conj(X[l,m,n]).  A fixed unitary change of basis per degree makes such
spectra real and turns the complex block product into a real one with a quarter of the multiply-adds.
These functions have no counterpart in the reference; the layer's results are the same.
"""
from functools import lru_cache

import numpy as np
import torch

from . import _hip, wigner
from .so3_mm import _nl_from_nspec


def _convert(name, x, out_shape):
    nspec = x.size(0)
    nl = _nl_from_nspec(nspec)
    out = x.new_empty(out_shape)
    ncols = out.numel() // out.size(0) // (2 if name.endswith("to_complex") else 1)
    if ncols == 0:
        return out
    _hip.call(name, _hip.ptr(x), _hip.ptr(out), nl, ncols, _hip.stream_ptr())
    return out


class _ToReal(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        _hip.require_gpu_f32(x)
        assert x.size(-1) == 2
        return _convert("s2cnn_so3_spectrum_to_real", x.contiguous(), x.shape[:-1])

    @staticmethod
    def backward(ctx, g):
        return _convert("s2cnn_so3_spectrum_to_complex", g.contiguous(), (*g.shape, 2))


class _ToComplex(torch.autograd.Function):
    @staticmethod
    def forward(ctx, r):
        _hip.require_gpu_f32(r)
        return _convert("s2cnn_so3_spectrum_to_complex", r.contiguous(), (*r.shape, 2))

    @staticmethod
    def backward(ctx, g):
        return _convert("s2cnn_so3_spectrum_to_real", g.contiguous(), g.shape[:-1])


def so3_spectrum_to_real(x):
    """[l * m * n, ..., complex] -> [l * m * n, ...]: Re(U x U^H) per degree (exact for the spectrum of a real signal)."""
    return _ToReal.apply(x)


def so3_spectrum_to_complex(r):
    """[l * m * n, ...] -> [l * m * n, ..., complex]: U^H r U per degree, the inverse of so3_spectrum_to_real."""
    return _ToComplex.apply(r)


class _SO3_mm_real(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, y):
        _hip.require_gpu_f32(x, y)
        assert x.dim() == 3 and y.dim() == 3
        nspec, nbatch, f_in = x.size()
        f_out = y.size(2)
        assert y.size(1) == f_in
        assert y.size(0) == nspec
        nl = _nl_from_nspec(nspec)
        x = x.contiguous()
        y = y.contiguous()
        ctx.save_for_backward(x, y)
        z = x.new_empty((nspec, nbatch, f_out))
        if nbatch > 0:
            _hip.call("s2cnn_so3_mm_real_fwd", _hip.ptr(x), _hip.ptr(y), _hip.ptr(z), nl, nbatch, f_in, f_out,
                      _hip.stream_ptr())
        return z

    @staticmethod
    def backward(ctx, gz):
        x, y = ctx.saved_tensors
        nspec, nbatch, f_in = x.size()
        f_out = y.size(2)
        nl = _nl_from_nspec(nspec)
        gz = gz.contiguous()
        gx = gy = None
        if ctx.needs_input_grad[0]:
            gx = gz.new_empty((nspec, nbatch, f_in))
            if nbatch > 0:
                _hip.call("s2cnn_so3_mm_real_gradx", _hip.ptr(gz), _hip.ptr(y), _hip.ptr(gx), nl, nbatch, f_in, f_out,
                          _hip.stream_ptr())
        if ctx.needs_input_grad[1]:
            gy = gz.new_empty((nspec, f_in, f_out))
            if nbatch > 0:
                _hip.call("s2cnn_so3_mm_real_grady", _hip.ptr(gz), _hip.ptr(x), _hip.ptr(gy), nl, nbatch, f_in, f_out,
                          _hip.stream_ptr())
            else:
                gy.zero_()
        return gx, gy


def so3_mm_real(x, y):
    '''
    :param x: [l * m * n,   batch,    feature_in ]  real-basis spectrum
    :param y: [l * m * n, feature_in, feature_out]  real-basis spectrum
    :return:  [l * m * n,   batch,    feature_out]  real-basis spectrum of so3_mm of the complex spectra
    '''
    return _SO3_mm_real.apply(x, y)


@lru_cache(maxsize=32)
def _setup_so3_ft_real(b, grid, device):
    F = wigner.so3_ft_matrix_real(b, grid)
    return torch.tensor(F.astype(np.float32), dtype=torch.float32, device=device)


@lru_cache(maxsize=32)
def _setup_so3_rft_plan(b, grid, device):
    """Factorised form of the matrix of `_setup_so3_ft_real` for grids with few distinct beta values
    (wigner.so3_rft_plan); None where it does not apply."""
    plan = wigner.so3_rft_plan(b, grid)
    if plan is None:
        return None
    idx, E, dtab = plan
    valid = torch.tensor(idx >= 0, device=device)
    sel = np.flatnonzero(idx.reshape(-1) >= 0)       # positions of the grid points in the padded [nbeta * P] layout
    return (torch.tensor(np.maximum(idx, 0), dtype=torch.long, device=device), valid,
            torch.tensor(E.astype(np.float32), device=device).contiguous(),
            torch.tensor(dtab.astype(np.float32), device=device).contiguous(),
            torch.tensor(sel, dtype=torch.long, device=device),
            torch.tensor(idx.reshape(-1)[sel], dtype=torch.long, device=device))


class _SO3RftRealFactorised(torch.autograd.Function):
    """x [ncols, n_grid] -> y [nspec, ncols]: plane coefficients per beta group by a batched GEMM, then the
    expansion over the degrees (s2cnn_so3_rft_expand_real) and its adjoint."""
    @staticmethod
    def forward(ctx, x2, b, plan, complex_out=False):
        idx, valid, E, dtab = plan[:4]
        _hip.require_gpu_f32(x2)
        ncols = x2.size(0)
        with torch.autocast(device_type="cuda", enabled=False):  # the expansion kernel reads G as float32
            xg = x2.t()[idx] * valid.unsqueeze(-1)                # [nbeta, P, ncols]
            G = torch.bmm(E.transpose(1, 2), xg).contiguous()    # [nbeta, R, ncols]
        _hip.require_gpu_f32(G)
        nspec = b * (4 * b * b - 1) // 3
        y = x2.new_empty((nspec, ncols, 2) if complex_out else (nspec, ncols))
        _hip.call("s2cnn_so3_rft_expand" if complex_out else "s2cnn_so3_rft_expand_real",
                  _hip.ptr(G), _hip.ptr(dtab), _hip.ptr(y), b, idx.size(0), ncols, _hip.stream_ptr())
        ctx.plan, ctx.b, ctx.n_grid, ctx.complex_out = plan, b, x2.size(1), complex_out
        return y

    @staticmethod
    def backward(ctx, gy):
        idx, valid, E, dtab, sel, idx_sel = ctx.plan
        gy = gy.contiguous()
        if ctx.complex_out:      # the adjoint of the change of basis, then the adjoint of the real-basis expansion
            _hip.require_gpu_f32(gy)
            gy = _convert("s2cnn_so3_spectrum_to_real", gy, gy.shape[:-1])
        _hip.require_gpu_f32(gy)
        ncols = gy.size(1)
        gG = gy.new_empty((idx.size(0), E.size(2), ncols))
        _hip.call("s2cnn_so3_rft_expand_real_grad", _hip.ptr(gy), _hip.ptr(dtab), _hip.ptr(gG), ctx.b, idx.size(0), ncols, _hip.stream_ptr())
        with torch.autocast(device_type="cuda", enabled=False):
            gxg = torch.bmm(E, gG)                                # [nbeta, P, ncols]
        gx = gy.new_zeros((ctx.n_grid, ncols))
        gx.index_add_(0, idx_sel, gxg.reshape(-1, ncols).index_select(0, sel))   # no boolean masks: they would sync with the host
        return gx.t(), None, None, None


def so3_rft_complex(x, b, grid):
    """
    so3_rft (s2cnn/so3_ft.py:8-24) of a real kernel on a grid with few distinct beta values: the factorised transform with
    its expansion written as complex pairs; None where the factorisation does not apply (the caller takes the dense product)
    :param x: [..., beta_alpha_gamma]
    :return: [l * m * n, ..., complex] or None
    """
    sz = x.size()
    ncols = x.numel() // sz[-1]
    if not (x.is_cuda and x.dtype == torch.float32 and ncols % 4 == 0):
        return None
    plan = _setup_so3_rft_plan(b, tuple(grid), x.device)
    if plan is None:
        return None
    assert sz[-1] == len(grid)
    out = _SO3RftRealFactorised.apply(x.reshape(-1, sz[-1]), b, plan, True)
    return out.view(-1, *sz[:-1], 2)


def so3_rft_real(x, b, grid):
    """
    so3_rft followed by so3_spectrum_to_real, as one real GEMM with the transformed matrix
    :param x: [..., beta_alpha_gamma]
    :return: [l * m * n, ...]
    """
    sz = x.size()
    ncols = x.numel() // sz[-1]
    fast = x.is_cuda and x.dtype == torch.float32 and ncols % 4 == 0 and so3_rft_real.factorised
    plan = _setup_so3_rft_plan(b, tuple(grid), x.device) if fast else None
    if plan is not None:
        assert sz[-1] == len(grid)
        out = _SO3RftRealFactorised.apply(x.reshape(-1, sz[-1]), b, plan)
        return out.view(-1, *sz[:-1])
    F = _setup_so3_ft_real(b, grid, x.device)  # [beta_alpha_gamma, l * m * n]
    assert x.size(-1) == F.size(0)
    out = torch.matmul(F.t(), x.reshape(-1, sz[-1]).t())
    return out.view(-1, *sz[:-1])


so3_rft_real.factorised = True   # False: always the dense product with the [len(grid), nspec] matrix
