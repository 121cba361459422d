"""S^2 Fourier transforms on the SOFT grid: mirrors s2cnn/soft/s2_fft.py of the reference."""
from functools import lru_cache

import torch

from .. import _hip, wigner


@lru_cache(maxsize=32)
def _setup_wigner(b, nl, weighted, device):
    """[2b, nl^2] float32 on `device` (s2cnn/soft/s2_fft.py:109-147)."""
    dss = wigner.s2_wigner_table(b, nl, bool(weighted))
    return torch.tensor(dss, dtype=torch.float32, device=device).contiguous()


def _analysis(x, b_in, b_out, for_grad, complex_in):
    _hip.require_gpu_f32(x)
    L = _hip.lib()
    nbatch = x.size(0)
    table = _setup_wigner(b_in, nl=b_out, weighted=not for_grad, device=x.device)
    out = x.new_empty((b_out ** 2, nbatch, 2))
    if nbatch == 0:
        return out
    ws = _hip.workspace(L.s2cnn_s2_analysis_workspace(b_in, b_out, nbatch, complex_in), x.device)
    _hip.call("s2cnn_s2_analysis", _hip.ptr(x), _hip.ptr(table), _hip.ptr(out), _hip.ptr(ws), ws.numel(),
                  b_in, b_out, nbatch, complex_in, _hip.stream_ptr())
    return out


def _synthesis(x, b_in, b_out, for_grad, complex_out):
    _hip.require_gpu_f32(x)
    L = _hip.lib()
    nbatch = x.size(1)
    table = _setup_wigner(b_out, nl=b_in, weighted=for_grad, device=x.device)
    out = x.new_empty((nbatch, 2 * b_out, 2 * b_out) + ((2,) if complex_out else ()))
    if nbatch == 0:
        return out
    ws = _hip.workspace(L.s2cnn_s2_synthesis_workspace(b_in, b_out, nbatch, complex_out), x.device)
    _hip.call("s2cnn_s2_synthesis", _hip.ptr(x), _hip.ptr(table), _hip.ptr(out), _hip.ptr(ws), ws.numel(),
                  b_in, b_out, nbatch, complex_out, _hip.stream_ptr())
    return out


def _count(sizes):
    """Product of the batch dimensions (explicit, so that views of empty batches are not ambiguous)."""
    n = 1
    for d in sizes:
        n *= d
    return n


def _grid_args(x, b_out, complex_in):
    off = 1 if complex_in else 0
    b_in = x.size(-1 - off) // 2
    assert x.size(-1 - off) == 2 * b_in
    assert x.size(-2 - off) == 2 * b_in
    if b_out is None:
        b_out = b_in
    assert b_out <= b_in
    batch_size = x.size()[:x.dim() - 2 - off]
    return b_in, b_out, batch_size


def s2_fft(x, for_grad=False, b_out=None):
    '''
    :param x: [..., beta, alpha, complex]
    :return:  [l * m, ..., complex]
    '''
    assert x.size(-1) == 2
    b_in, b_out, batch_size = _grid_args(x, b_out, True)
    x = x.contiguous().view(_count(batch_size), 2 * b_in, 2 * b_in, 2)
    return _analysis(x, b_in, b_out, for_grad, 1).view(b_out ** 2, *batch_size, 2)


def s2_rfft(x, for_grad=False, b_out=None):
    '''
    s2_fft of a real signal without materialising the zero imaginary part
    (what S2_fft_real does through as_complex at s2cnn/soft/s2_fft.py:226-232).
    :param x: [..., beta, alpha]
    :return:  [l * m, ..., complex]
    '''
    b_in, b_out, batch_size = _grid_args(x, b_out, False)
    x = x.contiguous().view(_count(batch_size), 2 * b_in, 2 * b_in)
    return _analysis(x, b_in, b_out, for_grad, 0).view(b_out ** 2, *batch_size, 2)


def _spectrum_args(x, b_out):
    assert x.size(-1) == 2
    nspec = x.size(0)
    b_in = round(nspec ** 0.5)
    assert nspec == b_in ** 2
    if b_out is None:
        b_out = b_in
    assert b_out >= b_in
    batch_size = x.size()[1:-1]
    return x.contiguous().view(nspec, _count(batch_size), 2), b_in, b_out, batch_size


def s2_ifft(x, for_grad=False, b_out=None):
    '''
    :param x: [l * m, ..., complex]
    :return:  [..., beta, alpha, complex]
    '''
    x, b_in, b_out, batch_size = _spectrum_args(x, b_out)
    return _synthesis(x, b_in, b_out, for_grad, 1).view(*batch_size, 2 * b_out, 2 * b_out, 2)


def s2_rifft(x, for_grad=False, b_out=None):
    '''
    Real part of s2_ifft.
    :param x: [l * m, ..., complex]
    :return:  [..., beta, alpha]
    '''
    x, b_in, b_out, batch_size = _spectrum_args(x, b_out)
    return _synthesis(x, b_in, b_out, for_grad, 0).view(*batch_size, 2 * b_out, 2 * b_out)


class S2_fft_real(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, b_out=None):  # pylint: disable=W
        ctx.b_out = b_out
        ctx.b_in = x.size(-1) // 2
        return s2_rfft(x, b_out=ctx.b_out)

    @staticmethod
    def backward(ctx, grad_output):  # pylint: disable=W
        return s2_rifft(grad_output, for_grad=True, b_out=ctx.b_in), None


class S2_ifft_real(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, b_out=None):  # pylint: disable=W
        nspec = x.size(0)
        ctx.b_out = b_out
        ctx.b_in = round(nspec ** 0.5)
        return s2_rifft(x, b_out=ctx.b_out)

    @staticmethod
    def backward(ctx, grad_output):  # pylint: disable=W
        return s2_rfft(grad_output, for_grad=True, b_out=ctx.b_in), None
