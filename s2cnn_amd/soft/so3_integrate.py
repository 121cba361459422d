"""Haar integral over SO(3): mirrors s2cnn/soft/so3_integrate.py of the reference."""
from functools import lru_cache

import torch

from .. import _hip, wigner


@lru_cache(maxsize=32)
def _setup_so3_integrate(b, device):
    return torch.tensor(wigner.quadrature_weights(b), dtype=torch.float32, device=device)  # [beta]


class _SO3_integrate(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        _hip.require_gpu_f32(x)
        b = x.size(-1) // 2
        ctx.b = b
        ctx.shape = x.size()
        lead = x.size()[:-3]
        n = 1
        for d in lead:
            n *= d
        x = x.contiguous().view(n, 2 * b, 2 * b, 2 * b)
        w = _setup_so3_integrate(b, x.device)
        out = x.new_empty((x.size(0),))
        if x.size(0) == 0:
            return out.view(*lead)
        _hip.call("s2cnn_so3_integrate", _hip.ptr(x), _hip.ptr(w), _hip.ptr(out), b, x.size(0),
                  _hip.stream_ptr())
        return out.view(*lead)

    @staticmethod
    def backward(ctx, g):
        b = ctx.b
        g = g.contiguous().view(g.numel())
        w = _setup_so3_integrate(b, g.device)
        gx = g.new_empty((g.numel(), 2 * b, 2 * b, 2 * b))
        if g.numel() == 0:
            return gx.view(ctx.shape)
        _hip.call("s2cnn_so3_integrate_grad", _hip.ptr(g), _hip.ptr(w), _hip.ptr(gx), b, g.numel(),
                  _hip.stream_ptr())
        return gx.view(ctx.shape)


def so3_integrate(x):
    """
    Integrate a signal on SO(3) using the Haar measure

    :param x: [..., beta, alpha, gamma] (..., 2b, 2b, 2b)
    :return y: [...] (...)
    """
    assert x.size(-1) == x.size(-2)
    assert x.size(-2) == x.size(-3)
    return _SO3_integrate.apply(x)
