"""Block-diagonal spectral product on SO(3): mirrors s2cnn/so3_mm.py of the reference."""
import torch

from . import _hip


def _nl_from_nspec(nspec):
    nl = round((3 / 4 * nspec) ** (1 / 3))
    assert nspec == nl * (4 * nl ** 2 - 1) // 3
    return nl


class _SO3_mm(torch.autograd.Function):
    """Same contract as the reference's _cuda_SO3_mm (s2cnn/so3_mm.py:64-122)."""

    @staticmethod
    def forward(ctx, x, y):
        assert y.size(3) == 2
        assert x.size(3) == 2
        nspec, nbatch, f_in = x.size(0), x.size(1), x.size(2)
        f_out = y.size(2)
        assert y.size(1) == f_in
        assert y.size(0) == nspec
        nl = _nl_from_nspec(nspec)
        _hip.require_gpu_f32(x, y)
        x = x.contiguous()
        y = y.contiguous()
        ctx.save_for_backward(x, y)
        z = x.new_empty((nspec, nbatch, f_out, 2))
        if nbatch > 0:
            _hip.call("s2cnn_so3_mm_fwd", _hip.ptr(x), _hip.ptr(y), _hip.ptr(z), nl, nbatch, f_in, f_out,
                      _hip.stream_ptr())
        return z

    @staticmethod
    def backward(ctx, gz):
        x, y = ctx.saved_tensors
        nspec, nbatch, f_in = x.size(0), x.size(1), x.size(2)
        f_out = y.size(2)
        nl = _nl_from_nspec(nspec)
        gz = gz.contiguous()
        gx = gy = None
        if ctx.needs_input_grad[0]:
            gx = gz.new_empty((nspec, nbatch, f_in, 2))
            if nbatch > 0:
                _hip.call("s2cnn_so3_mm_gradx", _hip.ptr(gz), _hip.ptr(y), _hip.ptr(gx), nl, nbatch, f_in, f_out,
                          _hip.stream_ptr())
        if ctx.needs_input_grad[1]:
            gy = gz.new_empty((nspec, f_in, f_out, 2))
            if nbatch > 0:
                _hip.call("s2cnn_so3_mm_grady", _hip.ptr(gz), _hip.ptr(x), _hip.ptr(gy), nl, nbatch, f_in, f_out,
                          _hip.stream_ptr())
            else:
                gy.zero_()
        return gx, gy


def so3_mm(x, y):
    '''
    :param x: [l * m * n,   batch,    feature_in,  complex]
    :param y: [l * m * n, feature_in, feature_out, complex]
    :return:  [l * m * n,   batch,    feature_out, complex]
    '''
    return _SO3_mm.apply(x, y)
