"""S^2 x S^2 -> SO(3) spectral product: mirrors s2cnn/s2_mm.py of the reference."""
import torch

from . import _hip


class _S2_mm(torch.autograd.Function):
    """Same contract as the reference's _cuda_S2_mm (s2cnn/s2_mm.py:61-137)."""

    @staticmethod
    def forward(ctx, x, y):
        assert y.size(3) == 2
        assert x.size(3) == 2
        nbatch, f_in, f_out = x.size(1), x.size(2), y.size(2)
        assert y.size(1) == f_in
        assert y.size(0) == x.size(0)
        nl = round(x.size(0) ** 0.5)
        assert x.size(0) == nl ** 2
        _hip.require_gpu_f32(x, y)
        nspec = (4 * nl ** 2 - 1) * nl // 3
        x = x.contiguous()
        y = y.contiguous()
        ctx.save_for_backward(x, y)
        z = x.new_empty((nspec, nbatch, f_out, 2))
        if nbatch > 0:
            _hip.call("s2cnn_s2_mm_fwd", _hip.ptr(x), _hip.ptr(y), _hip.ptr(z), nl, nbatch, f_in, f_out,
                      _hip.stream_ptr())
        return z

    @staticmethod
    def backward(ctx, gz):
        x, y = ctx.saved_tensors
        nl = round(x.size(0) ** 0.5)
        nbatch, f_in, f_out = x.size(1), x.size(2), y.size(2)
        gz = gz.contiguous()
        gx = gy = None
        if ctx.needs_input_grad[0]:
            gx = gz.new_empty((nl ** 2, nbatch, f_in, 2))
            if nbatch > 0:
                _hip.call("s2cnn_s2_mm_gradx", _hip.ptr(gz), _hip.ptr(y), _hip.ptr(gx), nl, nbatch, f_in, f_out,
                          _hip.stream_ptr())
        if ctx.needs_input_grad[1]:
            gy = gz.new_empty((nl ** 2, f_in, f_out, 2))
            if nbatch > 0:
                _hip.call("s2cnn_s2_mm_grady", _hip.ptr(gz), _hip.ptr(x), _hip.ptr(gy), nl, nbatch, f_in, f_out,
                          _hip.stream_ptr())
            else:
                gy.zero_()
        return gx, gy


def s2_mm(x, y):
    '''
    :param x: [l * m,     batch,      feature_in,  complex]
    :param y: [l * m,     feature_in, feature_out, complex]
    :return:  [l * m * n, batch,      feature_out, complex]
    '''
    return _S2_mm.apply(x, y)
