"""Batch normalisation and ReLU between two spectral layers without passes of their own over the activations.

The reference's shape networks are nn.Sequential(conv, BatchNorm3d, ReLU, conv, ...) (examples/shrec17/model.py:17-38,
model_original.py:17-38).  Between two layers that is

    y = synthesis(z_hat) + bias                         the first layer's output, [batch, feature, 2b, 2b, 2b]
    u = max(weight (y - mean) / sqrt(var + eps) + bias_bn, 0)
    x_hat = analysis(u)                                 the second layer's input spectrum

Here y is written once and read by the kernels that need it anyway: one read for the two sums per volume that the
statistics are made of, and the analysis of the second layer applies `max(a y + b, 0)` as it loads y
(a = weight / sqrt(var + eps), b = bias_bn - mean a).  Backward, the synthesis that produces the gradient g with respect
to u is followed by one read of (g, y) for the two reductions of the normalisation's backward pass, and the analysis
that carries the gradient on to z_hat forms `a (u > 0 ? g : 0) + p + q y` as it loads g and y.  The module objects, their
parameters and buffers (running statistics, num_batches_tracked) stay those of the reference's models.
"""
import torch
from torch import nn

from .. import _hip
from .so3_conv import SO3Convolution
from .so3_integrate import _setup_so3_integrate, so3_integrate
from .so3_fft import (LoadAffineReLU, LoadBNReLUGrad, analysis_prologue_available, so3_rfft_real_basis,
                      so3_rifft_real_basis)


def _moments(name, n_per_volume, *operands):
    """[volumes, 2] float32: the two sums per volume of s2cnn_volume_moments / s2cnn_bn_relu_grad_moments."""
    first = operands[0]
    nvol = first.numel() // n_per_volume
    out = first.new_empty((nvol, 2))
    args = [_hip.ptr(t) if torch.is_tensor(t) else t for t in operands]
    _hip.call(name, *args, _hip.ptr(out), nvol, n_per_volume, _hip.stream_ptr())
    return out


def _synthesis_and_statistics(ctx, zr, conv_bias, weight, bias, running_mean, running_var, b_grid, eps, training):
    """y = synthesis(zr) + conv_bias, the batch statistics of y and the affine map (a, b) of the normalisation."""
    nspec, batch, nf = zr.shape
    ctx.b_z = round((3 / 4 * nspec) ** (1 / 3))
    ctx.b_grid, ctx.training = b_grid, training
    ctx.bias_shape = conv_bias.shape
    y = so3_rifft_real_basis(zr, b_out=b_grid, bias=conv_bias)                       # [batch, feature, 2b, 2b, 2b]
    nvox = (2 * b_grid) ** 3
    ctx.count = batch * nvox
    s = _moments("s2cnn_volume_moments", nvox, y).view(batch, nf, 2).double().sum(0)    # [feature, 2]
    mean = s[:, 0] / ctx.count
    var = (s[:, 1] / ctx.count - mean * mean).clamp_min(0.0)
    use_mean, use_var = (mean, var) if training else (running_mean.double(), running_var.double())
    invstd = torch.rsqrt(use_var + eps)
    w = weight.double() if weight is not None else torch.ones_like(invstd)
    a = w * invstd
    b = (bias.double() if bias is not None else torch.zeros_like(a)) - use_mean * a
    ab = torch.stack([a, b]).float()
    ctx.save_for_backward(y, ab, use_mean, invstd)
    ctx.has_affine = (weight is not None, bias is not None)
    mean_f, var_f = mean.float(), var.float()
    ctx.mark_non_differentiable(mean_f, var_f)
    return y, ab, mean_f, var_f


def _gradients_from(ctx, g):
    """g: the gradient with respect to u = max(a y + b, 0).  Returns the gradients with respect to the spectrum zr, the
    bias of the layer, and the weight and bias of the normalisation."""
    y, ab, mean, invstd = ctx.saved_tensors
    batch, nf = y.shape[:2]
    nvox = (2 * ctx.b_grid) ** 3
    d = _moments("s2cnn_bn_relu_grad_moments", nvox, g, y, ab, nf).view(batch, nf, 2).double().sum(0)
    d1, d2 = d[:, 0], d[:, 1]                                                        # sum g m, sum g m y
    a = ab[0].double()
    gxhat = invstd * (d2 - mean * d1)                                                # sum g m (y - mean) / std
    if ctx.training:
        k2 = invstd * gxhat / ctx.count
        p = -a * d1 / ctx.count + a * k2 * mean
        q = -a * k2
    else:
        p = torch.zeros_like(a)
        q = torch.zeros_like(a)
    params = torch.stack([a, ab[1].double(), p, q]).float()
    gz = so3_rfft_real_basis(g, for_grad=True, b_out=ctx.b_z, mask=LoadBNReLUGrad(y, params))
    g_conv_bias = gz[0].reshape(-1, nf).sum(0).reshape(ctx.bias_shape) if ctx.needs_input_grad[1] else None
    g_weight = gxhat.to(gz.dtype) if ctx.has_affine[0] else None
    g_bias = d1.to(gz.dtype) if ctx.has_affine[1] else None
    return gz, g_conv_bias, g_weight, g_bias


class _SynthesisBNReLUAnalysis(torch.autograd.Function):
    """z_hat (real-basis spectrum [l m n, batch, feature]) of one layer -> the input spectrum of the next one.
    Returns (x_hat, batch mean, biased batch variance); the statistics are not differentiable outputs (they feed the
    running averages)."""

    @staticmethod
    def forward(ctx, zr, conv_bias, weight, bias, running_mean, running_var, b_grid, b_next, eps, training):  # pylint: disable=W
        y, ab, mean, var = _synthesis_and_statistics(ctx, zr, conv_bias, weight, bias, running_mean, running_var, b_grid, eps, training)
        return so3_rfft_real_basis(y, b_out=b_next, mask=LoadAffineReLU(ab)), mean, var

    @staticmethod
    def backward(ctx, gxh, _gm, _gv):  # pylint: disable=W
        g = so3_rifft_real_basis(gxh.contiguous(), for_grad=True, b_out=ctx.b_grid)      # gradient with respect to u
        return (*_gradients_from(ctx, g), None, None, None, None, None, None)


class _SynthesisBNReLUIntegrate(torch.autograd.Function):
    """z_hat of the last layer -> so3_integrate(max(batch_norm(y), 0)), [batch, feature]: the end of the reference's shape
    network (examples/shrec17/model.py:36-45).  The integral applies the normalisation and the activation in its loads."""

    @staticmethod
    def forward(ctx, zr, conv_bias, weight, bias, running_mean, running_var, b_grid, eps, training):  # pylint: disable=W
        y, ab, mean, var = _synthesis_and_statistics(ctx, zr, conv_bias, weight, bias, running_mean, running_var, b_grid, eps, training)
        batch, nf = y.shape[:2]
        out = y.new_empty((batch, nf))
        _hip.call("s2cnn_so3_integrate_affine_relu", _hip.ptr(y), _hip.ptr(ab), nf, _hip.ptr(_setup_so3_integrate(b_grid, y.device)),
                  _hip.ptr(out), b_grid, batch * nf, _hip.stream_ptr())
        return out, mean, var

    @staticmethod
    def backward(ctx, gout, _gm, _gv):  # pylint: disable=W
        y = ctx.saved_tensors[0]
        g = torch.empty_like(y)                                                          # gradient with respect to u: gout[z] w[beta]
        _hip.call("s2cnn_so3_integrate_grad", _hip.ptr(gout.contiguous()), _hip.ptr(_setup_so3_integrate(ctx.b_grid, y.device)), _hip.ptr(g),
                  ctx.b_grid, gout.numel(), _hip.stream_ptr())
        return (*_gradients_from(ctx, g), None, None, None, None, None)


def _update_running_statistics(bn, mean, var_biased, count):
    """What nn.BatchNorm3d does to its buffers in training mode (unbiased variance, momentum or cumulative average)."""
    if not bn.track_running_stats or bn.running_mean is None:
        return
    with torch.no_grad():
        bn.num_batches_tracked += 1
        momentum = 1.0 / float(bn.num_batches_tracked) if bn.momentum is None else bn.momentum
        unbiased = var_biased * (count / max(count - 1, 1))
        bn.running_mean.mul_(1 - momentum).add_(mean.to(bn.running_mean.dtype), alpha=momentum)
        bn.running_var.mul_(1 - momentum).add_(unbiased.to(bn.running_var.dtype), alpha=momentum)


def _normalised(conv, bn, act):
    return (isinstance(bn, nn.BatchNorm3d) and isinstance(act, nn.ReLU) and conv.real_basis and conv.activation is None
            and conv.nfeature_out == bn.num_features and analysis_prologue_available(conv.b_out, conv.b_out))


def _fusable(conv, bn, act, nxt):
    return (_normalised(conv, bn, act) and isinstance(nxt, SO3Convolution) and nxt.real_basis and nxt.b_in == conv.b_out
            and analysis_prologue_available(nxt.b_in, nxt.b_out))


def run_sequence(sequence, x, integrate=False):
    """`nn.Sequential(conv, [BatchNorm3d, ReLU, SO3Convolution] ..., ...)(x)` with every (BatchNorm3d, ReLU) that stands
    between two spectral layers evaluated inside the transforms of its neighbours.  Same function, same parameters, same
    buffer updates; whatever does not match the pattern runs as the module it is.
    integrate: return so3_integrate of the result, [batch, feature]; a (BatchNorm3d, ReLU) that ends the sequence is then
    evaluated in the loads of the integral."""
    mods = list(sequence)
    if not mods or not hasattr(mods[0], "product_spectrum") or not x.is_cuda:
        return so3_integrate(sequence(x)) if integrate else sequence(x)
    conv = mods[0]
    zr = None
    i = 1
    while i + 2 < len(mods) and _fusable(conv, mods[i], mods[i + 1], mods[i + 2]):
        bn, nxt = mods[i], mods[i + 2]
        if zr is None:
            zr = conv.product_spectrum(x)
        training = bn.training or not bn.track_running_stats
        xh, mean, var = _SynthesisBNReLUAnalysis.apply(zr, conv.bias, bn.weight, bn.bias, bn.running_mean, bn.running_var,
                                                       conv.b_out, nxt.b_out, bn.eps, training)
        if bn.training:
            _update_running_statistics(bn, mean, var, x.size(0) * (2 * conv.b_out) ** 3)
        conv = nxt
        zr = conv.product_spectrum(None, xh)
        i += 3
    if integrate and len(mods) == i + 2 and _normalised(conv, mods[i], mods[i + 1]):
        bn = mods[i]
        if zr is None:
            zr = conv.product_spectrum(x)
        training = bn.training or not bn.track_running_stats
        out, mean, var = _SynthesisBNReLUIntegrate.apply(zr, conv.bias, bn.weight, bn.bias, bn.running_mean, bn.running_var,
                                                         conv.b_out, bn.eps, training)
        if bn.training:
            _update_running_statistics(bn, mean, var, x.size(0) * (2 * conv.b_out) ** 3)
        return out
    y = conv(x) if zr is None else conv.from_spectrum(zr)
    for m in mods[i:]:
        y = m(y)
    return so3_integrate(y) if integrate else y
