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
                      so3_rifft_real_basis, synthesis_moment_parts)


def _moments(name, n_per_volume, *operands):
    """[volumes, 2] float32: the two sums per volume of s2cnn_volume_moments / s2cnn_bn_relu_grad_moments."""
    first = operands[0]
    nvol = first.numel() // n_per_volume
    out = first.new_empty((nvol, 2))
    args = [_hip.ptr(t) if torch.is_tensor(t) else t for t in operands]
    _hip.call(name, *args, _hip.ptr(out), nvol, n_per_volume, _hip.stream_ptr())
    return out


def _ptr_or_none(t):
    return _hip.ptr(t) if t is not None else None


def _synthesis_and_statistics(ctx, zr, conv_bias, weight, bias, running_mean, running_var, b_grid, eps, training, momentum):
    """y = synthesis(zr) + conv_bias, the statistics of y and the affine map (a, b) of the normalisation; when training,
    the running averages (if given) move by `momentum`."""
    nspec, batch, nf = zr.shape
    ctx.b_z = round((3 / 4 * nspec) ** (1 / 3))
    ctx.b_grid, ctx.training = b_grid, training
    ctx.bias_shape = conv_bias.shape
    nvox = (2 * b_grid) ** 3
    ctx.count = batch * nvox
    parts = synthesis_moment_parts(ctx.b_z, b_grid)                # > 0: the synthesis forms the sums itself, one pair per plane or volume
    if parts:
        mom = zr.new_empty((batch * nf * parts, 2))
        y = so3_rifft_real_basis(zr, b_out=b_grid, bias=conv_bias, moments=(mom, None, None))
    else:
        parts = 1
        y = so3_rifft_real_basis(zr, b_out=b_grid, bias=conv_bias)                   # [batch, feature, 2b, 2b, 2b]
        mom = _moments("s2cnn_volume_moments", nvox, y)                              # [batch * feature, 2]
    ab = y.new_empty((2, nf))
    stats = y.new_empty((4, nf))          # batch mean, biased batch variance, mean in use, 1 / sqrt(variance in use + eps)
    for t in (weight, bias, running_mean, running_var):
        if t is not None:
            _hip.require_gpu_f32(t)
            assert t.is_contiguous() and t.numel() == nf
    _hip.call("s2cnn_bn_forward_from_moments", _hip.ptr(mom), batch, nf, parts, float(ctx.count), _ptr_or_none(weight), _ptr_or_none(bias),
              _ptr_or_none(running_mean), _ptr_or_none(running_var), float(eps), float(momentum), int(training), _hip.ptr(ab),
              _hip.ptr(stats), _hip.stream_ptr())
    ctx.save_for_backward(y, ab, stats)
    ctx.has_affine = (weight is not None, bias is not None)
    return y, ab


def _gradients_from(ctx, g, mom=None, parts=1):
    """g: the gradient with respect to u = max(a y + b, 0); mom: its sums (sum g m, sum g m y), `parts` pairs per volume, if
    the kernel that produced g has formed them.  Returns the gradients with respect to the spectrum zr, the bias of the
    layer, and the weight and bias of the normalisation."""
    y, ab, stats = ctx.saved_tensors
    batch, nf = y.shape[:2]
    nvox = (2 * ctx.b_grid) ** 3
    if mom is None:
        mom = _moments("s2cnn_bn_relu_grad_moments", nvox, g, y, ab, nf)             # per volume
    params = y.new_empty((4, nf))
    gwb = y.new_empty((2, nf))
    _hip.call("s2cnn_bn_backward_from_moments", _hip.ptr(mom), batch, nf, parts, float(ctx.count), _hip.ptr(ab), _hip.ptr(stats),
              int(ctx.training), _hip.ptr(params), _hip.ptr(gwb), _hip.stream_ptr())
    gz = so3_rfft_real_basis(g, for_grad=True, b_out=ctx.b_z, mask=LoadBNReLUGrad(y, params))
    g_conv_bias = gz[0].reshape(-1, nf).sum(0).reshape(ctx.bias_shape) if ctx.needs_input_grad[1] else None
    return gz, g_conv_bias, (gwb[0] if ctx.has_affine[0] else None), (gwb[1] if ctx.has_affine[1] else None)


class _SynthesisBNReLUAnalysis(torch.autograd.Function):
    """z_hat (real-basis spectrum [l m n, batch, feature]) of one layer -> the input spectrum of the next one.
    running_mean / running_var (buffers, may be None) are read in evaluation mode and updated in training mode."""

    @staticmethod
    def forward(ctx, zr, conv_bias, weight, bias, running_mean, running_var, b_grid, b_next, eps, training, momentum):  # pylint: disable=W
        y, ab = _synthesis_and_statistics(ctx, zr, conv_bias, weight, bias, running_mean, running_var, b_grid, eps, training, momentum)
        return so3_rfft_real_basis(y, b_out=b_next, mask=LoadAffineReLU(ab))

    @staticmethod
    def backward(ctx, gxh):  # pylint: disable=W
        gxh = gxh.contiguous()
        b_next = round((3 / 4 * gxh.size(0)) ** (1 / 3))
        parts = synthesis_moment_parts(b_next, ctx.b_grid, grad=True)
        if parts:           # the synthesis that produces the gradient with respect to u forms its two sums as well
            y, ab, _ = ctx.saved_tensors
            mom = gxh.new_empty((y.size(0) * y.size(1) * parts, 2))
            g = so3_rifft_real_basis(gxh, for_grad=True, b_out=ctx.b_grid, moments=(mom, y, ab))
            return (*_gradients_from(ctx, g, mom, parts), None, None, None, None, None, None, None)
        g = so3_rifft_real_basis(gxh, for_grad=True, b_out=ctx.b_grid)                   # gradient with respect to u
        return (*_gradients_from(ctx, g), None, None, None, None, None, None, None)


class _SynthesisBNReLUIntegrate(torch.autograd.Function):
    """z_hat of the last layer -> so3_integrate(max(batch_norm(y), 0)), [batch, feature]: the end of the reference's shape
    network (examples/shrec17/model.py:36-45).  The integral applies the normalisation and the activation in its loads."""

    @staticmethod
    def forward(ctx, zr, conv_bias, weight, bias, running_mean, running_var, b_grid, eps, training, momentum):  # pylint: disable=W
        y, ab = _synthesis_and_statistics(ctx, zr, conv_bias, weight, bias, running_mean, running_var, b_grid, eps, training, momentum)
        batch, nf = y.shape[:2]
        out = y.new_empty((batch, nf))
        _hip.call("s2cnn_so3_integrate_affine_relu", _hip.ptr(y), _hip.ptr(ab), nf, _hip.ptr(_setup_so3_integrate(b_grid, y.device)),
                  _hip.ptr(out), b_grid, batch * nf, _hip.stream_ptr())
        return out

    @staticmethod
    def backward(ctx, gout):  # pylint: disable=W
        y = ctx.saved_tensors[0]
        g = torch.empty_like(y)                                                          # gradient with respect to u: gout[z] w[beta]
        _hip.call("s2cnn_so3_integrate_grad", _hip.ptr(gout.contiguous()), _hip.ptr(_setup_so3_integrate(ctx.b_grid, y.device)), _hip.ptr(g),
                  ctx.b_grid, gout.numel(), _hip.stream_ptr())
        return (*_gradients_from(ctx, g), None, None, None, None, None, None)


class _SynthesisBNReLUMax(torch.autograd.Function):
    """z_hat of the last layer -> the maximum over the grid of max(batch_norm(y), 0), [batch, feature]: the end of the
    reference's original shape network (examples/shrec17/model_original.py:36-47).  max(a y + b, 0) is monotone in y, so
    its maximum sits at the largest (a >= 0) or smallest (a < 0) sample of y: the normalised tensor is never formed."""

    @staticmethod
    def forward(ctx, zr, conv_bias, weight, bias, running_mean, running_var, b_grid, eps, training, momentum):  # pylint: disable=W
        y, ab = _synthesis_and_statistics(ctx, zr, conv_bias, weight, bias, running_mean, running_var, b_grid, eps, training, momentum)
        batch, nf = y.shape[:2]
        flat = y.view(batch, nf, -1)
        hi, ihi = flat.max(-1)
        lo, ilo = flat.min(-1)
        a, b = ab[0].view(1, nf), ab[1].view(1, nf)
        up = a >= 0
        ctx.where = torch.where(up, ihi, ilo)                                            # [batch, feature]: the sample that carries the maximum
        return torch.relu(a * torch.where(up, hi, lo) + b)

    @staticmethod
    def backward(ctx, gout):  # pylint: disable=W
        y = ctx.saved_tensors[0]
        batch, nf = y.shape[:2]
        g = torch.zeros_like(y)                                                          # gradient with respect to u: one sample per volume
        g.view(batch, nf, -1).scatter_(-1, ctx.where.unsqueeze(-1), gout.contiguous().unsqueeze(-1))
        return (*_gradients_from(ctx, g), None, None, None, None, None, None)


def _statistics_mode(bn):
    """(training, momentum, running_mean, running_var) as nn.BatchNorm3d uses them, and its step counter moved on."""
    training = bn.training or not bn.track_running_stats
    momentum = 0.0
    if bn.training and bn.track_running_stats and bn.running_mean is not None:
        with torch.no_grad():
            bn.num_batches_tracked += 1
        if bn.momentum is None:                           # cumulative average: the factor 1 / n is read on the host
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError("BatchNorm3d(momentum=None) cannot be recorded into a HIP graph: its averaging factor 1 / "
                                   "num_batches_tracked is read on the host and would be frozen at the value of the capture; "
                                   "give the module a numeric momentum, or run this step eagerly")
            momentum = 1.0 / float(bn.num_batches_tracked)
        else:
            momentum = bn.momentum
        return training, momentum, bn.running_mean, bn.running_var
    if training:
        return training, momentum, None, None
    return training, momentum, bn.running_mean, bn.running_var


def _normalised(conv, bn, act):
    return (isinstance(bn, nn.BatchNorm3d) and isinstance(act, nn.ReLU) and conv.real_basis and conv.activation is None
            and conv.nfeature_out == bn.num_features and analysis_prologue_available(conv.b_out, conv.b_out))


def _fusable(conv, bn, act, nxt):
    return (_normalised(conv, bn, act) and isinstance(nxt, SO3Convolution) and nxt.real_basis and nxt.b_in == conv.b_out
            and analysis_prologue_available(nxt.b_in, nxt.b_out))


def run_sequence(sequence, x, head=None):
    """`nn.Sequential(conv, [BatchNorm3d, ReLU, SO3Convolution] ..., ...)(x)` with every (BatchNorm3d, ReLU) that stands
    between two spectral layers evaluated inside the transforms of its neighbours.  Same function, same parameters, same
    buffer updates; whatever does not match the pattern runs as the module it is.
    head: None, or what follows the sequence in the reference's networks, with a (BatchNorm3d, ReLU) that ends the sequence
    evaluated inside it: "integrate" = so3_integrate of the result (the pair in the loads of the integral), "max" = the
    maximum over the grid (taken on the samples before the pair); either returns [batch, feature]."""
    assert head in (None, "integrate", "max"), head

    def finish(y):
        if head == "integrate":
            return so3_integrate(y)
        return y.view(y.size(0), y.size(1), -1).max(-1)[0] if head == "max" else y

    mods = list(sequence)
    if not mods or not hasattr(mods[0], "product_spectrum") or not x.is_cuda or x.size(0) == 0:
        return finish(sequence(x))      # nothing to fuse (an empty batch behaves as the modules themselves do)
    conv = mods[0]
    zr = None
    i = 1
    while i + 2 < len(mods) and _fusable(conv, mods[i], mods[i + 1], mods[i + 2]):
        bn, nxt = mods[i], mods[i + 2]
        if zr is None:
            zr = conv.product_spectrum(x)
        training, momentum, rmean, rvar = _statistics_mode(bn)
        xh = _SynthesisBNReLUAnalysis.apply(zr, conv.bias, bn.weight, bn.bias, rmean, rvar, conv.b_out, nxt.b_out, bn.eps, training, momentum)
        conv = nxt
        zr = conv.product_spectrum(None, xh)
        i += 3
    if head is not None and len(mods) == i + 2 and _normalised(conv, mods[i], mods[i + 1]):
        bn = mods[i]
        if zr is None:
            zr = conv.product_spectrum(x)
        training, momentum, rmean, rvar = _statistics_mode(bn)
        last = _SynthesisBNReLUIntegrate if head == "integrate" else _SynthesisBNReLUMax
        return last.apply(zr, conv.bias, bn.weight, bn.bias, rmean, rvar, conv.b_out, bn.eps, training, momentum)
    y = conv(x) if zr is None else conv.from_spectrum(zr)
    for m in mods[i:]:
        y = m(y)
    return finish(y)
