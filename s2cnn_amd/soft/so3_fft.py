"""SO(3) Fourier transforms on the SOFT grid: mirrors s2cnn/soft/so3_fft.py of the reference
(same functions, arguments, layouts and autograd rules), running on the HIP kernels behind
s2cnn_so3_analysis / s2cnn_so3_synthesis."""
from functools import lru_cache

import torch

from .. import _hip, wigner


def _nspec(b):
    return b * (4 * b ** 2 - 1) // 3


@lru_cache(maxsize=32)
def _wigner_table(b, nl, weighted, device):
    dss = wigner.so3_wigner_table(b, nl, weighted)
    return torch.tensor(dss, dtype=torch.float32, device=device).contiguous()


def _setup_wigner(b, nl, weighted, device):
    """[2b, nspec(nl)] float32 on `device`, computed in float64 (s2cnn/soft/so3_fft.py:205-243).  One cache entry per
    table, whichever way the arguments are passed (lru_cache keys positional and keyword calls differently)."""
    return _wigner_table(int(b), int(nl), bool(weighted), torch.device(device))


@lru_cache(maxsize=32)
def _setup_packed_wigner(b_in, b_out, weighted, synthesis, device):
    """The table of `_setup_wigner` repacked once for the tiled kernels (None where they do not apply).  The first
    call for a table synchronizes: make it (one transform of each size) before capturing a HIP graph."""
    L = _hip.lib()
    nbytes = L.s2cnn_so3_packed_table_bytes(b_in, b_out, int(synthesis))
    if nbytes == 0:
        return None
    table = _setup_wigner(b_out, b_in, weighted, device) if synthesis else _setup_wigner(b_in, b_out, weighted, device)
    packed = torch.empty(nbytes // 4, dtype=torch.float32, device=device)
    with torch.cuda.device(device):
        _hip.check(L.s2cnn_so3_pack_table(_hip.ptr(table), _hip.ptr(packed), b_in, b_out, int(synthesis), _hip.stream_ptr()))
        torch.cuda.current_stream().synchronize()
    return packed


# Complex signals (so3_fft / so3_ifft; no layer uses them) run as two transforms of real signals.  False: the
# library's own kernels for complex signals (s2cnn_so3_analysis / s2cnn_so3_synthesis with complex = 1).
complex_via_real = True


def _null_or_ptr(t):
    return _hip.ptr(t) if t is not None else None


def _same_shape_operand(mask, x):
    """`mask` as a contiguous, 16-byte aligned float32 GPU tensor of the shape of x."""
    _hip.require_gpu_f32(mask)
    assert mask.shape == x.shape, (mask.shape, x.shape)
    mask = mask.contiguous()
    return mask.clone() if mask.data_ptr() % 16 else mask


class LoadAffineReLU:
    """Passed as `mask` to the real analyses: the signal that is transformed is max(a x + b, 0), a = params[0][z % F],
    b = params[1][z % F] for volume z (params: float32 [2, F] on the device of x)."""

    def __init__(self, params):
        _hip.require_gpu_f32(params)
        assert params.dim() == 2 and params.size(0) == 2
        self.params = params.contiguous()


class LoadBNReLUGrad:
    """Passed as `mask` to the real analyses of a gradient g: the signal that is transformed is
    a (a y + b > 0 ? g : 0) + p + q y, with a, b, p, q = params[0..3][z % F] (float32 [4, F]) and y of the shape of g:
    the gradient of max(batch_norm(y), 0) with respect to y."""

    def __init__(self, y, params):
        _hip.require_gpu_f32(params)
        assert params.dim() == 2 and params.size(0) == 4
        self.y, self.params = y, params.contiguous()


def analysis_prologue_available(b_in, b_out):
    """Whether the real analysis b_in -> b_out can apply LoadAffineReLU / LoadBNReLUGrad in its loads."""
    return bool(_hip.lib().s2cnn_so3_analysis_prologue_available(b_in, b_out))


def _analysis_with_loads(x, mask, table, packed, out, ws, b_in, b_out, nbatch, real_basis):
    """The analysis of x with what `mask` asks for done in its loads."""
    tail = (_hip.ptr(table), _null_or_ptr(packed), _hip.ptr(out), _hip.ptr(ws), ws.numel(), b_in, b_out, nbatch, real_basis, _hip.stream_ptr())
    if isinstance(mask, LoadAffineReLU):
        assert nbatch % mask.params.size(1) == 0
        _hip.call("s2cnn_so3_analysis_real_affine_relu", _hip.ptr(x), _hip.ptr(mask.params), mask.params.size(1), *tail)
    elif isinstance(mask, LoadBNReLUGrad):
        assert nbatch % mask.params.size(1) == 0
        y = _same_shape_operand(mask.y, x)
        _hip.call("s2cnn_so3_analysis_real_bn_relu_grad", _hip.ptr(x), _hip.ptr(y), _hip.ptr(mask.params), mask.params.size(1), *tail)
    elif _is_bit_mask(mask):
        _hip.call("s2cnn_so3_analysis_real_masked_bits", _hip.ptr(x), _hip.ptr(mask), *tail)
    else:
        mask = _same_shape_operand(mask, x)
        _hip.call("s2cnn_so3_analysis_real_masked", _hip.ptr(x), _hip.ptr(mask), *tail)
    return out


def _is_bit_mask(mask):
    """A mask of one bit per sample, as `_relu_bits` allocates it and the transforms with relu=True fill it."""
    return mask is not None and mask.dtype == torch.int64


def _relu_bits(b_grid, nbatch, device):
    """Where the synthesis onto the (2 b_grid)^3 grid can record the sign of its output as one bit per sample: an int64
    tensor for them (s2cnn_so3_relu_bits_bytes), else None (the float output then serves as the mask)."""
    nbytes = _hip.lib().s2cnn_so3_relu_bits_bytes(b_grid, nbatch) if nbatch > 0 else 0
    return torch.empty(nbytes // 8, dtype=torch.int64, device=device) if nbytes else None


def _analysis(x, b_in, b_out, batch_size, for_grad, complex_in, mask=None):
    """x: contiguous grid tensor whose leading dims are `batch_size`; the result is allocated in its
    final shape (never a view: autograd can then take ownership of it as a gradient without a copy).
    mask (real x only): the transform is that of x where mask > 0 and of zero elsewhere."""
    _hip.require_gpu_f32(x)
    assert mask is None or not complex_in
    if complex_in and complex_via_real:
        # the transform is linear over the complex numbers: analysis(x) = analysis(Re x) + i analysis(Im x), and the
        # kernels for real signals are the tuned ones; both parts go through them as one batch of twice the volumes
        AB = _analysis(torch.stack((x[..., 0], x[..., 1]), 0), b_in, b_out, (2, *batch_size), for_grad, 0)
        A, B = AB[:, 0], AB[:, 1]
        return torch.stack((A[..., 0] - B[..., 1], A[..., 1] + B[..., 0]), -1)
    if x.data_ptr() % 16:
        x = x.clone()
    L = _hip.lib()
    nbatch = 1
    for d in batch_size:
        nbatch *= d
    table = _setup_wigner(b_in, nl=b_out, weighted=not for_grad, device=x.device)
    packed = None if complex_in else _setup_packed_wigner(b_in, b_out, not for_grad, False, x.device)
    out = x.new_empty((_nspec(b_out), *batch_size, 2))
    if nbatch == 0:
        return out
    ws = _hip.workspace(L.s2cnn_so3_analysis_workspace(b_in, b_out, nbatch, complex_in), x.device)
    if mask is not None:
        return _analysis_with_loads(x, mask, table, packed, out, ws, b_in, b_out, nbatch, 0)
    _hip.call("s2cnn_so3_analysis", _hip.ptr(x), _hip.ptr(table), _null_or_ptr(packed), _hip.ptr(out), _hip.ptr(ws), ws.numel(),
                  b_in, b_out, nbatch, complex_in, _hip.stream_ptr())
    return out


def synthesis_moment_parts(b_in, b_out, grad=False):
    """How many pairs of sums per volume the real synthesis b_in -> b_out of a real-basis spectrum can form while it
    writes its output (0: none).  grad: the sums of the gradient of a normalisation (they need a second tensor) instead
    of the output's own (the per-volume kernels of the 64^3 grid form those for truncated spectra only)."""
    if _real_basis_direct(b_in, b_out, True):
        return _hip.lib().s2cnn_so3_synthesis_real_basis_moment_parts(b_in, b_out, int(grad))
    return _hip.lib().s2cnn_so3_synthesis_moment_parts(b_in, b_out)


def _synthesis(x, b_in, b_out, batch_size, for_grad, complex_out, bias=None, relu=False, bits=None, moments=None):
    """bits (with relu): an int64 tensor from `_relu_bits` that receives one bit per sample (the output is not <= 0).
    moments: None, or (out [volumes * parts, 2], yref or None, params or None) for s2cnn_so3_synthesis_real_moments."""
    _hip.require_gpu_f32(x)
    assert not (relu and complex_out)
    if complex_out and complex_via_real:
        # y = synthesis(x) is complex-linear in x and the real-output kernels return Re y for ANY spectrum:
        # Re y = real_synthesis(x), Im y = Re(-i y) = real_synthesis(-i x): one batch of twice the volumes
        both = torch.stack((x, torch.stack((x[..., 1], -x[..., 0]), -1)), 1)          # [nspec, 2, ..., 2]
        y = _synthesis(both, b_in, b_out, (2, *batch_size), for_grad, 0)
        return torch.stack((y[0], y[1]), -1)
    L = _hip.lib()
    nbatch = 1
    for d in batch_size:
        nbatch *= d
    table = _setup_wigner(b_out, nl=b_in, weighted=for_grad, device=x.device)
    packed = None if complex_out else _setup_packed_wigner(b_in, b_out, for_grad, True, x.device)
    shape = (*batch_size, 2 * b_out, 2 * b_out, 2 * b_out) + ((2,) if complex_out else ())
    out = x.new_empty(shape)
    if nbatch == 0:
        return out
    ws = _hip.workspace(L.s2cnn_so3_synthesis_workspace(b_in, b_out, nbatch, complex_out), x.device)
    if bias is not None:
        assert not complex_out
        _hip.require_gpu_f32(bias)
        bias = bias.reshape(-1).contiguous()
        assert len(batch_size) >= 1 and batch_size[-1] == bias.numel()
    if moments is not None:
        assert not relu and not complex_out
        mom, yref, params = moments
        nfeature = params.size(1) if params is not None else (1 if bias is None else bias.numel())
        _hip.call("s2cnn_so3_synthesis_real_moments", _hip.ptr(x), _hip.ptr(table), _null_or_ptr(packed), _hip.ptr(out), _hip.ptr(ws),
                  ws.numel(), b_in, b_out, nbatch, _null_or_ptr(bias), nfeature, _hip.ptr(mom), _null_or_ptr(yref), _null_or_ptr(params),
                  _hip.stream_ptr())
        return out
    if relu and bits is not None:
        _hip.call("s2cnn_so3_synthesis_real_relu_bits", _hip.ptr(x), _hip.ptr(table), _null_or_ptr(packed), _hip.ptr(out), _hip.ptr(bits),
                  _hip.ptr(ws), ws.numel(), b_in, b_out, nbatch, _null_or_ptr(bias), 1 if bias is None else bias.numel(), 0, _hip.stream_ptr())
        return out
    if relu:
        _hip.call("s2cnn_so3_synthesis_real_relu", _hip.ptr(x), _hip.ptr(table), _null_or_ptr(packed), _hip.ptr(out), _hip.ptr(ws),
                  ws.numel(), b_in, b_out, nbatch, _null_or_ptr(bias), 1 if bias is None else bias.numel(), 0, _hip.stream_ptr())
        return out
    if bias is not None:
        _hip.call("s2cnn_so3_synthesis_real_bias", _hip.ptr(x), _hip.ptr(table), _null_or_ptr(packed), _hip.ptr(out), _hip.ptr(ws),
                  ws.numel(), b_in, b_out, nbatch, _hip.ptr(bias), bias.numel(), _hip.stream_ptr())
        return out
    _hip.call("s2cnn_so3_synthesis", _hip.ptr(x), _hip.ptr(table), _null_or_ptr(packed), _hip.ptr(out), _hip.ptr(ws), ws.numel(),
                  b_in, b_out, nbatch, complex_out, _hip.stream_ptr())
    return out


def so3_fft(x, for_grad=False, b_out=None):
    '''
    :param x: [..., beta, alpha, gamma, complex]
    :return: [l * m * n, ..., complex]
    '''
    assert x.size(-1) == 2, x.size()
    b_in = x.size(-2) // 2
    assert x.size(-2) == 2 * b_in
    assert x.size(-3) == 2 * b_in
    assert x.size(-4) == 2 * b_in
    if b_out is None:
        b_out = b_in
    batch_size = x.size()[:-4]
    return _analysis(x.contiguous(), b_in, b_out, batch_size, for_grad, 1)


def so3_rfft(x, for_grad=False, b_out=None, mask=None):
    '''
    :param x: [..., beta, alpha, gamma]
    :param mask: None, or a tensor of the shape of x: samples of x where it is not positive count as zero
                 (or the bit mask that so3_rifft(..., relu=True, bits=...) filled)
    :return: [l * m * n, ..., complex]
    '''
    b_in = x.size(-1) // 2
    assert x.size(-1) == 2 * b_in
    assert x.size(-2) == 2 * b_in
    assert x.size(-3) == 2 * b_in
    if b_out is None:
        b_out = b_in
    batch_size = x.size()[:-3]
    return _analysis(x.contiguous(), b_in, b_out, batch_size, for_grad, 0, mask)


def _spectrum_args(x, b_out):
    assert x.size(-1) == 2
    nspec = x.size(0)
    b_in = round((3 / 4 * nspec) ** (1 / 3))
    assert nspec == b_in * (4 * b_in ** 2 - 1) // 3
    if b_out is None:
        b_out = b_in
    batch_size = x.size()[1:-1]
    return x.contiguous(), b_in, b_out, batch_size


def so3_ifft(x, for_grad=False, b_out=None):
    '''
    :param x: [l * m * n, ..., complex]
    :return: [..., beta, alpha, gamma, complex]
    '''
    x, b_in, b_out, batch_size = _spectrum_args(x, b_out)
    return _synthesis(x, b_in, b_out, batch_size, for_grad, 1)


def so3_rifft(x, for_grad=False, b_out=None, bias=None, relu=False, bits=None, moments=None):
    '''
    :param x: [l * m * n, ..., complex]
    :param bias: None, or one value per entry of the last batch dimension, added to every sample of its volumes
    :param relu: negative samples (after the bias) come out as zero
    :param bits: None, or (with relu) the int64 tensor of `_relu_bits` that receives one bit per sample: the output is not <= 0
    :return: [..., beta, alpha, gamma]  (the real part of so3_ifft, whatever the symmetry of x)
    '''
    x, b_in, b_out, batch_size = _spectrum_args(x, b_out)
    return _synthesis(x, b_in, b_out, batch_size, for_grad, 0, bias, relu, bits, moments)


class SO3_fft_real(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, b_out=None):  # pylint: disable=W
        ctx.b_out = b_out
        ctx.b_in = x.size(-1) // 2
        return so3_rfft(x, b_out=ctx.b_out)

    @staticmethod
    def backward(ctx, grad_output):  # pylint: disable=W
        # real part of the complex inverse of a spectrum that need not be Hermitian
        # (s2cnn/soft/so3_fft.py:453-456); the real-output kernel computes exactly that
        return so3_rifft(grad_output, for_grad=True, b_out=ctx.b_in), None


class SO3_ifft_real(torch.autograd.Function):
    """s2cnn/soft/so3_fft.py:224-236, with the bias of the convolution layers as an optional third argument
    (x [l * m * n, batch, feature, complex], bias with `feature` entries in any shape): it is added in the
    epilogue of the transform, and its gradient is read off the degree-0 coefficient of the unweighted analysis
    of grad_output, which IS the sum of grad_output over the grid.  relu = True applies max(., 0) in the same
    epilogue (the activation that follows the layers in the reference's models)."""
    @staticmethod
    def forward(ctx, x, b_out=None, bias=None, relu=False):  # pylint: disable=W
        nspec = x.size(0)
        ctx.b_out = b_out
        ctx.b_in = round((3 / 4 * nspec) ** (1 / 3))
        ctx.bias_shape = None if bias is None else bias.shape
        bits = None
        b_grid = ctx.b_in if b_out is None else b_out
        if relu and x.is_cuda and ctx.b_in <= b_grid:      # one bit per sample where the library can record it and its
            bits = _relu_bits(b_grid, x[..., 0].numel() // nspec, x.device)     # analysis can read it; else the output is the mask
        out = so3_rifft(x, b_out=ctx.b_out, bias=bias, relu=relu, bits=bits)
        ctx.relu = bool(relu)
        if relu:
            ctx.save_for_backward(out if bits is None else bits)
        return out

    @staticmethod
    def backward(ctx, grad_output):  # pylint: disable=W
        # with the relu in the epilogue, the gradient passes where the output is positive: the mask is applied as the
        # analysis reads grad_output
        g = so3_rfft(grad_output, for_grad=True, b_out=ctx.b_in, mask=ctx.saved_tensors[0] if ctx.relu else None)
        gb = None
        if ctx.bias_shape is not None and ctx.needs_input_grad[2]:
            gb = g[0, ..., 0].reshape(g[0, ..., 0].numel() // g.size(-2), g.size(-2)).sum(0).reshape(ctx.bias_shape)
        return g, None, gb, None


# ---------------------------------------------------------------------------------------------------
# The two real transforms with the spectrum in the real basis of s2cnn_amd.so3_real (one float per
# entry).  No counterpart in the reference; used by SO3Convolution, whose spectra are those of real
# signals throughout.  Where the library has no direct kernel for the sizes, the two steps are composed.
# ---------------------------------------------------------------------------------------------------
def _real_basis_direct(b_in, b_out, synthesis):
    return bool(_hip.lib().s2cnn_so3_real_basis_transform_available(b_in, b_out, int(synthesis)))


def so3_rfft_real_basis(x, for_grad=False, b_out=None, mask=None):
    '''
    :param x: [..., beta, alpha, gamma]
    :param mask: None, or a tensor of the shape of x: samples of x where it is not positive count as zero
    :return: [l * m * n, ...]  = so3_spectrum_to_real(so3_rfft(x))
    '''
    b_in = x.size(-1) // 2
    assert x.size(-1) == 2 * b_in and x.size(-2) == 2 * b_in and x.size(-3) == 2 * b_in
    if b_out is None:
        b_out = b_in
    if not (x.is_cuda and _real_basis_direct(b_in, b_out, False)):
        from ..so3_real import _convert
        y = so3_rfft(x, for_grad, b_out, mask)
        return _convert("s2cnn_so3_spectrum_to_real", y, y.shape[:-1])
    _hip.require_gpu_f32(x)
    x = x.contiguous()
    if x.data_ptr() % 16:
        x = x.clone()
    batch_size = x.size()[:-3]
    nbatch = 1
    for d in batch_size:
        nbatch *= d
    L = _hip.lib()
    table = _setup_wigner(b_in, nl=b_out, weighted=not for_grad, device=x.device)
    packed = _setup_packed_wigner(b_in, b_out, not for_grad, False, x.device)
    out = x.new_empty((_nspec(b_out), *batch_size))
    if nbatch == 0:
        return out
    ws = _hip.workspace(L.s2cnn_so3_analysis_workspace(b_in, b_out, nbatch, 0), x.device)
    if mask is not None:
        return _analysis_with_loads(x, mask, table, packed, out, ws, b_in, b_out, nbatch, 1)
    _hip.call("s2cnn_so3_analysis_real_basis", _hip.ptr(x), _hip.ptr(table), _null_or_ptr(packed), _hip.ptr(out), _hip.ptr(ws),
              ws.numel(), b_in, b_out, nbatch, _hip.stream_ptr())
    return out


def so3_rifft_real_basis(r, for_grad=False, b_out=None, bias=None, relu=False, bits=None, moments=None):
    '''
    :param r: [l * m * n, ...]  real-basis spectrum
    :param bias: None, or one value per entry of the last batch dimension, added to every sample of its volumes
    :param relu: negative samples (after the bias) come out as zero
    :return: [..., beta, alpha, gamma]  = so3_rifft(so3_spectrum_to_complex(r)) (+ bias)
    '''
    nspec = r.size(0)
    b_in = round((3 / 4 * nspec) ** (1 / 3))
    assert nspec == b_in * (4 * b_in ** 2 - 1) // 3
    if b_out is None:
        b_out = b_in
    if not (r.is_cuda and _real_basis_direct(b_in, b_out, True)):
        from ..so3_real import _convert
        return so3_rifft(_convert("s2cnn_so3_spectrum_to_complex", r.contiguous(), (*r.shape, 2)), for_grad, b_out, bias, relu, bits, moments)
    _hip.require_gpu_f32(r)
    r = r.contiguous()
    batch_size = r.size()[1:]
    nbatch = 1
    for d in batch_size:
        nbatch *= d
    L = _hip.lib()
    table = _setup_wigner(b_out, nl=b_in, weighted=for_grad, device=r.device)
    packed = _setup_packed_wigner(b_in, b_out, for_grad, True, r.device)
    out = r.new_empty((*batch_size, 2 * b_out, 2 * b_out, 2 * b_out))
    if nbatch == 0:
        return out
    ws = _hip.workspace(L.s2cnn_so3_synthesis_workspace(b_in, b_out, nbatch, 0), r.device)
    nfeature = 1
    if bias is not None:
        _hip.require_gpu_f32(bias)
        bias = bias.reshape(-1).contiguous()
        nfeature = bias.numel()
        assert r.dim() >= 2 and r.size(-1) == nfeature
    if moments is not None:
        mom, yref, params = moments
        assert not relu
        if params is not None:
            nfeature = params.size(1)
        _hip.call("s2cnn_so3_synthesis_real_basis_moments", _hip.ptr(r), _hip.ptr(table), _null_or_ptr(packed), _hip.ptr(out), _hip.ptr(ws),
                  ws.numel(), b_in, b_out, nbatch, _null_or_ptr(bias), nfeature, _hip.ptr(mom), _null_or_ptr(yref), _null_or_ptr(params),
                  _hip.stream_ptr())
        return out
    if relu and bits is not None:
        _hip.call("s2cnn_so3_synthesis_real_relu_bits", _hip.ptr(r), _hip.ptr(table), _null_or_ptr(packed), _hip.ptr(out), _hip.ptr(bits),
                  _hip.ptr(ws), ws.numel(), b_in, b_out, nbatch, _null_or_ptr(bias), nfeature, 1, _hip.stream_ptr())
        return out
    if relu:
        _hip.call("s2cnn_so3_synthesis_real_relu", _hip.ptr(r), _hip.ptr(table), _null_or_ptr(packed), _hip.ptr(out), _hip.ptr(ws),
                  ws.numel(), b_in, b_out, nbatch, _null_or_ptr(bias), nfeature, 1, _hip.stream_ptr())
        return out
    _hip.call("s2cnn_so3_synthesis_real_basis", _hip.ptr(r), _hip.ptr(table), _null_or_ptr(packed), _hip.ptr(out), _hip.ptr(ws),
              ws.numel(), b_in, b_out, nbatch, _null_or_ptr(bias), nfeature, _hip.stream_ptr())
    return out


class SO3_fft_real_basis(torch.autograd.Function):
    """SO3_fft_real followed by the change to the real basis; the backward is the adjoint pair of
    SO3_fft_real.backward and so3_spectrum_to_complex."""
    @staticmethod
    def forward(ctx, x, b_out=None):  # pylint: disable=W
        ctx.b_in = x.size(-1) // 2
        return so3_rfft_real_basis(x, b_out=b_out)

    @staticmethod
    def backward(ctx, grad_output):  # pylint: disable=W
        return so3_rifft_real_basis(grad_output, for_grad=True, b_out=ctx.b_in), None


class SO3_ifft_real_basis(torch.autograd.Function):
    """The change from the real basis followed by SO3_ifft_real and, optionally, the bias of the convolution
    layer (r [l * m * n, batch, feature], bias with `feature` entries in any shape).  The gradient of the bias
    costs nothing: the degree-0 coefficient of the unweighted analysis of grad_output IS its sum over the grid."""
    @staticmethod
    def forward(ctx, r, b_out=None, bias=None, relu=False):  # pylint: disable=W
        nspec = r.size(0)
        ctx.b_in = round((3 / 4 * nspec) ** (1 / 3))
        ctx.bias_shape = None if bias is None else bias.shape
        bits = None
        b_grid = ctx.b_in if b_out is None else b_out
        if relu and r.is_cuda and ctx.b_in <= b_grid:
            bits = _relu_bits(b_grid, r.numel() // nspec, r.device)
        out = so3_rifft_real_basis(r, b_out=b_out, bias=bias, relu=relu, bits=bits)
        ctx.relu = bool(relu)
        if relu:
            ctx.save_for_backward(out if bits is None else bits)
        return out

    @staticmethod
    def backward(ctx, grad_output):  # pylint: disable=W
        g = so3_rfft_real_basis(grad_output, for_grad=True, b_out=ctx.b_in, mask=ctx.saved_tensors[0] if ctx.relu else None)
        gb = None
        if ctx.bias_shape is not None and ctx.needs_input_grad[2]:
            gb = g[0].reshape(g[0].numel() // g.size(-1), g.size(-1)).sum(0).reshape(ctx.bias_shape)
        return g, None, gb, None
