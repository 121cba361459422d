"""TEST INFRASTRUCTURE ONLY - never imported by the product package.

CPU restatement (torch, any float dtype) of the reference's CPU branches for the
spectral path.  Only tests/, the smoke check and bench.py's cpu_baseline leg use
it, as the checker / the timed baseline, never as a code path of the product.

Each function names the reference lines whose arithmetic it restates.  The
algorithmic shape is kept (a Python loop over degrees l, a gather of the used
FFT bins followed by an einsum with the Wigner table, complex products as four
real matrix products, autograd for the backward of the matmuls) so that timing
it is timing the reference's CPU algorithm; the wording is this project's own.

Two defects of the reference as shipped are repaired, not reproduced, because
they make it raise instead of compute: torch.fft.rfftn on a complex tensor
(s2cnn/soft/so3_fft.py:94 - the full complex 2-D FFT is what lines 101-106
index into) and np.float (s2cnn/so3_grid.py:14, s2cnn/s2_grid.py:10).

Tables come from oracle/wigner_ref.py (Jacobi closed form, linear-system
quadrature weights): see that file's header for what pins them and for the one
convention bit that stays PARITY UNPINNED without lie_learn.
"""
import math
from functools import lru_cache

import numpy as np
import torch

from . import wigner_ref


# ----------------------------------------------------------------------------
# tables
# ----------------------------------------------------------------------------

def nspec_so3(b):
    return b * (4 * b * b - 1) // 3


@lru_cache(maxsize=64)
def _so3_table64(b, nl, weighted):
    """Vectorised over beta; same values as wigner_ref.so3_table_ref."""
    from scipy.special import eval_jacobi, gammaln

    betas = (np.arange(2 * b) + 0.5) / (2 * b) * np.pi
    w = wigner_ref.quadrature_weights_ref(b)
    sb, cb, x = np.sin(betas / 2), np.cos(betas / 2), np.cos(betas)
    out = np.zeros((2 * b, nspec_so3(nl)))
    pos = 0
    for l in range(nl):
        for mp in range(-l, l + 1):
            for m in range(-l, l + 1):
                k = min(l + m, l - m, l + mp, l - mp)
                if k == l + m:
                    a, lam = mp - m, mp - m
                elif k == l - m:
                    a, lam = m - mp, 0
                elif k == l + mp:
                    a, lam = m - mp, 0
                else:
                    a, lam = mp - m, mp - m
                bb = 2 * l - 2 * k - a
                logc = 0.5 * (gammaln(2 * l - k + 1) - gammaln(k + a + 1) - gammaln(2 * l - 2 * k - a + 1)
                              - gammaln(k + bb + 1) + gammaln(bb + 1) + gammaln(k + 1))
                v = math.exp(logc) * sb ** a * cb ** bb * eval_jacobi(k, a, bb, x)
                if lam % 2:
                    v = -v
                out[:, pos] = v * w if weighted else v * (2 * l + 1)
                pos += 1
    return out


def so3_table(b, nl, weighted, dtype=torch.float32):
    """[2b, nspec(nl)] (s2cnn/soft/so3_fft.py:205-243)."""
    return torch.tensor(_so3_table64(b, nl, bool(weighted)), dtype=dtype)


@lru_cache(maxsize=64)
def _s2_table64(b, nl, weighted):
    full = _so3_table64(b, nl, False)  # (2l+1) d^l_mn
    w = wigner_ref.quadrature_weights_ref(b) * 2 * b
    out = np.zeros((2 * b, nl * nl))
    for l in range(nl):
        L = 2 * l + 1
        blk = full[:, nspec_so3(l):nspec_so3(l) + L * L].reshape(2 * b, L, L)[:, :, l] / L  # d^l_{m0}
        out[:, l * l:l * l + L] = blk * w[:, None] if weighted else blk * L
    return out


def s2_table(b, nl, weighted, dtype=torch.float32):
    """[2b, nl^2] (s2cnn/soft/s2_fft.py:109-147)."""
    return torch.tensor(_s2_table64(b, nl, bool(weighted)), dtype=dtype)


def quadrature_weights(b, dtype=torch.float32):
    return torch.tensor(wigner_ref.quadrature_weights_ref(b), dtype=dtype)


@lru_cache(maxsize=4096)
def _d_jacobi_cached(l, beta):
    return wigner_ref.wigner_d_jacobi(l, beta)


def _wigner_D64(l, alpha, beta, gamma):
    """D^l_mn = exp(i m alpha) d^l_mn(beta) exp(i n gamma) (s2cnn/soft/so3_rotation.py:58)."""
    d = _d_jacobi_cached(l, float(beta))
    m = np.arange(-l, l + 1)
    return np.exp(1j * m * alpha)[:, None] * d * np.exp(1j * m * gamma)[None, :]


# ----------------------------------------------------------------------------
# complex helpers (s2cnn/utils/complex.py:5-40)
# ----------------------------------------------------------------------------

def as_complex(x):
    return torch.stack((x, torch.zeros_like(x)), dim=-1)


def complex_mm(x, y, conj_x=False, conj_y=False):
    """[M,K,2] x [K,N,2] -> [M,N,2] as four real products (complex.py:15-40)."""
    xr, xi = x[..., 0], x[..., 1]
    yr, yi = y[..., 0], y[..., 1]
    sx = -1.0 if conj_x else 1.0
    sy = -1.0 if conj_y else 1.0
    rr, ii = torch.mm(xr, yr), torch.mm(xi, yi)
    ri, ir = torch.mm(xr, yi), torch.mm(xi, yr)
    return torch.stack((rr - (sx * sy) * ii, sy * ri + sx * ir), dim=-1)


# ----------------------------------------------------------------------------
# SO(3) transforms (s2cnn/soft/so3_fft.py)
# ----------------------------------------------------------------------------

def _gather_bins(x, l, b_in, dims):
    """Pick FFT bins of signed frequencies -l..l (zero where |freq| >= b_in)
    along each of `dims` - the zero-padded copy of so3_fft.py:47-55/98-106."""
    f = torch.arange(-l, l + 1)
    keep = (f.abs() < b_in)
    idx = torch.where(keep, f % (2 * b_in), torch.zeros_like(f))
    for d in dims:
        x = x.index_select(d, idx)
        shape = [1] * x.dim()
        shape[d] = -1
        x = x * keep.to(x.dtype).view(shape)
    return x


def _so3_analysis(X, b_in, b_out, table):
    """X: [z, beta, m_bin, n_bin, 2] full complex 2-D spectrum -> [nspec, z, 2]
    (so3_fft.py:44-58, 95-109)."""
    out = X.new_zeros((nspec_so3(b_out), X.size(0), 2))
    for l in range(b_out):
        L = 2 * l + 1
        lo = nspec_so3(l)
        xx = _gather_bins(X, l, b_in, (2, 3))                      # [z, beta, m, n, 2]
        w = table[:, lo:lo + L * L].view(-1, L, L)                  # [beta, m, n]
        out[lo:lo + L * L] = torch.einsum("bmn,zbmnc->mnzc", w, xx).reshape(L * L, -1, 2)
    return out


def so3_fft(x, for_grad=False, b_out=None):
    """[..., beta, alpha, gamma, 2] -> [nspec(b_out), ..., 2] (so3_fft.py:12-61)."""
    assert x.size(-1) == 2
    b_in = x.size(-2) // 2
    assert x.size(-2) == x.size(-3) == x.size(-4) == 2 * b_in
    b_out = b_in if b_out is None else b_out
    lead = x.size()[:-4]
    x = x.reshape(-1, 2 * b_in, 2 * b_in, 2 * b_in, 2)
    table = so3_table(b_in, b_out, not for_grad, x.dtype)
    X = torch.view_as_real(torch.fft.fftn(torch.view_as_complex(x.contiguous()), dim=[2, 3]))
    return _so3_analysis(X, b_in, b_out, table).view(-1, *lead, 2)


def so3_rfft(x, for_grad=False, b_out=None):
    """[..., beta, alpha, gamma] real -> [nspec(b_out), ..., 2] (so3_fft.py:64-112)."""
    b_in = x.size(-1) // 2
    assert x.size(-1) == x.size(-2) == x.size(-3) == 2 * b_in
    b_out = b_in if b_out is None else b_out
    lead = x.size()[:-3]
    x = x.reshape(-1, 2 * b_in, 2 * b_in, 2 * b_in)
    table = so3_table(b_in, b_out, not for_grad, x.dtype)
    X = torch.view_as_real(torch.fft.fftn(x.to(torch.complex128 if x.dtype == torch.float64 else torch.complex64),
                                          dim=[2, 3]))
    return _so3_analysis(X, b_in, b_out, table).view(-1, *lead, 2)


def _so3_synthesis(x, b_in, b_out, table):
    """[nspec(b_in), z, 2] -> [z, beta, alpha, gamma, 2], unnormalised inverse
    DFT (so3_fft.py:141-153, 186-197)."""
    nz = x.size(1)
    n2 = 2 * b_out
    S = x.new_zeros((nz, n2, n2, n2, 2))
    for l in range(min(b_in, b_out)):
        L = 2 * l + 1
        lo = nspec_so3(l)
        w = table[:, lo:lo + L * L].view(-1, L, L)
        o = torch.einsum("mnzc,bmn->zbmnc", x[lo:lo + L * L].view(L, L, nz, 2), w)  # [z, beta, m, n, 2]
        f = torch.arange(-l, l + 1) % n2
        S[:, :, f[:, None], f[None, :]] += o          # bins are distinct: |m|, |n| < b_out
    y = torch.fft.ifftn(torch.view_as_complex(S), dim=[2, 3]) * float(n2 * n2)
    return torch.view_as_real(y)


def so3_ifft(x, for_grad=False, b_out=None):
    """[nspec(b_in), ..., 2] -> [..., 2b_out, 2b_out, 2b_out, 2] (so3_fft.py:115-155)."""
    assert x.size(-1) == 2
    nspec = x.size(0)
    b_in = round((3 / 4 * nspec) ** (1 / 3))
    assert nspec == nspec_so3(b_in)
    b_out = b_in if b_out is None else b_out
    lead = x.size()[1:-1]
    x = x.reshape(nspec, -1, 2)
    table = so3_table(b_out, b_in, for_grad, x.dtype)
    y = _so3_synthesis(x, b_in, b_out, table)
    return y.reshape(*lead, 2 * b_out, 2 * b_out, 2 * b_out, 2)


def so3_rifft(x, for_grad=False, b_out=None):
    """Real part of so3_ifft (so3_fft.py:158-202; CPU branch semantics)."""
    return so3_ifft(x, for_grad=for_grad, b_out=b_out)[..., 0].contiguous()


class SO3_fft_real(torch.autograd.Function):
    """so3_fft.py:446-456."""

    @staticmethod
    def forward(ctx, x, b_out=None):
        ctx.b_in = x.size(-1) // 2
        return so3_rfft(x, b_out=b_out)

    @staticmethod
    def backward(ctx, g):
        return so3_ifft(g, for_grad=True, b_out=ctx.b_in)[..., 0], None


class SO3_ifft_real(torch.autograd.Function):
    """so3_fft.py:459-469."""

    @staticmethod
    def forward(ctx, x, b_out=None):
        ctx.b_in = round((3 / 4 * x.size(0)) ** (1 / 3))
        return so3_rifft(x, b_out=b_out)

    @staticmethod
    def backward(ctx, g):
        return so3_rfft(g, for_grad=True, b_out=ctx.b_in), None


# ----------------------------------------------------------------------------
# S^2 transforms (s2cnn/soft/s2_fft.py)
# ----------------------------------------------------------------------------

def s2_fft(x, for_grad=False, b_out=None):
    """[..., beta, alpha, 2] -> [b_out^2, ..., 2] (s2_fft.py:13-58)."""
    assert x.size(-1) == 2
    b_in = x.size(-2) // 2
    assert x.size(-2) == x.size(-3) == 2 * b_in
    b_out = b_in if b_out is None else b_out
    assert b_out <= b_in
    lead = x.size()[:-3]
    x = x.reshape(-1, 2 * b_in, 2 * b_in, 2)
    table = s2_table(b_in, b_out, not for_grad, x.dtype)
    X = torch.view_as_real(torch.fft.fft(torch.view_as_complex(x.contiguous())))  # [z, beta, m_bin, 2]
    out = X.new_empty((b_out * b_out, X.size(0), 2))
    for l in range(b_out):
        s = slice(l * l, l * l + 2 * l + 1)
        xx = _gather_bins(X, l, b_in, (2,))
        out[s] = torch.einsum("bm,zbmc->mzc", table[:, s], xx)
    return out.view(-1, *lead, 2)


def s2_ifft(x, for_grad=False, b_out=None):
    """[b_in^2, ..., 2] -> [..., 2b_out, 2b_out, 2] (s2_fft.py:61-106)."""
    assert x.size(-1) == 2
    nspec = x.size(0)
    b_in = round(nspec ** 0.5)
    assert nspec == b_in * b_in
    b_out = b_in if b_out is None else b_out
    assert b_out >= b_in
    lead = x.size()[1:-1]
    x = x.reshape(nspec, -1, 2)
    table = s2_table(b_out, b_in, for_grad, x.dtype)
    n2 = 2 * b_out
    S = x.new_zeros((x.size(1), n2, n2, 2))
    for l in range(b_in):
        s = slice(l * l, l * l + 2 * l + 1)
        o = torch.einsum("mzc,bm->zbmc", x[s], table[:, s])
        f = torch.arange(-l, l + 1) % n2
        S.index_add_(2, f, o)
    y = torch.view_as_real(torch.fft.ifft(torch.view_as_complex(S))) * float(n2)
    return y.reshape(*lead, n2, n2, 2)


class S2_fft_real(torch.autograd.Function):
    """s2_fft.py:226-236."""

    @staticmethod
    def forward(ctx, x, b_out=None):
        ctx.b_in = x.size(-1) // 2
        return s2_fft(as_complex(x), b_out=b_out)

    @staticmethod
    def backward(ctx, g):
        return s2_ifft(g, for_grad=True, b_out=ctx.b_in)[..., 0], None


class S2_ifft_real(torch.autograd.Function):
    """s2_fft.py:239-250."""

    @staticmethod
    def forward(ctx, x, b_out=None):
        ctx.b_in = round(x.size(0) ** 0.5)
        return s2_ifft(x, b_out=b_out)[..., 0]

    @staticmethod
    def backward(ctx, g):
        return s2_fft(as_complex(g), for_grad=True, b_out=ctx.b_in), None


# ----------------------------------------------------------------------------
# block-diagonal spectral products (s2cnn/so3_mm.py:8-61, s2cnn/s2_mm.py:10-58)
# ----------------------------------------------------------------------------

def so3_mm(x, y):
    """x [nspec, B, Fi, 2], y [nspec, Fi, Fo, 2] -> [nspec, B, Fo, 2];
    z[l,m,n] = sum_p x[l,m,p] conj(y[l,n,p]) over features (so3_mm.py:31-61)."""
    assert x.size(3) == 2 and y.size(3) == 2
    nspec, B, Fi = x.size(0), x.size(1), x.size(2)
    Fo = y.size(2)
    assert y.size(0) == nspec and y.size(1) == Fi
    nl = math.ceil((3 / 4 * nspec) ** (1 / 3))
    assert nspec == nspec_so3(nl)
    parts = []
    for l in range(nl):
        L = 2 * l + 1
        lo = nspec_so3(l)
        # rows (batch, m), contraction (f_in, p)
        X = x[lo:lo + L * L].view(L, L, B, Fi, 2).permute(2, 0, 3, 1, 4).reshape(B * L, Fi * L, 2)
        # contraction (f_in, p), columns (n, f_out)
        Y = y[lo:lo + L * L].view(L, L, Fi, Fo, 2).permute(2, 1, 0, 3, 4).reshape(Fi * L, L * Fo, 2)
        Z = complex_mm(X, Y, conj_y=True)                     # [(batch, m), (n, f_out), 2]
        parts.append(Z.view(B, L * L, Fo, 2).transpose(0, 1))
    return torch.cat(parts, 0)


def s2_mm(x, y):
    """x [b^2, B, Fi, 2], y [b^2, Fi, Fo, 2] -> [nspec(b), B, Fo, 2];
    z[l,m,n] = x[l,m] conj(y[l,n]) over features (s2_mm.py:30-58)."""
    assert x.size(3) == 2 and y.size(3) == 2
    nspec, B, Fi = x.size(0), x.size(1), x.size(2)
    Fo = y.size(2)
    assert y.size(0) == nspec and y.size(1) == Fi
    nl = round(nspec ** 0.5)
    parts = []
    for l in range(nl):
        L = 2 * l + 1
        X = x[l * l:l * l + L].reshape(L * B, Fi, 2)
        Y = y[l * l:l * l + L].transpose(0, 1).reshape(Fi, L * Fo, 2)
        Z = complex_mm(X, Y, conj_y=True).view(L, B, L, Fo, 2).transpose(1, 2)
        parts.append(Z.reshape(L * L, B, Fo, 2))
    return torch.cat(parts, 0)


# ----------------------------------------------------------------------------
# kernel -> spectrum on an arbitrary grid (s2cnn/so3_ft.py, s2cnn/s2_ft.py)
# ----------------------------------------------------------------------------

@lru_cache(maxsize=32)
def _so3_ft_matrix64(b, grid):
    F = np.zeros((len(grid), nspec_so3(b)), dtype=complex)
    for i, (beta, alpha, gamma) in enumerate(grid):
        F[i] = np.concatenate([_wigner_D64(l, alpha, beta, gamma).conj().reshape(-1) for l in range(b)])
    return F


@lru_cache(maxsize=32)
def _s2_ft_matrix64(b, grid):
    F = np.zeros((len(grid), b * b), dtype=complex)
    for i, (beta, alpha) in enumerate(grid):
        F[i] = np.concatenate([2 * b * _wigner_D64(l, alpha, beta, 0.0).conj()[:, l] for l in range(b)])
    return F


def _rft(x, F):
    Fr = torch.tensor(np.stack((F.real, F.imag), -1), dtype=x.dtype)      # [a, spec, 2]
    sz = x.size()
    out = torch.einsum("ia,afc->fic", x.reshape(-1, sz[-1]), Fr)
    return out.reshape(-1, *sz[:-1], 2)


def so3_rft(x, b, grid):
    """[..., n_grid] -> [nspec(b), ..., 2] (so3_ft.py:8-24)."""
    return _rft(x, _so3_ft_matrix64(b, tuple(map(tuple, grid))))


def s2_rft(x, b, grid):
    """[..., n_grid] -> [b^2, ..., 2] (s2_ft.py:8-24)."""
    return _rft(x, _s2_ft_matrix64(b, tuple(map(tuple, grid))))


# ----------------------------------------------------------------------------
# grids (s2cnn/s2_grid.py, s2cnn/so3_grid.py)
# ----------------------------------------------------------------------------

def _mesh(*axes):
    g = np.meshgrid(*axes, indexing="ij")
    return [a.flatten() for a in g]


def s2_near_identity_grid(max_beta=np.pi / 8, n_alpha=8, n_beta=3):
    beta = np.arange(1, n_beta + 1, dtype=float) * max_beta / n_beta
    alpha = np.linspace(0, 2 * np.pi, n_alpha, endpoint=False)
    B, A = _mesh(beta, alpha)
    return tuple(tuple(float(v) for v in ba) for ba in np.stack((B, A), 1))


def s2_equatorial_grid(max_beta=0, n_alpha=32, n_beta=1):
    beta = np.linspace(np.pi / 2 - max_beta, np.pi / 2 + max_beta, n_beta, endpoint=True)
    alpha = np.linspace(0, 2 * np.pi, n_alpha, endpoint=False)
    B, A = _mesh(beta, alpha)
    return tuple(tuple(float(v) for v in ba) for ba in np.stack((B, A), 1))


def s2_soft_grid(b):
    beta = (np.arange(2 * b) + 0.5) / (2 * b) * np.pi
    alpha = np.linspace(0, 2 * np.pi, 2 * b, endpoint=False)
    B, A = _mesh(beta, alpha)
    return tuple(tuple(float(v) for v in ba) for ba in np.stack((B, A), 1))


def so3_near_identity_grid(max_beta=np.pi / 8, max_gamma=2 * np.pi, n_alpha=8, n_beta=3, n_gamma=None):
    n_gamma = n_alpha if n_gamma is None else n_gamma
    beta = np.arange(1, n_beta + 1, dtype=float) * max_beta / n_beta
    alpha = np.linspace(0, 2 * np.pi, n_alpha, endpoint=False)
    pre_gamma = np.linspace(-max_gamma, max_gamma, n_gamma, endpoint=True)
    B, A, P = _mesh(beta, alpha, pre_gamma)
    return tuple(tuple(float(v) for v in bac) for bac in np.stack((B, A, P - A), 1))


def so3_equatorial_grid(max_beta=0, max_gamma=np.pi / 8, n_alpha=32, n_beta=1, n_gamma=2):
    beta = np.linspace(np.pi / 2 - max_beta, np.pi / 2 + max_beta, n_beta, endpoint=True)
    alpha = np.linspace(0, 2 * np.pi, n_alpha, endpoint=False)
    gamma = np.linspace(-max_gamma, max_gamma, n_gamma, endpoint=True)
    B, A, C = _mesh(beta, alpha, gamma)
    return tuple(tuple(float(v) for v in bac) for bac in np.stack((B, A, C), 1))


def so3_soft_grid(b):
    beta = (np.arange(2 * b) + 0.5) / (2 * b) * np.pi
    alpha = gamma = np.linspace(0, 2 * np.pi, 2 * b, endpoint=False)
    B, A, C = _mesh(beta, alpha, gamma)
    return tuple(tuple(float(v) for v in bac) for bac in np.stack((B, A, C), 1))


# ----------------------------------------------------------------------------
# Haar integral, layers, rotation
# ----------------------------------------------------------------------------

def so3_integrate(x):
    """[..., 2b, 2b, 2b] -> [...] (s2cnn/soft/so3_integrate.py:7-29)."""
    b = x.size(-1) // 2
    w = quadrature_weights(b, x.dtype)
    s = x.sum(-1).sum(-1)                      # [..., beta]
    return torch.mm(s.reshape(-1, 2 * b), w.view(2 * b, 1)).view(s.size()[:-1])


def so3_conv_scaling(n_grid, f_in, b_in, b_out):
    return 1.0 / math.sqrt(n_grid * f_in * (b_out ** 3.0) / (b_in ** 3.0))   # so3_conv.py:34


def s2_conv_scaling(n_grid, f_in, b_in, b_out):
    return 1.0 / math.sqrt(n_grid * f_in * (b_out ** 4.0) / (b_in ** 2.0))   # s2_conv.py:29


def so3_conv(x, kernel, bias, b_in, b_out, grid):
    """SO3Convolution.forward (s2cnn/soft/so3_conv.py:36-58)."""
    f_in = kernel.size(0)
    xs = SO3_fft_real.apply(x, b_out)
    ys = so3_rft(kernel * so3_conv_scaling(len(grid), f_in, b_in, b_out), b_out, grid)
    zs = so3_mm(xs, ys)
    return SO3_ifft_real.apply(zs) + bias


def s2_conv(x, kernel, bias, b_in, b_out, grid):
    """S2Convolution.forward (s2cnn/soft/s2_conv.py:32-47)."""
    f_in = kernel.size(0)
    xs = S2_fft_real.apply(x, b_out)
    ys = s2_rft(kernel * s2_conv_scaling(len(grid), f_in, b_in, b_out), b_out, grid)
    zs = s2_mm(xs, ys)
    return SO3_ifft_real.apply(zs) + bias


def so3_rotation(x, alpha, beta, gamma):
    """[..., 2b, 2b, 2b] rotated spectrally (s2cnn/soft/so3_rotation.py:11-49)."""
    b = x.size(-1) // 2
    shape = x.size()
    xs = SO3_fft_real.apply(x)
    parts = []
    for l in range(b):
        L = 2 * l + 1
        lo = nspec_so3(l)
        U = _wigner_D64(l, alpha, beta, gamma)
        U = torch.tensor(np.stack((U.real, U.imag), -1), dtype=x.dtype)
        Fx = xs[lo:lo + L * L].reshape(L, -1, 2)
        parts.append(complex_mm(U, Fx, conj_x=True).reshape(L * L, -1, 2))
    z = SO3_ifft_real.apply(torch.cat(parts, 0))
    return z.contiguous().view(*shape)
