"""TEST INFRASTRUCTURE ONLY - never imported by the product package.

Direct O(b^6) evaluation, in float64 numpy, of the definitions the transforms
implement (s2cnn/soft/calculus.pdf: U^l_mn = e^{i m alpha} d^l_mn(beta)
e^{i n gamma}; forward transform = quadrature against conj(U), inverse =
sum_l (2l+1) sum_mn F^l_mn U^l_mn).  No FFT, no bin bookkeeping, Wigner values
from the explicit factorial sum: a dropped term, a wrong sign or a transposed
index in oracle/cpu_path.py or in the HIP kernels cannot cancel here.
Only for b <= 4.
"""
import numpy as np

from . import wigner_ref


def _d_tables(b_grid, nl):
    betas = (np.arange(2 * b_grid) + 0.5) / (2 * b_grid) * np.pi
    return [np.stack([wigner_ref.wigner_d_sum(l, bt) for bt in betas]) for l in range(nl)]  # [l][beta, m, n]


def so3_analysis(x, b_out, weighted=True):
    """x complex [z, 2b, 2b, 2b] (beta, alpha, gamma) -> complex [nspec(b_out), z]."""
    b_in = x.shape[-1] // 2
    ang = 2 * np.pi * np.arange(2 * b_in) / (2 * b_in)
    w = wigner_ref.quadrature_weights_ref(b_in)
    d = _d_tables(b_in, b_out)
    out = []
    for l in range(b_out):
        for m in range(-l, l + 1):
            for n in range(-l, l + 1):
                if abs(m) >= b_in or abs(n) >= b_in:
                    out.append(np.zeros(x.shape[0], dtype=complex))
                    continue
                scale = w if weighted else np.full(2 * b_in, 2 * l + 1.0)
                ker = (scale * d[l][:, m + l, n + l])[:, None, None] \
                    * np.exp(-1j * m * ang)[None, :, None] * np.exp(-1j * n * ang)[None, None, :]
                out.append(np.einsum("zbac,bac->z", x, ker))
    return np.stack(out)


def so3_synthesis(xh, b_out, weighted=False):
    """xh complex [nspec(b_in), z] -> complex [z, 2b_out, 2b_out, 2b_out]."""
    nspec = xh.shape[0]
    b_in = round((3 / 4 * nspec) ** (1 / 3))
    ang = 2 * np.pi * np.arange(2 * b_out) / (2 * b_out)
    w = wigner_ref.quadrature_weights_ref(b_out)
    nl = min(b_in, b_out)
    d = _d_tables(b_out, nl)
    y = np.zeros((xh.shape[1], 2 * b_out, 2 * b_out, 2 * b_out), dtype=complex)
    pos = 0
    for l in range(b_in):
        for m in range(-l, l + 1):
            for n in range(-l, l + 1):
                if l < nl:
                    scale = w if weighted else np.full(2 * b_out, 2 * l + 1.0)
                    ker = (scale * d[l][:, m + l, n + l])[:, None, None] \
                        * np.exp(1j * m * ang)[None, :, None] * np.exp(1j * n * ang)[None, None, :]
                    y += xh[pos][:, None, None, None] * ker[None]
                pos += 1
    return y


def s2_analysis(x, b_out, weighted=True):
    """x complex [z, 2b, 2b] (beta, alpha) -> complex [b_out^2, z]."""
    b_in = x.shape[-1] // 2
    ang = 2 * np.pi * np.arange(2 * b_in) / (2 * b_in)
    w = wigner_ref.quadrature_weights_ref(b_in) * 2 * b_in
    d = _d_tables(b_in, b_out)
    out = []
    for l in range(b_out):
        for m in range(-l, l + 1):
            scale = w if weighted else np.full(2 * b_in, 2 * l + 1.0)
            ker = (scale * d[l][:, m + l, l])[:, None] * np.exp(-1j * m * ang)[None, :]
            out.append(np.einsum("zba,ba->z", x, ker))
    return np.stack(out)


def s2_synthesis(xh, b_out, weighted=False):
    """xh complex [b_in^2, z] -> complex [z, 2b_out, 2b_out]."""
    b_in = round(xh.shape[0] ** 0.5)
    ang = 2 * np.pi * np.arange(2 * b_out) / (2 * b_out)
    w = wigner_ref.quadrature_weights_ref(b_out) * 2 * b_out
    d = _d_tables(b_out, b_in)
    y = np.zeros((xh.shape[1], 2 * b_out, 2 * b_out), dtype=complex)
    pos = 0
    for l in range(b_in):
        for m in range(-l, l + 1):
            scale = w if weighted else np.full(2 * b_out, 2 * l + 1.0)
            ker = (scale * d[l][:, m + l, l])[:, None] * np.exp(1j * m * ang)[None, :]
            y += xh[pos][:, None, None] * ker[None]
            pos += 1
    return y


def so3_mm(x, y, nl):
    """complex x [nspec, B, Fi], y [nspec, Fi, Fo] -> z [nspec, B, Fo] with
    z[l,m,n,i,j] = sum_{p,k} x[l,m,p,i,k] conj(y[l,n,p,k,j])  (s2cnn/so3_mm.py:31-61)."""
    out = []
    pos = 0
    for l in range(nl):
        L = 2 * l + 1
        X = x[pos:pos + L * L].reshape(L, L, *x.shape[1:])
        Y = y[pos:pos + L * L].reshape(L, L, *y.shape[1:])
        out.append(np.einsum("mpik,npkj->mnij", X, Y.conj()).reshape(L * L, x.shape[1], y.shape[2]))
        pos += L * L
    return np.concatenate(out)


def s2_mm(x, y, nl):
    """complex x [nl^2, B, Fi], y [nl^2, Fi, Fo] -> z [nspec(nl), B, Fo] with
    z[l,m,n,i,j] = sum_k x[l,m,i,k] conj(y[l,n,k,j])  (s2cnn/s2_mm.py:30-58)."""
    out = []
    for l in range(nl):
        L = 2 * l + 1
        X = x[l * l:l * l + L]
        Y = y[l * l:l * l + L]
        out.append(np.einsum("mik,nkj->mnij", X, Y.conj()).reshape(L * L, x.shape[1], y.shape[2]))
    return np.concatenate(out)
