"""Float64 host-side generator for everything the spectral path takes from the
representation theory of SO(3): SOFT quadrature weights, Wigner small-d tables
on the SOFT beta grid, and Wigner-D samples on arbitrary (beta, alpha, gamma)
points.

It stands in for the third-party package the reference calls at
s2cnn/soft/so3_fft.py:214-230, s2cnn/soft/s2_fft.py:118-142,
s2cnn/so3_ft.py:29-42, s2cnn/s2_ft.py:29-40, s2cnn/soft/so3_integrate.py:35-37
and s2cnn/soft/so3_rotation.py:53-56.

Conventions (rows m, columns n, both ascending -l..l, "centered" order):

    d^l_{mn}(beta) = <l m| exp(-i beta J_y) |l n>          (d^1_{1,0} = -sin(beta)/sqrt 2)
    D^l_{mn}(alpha, beta, gamma) = exp(i m alpha) d^l_{mn}(beta) exp(i n gamma)

The second line is the convention stated at s2cnn/soft/so3_rotation.py:58.

Method: d^l(beta) = V exp(-i beta Lambda) V^H where J_y = V Lambda V^H is the
eigendecomposition of the (2l+1)x(2l+1) Hermitian tridiagonal J_y and Lambda is
known exactly (-l..l).  The result is real; accuracy is a few 1e-15 * l.
"""
from functools import lru_cache

import numpy as np


def soft_betas(b):
    """beta_j = pi (2j+1) / (4b), j < 2b  (s2cnn/soft/so3_fft.py:219)."""
    return (np.arange(2 * b) + 0.5) / (2 * b) * np.pi


def quadrature_weights(b):
    """SOFT quadrature weights over beta, normalised so that the sum over the
    whole 2b x 2b x 2b grid of w[beta] is 1 (so the sum over beta alone is
    1/(2b)^2).  This is what s2cnn/soft/so3_fft.py:220 and
    s2cnn/soft/so3_integrate.py:37 obtain from S3.quadrature_weights(b).

    Closed form (Kostelec & Rockmore): w_j = (2/b) sin(beta_j) sum_{k<b}
    sin((2k+1) beta_j)/(2k+1), which integrates Legendre polynomials of degree
    < 2b exactly against sin(beta) dbeta (total 2); divided by 2 (2b)^2.
    """
    j = np.arange(2 * b)
    k = np.arange(b)
    beta = np.pi * (2 * j + 1) / (4 * b)
    inner = np.sum(np.sin(np.outer(2 * j + 1, 2 * k + 1) * np.pi / (4 * b)) / (2 * k + 1), axis=1)
    w = (2.0 / b) * np.sin(beta) * inner
    return w / (2.0 * (2 * b) ** 2)


@lru_cache(maxsize=512)
def _jy_eigvecs(l):
    """Eigenvectors of J_y for degree l, columns ordered by eigenvalue -l..l."""
    n = 2 * l + 1
    m = np.arange(-l, l)  # couples m -> m+1
    c = np.sqrt((l - m) * (l + m + 1.0))
    jy = np.zeros((n, n), dtype=np.complex128)
    idx = np.arange(n - 1)
    jy[idx + 1, idx] = -0.5j * c  # <m+1| J_y |m>
    jy[idx, idx + 1] = 0.5j * c   # <m| J_y |m+1>
    w, v = np.linalg.eigh(jy)
    assert np.allclose(w, np.arange(-l, l + 1), atol=1e-9 * (l + 1))
    return v


def wigner_d(l, betas):
    """d^l(beta) for an array of betas: float64 [len(betas), 2l+1, 2l+1]."""
    betas = np.atleast_1d(np.asarray(betas, dtype=np.float64))
    if l == 0:
        return np.ones((len(betas), 1, 1))
    v = _jy_eigvecs(l)
    lam = np.arange(-l, l + 1)
    phase = np.exp(-1j * np.outer(betas, lam))  # [beta, k]
    # d[b, m, n] = sum_k v[m, k] phase[b, k] conj(v[n, k])
    d = np.matmul(v[None, :, :] * phase[:, None, :], v.conj().T[None, :, :])
    return np.ascontiguousarray(d.real)


def wigner_D(l, alpha, beta, gamma):
    """D^l_{mn}(alpha, beta, gamma) = exp(i m alpha) d^l_{mn}(beta) exp(i n gamma)
    for arrays of angles of equal length: complex128 [npts, 2l+1, 2l+1]."""
    alpha = np.atleast_1d(np.asarray(alpha, dtype=np.float64))
    beta = np.atleast_1d(np.asarray(beta, dtype=np.float64))
    gamma = np.atleast_1d(np.asarray(gamma, dtype=np.float64))
    ub, inv = np.unique(beta, return_inverse=True)
    d = wigner_d(l, ub)[inv]
    m = np.arange(-l, l + 1)
    ea = np.exp(1j * np.outer(alpha, m))
    eg = np.exp(1j * np.outer(gamma, m))
    return ea[:, :, None] * d * eg[:, None, :]


def so3_nspec(b):
    return b * (4 * b * b - 1) // 3


@lru_cache(maxsize=32)
def so3_wigner_table(b, nl, weighted):
    """Table [2b, nspec(nl)] of d^l_{mn}(beta_j), degree-major then m then n,
    scaled per row by w[j] (weighted) or per degree by 2l+1 (not weighted).
    Same contents as s2cnn/soft/so3_fft.py:212-243, float64."""
    betas = soft_betas(b)
    w = quadrature_weights(b)
    out = np.empty((2 * b, so3_nspec(nl)), dtype=np.float64)
    pos = 0
    for l in range(nl):
        n = (2 * l + 1) ** 2
        d = wigner_d(l, betas).reshape(2 * b, n)
        out[:, pos:pos + n] = d * w[:, None] if weighted else d * (2 * l + 1)
        pos += n
    return out


@lru_cache(maxsize=32)
def s2_wigner_table(b, nl, weighted):
    """Table [2b, nl^2] of d^l_{m0}(beta_j), degree-major then m, scaled by
    2b w[j] (weighted) or 2l+1 (not weighted): s2cnn/soft/s2_fft.py:116-147."""
    betas = soft_betas(b)
    w = quadrature_weights(b) * 2 * b
    out = np.empty((2 * b, nl * nl), dtype=np.float64)
    for l in range(nl):
        d = wigner_d(l, betas)[:, :, l]  # column n = 0
        out[:, l * l:l * l + 2 * l + 1] = d * w[:, None] if weighted else d * (2 * l + 1)
    return out


def so3_ft_matrix(b, grid):
    """F[a, lmn] = conj(D^l_{mn}(alpha_a, beta_a, gamma_a)) for grid points given
    as (beta, alpha, gamma) tuples: complex128 [len(grid), nspec(b)]
    (s2cnn/so3_ft.py:28-52)."""
    g = np.asarray(grid, dtype=np.float64).reshape(-1, 3)
    beta, alpha, gamma = g[:, 0], g[:, 1], g[:, 2]
    out = np.empty((len(g), so3_nspec(b)), dtype=np.complex128)
    pos = 0
    for l in range(b):
        n = (2 * l + 1) ** 2
        out[:, pos:pos + n] = wigner_D(l, alpha, beta, gamma).conj().reshape(len(g), n)
        pos += n
    return out


def real_basis_matrix(l):
    """Unitary U_l [2l+1, 2l+1] (complex128) that makes the degree-l block of a real signal's SO(3)
    spectrum real: for X[-m,-n] = (-1)^(m-n) conj(X[m,n]) the matrix U X U^H has no imaginary part.
    Rows are the real index r = -l..l (r > 0 cosine-like, r < 0 sine-like), columns m = -l..l."""
    L = 2 * l + 1
    U = np.zeros((L, L), dtype=np.complex128)
    U[l, l] = 1.0
    s = 1.0 / np.sqrt(2.0)
    for m in range(1, l + 1):
        sg = -1.0 if m & 1 else 1.0
        U[l + m, l + m] = s
        U[l + m, l - m] = sg * s
        U[l - m, l + m] = -1j * s
        U[l - m, l - m] = 1j * sg * s
    return U


def so3_ft_matrix_real(b, grid):
    """The matrix of so3_ft_matrix in the real basis: Re(U_l F[a, l] U_l^H) per grid point and degree,
    float64 [len(grid), nspec(b)].  The imaginary part that is dropped vanishes identically because
    Wigner D-functions obey D^l_{-m,-n} = (-1)^(m-n) conj(D^l_{mn})."""
    F = so3_ft_matrix(b, grid)
    out = np.empty(F.shape, dtype=np.float64)
    pos = 0
    for l in range(b):
        L = 2 * l + 1
        U = real_basis_matrix(l)
        blk = F[:, pos:pos + L * L].reshape(-1, L, L)
        out[:, pos:pos + L * L] = np.einsum("rm,amn,sn->ars", U, blk, U.conj()).real.reshape(-1, L * L)
        pos += L * L
    return out


def s2_ft_matrix(b, grid):
    """F[a, lm] = 2b conj(D^l_{m0}(alpha_a, beta_a, 0)) for grid points given as
    (beta, alpha) tuples: complex128 [len(grid), b^2] (s2cnn/s2_ft.py:28-50)."""
    g = np.asarray(grid, dtype=np.float64).reshape(-1, 2)
    beta, alpha = g[:, 0], g[:, 1]
    out = np.empty((len(g), b * b), dtype=np.complex128)
    zero = np.zeros_like(alpha)
    for l in range(b):
        D = wigner_D(l, alpha, beta, zero).conj()
        out[:, l * l:l * l + 2 * l + 1] = (2 * b) * D[:, :, l]
    return out


def so3_rft_plan(b, grid, max_betas=4):
    """Factorisation of so3_ft_matrix for grids with few distinct beta values (every grid of
    s2cnn/so3_grid.py:6-37 is of that kind): with A_i the points whose beta is beta_i,

        F[a, (l,m,n)] = d^l_{mn}(beta_i) * E_a[m, n],   E_a[m, n] = exp(-i (m alpha_a + n gamma_a)),   a in A_i,

    so the transform of x is  y[l,m,n] = sum_i d^l_{mn}(beta_i) G_i[m,n],  G_i = sum_{a in A_i} x_a E_a:
    a small GEMM per beta_i followed by a pass that is linear in the size of the result.

    Returns None when the grid has more than `max_betas` distinct betas, else (idx, E, dtab), float64:
      idx  [nbeta, P] int64   grid index of each group member (-1: padding)
      E    [nbeta, P, R]      R = (2b-1) * b * 2; column ((m + b-1) * b + n) * 2 + (0: re, 1: im), m in -(b-1)..b-1,
                              n in 0..b-1 (the half n >= 0 suffices for real x)
      dtab [nbeta, nspec(b)]  d^l_{mn}(beta_i), degree-major then m then n
    """
    g = np.asarray(grid, dtype=np.float64).reshape(-1, 3)
    ub, inv = np.unique(np.round(g[:, 0], 12), return_inverse=True)
    if len(ub) > max_betas:
        return None
    groups = [np.nonzero(inv == i)[0] for i in range(len(ub))]
    P = max(len(q) for q in groups)
    idx = -np.ones((len(ub), P), dtype=np.int64)
    m = np.arange(-(b - 1), b)[:, None]
    n = np.arange(b)[None, :]
    E = np.zeros((len(ub), P, (2 * b - 1) * b * 2), dtype=np.float64)
    for i, q in enumerate(groups):
        idx[i, :len(q)] = q
        for p, a in enumerate(q):
            ang = m * g[a, 1] + n * g[a, 2]
            E[i, p, 0::2] = np.cos(ang).reshape(-1)
            E[i, p, 1::2] = -np.sin(ang).reshape(-1)
    dtab = np.empty((len(ub), so3_nspec(b)), dtype=np.float64)
    pos = 0
    for l in range(b):
        cnt = (2 * l + 1) ** 2
        dtab[:, pos:pos + cnt] = wigner_d(l, g[[q[0] for q in groups], 0]).reshape(len(ub), cnt)
        pos += cnt
    return idx, E, dtab
