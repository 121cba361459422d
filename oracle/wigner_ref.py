"""TEST INFRASTRUCTURE ONLY - never imported by the product package.

Independent evaluation of the special functions the spectral path needs, by
formulas that share nothing with the product's eigendecomposition generator:

  * wigner_d_jacobi : Jacobi-polynomial closed form (scipy.special.eval_jacobi)
  * wigner_d_sum    : Wigner's explicit factorial sum in mpmath arithmetic
                      (exact coefficients; use for small l)
  * quadrature_weights_ref : SOFT weights from the defining linear system
                      (exact integration of Legendre polynomials), not from the
                      closed-form sine series

They stand in for lie_learn (absent, unpinned version), which the reference
calls at s2cnn/soft/so3_fft.py:214-230 (wigner_d_matrix, field='complex',
normalization='quantum', order='centered', condon_shortley='cs') and
s2cnn/soft/so3_fft.py:220 (S3.quadrature_weights).

Convention: d^l_{mn}(beta) = <l m|exp(-i beta J_y)|l n>, rows m and columns n
ascending -l..l.  PARITY UNPINNED for one bit: whether lie_learn's d equals this
or its transpose (= S d S, S = diag((-1)^m)) cannot be checked without
lie_learn.  Convolution outputs, fft->ifft round trips and all gradients are
invariant to that choice (tests/test_oracle_math.py::test_transpose_invariance).
"""
import math

import numpy as np


def wigner_d_jacobi(l, beta):
    """d^l(beta) [2l+1, 2l+1] float64 via the Jacobi-polynomial form."""
    from scipy.special import eval_jacobi, gammaln

    out = np.zeros((2 * l + 1, 2 * l + 1))
    sb, cb = math.sin(beta / 2), math.cos(beta / 2)
    for mp in range(-l, l + 1):      # row index  m'
        for m in range(-l, l + 1):   # column index m
            k = min(l + m, l - m, l + mp, l - mp)
            if k == l + m:
                a, lam = mp - m, mp - m
            elif k == l - m:
                a, lam = m - mp, 0
            elif k == l + mp:
                a, lam = m - mp, 0
            else:
                a, lam = mp - m, mp - m
            b = 2 * l - 2 * k - a
            # sqrt( C(2l-k, k+a) / C(k+b, b) ) in log space
            logc = 0.5 * (gammaln(2 * l - k + 1) - gammaln(k + a + 1) - gammaln(2 * l - 2 * k - a + 1)
                          - gammaln(k + b + 1) + gammaln(b + 1) + gammaln(k + 1))
            val = math.exp(logc) * (sb ** a) * (cb ** b) * eval_jacobi(k, a, b, math.cos(beta))
            out[mp + l, m + l] = -val if lam % 2 else val
    return out


def wigner_d_sum(l, beta, dps=60):
    """d^l(beta) by Wigner's explicit sum, evaluated in mpmath with `dps` digits
    so the alternating sum does not cancel; returned as float64."""
    import mpmath as mp

    mp.mp.dps = dps
    c, s = mp.cos(mp.mpf(beta) / 2), mp.sin(mp.mpf(beta) / 2)
    f = [mp.factorial(i) for i in range(2 * l + 2)]
    out = np.zeros((2 * l + 1, 2 * l + 1))
    for mp_ in range(-l, l + 1):
        for m in range(-l, l + 1):
            pref = mp.sqrt(f[l + mp_] * f[l - mp_] * f[l + m] * f[l - m])
            tot = mp.mpf(0)
            for t in range(max(0, m - mp_), min(l + m, l - mp_) + 1):
                term = (c ** (2 * l + m - mp_ - 2 * t)) * (s ** (mp_ - m + 2 * t))
                term /= f[l + m - t] * f[t] * f[mp_ - m + t] * f[l - mp_ - t]
                tot += -term if (mp_ - m + t) % 2 else term
            out[mp_ + l, m + l] = float(pref * tot)
    return out


def quadrature_weights_ref(b):
    """Weights on beta_j = pi(2j+1)/(4b) such that sum_j w_j P_k(cos beta_j) =
    2 delta_{k0} for all k < 2b (2b equations, 2b unknowns), then divided by
    2 (2b)^2 as the reference's S3.quadrature_weights is (see the normalisation
    forced by tests/so3_fft.py:34-64 of the reference: unnormalised forward and
    inverse DFTs with idempotent fft->ifft)."""
    from numpy.polynomial import legendre

    beta = np.pi * (2 * np.arange(2 * b) + 1) / (4 * b)
    x = np.cos(beta)
    A = np.stack([legendre.legval(x, [0] * k + [1]) for k in range(2 * b)])  # [k, j]
    rhs = np.zeros(2 * b)
    rhs[0] = 2.0
    w = np.linalg.solve(A, rhs)
    return w / (2.0 * (2 * b) ** 2)


def so3_table_ref(b, nl, weighted):
    """[2b, nspec(nl)] table as in s2cnn/soft/so3_fft.py:212-243, from the
    Jacobi form and the linear-system weights."""
    betas = (np.arange(2 * b) + 0.5) / (2 * b) * np.pi
    w = quadrature_weights_ref(b)
    rows = []
    for j, beta in enumerate(betas):
        ds = []
        for l in range(nl):
            d = wigner_d_jacobi(l, beta).reshape(-1)
            ds.append(d * w[j] if weighted else d * (2 * l + 1))
        rows.append(np.concatenate(ds))
    return np.stack(rows)


def s2_table_ref(b, nl, weighted):
    """[2b, nl^2] table as in s2cnn/soft/s2_fft.py:116-147."""
    betas = (np.arange(2 * b) + 0.5) / (2 * b) * np.pi
    w = quadrature_weights_ref(b) * 2 * b
    rows = []
    for j, beta in enumerate(betas):
        ds = []
        for l in range(nl):
            d = wigner_d_jacobi(l, beta)[:, l]
            ds.append(d * w[j] if weighted else d * (2 * l + 1))
        rows.append(np.concatenate(ds))
    return np.stack(rows)
