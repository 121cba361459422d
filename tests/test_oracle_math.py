"""Pins for the oracle's special functions (oracle/wigner_ref.py) and for the
product's generator (s2cnn_amd/wigner.py): closed forms, invariants, library
routines and three mutually independent formulas."""
import math

import numpy as np
import pytest

from oracle import wigner_ref as R
from s2cnn_amd import wigner as W

BETAS = [0.0, 0.3, 1.1, math.pi / 2, 2.9, math.pi]


def test_closed_forms_l1_l2():
    for b in BETAS:
        c, s = math.cos(b), math.sin(b)
        d1 = np.array([[(1 + c) / 2, s / math.sqrt(2), (1 - c) / 2],
                       [-s / math.sqrt(2), c, s / math.sqrt(2)],
                       [(1 - c) / 2, -s / math.sqrt(2), (1 + c) / 2]])
        for f in (R.wigner_d_jacobi, R.wigner_d_sum, lambda l, x: W.wigner_d(l, [x])[0]):
            assert np.allclose(f(1, b), d1, atol=1e-13)
            d2 = f(2, b)
            assert abs(d2[2 + 2, 2 + 2] - ((1 + c) / 2) ** 2) < 1e-13           # d^2_{22}
            assert abs(d2[2 + 2, 2 + 1] - (-(1 + c) * s / 2)) < 1e-13          # d^2_{21}
            assert abs(d2[2 + 2, 2 + 0] - math.sqrt(6) / 4 * s * s) < 1e-13    # d^2_{20}
            assert abs(d2[2 + 1, 2 + 0] - (-math.sqrt(1.5) * s * c)) < 1e-13   # d^2_{10}
            assert abs(d2[2 + 0, 2 + 0] - (3 * c * c - 1) / 2) < 1e-13         # d^2_{00}
            assert abs(d2[2 + 1, 2 - 1] - (1 - c) * (2 * c + 1) / 2) < 1e-13   # d^2_{1,-1}


def test_sympy_rotation_d():
    from sympy import N, Rational
    from sympy.physics.quantum.spin import Rotation
    beta = Rational(7, 10)
    for l in (1, 2, 3):
        d = R.wigner_d_jacobi(l, 0.7)
        for m in range(-l, l + 1):
            for n in range(-l, l + 1):
                ref = float(N(Rotation.d(l, m, n, beta).doit()))
                assert abs(d[m + l, n + l] - ref) < 1e-12


@pytest.mark.parametrize("l", [0, 1, 2, 5, 9, 17, 31])
def test_three_formulas_agree(l):
    for b in BETAS[1:-1]:
        a = W.wigner_d(l, [b])[0]
        j = R.wigner_d_jacobi(l, b)
        assert np.abs(a - j).max() < 1e-12
        if l <= 9:
            assert np.abs(R.wigner_d_sum(l, b) - j).max() < 1e-12


@pytest.mark.parametrize("l", [1, 4, 12, 31])
def test_invariants(l):
    m = np.arange(-l, l + 1)
    sgn = (-1.0) ** (m[:, None] - m[None, :])
    for f in (R.wigner_d_jacobi, lambda l_, x: W.wigner_d(l_, [x])[0]):
        assert np.allclose(f(l, 0.0), np.eye(2 * l + 1), atol=1e-12)
        dpi = f(l, math.pi)
        expect = np.zeros_like(dpi)
        for n in m:
            expect[-n + l, n + l] = (-1.0) ** (l - n)        # d^l_{mn}(pi) = (-1)^{l-n} delta_{m,-n}
        assert np.allclose(dpi, expect, atol=1e-11)
        d = f(l, 0.9)
        assert np.allclose(d @ d.T, np.eye(2 * l + 1), atol=1e-12)               # orthogonal
        assert np.allclose(d[::-1, ::-1], sgn * d, atol=1e-12)                    # d_{-m,-n} = (-1)^{m-n} d_{mn}
        assert np.allclose(d.T, sgn * d, atol=1e-12)                              # d_{nm} = (-1)^{m-n} d_{mn}
        assert np.allclose(f(l, 0.4) @ f(l, 0.5), d, atol=1e-12)                  # one-parameter group


def test_legendre_column():
    from scipy.special import eval_legendre, lpmv
    for l in (1, 3, 8, 20):
        for b in (0.4, 1.7, 2.8):
            d = R.wigner_d_jacobi(l, b)
            assert abs(d[l, l] - eval_legendre(l, math.cos(b))) < 1e-12
            for m in range(0, l + 1):
                # d^l_{m0} = sqrt((l-m)!/(l+m)!) P_l^m(cos b), Condon-Shortley phase in lpmv
                ref = math.sqrt(math.factorial(l - m) / math.factorial(l + m)) * lpmv(m, l, math.cos(b))
                assert abs(d[m + l, l] - ref) < 1e-11


@pytest.mark.parametrize("b", [1, 2, 5, 16, 32])
def test_quadrature_weights(b):
    w_closed = W.quadrature_weights(b)
    w_ref = R.quadrature_weights_ref(b)
    assert np.allclose(w_closed, w_ref, rtol=1e-10, atol=1e-16)
    assert abs(w_ref.sum() * (2 * b) ** 2 - 1) < 1e-12
    assert (w_ref > 0).all()


@pytest.mark.parametrize("b", [3, 8])
def test_quadrature_exact_orthogonality(b):
    """sum_beta w d^l_mn d^l'_mn = delta_ll' / ((2l+1)(2b)^2) for l, l' < b: what
    makes fft -> ifft the identity on band-limited signals (tests/so3_fft.py:34-91)."""
    w = R.quadrature_weights_ref(b)
    betas = W.soft_betas(b)
    d = [np.stack([R.wigner_d_jacobi(l, x) for x in betas]) for l in range(b)]
    for l in range(b):
        for lp in range(b):
            k = min(l, lp)
            a = d[l][:, l - k:l + k + 1, l - k:l + k + 1]
            c = d[lp][:, lp - k:lp + k + 1, lp - k:lp + k + 1]
            g = np.einsum("b,bmn,bmn->mn", w, a, c)
            want = (1.0 / ((2 * l + 1) * (2 * b) ** 2)) if l == lp else 0.0
            assert np.allclose(g, want, atol=1e-14)


@pytest.mark.parametrize("b,nl", [(4, 4), (6, 3), (3, 5), (32, 32)])
def test_product_tables_match_oracle_tables(b, nl):
    from oracle import cpu_path
    for weighted in (True, False):
        a = W.so3_wigner_table(b, nl, weighted)
        r = cpu_path._so3_table64(b, nl, weighted)
        assert a.shape == r.shape
        assert np.abs(a - r).max() < 1e-12 * max(1.0, np.abs(r).max())
        a2 = W.s2_wigner_table(b, nl, weighted)
        r2 = cpu_path._s2_table64(b, nl, weighted)
        assert np.abs(a2 - r2).max() < 1e-12 * max(1.0, np.abs(r2).max())
    if b <= 6:
        assert np.allclose(cpu_path._so3_table64(b, nl, True), R.so3_table_ref(b, nl, True), atol=1e-15)
        assert np.allclose(cpu_path._s2_table64(b, nl, False), R.s2_table_ref(b, nl, False), atol=1e-13)


def test_ft_matrices_match():
    from oracle import cpu_path
    g3 = cpu_path.so3_near_identity_grid(n_alpha=4, n_beta=2, n_gamma=3)
    a = W.so3_ft_matrix(5, g3)
    r = cpu_path._so3_ft_matrix64(5, g3)
    assert np.abs(a - r).max() < 1e-12
    g2 = cpu_path.s2_near_identity_grid(n_alpha=5, n_beta=2)
    assert np.abs(W.s2_ft_matrix(6, g2) - cpu_path._s2_ft_matrix64(6, g2)).max() < 1e-11
