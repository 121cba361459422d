"""Pins for oracle/cpu_path.py: brute-force evaluation of the definitions on tiny
bandwidths, the identities the reference's own test script asserts
(tests/so3_fft.py of the reference), adjoint pairs, and convention invariance."""
import math

import numpy as np
import pytest
import torch

from oracle import brute, cpu_path as O

torch.manual_seed(0)
D = torch.float64


def c2np(t):
    return t[..., 0].numpy() + 1j * t[..., 1].numpy()


def np2c(a):
    return torch.tensor(np.stack((a.real, a.imag), -1), dtype=D)


# ---------------- brute force ----------------

@pytest.mark.parametrize("b_in,b_out", [(2, 2), (3, 2), (2, 3), (3, 3), (4, 2)])
@pytest.mark.parametrize("for_grad", [False, True])
def test_so3_fft_vs_definition(b_in, b_out, for_grad):
    g = torch.Generator().manual_seed(b_in * 10 + b_out)
    x = torch.randn(2, 2 * b_in, 2 * b_in, 2 * b_in, 2, dtype=D, generator=g)
    want = brute.so3_analysis(c2np(x), b_out, weighted=not for_grad)
    got = c2np(O.so3_fft(x, for_grad=for_grad, b_out=b_out))
    assert np.abs(got - want).max() < 1e-12 * max(1, np.abs(want).max())
    xr = x[..., 0].contiguous()
    want_r = brute.so3_analysis(xr.numpy().astype(complex), b_out, weighted=not for_grad)
    got_r = c2np(O.so3_rfft(xr, for_grad=for_grad, b_out=b_out))
    assert np.abs(got_r - want_r).max() < 1e-12 * max(1, np.abs(want_r).max())


@pytest.mark.parametrize("b_in,b_out", [(2, 2), (3, 2), (2, 3), (3, 3), (2, 4)])
@pytest.mark.parametrize("for_grad", [False, True])
def test_so3_ifft_vs_definition(b_in, b_out, for_grad):
    g = torch.Generator().manual_seed(b_in * 10 + b_out)
    xh = torch.randn(O.nspec_so3(b_in), 2, 2, dtype=D, generator=g)
    want = brute.so3_synthesis(c2np(xh), b_out, weighted=for_grad)
    got = c2np(O.so3_ifft(xh, for_grad=for_grad, b_out=b_out))
    assert np.abs(got - want).max() < 1e-11 * max(1, np.abs(want).max())
    got_r = O.so3_rifft(xh, for_grad=for_grad, b_out=b_out).numpy()
    assert np.abs(got_r - want.real).max() < 1e-11 * max(1, np.abs(want).max())


@pytest.mark.parametrize("b_in,b_out", [(2, 2), (3, 2), (4, 3), (4, 1)])
@pytest.mark.parametrize("for_grad", [False, True])
def test_s2_fft_vs_definition(b_in, b_out, for_grad):
    g = torch.Generator().manual_seed(b_in * 10 + b_out)
    x = torch.randn(3, 2 * b_in, 2 * b_in, 2, dtype=D, generator=g)
    want = brute.s2_analysis(c2np(x), b_out, weighted=not for_grad)
    got = c2np(O.s2_fft(x, for_grad=for_grad, b_out=b_out))
    assert np.abs(got - want).max() < 1e-12 * max(1, np.abs(want).max())
    xh = torch.randn(b_out ** 2, 3, 2, dtype=D, generator=g)
    want = brute.s2_synthesis(c2np(xh), b_in, weighted=for_grad)
    got = c2np(O.s2_ifft(xh, for_grad=for_grad, b_out=b_in))
    assert np.abs(got - want).max() < 1e-11 * max(1, np.abs(want).max())


def test_mm_vs_definition():
    g = torch.Generator().manual_seed(5)
    nl, B, Fi, Fo = 4, 2, 3, 5                         # sizes of s2cnn/so3_mm.py:264-271
    x = torch.randn(O.nspec_so3(nl), B, Fi, 2, dtype=D, generator=g)
    y = torch.randn(O.nspec_so3(nl), Fi, Fo, 2, dtype=D, generator=g)
    assert np.abs(c2np(O.so3_mm(x, y)) - brute.so3_mm(c2np(x), c2np(y), nl)).max() < 1e-12
    x = torch.randn(nl * nl, B, Fi, 2, dtype=D, generator=g)
    y = torch.randn(nl * nl, Fi, Fo, 2, dtype=D, generator=g)
    assert np.abs(c2np(O.s2_mm(x, y)) - brute.s2_mm(c2np(x), c2np(y), nl)).max() < 1e-12


def test_complex_mm_flags():
    g = torch.Generator().manual_seed(6)
    x = torch.randn(4, 3, 2, dtype=D, generator=g)
    y = torch.randn(3, 5, 2, dtype=D, generator=g)
    for cx in (False, True):
        for cy in (False, True):
            X = c2np(x).conj() if cx else c2np(x)
            Y = c2np(y).conj() if cy else c2np(y)
            assert np.abs(c2np(O.complex_mm(x, y, cx, cy)) - X @ Y).max() < 1e-13


# ---------------- identities asserted by the reference's test script ----------------

def test_rfft_equals_rft_on_soft_grid():
    """tests/so3_fft.py:8-24 of the reference at (b_in, b_out) = (7, 5), and
    examples/fast_ft/main.py:9-32 at b = 6."""
    for b_in, b_out in ((7, 5), (6, 6)):
        x = torch.randn(2 * b_in, 2 * b_in, 2 * b_in, dtype=D)
        y1 = O.so3_rfft(x, b_out=b_out)
        x2 = torch.einsum("bac,b->bac", x, O.quadrature_weights(b_in, D))
        y2 = O.so3_rft(x2.reshape(-1), b_out, O.so3_soft_grid(b_in))
        assert (y1 - y2).abs().max().item() < 1e-10 * y1.abs().mean().item()


@pytest.mark.parametrize("b_in,b_out", [(7, 5), (6, 6), (9, 2)])
def test_s2_fft_equals_s2_rft_on_soft_grid(b_in, b_out):
    """The S^2 twin of tests/so3_fft.py:8-24 of the reference: s2_fft's table carries 2 b_in w_beta
    (s2cnn/soft/s2_fft.py:124) and s2_rft's matrix 2 b_out (s2cnn/s2_ft.py:38-45), hence
    s2_fft(x, b_out) = (b_in / b_out) s2_rft(w * x, b_out, s2_soft_grid(b_in)).  s2_fft is pinned by brute force above,
    so a dropped factor, a wrong column of D or a swapped (beta, alpha) in s2_rft fails here."""
    x = torch.randn(2, 2 * b_in, 2 * b_in, dtype=D)
    y1 = O.s2_fft(O.as_complex(x), b_out=b_out)
    xw = torch.einsum("zba,b->zba", x, O.quadrature_weights(b_in, D))
    y2 = O.s2_rft(xw.reshape(2, -1), b_out, O.s2_soft_grid(b_in)) * (b_in / b_out)
    assert (y1 - y2).abs().max().item() < 1e-12 * y1.abs().mean().item()


def _idem(f, g, x, b_in, b_out):
    x = g(f(x, b_out=b_out), b_out=b_in)
    y = g(f(x, b_out=b_out), b_out=b_in)
    assert (x - y).abs().max().item() < 1e-10 * y.abs().mean().item()
    return x


@pytest.mark.parametrize("b_in,b_out", [(7, 7), (5, 4), (7, 4), (4, 6)])
def test_projector_idempotent_grid(b_in, b_out):
    """tests/so3_fft.py:34-44,57-91 of the reference."""
    _idem(O.so3_fft, O.so3_ifft, torch.randn(2 * b_in, 2 * b_in, 2 * b_in, 2, dtype=D), b_in, b_out)
    _idem(O.so3_rfft, O.so3_rifft, torch.randn(2 * b_in, 2 * b_in, 2 * b_in, dtype=D), b_in, b_out)


@pytest.mark.parametrize("b_in,b_out", [(7, 7), (5, 4), (4, 7)])
def test_projector_idempotent_spectrum(b_in, b_out):
    """tests/so3_fft.py:47-54,62-64,88-91 of the reference."""
    _idem(O.so3_ifft, O.so3_fft, torch.randn(O.nspec_so3(b_in), 2, dtype=D), b_in, b_out)
    _idem(O.so3_rifft, O.so3_rfft, torch.randn(O.nspec_so3(b_in), 2, dtype=D), b_in, b_out)


def test_fft_ifft_is_identity_on_bandlimited():
    b = 5
    xh = torch.randn(O.nspec_so3(b), 3, 2, dtype=D)
    back = O.so3_fft(O.so3_ifft(xh), b_out=b)
    assert (back - xh).abs().max().item() < 1e-11
    xh2 = torch.randn(b * b, 3, 2, dtype=D)
    back2 = O.s2_fft(O.s2_ifft(xh2), b_out=b)
    assert (back2 - xh2).abs().max().item() < 1e-11


# ---------------- adjoints (the autograd Functions' backward rules) ----------------

@pytest.mark.parametrize("b_in,b_out", [(4, 4), (5, 3)])
def test_so3_fft_real_backward_is_adjoint(b_in, b_out):
    """so3_fft.py:453-456.  Exact adjoint when b_out <= b_in (the layers' case); for
    b_out > b_in the reference's rule drops degrees l >= b_in that its forward fills,
    and the restatement keeps that rule as it is."""
    x = torch.randn(2, 2 * b_in, 2 * b_in, 2 * b_in, dtype=D, requires_grad=True)
    gy = torch.randn(O.nspec_so3(b_out), 2, 2, dtype=D)
    y = O.SO3_fft_real.apply(x, b_out)
    (gx,) = torch.autograd.grad(y, x, gy)
    x0 = torch.randn_like(x)
    lhs = (O.so3_rfft(x0, b_out=b_out) * gy).sum()
    assert abs(lhs - (x0 * gx).sum()).item() < 1e-10 * abs(lhs.item()) + 1e-12


@pytest.mark.parametrize("b_in,b_out", [(4, 4), (3, 5)])
def test_so3_ifft_real_backward_is_adjoint(b_in, b_out):
    """so3_fft.py:467-469.  Exact adjoint when b_out >= b_in (the layers call it with
    b_out = b_in)."""
    s = torch.randn(O.nspec_so3(b_in), 2, 2, dtype=D, requires_grad=True)
    gz = torch.randn(2, 2 * b_out, 2 * b_out, 2 * b_out, dtype=D)
    z = O.SO3_ifft_real.apply(s, b_out)
    (gs,) = torch.autograd.grad(z, s, gz)
    s0 = torch.randn_like(s)
    lhs = (O.so3_rifft(s0, b_out=b_out) * gz).sum()
    assert abs(lhs - (s0 * gs).sum()).item() < 1e-10 * abs(lhs.item()) + 1e-12


@pytest.mark.parametrize("b_in,b_out", [(4, 4), (5, 3)])
def test_s2_backward_rules_are_adjoints(b_in, b_out):
    x = torch.randn(2, 2 * b_in, 2 * b_in, dtype=D, requires_grad=True)
    gy = torch.randn(b_out ** 2, 2, 2, dtype=D)
    (gx,) = torch.autograd.grad(O.S2_fft_real.apply(x, b_out), x, gy)
    x0 = torch.randn_like(x)
    lhs = (O.S2_fft_real.apply(x0, b_out) * gy).sum()
    assert abs(lhs - (x0 * gx).sum()).item() < 1e-10 * abs(lhs.item())


def test_mm_gradients_match_closed_form():
    """gx = gz . y, gy = conj(gz) . x, the contractions of s2cnn/so3_mm.py:96-122
    and s2cnn/s2_mm.py:231-241,288-298, against autograd through the CPU loop."""
    nl, B, Fi, Fo = 3, 2, 3, 4
    g = torch.Generator().manual_seed(11)
    x = torch.randn(O.nspec_so3(nl), B, Fi, 2, dtype=D, generator=g, requires_grad=True)
    y = torch.randn(O.nspec_so3(nl), Fi, Fo, 2, dtype=D, generator=g, requires_grad=True)
    gz = torch.randn(O.nspec_so3(nl), B, Fo, 2, dtype=D, generator=g)
    gx, gy = torch.autograd.grad(O.so3_mm(x, y), (x, y), gz)
    X, Y, GZ = c2np(x.detach()), c2np(y.detach()), c2np(gz)
    pos = 0
    for l in range(nl):
        L = 2 * l + 1
        s = slice(pos, pos + L * L)
        Xl, Yl, Gl = (a[s].reshape(L, L, *a.shape[1:]) for a in (X, Y, GZ))
        wx = np.einsum("mnij,npkj->mpik", Gl, Yl).reshape(L * L, B, Fi)
        wy = np.einsum("mnij,mpik->npkj", Gl.conj(), Xl).reshape(L * L, Fi, Fo)
        assert np.abs(c2np(gx)[s] - wx).max() < 1e-12
        assert np.abs(c2np(gy)[s] - wy).max() < 1e-12
        pos += L * L

    x = torch.randn(nl * nl, B, Fi, 2, dtype=D, generator=g, requires_grad=True)
    y = torch.randn(nl * nl, Fi, Fo, 2, dtype=D, generator=g, requires_grad=True)
    gx, gy = torch.autograd.grad(O.s2_mm(x, y), (x, y), gz)
    X, Y = c2np(x.detach()), c2np(y.detach())
    pos = 0
    for l in range(nl):
        L = 2 * l + 1
        Gl = GZ[pos:pos + L * L].reshape(L, L, B, Fo)
        s = slice(l * l, l * l + L)
        assert np.abs(c2np(gx)[s] - np.einsum("mnij,nkj->mik", Gl, Y[s])).max() < 1e-12
        assert np.abs(c2np(gy)[s] - np.einsum("mnij,mik->nkj", Gl.conj(), X[s])).max() < 1e-12
        pos += L * L


def test_gradcheck_small_conv():
    grid = O.so3_near_identity_grid(n_alpha=3, n_beta=1, n_gamma=2)
    x = torch.randn(1, 2, 4, 4, 4, dtype=D, requires_grad=True)
    k = torch.randn(2, 2, len(grid), dtype=D, requires_grad=True)
    bias = torch.zeros(1, 2, 1, 1, 1, dtype=D, requires_grad=True)
    assert torch.autograd.gradcheck(lambda a, c, d: O.so3_conv(a, c, d, 2, 2, grid), (x, k, bias), atol=1e-6)
    grid2 = O.s2_near_identity_grid(n_alpha=3, n_beta=1)
    x2 = torch.randn(1, 2, 6, 6, dtype=D, requires_grad=True)
    k2 = torch.randn(2, 2, len(grid2), dtype=D, requires_grad=True)
    assert torch.autograd.gradcheck(lambda a, c, d: O.s2_conv(a, c, d, 3, 2, grid2), (x2, k2, bias), atol=1e-6)


# ---------------- layer-level invariants ----------------

def test_integrate_and_grids():
    assert abs(O.so3_integrate(torch.ones(3, 8, 8, 8, dtype=D)) - 1).abs().max().item() < 1e-13
    g = O.so3_near_identity_grid()
    assert len(g) == 192 and len(g[0]) == 3
    beta = sorted({p[0] for p in g})
    assert np.allclose(beta, np.arange(1, 4) * (np.pi / 8) / 3)
    # gamma = pre_gamma - alpha (s2cnn/so3_grid.py:14-18)
    assert abs(g[0][2] - (-2 * np.pi)) < 1e-15 and abs(g[8][1] - np.pi / 4) < 1e-15 and abs(g[8][2] - (-2 * np.pi - np.pi / 4)) < 1e-15
    assert len(O.s2_near_identity_grid()) == 24 and len(O.s2_equatorial_grid()) == 32
    assert len(O.so3_equatorial_grid()) == 64 and len(O.so3_soft_grid(3)) == 216 and len(O.s2_soft_grid(3)) == 36
    assert O.so3_soft_grid(2)[5] == (np.pi / 8, np.pi / 2, np.pi / 2)


def test_z_rotation_equivariance():
    """examples/equivariance_error/main.py:18-46 of the reference, reduced sizes."""
    g = torch.Generator().manual_seed(3)
    s2g = O.s2_equatorial_grid(max_beta=0, n_alpha=16, n_beta=1)
    so3g = O.so3_equatorial_grid(max_beta=0, max_gamma=0, n_alpha=16, n_beta=1, n_gamma=1)
    k1 = torch.rand(2, 3, len(s2g), dtype=D, generator=g) * 2 - 1
    k2 = torch.rand(3, 2, len(so3g), dtype=D, generator=g) * 2 - 1
    z3 = torch.zeros(1, 3, 1, 1, 1, dtype=D)
    z2 = torch.zeros(1, 2, 1, 1, 1, dtype=D)

    def phi(x):
        return O.so3_conv(torch.relu(O.s2_conv(x, k1, z3, 8, 4, s2g)), k2, z2, 4, 3, so3g)

    def rot(x, n):
        return torch.cat([x[:, :, :, n:], x[:, :, :, :n]], dim=3)

    x = torch.randn(1, 2, 16, 16, dtype=D, generator=g)
    y = phi(x)
    y1 = rot(phi(x), y.size(3) // 8 * 1 * 0 + 0)  # identity sanity
    assert torch.equal(y1, y)
    # an alpha-roll of the input by 2 of 16 samples = roll of the output alpha axis by 2*(6/16)?  only
    # commensurate shifts map grid to grid: 16 -> 6 samples needs a shift of 8 (half turn) <-> 3
    ya = rot(phi(x), 3)
    yb = phi(rot(x, 8))
    assert (ya - yb).std().item() / y.std().item() < 1e-10


def test_transpose_convention_invariance():
    """Replacing d by its transpose (d^T = S d S, S = diag((-1)^m)) - the one bit
    lie_learn's absence leaves unpinned - changes standalone spectra by the sign
    (-1)^(m-n) but leaves fft->mm->ifft (the conv layers) unchanged."""
    b = 3
    g = torch.Generator().manual_seed(4)
    x = torch.randn(2, 2, 2 * b, 2 * b, 2 * b, dtype=D, generator=g)
    grid = O.so3_near_identity_grid(n_alpha=4, n_beta=2, n_gamma=3)
    k = torch.randn(2, 3, len(grid), dtype=D, generator=g)
    xs = O.so3_rfft(x, b_out=b)
    ys = O.so3_rft(k, b, grid)
    sign = torch.cat([torch.tensor([[(-1.0) ** (m - n) for n in range(-l, l + 1)] for m in range(-l, l + 1)],
                                   dtype=D).reshape(-1) for l in range(b)])
    s4 = sign.view(-1, 1, 1, 1)
    zs = O.so3_mm(xs, ys)
    zs_t = O.so3_mm(xs * s4, ys * s4)          # what the transposed tables would have produced
    assert (zs_t - zs * s4).abs().max().item() < 1e-12
    out = O.so3_rifft(zs)
    out_t = O.so3_rifft(zs_t * s4)              # synthesis with transposed table = sign then same table
    assert (out - out_t).abs().max().item() < 1e-12
