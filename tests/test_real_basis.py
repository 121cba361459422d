"""The real basis of SO(3) spectra of real signals (no counterpart in the reference, so pinned by
mathematics and by the oracle's complex path): unitarity, reality of transformed spectra that the
oracle computes from real signals, the product identity U (X Y^H) U^H = X_r Y_r^T against the oracle's
complex so3_mm, and the real-basis kernel matrix against the complex one."""
import numpy as np
import pytest
import torch

from oracle import cpu_path as O
from s2cnn_amd import wigner


def dense_to_real(x):
    """x [nspec, ...] complex128 ndarray -> U x U^H per degree (complex; caller checks / takes the real part)."""
    out = np.empty_like(x)
    pos, l = 0, 0
    while pos < x.shape[0]:
        L = 2 * l + 1
        U = wigner.real_basis_matrix(l)
        blk = x[pos:pos + L * L].reshape(L, L, -1)
        out[pos:pos + L * L] = np.einsum("rm,mnc,sn->rsc", U, blk, U.conj()).reshape(L * L, *x.shape[1:])
        pos += L * L
        l += 1
    return out


def dense_to_complex(r):
    out = np.empty(r.shape, dtype=np.complex128)
    pos, l = 0, 0
    while pos < r.shape[0]:
        L = 2 * l + 1
        U = wigner.real_basis_matrix(l)
        blk = r[pos:pos + L * L].reshape(L, L, -1)
        out[pos:pos + L * L] = np.einsum("rm,rsc,sn->mnc", U.conj(), blk, U).reshape(L * L, *r.shape[1:])
        pos += L * L
        l += 1
    return out


def as_np(t):
    t = t.detach().double().numpy()
    return t[..., 0] + 1j * t[..., 1]


@pytest.mark.parametrize("l", [0, 1, 2, 5, 8])
def test_unitary(l):
    U = wigner.real_basis_matrix(l)
    assert np.allclose(U @ U.conj().T, np.eye(2 * l + 1), atol=1e-14)


@pytest.mark.parametrize("b", [3, 6])
def test_spectrum_of_real_signal_becomes_real(b):
    x = torch.randn(2, 2 * b, 2 * b, 2 * b, dtype=torch.float64, generator=torch.Generator().manual_seed(b))
    X = as_np(O.so3_rfft(x))
    R = dense_to_real(X)
    assert np.abs(R.imag).max() < 1e-12 * np.abs(R).max()
    assert np.allclose(dense_to_complex(R.real), X, atol=1e-12)
    # an asymmetric spectrum does NOT become real: the test above is not vacuous
    Y = X.copy()
    Y[4] += 1.0          # (l, m, n) = (1, 0, -1) alone
    assert np.abs(dense_to_real(Y).imag).max() > 0.1


def test_product_identity_against_oracle_so3_mm():
    b, B, Fi, Fo = 4, 2, 3, 2
    g = torch.Generator().manual_seed(1)
    x = O.so3_rfft(torch.randn(B * Fi, 2 * b, 2 * b, 2 * b, dtype=torch.float64, generator=g))
    y = O.so3_rfft(torch.randn(Fi * Fo, 2 * b, 2 * b, 2 * b, dtype=torch.float64, generator=g))
    ns = x.shape[0]
    x = x.reshape(ns, B, Fi, 2)
    y = y.reshape(ns, Fi, Fo, 2)
    z = as_np(O.so3_mm(x, y))
    xr, yr = dense_to_real(as_np(x)).real, dense_to_real(as_np(y)).real
    zr = np.empty((ns, B, Fo))
    pos = 0
    for l in range(b):
        L = 2 * l + 1
        xa = xr[pos:pos + L * L].reshape(L, L, B, Fi)
        ya = yr[pos:pos + L * L].reshape(L, L, Fi, Fo)
        zr[pos:pos + L * L] = np.einsum("mpik,npkj->mnij", xa, ya).reshape(L * L, B, Fo)
        pos += L * L
    assert np.allclose(dense_to_complex(zr), z, atol=1e-10 * np.abs(z).max())


def test_real_kernel_matrix_matches_complex_one():
    b = 5
    grid = tuple((0.1 * i + 0.05, 0.3 * i, -0.2 * i + 1.0) for i in range(7))
    F = wigner.so3_ft_matrix(b, grid)
    Fr = wigner.so3_ft_matrix_real(b, grid)
    assert np.allclose(dense_to_complex(Fr.T.copy()).T, F, atol=1e-12)
    # and against the oracle's so3_rft of a real kernel
    k = torch.randn(3, len(grid), dtype=torch.float64, generator=torch.Generator().manual_seed(2))
    Y = as_np(O.so3_rft(k, b, grid))                       # [nspec, 3]
    Yr = (k.numpy() @ Fr).T
    assert np.allclose(dense_to_real(Y).real, Yr, atol=1e-12)
    assert np.abs(dense_to_real(Y).imag).max() < 1e-12


# ------------------------------------------------------------------ GPU kernels
def _close(got, want, tol=1e-4):
    got = got.detach().double().cpu().numpy()
    scale = max(want.std(), 1e-30)
    q = np.abs(got - want).max() / scale
    print(f"max|d|/std={q:.2e}", flush=True)
    assert got.shape == want.shape and q < tol, q


@pytest.mark.gpu
@pytest.mark.parametrize("nl,cols", [(1, (3,)), (4, (2, 3)), (7, (5, 1)), (12, (16, 20))])
def test_basis_kernels_against_dense(hip, nl, cols):
    import s2cnn_amd
    print(f"real basis kernels nl={nl} cols={cols}", flush=True)
    ns = O.nspec_so3(nl)
    g = torch.Generator().manual_seed(nl)
    x = torch.randn(ns, *cols, 2, generator=g)          # arbitrary, not symmetric: to_real is Re(U x U^H)
    r = torch.randn(ns, *cols, generator=g)
    xr = s2cnn_amd.so3_spectrum_to_real(x.cuda())
    _close(xr, dense_to_real(as_np(x).reshape(ns, -1)).real.reshape(ns, *cols))
    xc = s2cnn_amd.so3_spectrum_to_complex(r.cuda())
    want = dense_to_complex(r.double().numpy().reshape(ns, -1)).reshape(ns, *cols)
    _close(xc, np.stack((want.real, want.imag), -1))
    # adjoint pair: <to_real x, r> = <x, to_complex r>
    lhs = (xr.double().cpu() * r.double()).sum().item()
    rhs = (x.double() * xc.double().cpu()).sum().item()
    assert abs(lhs - rhs) < 1e-4 * max(abs(lhs), 1.0)
    # autograd wiring
    xg = x.cuda().requires_grad_()
    (s2cnn_amd.so3_spectrum_to_real(xg) * r.cuda()).sum().backward()
    _close(xg.grad, np.stack((want.real, want.imag), -1))


@pytest.mark.gpu
@pytest.mark.parametrize("nl,B,Fi,Fo", [(4, 2, 3, 5), (3, 32, 20, 40), (6, 3, 7, 55), (8, 16, 64, 64), (5, 1, 1, 1),
                                        (12, 16, 32, 48), (9, 4, 100, 36),
                                        # block sizes that divide / are multiples of the K stage (32): scalar-stepped loaders,
                                        # several blocks per stage (8, 16), several stages per block (96, 128), ragged last stage
                                        (5, 8, 64, 32), (4, 4, 128, 64), (7, 32, 96, 32), (6, 16, 16, 8),
                                        # one operand with 16-byte accesses, the other with 4-byte ones
                                        (5, 6, 20, 7), (4, 3, 7, 8), (7, 32, 100, 55),
                                        # even sizes that are no multiples of four: 8-byte accesses, alone and beside 16-byte ones
                                        (6, 2, 50, 70), (5, 6, 10, 14), (4, 16, 70, 350), (5, 4, 6, 20), (5, 2, 20, 6), (3, 6, 2, 2),
                                        # ... through the scalar-stepped loaders: blocks that divide the stage (16, 2) and blocks
                                        # that stages run across (34, 50, 66, 70), ragged last stages
                                        (7, 16, 50, 70), (5, 6, 34, 66), (6, 6, 16, 18), (4, 10, 66, 34), (9, 2, 38, 2)])
def test_so3_mm_real_forward_backward(hip, nl, B, Fi, Fo):
    import s2cnn_amd
    print(f"so3_mm_real nl={nl} B={B} Fi={Fi} Fo={Fo}", flush=True)
    ns = O.nspec_so3(nl)
    g = torch.Generator().manual_seed(7)
    x = torch.randn(ns, B, Fi, generator=g)
    y = torch.randn(ns, Fi, Fo, generator=g) * Fi ** -0.5
    gz = torch.randn(ns, B, Fo, generator=g)
    xd, yd, gd = x.double().numpy(), y.double().numpy(), gz.double().numpy()
    z = np.empty((ns, B, Fo)); gx = np.empty((ns, B, Fi)); gy = np.empty((ns, Fi, Fo))
    pos = 0
    for l in range(nl):
        L = 2 * l + 1
        sl = slice(pos, pos + L * L)
        xa, ya, ga = xd[sl].reshape(L, L, B, Fi), yd[sl].reshape(L, L, Fi, Fo), gd[sl].reshape(L, L, B, Fo)
        z[sl] = np.einsum("mpik,npkj->mnij", xa, ya).reshape(L * L, B, Fo)
        gx[sl] = np.einsum("mnij,npkj->mpik", ga, ya).reshape(L * L, B, Fi)
        gy[sl] = np.einsum("mnij,mpik->npkj", ga, xa).reshape(L * L, Fi, Fo)
        pos += L * L
    xg, yg = x.cuda().requires_grad_(), y.cuda().requires_grad_()
    zg = s2cnn_amd.so3_mm_real(xg, yg)
    gxg, gyg = torch.autograd.grad(zg, (xg, yg), gz.cuda())
    _close(zg, z)
    _close(gxg, gx)
    _close(gyg, gy)


@pytest.mark.gpu
def test_real_product_equals_oracle_complex_product(hip):
    """to_complex(mm_real(to_real x, to_real y)) against the oracle's so3_mm on spectra of real signals."""
    import s2cnn_amd
    b, B, Fi, Fo = 6, 3, 4, 5
    g = torch.Generator().manual_seed(3)
    x = O.so3_rfft(torch.randn(B * Fi, 2 * b, 2 * b, 2 * b, generator=g))
    y = O.so3_rfft(torch.randn(Fi * Fo, 2 * b, 2 * b, 2 * b, generator=g))
    ns = x.shape[0]
    x, y = x.reshape(ns, B, Fi, 2), y.reshape(ns, Fi, Fo, 2)
    want = O.so3_mm(x.double(), y.double()).numpy()
    got = s2cnn_amd.so3_spectrum_to_complex(
        s2cnn_amd.so3_mm_real(s2cnn_amd.so3_spectrum_to_real(x.cuda()), s2cnn_amd.so3_spectrum_to_real(y.cuda())))
    _close(got, want)


@pytest.mark.gpu
def test_so3_rft_real_matches_complex(hip):
    import s2cnn_amd
    b = 6
    grid = s2cnn_amd.so3_near_identity_grid()
    k = torch.randn(3, 4, len(grid), generator=torch.Generator().manual_seed(5))
    want = O.so3_rft(k.double(), b, grid).numpy()
    got = s2cnn_amd.so3_spectrum_to_complex(s2cnn_amd.so3_rft_real(k.cuda(), b, grid))
    _close(got, want)


@pytest.mark.gpu
def test_convolution_real_and_complex_paths_agree(hip):
    import s2cnn_amd
    from s2cnn_amd.soft.so3_conv import SO3Convolution
    torch.manual_seed(0)
    conv = SO3Convolution(3, 4, 6, 4, s2cnn_amd.so3_near_identity_grid()).cuda()
    x = torch.randn(2, 3, 12, 12, 12, device="cuda", requires_grad=True)
    out = {}
    for flag in (True, False):
        conv.real_basis = flag
        conv.zero_grad()
        x.grad = None
        z = conv(x)
        z.pow(2).sum().backward()
        out[flag] = (z.detach(), x.grad.clone(), conv.kernel.grad.clone())
    for a, c in zip(out[True], out[False]):
        _close(a, c.double().cpu().numpy())


@pytest.mark.gpu
@pytest.mark.parametrize("b_in,b_out,nz", [(32, 32, 3), (32, 20, 33), (20, 32, 5), (6, 4, 2), (4, 6, 3), (22, 22, 17), (16, 16, 5),
                                           (7, 22, 4), (22, 7, 9), (36, 40, 2), (40, 36, 2), (40, 20, 2), (12, 30, 3), (10, 6, 24),
                                           (1, 1, 3), (17, 17, 9), (25, 16, 13), (16, 25, 3), (33, 20, 2), (20, 33, 1)])
def test_transforms_in_the_real_basis(hip, b_in, b_out, nz):
    """so3_rfft_real_basis / so3_rifft_real_basis against the two-step compositions they replace (per-volume
    kernels on the 64^3 grid, elsewhere the tiled Wigner stage reads or writes the real basis; composed where that stage
    does not apply: an analysis onto more than 32 degrees), for both tables, and the autograd pair by a dot-product test."""
    from s2cnn_amd.soft import so3_fft as P
    from s2cnn_amd.so3_real import so3_spectrum_to_complex, so3_spectrum_to_real
    g = torch.Generator().manual_seed(b_in * 100 + b_out)
    x = torch.randn(nz, 2 * b_in, 2 * b_in, 2 * b_in, generator=g).cuda()
    ns = b_in * (4 * b_in ** 2 - 1) // 3
    r = torch.randn(ns, nz, generator=g).cuda()
    for for_grad in (False, True):
        got = P.so3_rfft_real_basis(x, for_grad, b_out)
        want = so3_spectrum_to_real(P.so3_rfft(x, for_grad, b_out))
        assert got.shape == want.shape
        assert (got - want).abs().max().item() < 1e-5 * want.abs().max().item(), (b_in, b_out, for_grad)
        got = P.so3_rifft_real_basis(r, for_grad, b_out)
        want = P.so3_rifft(so3_spectrum_to_complex(r), for_grad, b_out)
        assert got.shape == want.shape
        assert (got - want).abs().max().item() < 1e-5 * want.abs().max().item(), (b_in, b_out, for_grad)
    # <fft(x), r'> = <x, fft.backward(r')> and the same for ifft
    xg = x.clone().requires_grad_()
    y = P.SO3_fft_real_basis.apply(xg, b_out)
    w = torch.randn(y.shape, generator=g).cuda()
    (gx,) = torch.autograd.grad(y, xg, w)
    lhs, rhs = (y.double() * w.double()).sum().item(), (x.double() * gx.double()).sum().item()
    if b_out <= b_in:   # the reference's backward is the exact adjoint only when no frequencies are cut off
        assert abs(lhs - rhs) < 1e-4 * abs(lhs), (lhs, rhs)
    rg = r.clone().requires_grad_()
    y = P.SO3_ifft_real_basis.apply(rg, b_out)
    w = torch.randn(y.shape, generator=g).cuda()
    (gr,) = torch.autograd.grad(y, rg, w)
    lhs, rhs = (y.double() * w.double()).sum().item(), (r.double() * gr.double()).sum().item()
    if b_out >= b_in:
        assert abs(lhs - rhs) < 1e-4 * abs(lhs), (lhs, rhs)


@pytest.mark.gpu
def test_convolution_on_the_64_grid_matches_oracle(hip):
    """SO3Convolution with b_in = b_out = 32 (direct real-basis transforms on both sides) against the oracle,
    forward and all gradients, at a small batch and few features."""
    import s2cnn_amd
    from oracle import cpu_path as O
    B, Fi, Fo, b = 2, 2, 3, 32
    grid = s2cnn_amd.so3_near_identity_grid()
    g = torch.Generator().manual_seed(5)
    x = torch.randn(B, Fi, 64, 64, 64, generator=g)
    layer = s2cnn_amd.SO3Convolution(Fi, Fo, b, b, grid)
    k = torch.rand(Fi, Fo, len(grid), generator=g) * 2 - 1
    bias = torch.randn(1, Fo, 1, 1, 1, generator=g) * 0.1
    with torch.no_grad():
        layer.kernel.copy_(k)
        layer.bias.copy_(bias)
    layer = layer.cuda()
    xg = x.cuda().requires_grad_()
    out = layer(xg)
    (out * out).sum().backward()
    xo, ko, bo = x.requires_grad_(), k.requires_grad_(), bias.requires_grad_()   # float32 oracle: b = 32 in float64 takes minutes
    outo = O.so3_conv(xo, ko, bo, b, b, grid)
    (outo * outo).sum().backward()
    for name, a, c in (("out", out, outo), ("grad_x", xg.grad, xo.grad), ("grad_kernel", layer.kernel.grad, ko.grad), ("grad_bias", layer.bias.grad, bo.grad)):
        q = (a.detach().cpu().double() - c.detach().double()).abs().max().item() / c.detach().double().std().item()
        print(name, q, flush=True)
        assert q < 1e-4, (name, q)


def test_factorised_kernel_transform_plan():
    """wigner.so3_rft_plan: plane coefficients per beta group, expanded with the real-basis formulas of
    csrc/so3_rft.hip in numpy, reproduce the dense real-basis matrix (itself pinned against the oracle above)."""
    import s2cnn_amd
    from s2cnn_amd import wigner
    b = 5
    for grid in (s2cnn_amd.so3_near_identity_grid(n_alpha=4, n_beta=3, n_gamma=5), s2cnn_amd.so3_equatorial_grid(n_alpha=6, n_gamma=3), ((0, 0, 0),)):
        idx, E, dtab = wigner.so3_rft_plan(b, grid)
        rng = np.random.default_rng(1)
        x = rng.standard_normal((3, len(grid)))
        want = wigner.so3_ft_matrix_real(b, grid).T @ x.T
        xg = np.where((idx >= 0)[..., None], x.T[np.maximum(idx, 0)], 0.0)
        G = np.einsum("ipr,ipc->irc", E, xg)

        def lmn(l, m, n):
            return l * (4 * l * l - 1) // 3 + (l + m) * (2 * l + 1) + (l + n)

        def row(i, m, n):
            r = ((m + b - 1) * b + n) * 2
            return G[i, r] + 1j * G[i, r + 1]
        got = np.zeros_like(want)
        for a in range(b):
            for n in range(b):
                s = -1.0 if a & 1 else 1.0
                for l in range(max(a, n), b):
                    A = sum(dtab[i, lmn(l, a, n)] * row(i, a, n) for i in range(len(idx)))
                    C = sum(dtab[i, lmn(l, -a, n)] * row(i, -a, n) for i in range(len(idx)))
                    if a > 0 and n > 0:
                        got[lmn(l, a, n)], got[lmn(l, a, -n)] = A.real + s * C.real, -A.imag - s * C.imag
                        got[lmn(l, -a, n)], got[lmn(l, -a, -n)] = A.imag - s * C.imag, A.real - s * C.real
                    elif a > 0:
                        got[lmn(l, a, 0)], got[lmn(l, -a, 0)] = (A.real + s * C.real) / np.sqrt(2), (A.imag - s * C.imag) / np.sqrt(2)
                    elif n > 0:
                        got[lmn(l, 0, n)], got[lmn(l, 0, -n)] = np.sqrt(2) * A.real, -np.sqrt(2) * A.imag
                    else:
                        got[lmn(l, 0, 0)] = A.real
        assert np.abs(got - want).max() < 1e-12 * max(1.0, np.abs(want).max())
    assert wigner.so3_rft_plan(3, s2cnn_amd.so3_soft_grid(3)) is None        # 6 distinct betas: dense product


@pytest.mark.gpu
def test_factorised_kernel_transform_matches_dense(hip):
    """so3_rft_real through the factorised path against the dense product, forward and gradient."""
    import s2cnn_amd
    from s2cnn_amd.so3_real import so3_rft_real
    for b, grid, shape in ((32, s2cnn_amd.so3_near_identity_grid(), (8, 12)), (7, s2cnn_amd.so3_equatorial_grid(n_alpha=8), (4, 5)),
                           (6, ((0, 0, 0),), (2, 2))):
        g = torch.Generator().manual_seed(b)
        x = torch.randn(*shape, len(grid), generator=g).cuda().requires_grad_()
        w = None
        res = {}
        for flag in (True, False):
            so3_rft_real.factorised = flag
            y = so3_rft_real(x, b, grid)
            if w is None:
                w = torch.randn(y.shape, generator=g).cuda()
            (gx,) = torch.autograd.grad(y, x, w)
            res[flag] = (y.detach(), gx)
        so3_rft_real.factorised = True
        for got, want in zip(res[True], res[False]):
            assert got.shape == want.shape
            assert (got - want).abs().max().item() < 2e-5 * want.abs().max().item(), (b, (got - want).abs().max().item(), want.abs().max().item())


@pytest.mark.gpu
@pytest.mark.parametrize("nl,B,Fi,Fo", [(4, 2, 3, 5), (10, 32, 1, 20), (7, 5, 6, 9), (6, 16, 12, 16), (5, 3, 6, 100), (3, 1, 1, 1),
                                        (4, 7, 20, 8), (2, 2, 3, 1028), (6, 16, 6, 50), (5, 3, 9, 2), (3, 4, 2, 70)])
def test_s2_mm_real_forward_backward(hip, nl, B, Fi, Fo):
    """The real outer product against numpy: odd sizes (4-byte accesses), even ones (8-byte), multiples of four (16-byte accesses), more
    input features than one register pass, an odd batch, rows longer than a workgroup."""
    import s2cnn_amd
    print(f"s2_mm_real nl={nl} B={B} Fi={Fi} Fo={Fo}", flush=True)
    g = torch.Generator().manual_seed(11)
    x = torch.randn(nl * nl, B, Fi, generator=g)
    y = torch.randn(nl * nl, Fi, Fo, generator=g) * Fi ** -0.5
    ns = O.nspec_so3(nl)
    gz = torch.randn(ns, B, Fo, generator=g)
    xd, yd, gd = x.double().numpy(), y.double().numpy(), gz.double().numpy()
    z = np.empty((ns, B, Fo)); gx = np.empty((nl * nl, B, Fi)); gy = np.empty((nl * nl, Fi, Fo))
    pos = 0
    for l in range(nl):
        L = 2 * l + 1
        xa, ya = xd[l * l:l * l + L], yd[l * l:l * l + L]
        ga = gd[pos:pos + L * L].reshape(L, L, B, Fo)
        z[pos:pos + L * L] = np.einsum("rik,skj->rsij", xa, ya).reshape(L * L, B, Fo)
        gx[l * l:l * l + L] = np.einsum("rsij,skj->rik", ga, ya)
        gy[l * l:l * l + L] = np.einsum("rsij,rik->skj", ga, xa)
        pos += L * L
    xg, yg = x.cuda().requires_grad_(), y.cuda().requires_grad_()
    zg = s2cnn_amd.s2_mm_real(xg, yg)
    gxg, gyg = torch.autograd.grad(zg, (xg, yg), gz.cuda())
    _close(zg, z)
    _close(gxg, gx)
    _close(gyg, gy)


@pytest.mark.gpu
def test_s2_real_product_equals_oracle_complex_product(hip):
    """to_complex(s2_mm_real(to_real x, to_real y)) against the oracle's s2_mm on spectra of real signals, and the
    real-basis kernel spectrum against the complex one."""
    import s2cnn_amd
    b, B, Fi, Fo = 6, 3, 4, 5
    g = torch.Generator().manual_seed(5)
    sig = torch.randn(B * Fi, 2 * b, 2 * b, generator=g).double()
    x = O.s2_fft(torch.stack((sig, torch.zeros_like(sig)), -1))
    grid = s2cnn_amd.s2_near_identity_grid()
    k = torch.randn(Fi, Fo, len(grid), generator=g)
    y = O.s2_rft(k.double(), b, grid)
    x = x.reshape(b * b, B, Fi, 2)
    want = O.s2_mm(x, y).numpy()
    xr = s2cnn_amd.s2_spectrum_to_real(x.float().cuda())
    yr = s2cnn_amd.s2_rft_real(k.cuda(), b, grid)
    _close(yr, s2cnn_amd.s2_spectrum_to_real(y.float().cuda()).cpu().double().numpy())
    got = s2cnn_amd.so3_spectrum_to_complex(s2cnn_amd.s2_mm_real(xr, yr))
    _close(got, want)


@pytest.mark.gpu
def test_so3_mm_real_at_the_benchmark_size(hip):
    """nl = 32, batch 16, 64 -> 64 features (the loaders with scalar stage offsets, 3 048 to 11 440 tiles per launch):
    forward and both gradients against float64 einsums per degree on the same device."""
    import s2cnn_amd
    nl, B, Fi, Fo = 32, 16, 64, 64
    ns = O.nspec_so3(nl)
    g = torch.Generator(device="cuda").manual_seed(21)
    x = torch.randn(ns, B, Fi, device="cuda", generator=g).requires_grad_()
    y = (torch.randn(ns, Fi, Fo, device="cuda", generator=g) * Fi ** -0.5).requires_grad_()
    gz = torch.randn(ns, B, Fo, device="cuda", generator=g)
    z = s2cnn_amd.so3_mm_real(x, y)
    gx, gy = torch.autograd.grad(z, (x, y), gz)
    worst = 0.0
    pos = 0
    for l in range(nl):
        L = 2 * l + 1
        sl = slice(pos, pos + L * L)
        xa = x.detach()[sl].double().reshape(L, L, B, Fi)
        ya = y.detach()[sl].double().reshape(L, L, Fi, Fo)
        ga = gz[sl].double().reshape(L, L, B, Fo)
        for got, want in ((z.detach()[sl], torch.einsum("mpik,npkj->mnij", xa, ya)),
                          (gx[sl], torch.einsum("mnij,npkj->mpik", ga, ya)),
                          (gy[sl], torch.einsum("mnij,mpik->npkj", ga, xa))):
            want = want.reshape(L * L, *got.shape[1:])
            worst = max(worst, ((got.double() - want).abs().max() / want.std()).item())
        pos += L * L
    print(f"worst max|d|/std over degrees and the three products: {worst:.2e}", flush=True)
    assert worst < 1e-4


@pytest.mark.gpu
def test_convolution_paths_agree_at_the_benchmark_size(hip, monkeypatch):
    """The layer of the headline benchmark (batch 16, 64 -> 64 features, b = 32), forward and all gradients, through
    two disjoint sets of kernels: real-basis spectra (per-volume transforms writing real rows, real product, factorised
    kernel spectrum) against complex spectra (complex rows, complex product, dense kernel transform)."""
    import s2cnn_amd
    B, F, b = 16, 64, 32
    torch.manual_seed(1)
    conv = s2cnn_amd.SO3Convolution(F, F, b, b, s2cnn_amd.so3_near_identity_grid()).cuda()
    with torch.no_grad():
        conv.bias.normal_(0, 0.1)
    x = torch.randn(B, F, 64, 64, 64, device="cuda", requires_grad=True)
    res = {}
    for flag in (True, False):
        conv.real_basis = flag
        monkeypatch.setattr(s2cnn_amd.so3_rft, "factorised", flag)
        conv.zero_grad()
        x.grad = None
        z = conv(x)
        loss = z.square().sum()
        loss.backward()
        res[flag] = (z.detach()[::5, ::7].clone(), x.grad[::5, ::7].clone(), conv.kernel.grad.clone(), conv.bias.grad.clone())
        del z, loss
    for name, a, c in zip(("out", "grad_x", "grad_kernel", "grad_bias"), res[True], res[False]):
        q = ((a.double() - c.double()).abs().max() / c.double().std()).item()
        print(name, f"{q:.2e}", flush=True)
        assert q < 1e-4, (name, q)
