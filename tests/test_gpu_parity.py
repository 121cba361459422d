"""Parity of the HIP path (through the C ABI) against the CPU oracle on identical seeded
inputs.  Bar: max|d| / std(ref) < 1e-4 (the reference's own CPU-vs-GPU metric,
tests/so3_fft.py:95-100, so3_mm.py:264-271 of the reference) and relative L2 < 1e-4."""
import pytest
import torch

import s2cnn_amd
from oracle import cpu_path as O
from s2cnn_amd.soft import s2_fft as PS2
from s2cnn_amd.soft import so3_fft as PSO3

pytestmark = pytest.mark.gpu
TOL = 1e-4


def close(got, want, what=""):
    got = got.detach().double().cpu()
    want = want.detach().double()
    assert got.shape == want.shape, (what, got.shape, want.shape)
    scale = want.std().item() if want.numel() > 1 else abs(want.item())
    scale = max(scale, 1e-3 * want.abs().max().item())      # a constant signal (one degree) has no spread to measure against
    q = (got - want).abs().max().item() / max(scale, 1e-30)
    r = (got - want).norm().item() / max(want.norm().item(), 1e-30)
    print(f"{what}: max|d|/std={q:.2e} relL2={r:.2e}", flush=True)
    assert q < TOL and r < TOL, (what, q, r)


def rnd(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


# ------------------------------------------------------------------ so3_mm
MM_SHAPES = [(4, 2, 3, 5),        # the reference's in-module test (so3_mm.py:264-271): odd sizes
             (3, 32, 20, 40),     # config 1 layer 2 features
             (6, 3, 7, 55),       # odd everything
             (8, 16, 64, 64),     # config 3/4 features at a small bandwidth
             (5, 1, 1, 1),
             (12, 16, 32, 48)]


@pytest.mark.parametrize("nl,B,Fi,Fo", MM_SHAPES)
def test_so3_mm_forward_backward(hip, nl, B, Fi, Fo):
    print(f"so3_mm nl={nl} B={B} Fi={Fi} Fo={Fo}", flush=True)
    ns = O.nspec_so3(nl)
    x = rnd((ns, B, Fi, 2), 3)
    y = rnd((ns, Fi, Fo, 2), 4, Fi ** -0.5)
    gz = rnd((ns, B, Fo, 2), 5)
    xo, yo = x.double().requires_grad_(), y.double().requires_grad_()
    zo = O.so3_mm(xo, yo)
    gxo, gyo = torch.autograd.grad(zo, (xo, yo), gz.double())
    xg, yg = x.cuda().requires_grad_(), y.cuda().requires_grad_()
    zg = s2cnn_amd.so3_mm(xg, yg)
    gxg, gyg = torch.autograd.grad(zg, (xg, yg), gz.cuda())
    close(zg, zo, "z")
    close(gxg, gxo, "gx")
    close(gyg, gyo, "gy")


@pytest.mark.parametrize("nl,B,Fi,Fo", [(4, 2, 3, 5), (10, 32, 1, 20), (7, 5, 6, 9), (6, 16, 12, 15),
                                        (5, 3, 10, 6), (8, 7, 6, 100)])      # even F_out: 16-byte accesses in the gradients
def test_s2_mm_forward_backward(hip, nl, B, Fi, Fo):
    print(f"s2_mm nl={nl} B={B} Fi={Fi} Fo={Fo}", flush=True)
    x = rnd((nl * nl, B, Fi, 2), 6)
    y = rnd((nl * nl, Fi, Fo, 2), 7)
    gz = rnd((O.nspec_so3(nl), B, Fo, 2), 8)
    xo, yo = x.double().requires_grad_(), y.double().requires_grad_()
    gxo, gyo = torch.autograd.grad(O.s2_mm(xo, yo), (xo, yo), gz.double())
    xg, yg = x.cuda().requires_grad_(), y.cuda().requires_grad_()
    zg = s2cnn_amd.s2_mm(xg, yg)
    gxg, gyg = torch.autograd.grad(zg, (xg, yg), gz.cuda())
    close(zg, O.s2_mm(x.double(), y.double()), "z")
    close(gxg, gxo, "gx")
    close(gyg, gyo, "gy")


# ------------------------------------------------------------------ SO(3) transforms
SO3_PAIRS = [(2, 9), (6, 6), (9, 2), (10, 11), (11, 10), (7, 5), (4, 6), (10, 10), (10, 6), (16, 16), (16, 10), (20, 16), (22, 22), (22, 18), (32, 32), (32, 12), (12, 32)]   # first five: tests/so3_fft.py:102


@pytest.mark.parametrize("b_in,b_out", SO3_PAIRS)
@pytest.mark.parametrize("for_grad", [False, True])
def test_so3_transforms(hip, b_in, b_out, for_grad):
    print(f"so3 transforms b_in={b_in} b_out={b_out} for_grad={for_grad}", flush=True)
    nz = 3
    x = rnd((nz, 2 * b_in, 2 * b_in, 2 * b_in, 2), 10)
    close(PSO3.so3_fft(x.cuda(), for_grad, b_out), O.so3_fft(x.double(), for_grad, b_out), "so3_fft")
    xr = x[..., 0].contiguous()
    close(PSO3.so3_rfft(xr.cuda(), for_grad, b_out), O.so3_rfft(xr.double(), for_grad, b_out), "so3_rfft")
    s = rnd((O.nspec_so3(b_in), nz, 2), 11)
    close(PSO3.so3_ifft(s.cuda(), for_grad, b_out), O.so3_ifft(s.double(), for_grad, b_out), "so3_ifft")
    close(PSO3.so3_rifft(s.cuda(), for_grad, b_out), O.so3_rifft(s.double(), for_grad, b_out), "so3_rifft (generic spectrum)")
    sh = O.so3_rfft(rnd((nz, 2 * b_in, 2 * b_in, 2 * b_in), 12).double()).float()      # Hermitian spectrum, tests/so3_fft.py:112-114
    close(PSO3.so3_rifft(sh.cuda(), for_grad, b_out), O.so3_rifft(sh.double(), for_grad, b_out), "so3_rifft (real signal)")


@pytest.mark.parametrize("b_in,b_out", [(6, 6), (9, 2), (4, 6), (32, 12)])
def test_so3_complex_transforms_library_kernels(hip, b_in, b_out, monkeypatch):
    """so3_fft / so3_ifft through the library's kernels for complex signals (the default composes two real transforms)."""
    monkeypatch.setattr(PSO3, "complex_via_real", False)
    x = rnd((2, 2 * b_in, 2 * b_in, 2 * b_in, 2), 17)
    close(PSO3.so3_fft(x.cuda(), False, b_out), O.so3_fft(x.double(), False, b_out), "so3_fft")
    s = rnd((O.nspec_so3(b_in), 2, 2), 18)
    close(PSO3.so3_ifft(s.cuda(), True, b_out), O.so3_ifft(s.double(), True, b_out), "so3_ifft")


def test_so3_transform_batch_dims_and_ragged(hip):
    x = rnd((2, 3, 8, 8, 8), 13)
    close(PSO3.so3_rfft(x.cuda(), b_out=3), O.so3_rfft(x.double(), b_out=3), "lead dims")
    x1 = rnd((17, 6, 6, 6), 14)              # nbatch not a multiple of the z tile
    close(PSO3.so3_rfft(x1.cuda()), O.so3_rfft(x1.double()), "ragged batch")
    s1 = rnd((O.nspec_so3(3), 17, 2), 15)
    close(PSO3.so3_rifft(s1.cuda()), O.so3_rifft(s1.double()), "ragged batch inv")
    x0 = rnd((1, 2, 2, 2), 16)               # b = 1: a single coefficient
    close(PSO3.so3_rfft(x0.cuda()), O.so3_rfft(x0.double()), "b=1")


@pytest.mark.parametrize("nz", [1, 9, 20])
def test_so3_one_kernel_path_batches(hip, nz):
    """Real signals on the 64^3 grid take the one-kernel path (one workgroup per volume): batch sizes that
    leave XCD slots empty, truncated and over-long spectra, weighted and unweighted tables."""
    print(f"so3 one-kernel path nz={nz}", flush=True)
    x = rnd((nz, 64, 64, 64), 50 + nz)
    for for_grad in (False, True):
        for b_out in (32, 20, 1):
            close(PSO3.so3_rfft(x.cuda(), for_grad, b_out), O.so3_rfft(x.double(), for_grad, b_out), f"rfft 32->{b_out} for_grad={for_grad}")
        for b_spec in (32, 20, 36, 1):
            s = rnd((O.nspec_so3(b_spec), nz, 2), 60 + b_spec)
            close(PSO3.so3_rifft(s.cuda(), for_grad, 32), O.so3_rifft(s.double(), for_grad, 32), f"rifft {b_spec}->32 for_grad={for_grad}")


@pytest.mark.parametrize("b,nz", [(10, 1), (10, 9), (10, 41), (16, 1), (16, 9), (16, 20), (22, 1), (22, 9), (22, 20)])
def test_so3_one_kernel_path_of_the_20_32_and_44_grids(hip, b, nz):
    """Real signals on the 20^3, 32^3 and 44^3 grids have per-volume kernels of their own (a line of 4 x 5, 4 x 8 or 4 x 11
    points, two or three item rounds): batch sizes that leave XCD slots empty, spectra that skip the later rounds and over-long ones,
    both tables; repeated calls agree bit for bit, and a truncated spectrum gives what its zero-extended form gives."""
    from s2cnn_amd.soft.so3_fft import so3_rifft_real_basis, so3_rfft_real_basis
    print(f"so3 one-kernel path of the {2 * b}^3 grid nz={nz}", flush=True)
    x = rnd((nz, 2 * b, 2 * b, 2 * b), 150 + nz)
    for for_grad in (False, True):
        for b_out in (b, b - 3, b - 4, 7, 1):
            close(PSO3.so3_rfft(x.cuda(), for_grad, b_out), O.so3_rfft(x.double(), for_grad, b_out), f"rfft {b}->{b_out} for_grad={for_grad}")
        for b_spec in (b, b - 4, 9, b + 3, 1):
            s = rnd((O.nspec_so3(b_spec), nz, 2), 160 + b_spec)
            close(PSO3.so3_rifft(s.cuda(), for_grad, b), O.so3_rifft(s.double(), for_grad, b), f"rifft {b_spec}->{b} for_grad={for_grad}")
    xg = x.cuda()
    bias = rnd((1,), 170).cuda()
    for bs in (b, b - 6):
        r = rnd((O.nspec_so3(bs), nz, 1), 171 + bs).cuda()
        a1, y1 = so3_rfft_real_basis(xg, b_out=bs), so3_rifft_real_basis(r, b_out=b, bias=bias)
        for _ in range(3):
            assert torch.equal(so3_rfft_real_basis(xg, b_out=bs), a1)
            assert torch.equal(so3_rifft_real_basis(r, b_out=b, bias=bias), y1)
        rz = torch.zeros(O.nspec_so3(b), nz, 1, device="cuda")
        rz[:r.size(0)] = r
        close(y1, so3_rifft_real_basis(rz, b_out=b, bias=bias).cpu().double(), f"synthesis from {bs} degrees")
        close(a1, so3_rfft_real_basis(xg, b_out=b)[:a1.size(0)].cpu().double(), f"analysis to {bs} degrees")


@pytest.mark.parametrize("b", [10, 16, 22, 32])
def test_so3_few_volumes_split_along_beta(hip, b):
    """Below 129 volumes the per-volume kernels give a volume to 2, 4 or 8 workgroups along beta.  The analysis then adds
    partial records (another order of the beta sum: equal to rounding), the synthesis writes the same planes from the same
    record (equal to the bit).  130 volumes run unsplit; 100, 40 and 3 of them run with 2, 4 and up to 8 parts."""
    print(f"so3 beta split b={b}", flush=True)
    x = rnd((130, 2 * b, 2 * b, 2 * b), 180 + b).cuda()
    m = rnd((130, 2 * b, 2 * b, 2 * b), 181 + b).cuda()
    s = PSO3.so3_rfft(x)
    sm = PSO3.so3_rfft(x, mask=m)
    y = PSO3.so3_rifft(s)
    for n in (100, 40, 3):
        close(PSO3.so3_rfft(x[:n].contiguous()), s[:, :n].cpu(), f"rfft of {n} volumes")
        close(PSO3.so3_rfft(x[:n].contiguous(), mask=m[:n].contiguous()), sm[:, :n].cpu(), f"masked rfft of {n} volumes")
        assert torch.equal(PSO3.so3_rifft(s[:, :n].contiguous()), y[:n]), n


def test_so3_one_kernel_path_is_reproducible(hip):
    """Both directions on the 64^3 grid form their sums in a fixed order: repeated calls agree bit for bit
    (this also guards the store sequence of the synthesis kernel, which once mixed two stores up now and then)."""
    x = rnd((5, 64, 64, 64), 90).cuda()
    s = rnd((O.nspec_so3(32), 5, 2), 91).cuda()
    a0, y0 = PSO3.so3_rfft(x), PSO3.so3_rifft(s)
    close(y0, O.so3_rifft(s.cpu().double()), "rifft")
    for _ in range(4):
        assert torch.equal(PSO3.so3_rfft(x), a0)
        assert torch.equal(PSO3.so3_rifft(s), y0)
    # the instantiations for truncated spectra (22 and 26 degrees), at a batch that fills the chip, with the bias
    from s2cnn_amd.soft.so3_fft import so3_rifft_real_basis, so3_rfft_real_basis
    xb = rnd((300, 64, 64, 64), 92).cuda()
    bias = rnd((4,), 93).cuda()
    for b in (22, 26):
        r = rnd((O.nspec_so3(b), 75, 4), 94).cuda()
        a1, y1 = so3_rfft_real_basis(xb, b_out=b), so3_rifft_real_basis(r, b_out=32, bias=bias)
        for _ in range(3):
            assert torch.equal(so3_rfft_real_basis(xb, b_out=b), a1)
            assert torch.equal(so3_rifft_real_basis(r, b_out=32, bias=bias), y1)
        # against the untruncated kernels: zero-extended spectrum in, leading rows out
        rz = torch.zeros(O.nspec_so3(32), 75, 4, device="cuda")
        rz[:r.size(0)] = r
        close(y1, so3_rifft_real_basis(rz, b_out=32, bias=bias).cpu().double(), f"synthesis from {b} degrees")
        close(a1, so3_rfft_real_basis(xb, b_out=32)[:a1.size(0)].cpu().double(), f"analysis to {b} degrees")


def test_so3_transforms_without_prepacked_table(hip):
    """packed_table = NULL (the library repacks into its workspace) gives the same bits as the prepacked path."""
    from s2cnn_amd import _hip
    for b_in, b_out in [(32, 32), (16, 16), (16, 9), (22, 22), (22, 13), (10, 10), (10, 6), (9, 5)]:
        nz = 5
        x = rnd((nz, 2 * b_in, 2 * b_in, 2 * b_in), 17).cuda()
        want = PSO3.so3_rfft(x, b_out=b_out)
        table = PSO3._setup_wigner(b_in, b_out, True, x.device)
        out = torch.empty_like(want)
        ws = _hip.workspace(hip.s2cnn_so3_analysis_workspace(b_in, b_out, nz, 0), x.device)
        _hip.check(hip.s2cnn_so3_analysis(_hip.ptr(x), _hip.ptr(table), None, _hip.ptr(out), _hip.ptr(ws), ws.numel(),
                                          b_in, b_out, nz, 0, _hip.stream_ptr()))
        assert torch.equal(out, want)
        s = rnd((O.nspec_so3(b_out), nz, 2), 18).cuda()
        want = PSO3.so3_rifft(s, b_out=b_in)
        table = PSO3._setup_wigner(b_in, b_out, False, x.device)
        out = torch.empty_like(want)
        ws = _hip.workspace(hip.s2cnn_so3_synthesis_workspace(b_out, b_in, nz, 0), x.device)
        _hip.check(hip.s2cnn_so3_synthesis(_hip.ptr(s), _hip.ptr(table), None, _hip.ptr(out), _hip.ptr(ws), ws.numel(),
                                           b_out, b_in, nz, 0, _hip.stream_ptr()))
        assert torch.equal(out, want)


@pytest.mark.parametrize("b", [10, 16, 22])
def test_so3_per_volume_kernels_take_any_float_pointer(hip, b):
    """Through the raw C ABI: the per-volume kernels of the 20^3, 32^3 and 44^3 grids ask for no more than float alignment
    of the signal, the mask and the output (the 64^3 grid wants 16 bytes and says so with S2CNN_EALIGN)."""
    from s2cnn_amd import _hip
    nz = 3
    n3 = nz * (2 * b) ** 3
    big = rnd((2 * n3 + 8,), 33).cuda()
    x = big[1:1 + n3].view(nz, 2 * b, 2 * b, 2 * b)                    # 4 bytes past a 16-byte boundary
    assert x.data_ptr() % 16 == 4
    table = PSO3._setup_wigner(b, b, True, x.device)
    want = PSO3.so3_rfft(x.clone())
    out = torch.empty_like(want)
    ws = _hip.workspace(hip.s2cnn_so3_analysis_workspace(b, b, nz, 0), x.device)
    _hip.check(hip.s2cnn_so3_analysis(_hip.ptr(x), _hip.ptr(table), None, _hip.ptr(out), _hip.ptr(ws), ws.numel(), b, b, nz, 0, _hip.stream_ptr()))
    assert torch.equal(out, want)
    s = rnd((O.nspec_so3(b), nz, 2), 34).cuda()
    want = PSO3.so3_rifft(s)
    y = big[n3 + 3:2 * n3 + 3].view(nz, 2 * b, 2 * b, 2 * b)
    assert y.data_ptr() % 16 == 12
    table = PSO3._setup_wigner(b, b, False, x.device)
    ws = _hip.workspace(hip.s2cnn_so3_synthesis_workspace(b, b, nz, 0), x.device)
    _hip.check(hip.s2cnn_so3_synthesis(_hip.ptr(s), _hip.ptr(table), None, _hip.ptr(y), _hip.ptr(ws), ws.numel(), b, b, nz, 0, _hip.stream_ptr()))
    assert torch.equal(y, want)
    x64 = rnd((64 ** 3 + 4,), 35).cuda()[1:]
    ws = _hip.workspace(hip.s2cnn_so3_analysis_workspace(32, 32, 1, 0), x.device)
    t64 = PSO3._setup_wigner(32, 32, True, x.device)
    o64 = torch.empty(O.nspec_so3(32), 1, 2, device="cuda")
    assert hip.s2cnn_so3_analysis(_hip.ptr(x64), _hip.ptr(t64), None, _hip.ptr(o64), _hip.ptr(ws), ws.numel(), 32, 32, 1, 0, _hip.stream_ptr()) == -3


def test_so3_reference_identities_on_gpu(hip):
    """tests/so3_fft.py:8-24 and :34-91 of the reference, run on the HIP path."""
    b_in, b_out = 7, 5
    x = rnd((2 * b_in, 2 * b_in, 2 * b_in), 20).cuda()
    y1 = PSO3.so3_rfft(x, b_out=b_out)
    w = torch.tensor(s2cnn_amd.wigner.quadrature_weights(b_in), dtype=torch.float32).cuda()
    y2 = s2cnn_amd.so3_rft((x * w.view(-1, 1, 1)).view(-1), b_out, s2cnn_amd.so3_soft_grid(b_in))
    assert (y1 - y2).abs().max().item() < 1e-4 * y1.abs().mean().item()
    for f, g, cplx, pairs in ((PSO3.so3_fft, PSO3.so3_ifft, True, [(7, 7), (5, 4), (7, 4), (7, 5), (4, 6)]),
                              (PSO3.so3_rfft, PSO3.so3_rifft, False, [(7, 7), (5, 4), (4, 6)])):
        for bi, bo in pairs:
            x = rnd((2 * bi,) * 3 + ((2,) if cplx else ()), 21).cuda()
            x = g(f(x, b_out=bo), b_out=bi)
            y = g(f(x, b_out=bo), b_out=bi)
            assert (x - y).abs().max().item() < 1e-4 * y.abs().mean().item(), (bi, bo, cplx)
    for f, g in ((PSO3.so3_ifft, PSO3.so3_fft), (PSO3.so3_rifft, PSO3.so3_rfft)):
        for bi, bo in [(7, 7), (5, 4), (4, 7)]:
            x = rnd((O.nspec_so3(bi), 2), 22).cuda()
            x = g(f(x, b_out=bo), b_out=bi)
            y = g(f(x, b_out=bo), b_out=bi)
            assert (x - y).abs().max().item() < 1e-4 * y.abs().mean().item(), (bi, bo)


# ------------------------------------------------------------------ S^2 transforms
@pytest.mark.parametrize("b_in,b_out", [(6, 5), (12, 12), (13, 12), (30, 10), (4, 1), (64, 16)])   # (6,5): s2_fft.py:253-259
@pytest.mark.parametrize("for_grad", [False, True])
def test_s2_transforms(hip, b_in, b_out, for_grad):
    print(f"s2 transforms b_in={b_in} b_out={b_out} for_grad={for_grad}", flush=True)
    x = rnd((1, 2, 2 * b_in, 2 * b_in, 2), 30)
    close(PS2.s2_fft(x.cuda(), for_grad, b_out), O.s2_fft(x.double(), for_grad, b_out), "s2_fft")
    xr = x[..., 0].contiguous()
    close(PS2.s2_rfft(xr.cuda(), for_grad, b_out), O.s2_fft(O.as_complex(xr.double()), for_grad, b_out), "s2_rfft")
    s = rnd((b_out ** 2, 10, 2), 31)                                                    # s2_fft.py:262-268 uses (12 -> 13)
    close(PS2.s2_ifft(s.cuda(), for_grad, b_in), O.s2_ifft(s.double(), for_grad, b_in), "s2_ifft")
    close(PS2.s2_rifft(s.cuda(), for_grad, b_in), O.s2_ifft(s.double(), for_grad, b_in)[..., 0], "s2_rifft")


@pytest.mark.parametrize("b,nbatch", [(12, 5), (32, 100), (20, 1)])
def test_s2_analysis_of_few_signals_at_full_bandwidth(hip, b, nbatch):
    """b_out = b_in with few signals: the analysis is split along beta and the partial spectra go through the workspace
    (s2cnn_s2_analysis_workspace covers them).  Checked against the oracle, and through the raw C ABI with a workspace of
    the two-kernel path's size only, where the library must run with as many splits as fit and give the same spectrum."""
    import ctypes
    x = rnd((nbatch, 2 * b, 2 * b), 33 + b)
    want = O.s2_fft(O.as_complex(x.double()), False, b)
    got = PS2.s2_rfft(x.cuda(), False, b)
    close(got, want, f"s2_rfft b={b}, {nbatch} signals")
    xg = x.cuda()
    table = PS2._setup_wigner(b, b, True, xg.device)
    small = nbatch * 2 * b * (2 * b - 1) * 8
    assert hip.s2cnn_s2_analysis_workspace(b, b, nbatch, 0) >= small
    ws = torch.empty(small, dtype=torch.uint8, device=xg.device)
    out = torch.full_like(got, float("nan"))
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    rc = hip.s2cnn_s2_analysis(p(xg), p(table), p(out), p(ws), small, b, b, nbatch, 0, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    close(out, want, "the same with the smaller workspace")


def test_so3_integrate(hip):
    for b in (1, 3, 6, 16, 32):                     # 32: the 16-byte-load path (planes of 4096 samples)
        x = rnd((2, 5, 2 * b, 2 * b, 2 * b), 40 + b)
        xg = x.cuda().requires_grad_()
        out = s2cnn_amd.so3_integrate(xg)
        close(out, O.so3_integrate(x.double()), f"integrate b={b}")
        g = rnd((2, 5), 41)
        (gx,) = torch.autograd.grad(out, xg, g.cuda())
        xo = x.double().requires_grad_()
        (gxo,) = torch.autograd.grad(O.so3_integrate(xo), xo, g.double())
        close(gx, gxo, f"integrate grad b={b}")
    ones = torch.ones(3, 8, 8, 8, device="cuda")
    assert (s2cnn_amd.so3_integrate(ones) - 1).abs().max().item() < 1e-5
    # an input that is not 16-byte aligned takes the 4-byte loads: same numbers up to the order of the sums
    big = rnd((3 * 14 ** 3 + 1,), 43).cuda()
    xo = big[1:].view(3, 14, 14, 14)
    close(s2cnn_amd.so3_integrate(xo), O.so3_integrate(xo.cpu().double()), "integrate, unaligned input")


# ------------------------------------------------------------------ layers, forward and gradients
def _conv_case(kind, B, Fi, Fo, b_in, b_out, grid, seed, real_basis=None, activation=None):
    if kind == "so3":
        x = rnd((B, Fi, 2 * b_in, 2 * b_in, 2 * b_in), seed)
        layer = s2cnn_amd.SO3Convolution(Fi, Fo, b_in, b_out, grid, activation=activation)
        ofun = O.so3_conv
    else:
        x = rnd((B, Fi, 2 * b_in, 2 * b_in), seed)
        layer = s2cnn_amd.S2Convolution(Fi, Fo, b_in, b_out, grid, activation=activation)
        ofun = O.s2_conv
    k = torch.rand(Fi, Fo, len(grid), generator=torch.Generator().manual_seed(seed + 1)) * 2 - 1
    bias = rnd((1, Fo, 1, 1, 1), seed + 2, 0.1)
    with torch.no_grad():
        layer.kernel.copy_(k)
        layer.bias.copy_(bias)
    if real_basis is not None:
        layer.real_basis = real_basis
    layer = layer.cuda()
    xg = x.cuda().requires_grad_()
    out = layer(xg)
    (out ** 2).sum().backward()
    xo, ko, bo = x.double().requires_grad_(), k.double().requires_grad_(), bias.double().requires_grad_()
    outo = ofun(xo, ko, bo, b_in, b_out, grid)
    if activation == "relu":
        outo = torch.relu(outo)
    (outo ** 2).sum().backward()
    close(out, outo, kind + " conv out")
    close(xg.grad, xo.grad, kind + " conv grad x")
    close(layer.kernel.grad, ko.grad, kind + " conv grad kernel")
    close(layer.bias.grad, bo.grad, kind + " conv grad bias")


def _random_grid(kind, rng):
    import math
    if kind == "so3":
        pick = rng.randrange(3)
        if pick == 0:
            return s2cnn_amd.so3_near_identity_grid(max_beta=math.pi / rng.choice((4, 8, 16)), n_alpha=rng.choice((3, 4, 6, 8)),
                                                    n_beta=rng.choice((1, 2, 3)), n_gamma=rng.choice((None, 1, 3, 5)))
        if pick == 1:
            return s2cnn_amd.so3_equatorial_grid(max_beta=rng.choice((0, 0.2)), max_gamma=rng.choice((0, 0.4)), n_alpha=rng.choice((4, 7, 12)),
                                                 n_beta=rng.choice((1, 2)), n_gamma=rng.choice((1, 2, 3)))
        return ((0.3, 1.0, 2.0), (1.1, 0.2, 5.0), (2.9, 4.0, 0.1), (0.3, 2.0, 2.5), (1.7, 3.3, 3.3))   # no two points share beta rings evenly
    pick = rng.randrange(2)
    if pick == 0:
        return s2cnn_amd.s2_near_identity_grid(max_beta=math.pi / rng.choice((4, 8)), n_alpha=rng.choice((3, 5, 8)), n_beta=rng.choice((1, 2, 3)))
    return s2cnn_amd.s2_equatorial_grid(max_beta=rng.choice((0, 0.3)), n_alpha=rng.choice((4, 9, 16)), n_beta=rng.choice((1, 3)))


@pytest.mark.parametrize("seed", range(10))
def test_layers_on_random_shapes(hip, seed):
    """Seeded random draws of batch, feature counts, bandwidths (b_out <= b_in as the layers are used, both parities,
    grids the fast paths do not cover) and kernel grids: forward and all gradients of both layers against the oracle,
    in the real-basis and the complex formulation, with and without the activation inside."""
    import random
    rng = random.Random(1234 + seed)
    for kind in ("so3", "s2"):
        b_in = rng.randint(2, 7) if kind == "so3" else rng.randint(2, 12)
        b_out = rng.randint(2, min(b_in, 6))       # b_out = 1 gives constant outputs: the std of the error metric vanishes
        B, Fi, Fo = rng.randint(1, 5), rng.randint(1, 9), rng.randint(1, 9)
        grid = _random_grid(kind, rng)
        real_basis = rng.random() < 0.6
        activation = rng.choice((None, "relu"))
        print(f"random case {seed} {kind}: B={B} {Fi}->{Fo} b {b_in}->{b_out} grid {len(grid)} real_basis={real_basis} activation={activation}", flush=True)
        _conv_case(kind, B, Fi, Fo, b_in, b_out, grid, 7000 + 10 * seed, real_basis, activation)


def test_empty_batch(hip):
    """A batch of zero samples runs through operators and layers like any other: empty outputs of the right shape,
    zero gradients for the weights (the reference's CPU branches behave so, being plain tensor algebra)."""
    c1 = s2cnn_amd.S2Convolution(2, 3, 6, 4, s2cnn_amd.s2_near_identity_grid()).cuda()
    c2 = s2cnn_amd.SO3Convolution(3, 5, 4, 3, s2cnn_amd.so3_near_identity_grid(), activation="relu").cuda()
    for real_basis in (True, False):
        c1.real_basis = c2.real_basis = real_basis
        x = torch.zeros(0, 2, 12, 12, device="cuda", requires_grad=True)
        y = c2(c1(x))
        assert y.shape == (0, 5, 6, 6, 6)
        v = s2cnn_amd.so3_integrate(y)
        assert v.shape == (0, 5)
        v.sum().backward()
        assert x.grad.shape == x.shape
        for c in (c1, c2):
            assert c.kernel.grad.shape == c.kernel.shape and float(c.kernel.grad.abs().max()) == 0.0
            assert float(c.bias.grad.abs().max()) == 0.0
            c.zero_grad()
    s = PSO3.so3_rfft(torch.zeros(0, 8, 8, 8, device="cuda"))
    assert s.shape == (O.nspec_so3(4), 0, 2) and PSO3.so3_rifft(s).shape == (0, 8, 8, 8)
    s = PS2.s2_rfft(torch.zeros(3, 0, 8, 8, device="cuda"))
    assert s.shape == (16, 3, 0, 2) and PS2.s2_rifft(s).shape == (3, 0, 8, 8)
    z = s2cnn_amd.so3_mm(torch.zeros(10, 0, 3, 2, device="cuda"), torch.zeros(10, 3, 4, 2, device="cuda"))
    assert z.shape == (10, 0, 4, 2)
    z = s2cnn_amd.s2_mm(torch.zeros(4, 0, 3, 2, device="cuda"), torch.zeros(4, 3, 4, 2, device="cuda"))
    assert z.shape == (10, 0, 4, 2)


def test_so3_convolution_parity(hip):
    _conv_case("so3", 2, 3, 4, 5, 4, s2cnn_amd.so3_near_identity_grid(n_alpha=4, n_beta=2, n_gamma=3), 50)
    _conv_case("so3", 3, 8, 8, 6, 6, s2cnn_amd.so3_near_identity_grid(), 53)
    _conv_case("so3", 2, 4, 6, 4, 4, s2cnn_amd.so3_equatorial_grid(n_alpha=8), 56)


@pytest.mark.parametrize("real_basis", [True, False])
def test_s2_convolution_parity(hip, real_basis):
    """Both paths of the layer: real-basis spectra (the default) and the reference's complex ones."""
    _conv_case("s2", 2, 1, 4, 8, 4, s2cnn_amd.s2_near_identity_grid(), 60, real_basis)
    _conv_case("s2", 3, 6, 5, 10, 5, s2cnn_amd.s2_equatorial_grid(n_alpha=16), 63, real_basis)
    _conv_case("s2", 3, 10, 8, 6, 6, s2cnn_amd.s2_near_identity_grid(), 66, real_basis)      # two feature passes, 16-byte rows


@pytest.mark.parametrize("b_in,b_out,nz,nf", [(32, 32, 4, 2),     # per-volume kernels (all item rounds)
                                              (32, 22, 6, 3), (32, 26, 2, 1),   # their truncated instantiations
                                              (10, 32, 6, 3),     # synthesis onto the 64^3 grid from a short spectrum
                                              (16, 16, 4, 2), (16, 10, 6, 3), (10, 16, 6, 3), (16, 18, 2, 1),   # the per-volume kernels of the 32^3 grid
                                              (22, 22, 4, 2), (22, 18, 2, 1), (12, 22, 6, 3), (22, 24, 2, 1),   # ... and of the 44^3 grid
                                              (10, 10, 4, 2), (10, 7, 6, 3), (6, 10, 6, 3), (10, 13, 2, 1),     # ... and of the 20^3 grid
                                              (32, 34, 2, 1),     # 64-point plane kernel + Wigner stage
                                              (22, 7, 6, 2), (6, 6, 10, 5), (5, 9, 3, 1), (11, 4, 2, 1),   # folded plane kernels
                                              (36, 36, 2, 1), (40, 33, 2, 2)])   # ... with the Wigner stage in parts
def test_so3_transforms_with_fused_relu(hip, b_in, b_out, nz, nf):
    """max(., 0) in the epilogue of the synthesis and its gradient mask in the loads of the analysis against the
    separate elementwise passes they replace: the results must be the same numbers, bit for bit, for complex and
    real-basis spectra."""
    from s2cnn_amd.soft import so3_fft as P
    from s2cnn_amd.so3_real import so3_spectrum_to_real
    print(f"fused relu b_in={b_in} b_out={b_out} nz={nz} nf={nf}", flush=True)
    g = torch.Generator().manual_seed(1000 * b_in + b_out)
    # synthesis b_in -> b_out
    xh = torch.randn(O.nspec_so3(b_in), nz // nf, nf, 2, generator=g).cuda()
    bias = torch.randn(nf, generator=g).cuda()
    for bb in (bias, None):
        plain = P.so3_rifft(xh, b_out=b_out, bias=bb)
        fused = P.so3_rifft(xh, b_out=b_out, bias=bb, relu=True)
        assert torch.equal(fused, torch.relu(plain))
        assert (fused == 0).float().mean().item() > 0.2
        r = so3_spectrum_to_real(xh)
        assert torch.equal(P.so3_rifft_real_basis(r, b_out=b_out, bias=bb, relu=True), torch.relu(P.so3_rifft_real_basis(r, b_out=b_out, bias=bb)))
    # analysis b_in -> b_out, both tables
    x = torch.randn(nz // nf, nf, 2 * b_in, 2 * b_in, 2 * b_in, generator=g).cuda()
    y = torch.relu(torch.randn(x.shape, generator=g)).cuda()        # what a relu leaves behind: zeros and positive values
    for for_grad in (False, True):
        want = P.so3_rfft(x * (y > 0), for_grad=for_grad, b_out=b_out)
        assert torch.equal(P.so3_rfft(x, for_grad=for_grad, b_out=b_out, mask=y), want)
        want = P.so3_rfft_real_basis(x * (y > 0), for_grad=for_grad, b_out=b_out)
        assert torch.equal(P.so3_rfft_real_basis(x, for_grad=for_grad, b_out=b_out, mask=y), want)
    # an operand that is not 16-byte aligned takes another loader (or a copy): same numbers
    big = torch.randn(x.numel() + 1, generator=g).cuda()
    xo, yo = big[1:].view(x.shape), torch.relu(big.flip(0))[1:].view(x.shape)
    assert torch.equal(P.so3_rfft(xo, b_out=b_out, mask=yo), P.so3_rfft(xo * (yo > 0), b_out=b_out))


@pytest.mark.parametrize("b_in", [32, 10, 22])
def test_one_bit_relu_mask_on_the_64_grid(hip, b_in):
    """The synthesis onto the 64^3 grid can record "the output is not <= 0" as one bit per sample (word
    [volume][beta][alpha % 8][alpha / 8], bit gamma), and the analysis from that grid can take those bits for the mask:
    the bits must say exactly what the float output says, and the masked analysis must give the numbers of the analysis
    with the float mask up to rounding (the two instantiations of the kernel need not contract their multiply-adds alike:
    2e-6 of the largest coefficient), for both kinds of spectra and both tables.  Other grids report that they keep no bits."""
    from s2cnn_amd.soft import so3_fft as P
    from s2cnn_amd.so3_real import so3_spectrum_to_real
    assert P._relu_bits(22, 3, "cuda") is None and P._relu_bits(32, 0, "cuda") is None
    nz, nf = 6, 3
    g = torch.Generator().manual_seed(77 + b_in)
    xh = torch.randn(O.nspec_so3(b_in), nz // nf, nf, 2, generator=g).cuda()
    bias = torch.randn(nf, generator=g).cuda()
    gy = torch.randn(nz // nf, nf, 64, 64, 64, generator=g).cuda()
    for real_basis in (False, True):
        spec = so3_spectrum_to_real(xh) if real_basis else xh
        synth = P.so3_rifft_real_basis if real_basis else P.so3_rifft
        ana = P.so3_rfft_real_basis if real_basis else P.so3_rfft
        bits = P._relu_bits(32, nz, "cuda")
        assert bits.numel() == nz * 64 * 64 and bits.dtype == torch.int64
        bits.fill_(0x5555555555555555)                                        # every word must be overwritten
        out = synth(spec, b_out=32, bias=bias, relu=True, bits=bits)
        assert torch.equal(out, synth(spec, b_out=32, bias=bias, relu=True))
        # unpack: [z, beta, alpha % 8, alpha / 8] words, bit gamma
        shifts = torch.arange(64, device="cuda")
        got = ((bits.view(nz, 64, 8, 8, 1) >> shifts) & 1).bool()             # [z, beta, a_lo, a_hi, gamma]
        got = got.permute(0, 1, 3, 2, 4).reshape(nz, 64, 64, 64)              # alpha = 8 a_hi + a_lo
        assert torch.equal(got, out.view(nz, 64, 64, 64) > 0)
        for for_grad in (False, True):
            for b_out in (32, 22, b_in):
                want = ana(gy, for_grad=for_grad, b_out=b_out, mask=out)
                got = ana(gy, for_grad=for_grad, b_out=b_out, mask=bits)
                err = (got - want).abs().max().item() / want.abs().max().item()
                assert err < 2e-6, (real_basis, for_grad, b_out, err)
        # a mask of all ones is no mask, a mask of zeros leaves nothing
        close(ana(gy, b_out=b_in, mask=torch.full_like(bits, -1)), ana(gy, b_out=b_in).double().cpu(), "all-ones bit mask")
        assert not ana(gy, b_out=b_in, mask=torch.zeros_like(bits)).any()


@pytest.mark.parametrize("kind,real_basis", [("so3", True), ("so3", False), ("s2", True), ("s2", False)])
def test_layers_with_fused_relu(hip, kind, real_basis):
    """activation="relu" is F.relu(layer(x)): same output, same gradients wrt input, kernel and bias; and the
    output against the oracle's layer followed by relu."""
    shapes = [(3, 4, 6, 5, 5), (2, 3, 5, 32, 32)] if kind == "so3" else [(3, 2, 6, 8, 5), (2, 3, 4, 40, 32)]
    for (B, fi, fo, b_in, b_out) in shapes:
        print(f"fused relu layer {kind} real_basis={real_basis} B={B} {fi}->{fo} b {b_in}->{b_out}", flush=True)
        torch.manual_seed(b_in)
        if kind == "so3":
            grid = s2cnn_amd.so3_near_identity_grid()
            ref = s2cnn_amd.SO3Convolution(fi, fo, b_in, b_out, grid)
            fus = s2cnn_amd.SO3Convolution(fi, fo, b_in, b_out, grid, activation="relu")
            x = torch.randn(B, fi, 2 * b_in, 2 * b_in, 2 * b_in)
        else:
            grid = s2cnn_amd.s2_near_identity_grid()
            ref = s2cnn_amd.S2Convolution(fi, fo, b_in, b_out, grid)
            fus = s2cnn_amd.S2Convolution(fi, fo, b_in, b_out, grid, activation="relu")
            x = torch.randn(B, fi, 2 * b_in, 2 * b_in)
        with torch.no_grad():
            ref.bias.normal_()
        fus.load_state_dict(ref.state_dict())
        ref.real_basis = fus.real_basis = real_basis
        if b_in <= 8:
            conv = O.so3_conv if kind == "so3" else O.s2_conv
            want = torch.relu(conv(x.double(), ref.kernel.detach().double(), ref.bias.detach().double(), b_in, b_out, grid))
        ref, fus = ref.cuda(), fus.cuda()
        xa, xb = x.cuda().requires_grad_(), x.cuda().requires_grad_()
        ya, yb = torch.relu(ref(xa)), fus(xb)
        assert torch.equal(ya, yb)
        if b_in <= 8:
            close(yb, want, "layer + relu against the oracle")
        w = torch.randn(ya.shape, generator=torch.Generator().manual_seed(5)).cuda()
        (ya * w).sum().backward()
        (yb * w).sum().backward()
        for a, b, name in ((xa.grad, xb.grad, "input"), (ref.kernel.grad, fus.kernel.grad, "kernel"), (ref.bias.grad, fus.bias.grad, "bias")):
            err = (a - b).abs().max().item() / a.abs().max().item()
            assert err < 1e-6, (name, err)


def test_config1_shaped_network(hip):
    """benchmark config 1 shapes at reduced batch: S2Conv 1->20 (b 30->10), ReLU, SO3Conv 20->40
    (b 10->6), ReLU, so3_integrate; forward only."""
    g = torch.Generator().manual_seed(1)
    x = torch.rand(4, 1, 60, 60, generator=g) * (torch.rand(4, 1, 60, 60, generator=g) < 0.3)
    g1 = s2cnn_amd.s2_near_identity_grid(max_beta=3.141592653589793 / 8, n_alpha=8, n_beta=3)
    g2 = s2cnn_amd.so3_near_identity_grid(max_beta=3.141592653589793 / 8, max_gamma=2 * 3.141592653589793, n_alpha=8, n_beta=3, n_gamma=8)
    torch.manual_seed(0)
    c1 = s2cnn_amd.S2Convolution(1, 20, 30, 10, g1)
    c2 = s2cnn_amd.SO3Convolution(20, 40, 10, 6, g2)
    want = O.so3_integrate(torch.relu(O.so3_conv(torch.relu(O.s2_conv(x.double(), c1.kernel.detach().double(), c1.bias.detach().double(), 30, 10, g1)),
                                                 c2.kernel.detach().double(), c2.bias.detach().double(), 10, 6, g2)))
    c1, c2 = c1.cuda(), c2.cuda()
    with torch.no_grad():
        got = s2cnn_amd.so3_integrate(torch.relu(c2(torch.relu(c1(x.cuda())))))
    close(got, want, "config-1 features")


def _config5_layers(seed=8):
    """benchmark config 5 (SHREC17-shaped): S2Conv 6->100 b128->32, SO3Conv 100->100 b32->22, SO3Conv 100->55 b22->7,
    near-identity grids with max_beta scaled by the bandwidth ratio (examples/shrec17/model_original.py:12-40)."""
    import math
    g1 = s2cnn_amd.s2_near_identity_grid(max_beta=math.pi / 8 * 30 / 128, n_alpha=8, n_beta=3)
    g2 = s2cnn_amd.so3_near_identity_grid(max_beta=math.pi / 8 * 30 / 32, max_gamma=2 * math.pi, n_alpha=8, n_beta=3, n_gamma=8)
    g3 = s2cnn_amd.so3_near_identity_grid(max_beta=math.pi / 8 * 30 / 22, max_gamma=2 * math.pi, n_alpha=8, n_beta=3, n_gamma=8)
    torch.manual_seed(seed)
    return (s2cnn_amd.S2Convolution(6, 100, 128, 32, g1), s2cnn_amd.SO3Convolution(100, 100, 32, 22, g2),
            s2cnn_amd.SO3Convolution(100, 55, 22, 7, g3)), (g1, g2, g3)


def test_config5_shaped_network(hip):
    """Forward parity against the oracle at batch 1; forward + backward at batch 4 on the GPU must reproduce the
    batch-1 result for its first sample (batch independence) and give finite gradients."""
    (c1, c2, c3), (g1, g2, g3) = _config5_layers()
    from s2cnn_amd.harness import smooth_spherical_batch
    x = smooth_spherical_batch(4, 6, 128, "cuda", seed=9).cpu()       # the input the configuration names: smooth, l < 16, plus noise
    assert 0.0 <= x.min().item() and x.max().item() < 1.0 and x.std().item() > 0.05
    x1 = x[:1].double()

    def kb(c):
        return c.kernel.detach().double(), c.bias.detach().double()

    y = O.s2_conv(x1, *kb(c1), 128, 32, g1)
    y = O.so3_conv(torch.relu(y), *kb(c2), 32, 22, g2)
    y = O.so3_conv(torch.relu(y), *kb(c3), 22, 7, g3)
    want = O.so3_integrate(y)
    c1, c2, c3 = c1.cuda(), c2.cuda(), c3.cuda()

    def net(t):
        return s2cnn_amd.so3_integrate(c3(torch.relu(c2(torch.relu(c1(t))))))

    with torch.no_grad():
        got1 = net(x[:1].cuda())
    close(got1, want, "config-5 features, batch 1")
    xg = x.cuda().requires_grad_()
    out = net(xg)
    (out ** 2).sum().backward()
    assert (out[:1] - got1).abs().max().item() < 1e-4 * got1.abs().max().item()
    for t in (xg.grad, c1.kernel.grad, c2.kernel.grad, c3.kernel.grad, c3.bias.grad):
        assert torch.isfinite(t).all() and t.abs().max().item() > 0


def test_z_rotation_equivariance_on_gpu(hip):
    """examples/equivariance_error/main.py:18-46 of the reference at reduced sizes."""
    torch.manual_seed(2)
    c1 = s2cnn_amd.S2Convolution(3, 5, 16, 8, s2cnn_amd.s2_equatorial_grid(max_beta=0, n_alpha=32, n_beta=1)).cuda()
    c2 = s2cnn_amd.SO3Convolution(5, 4, 8, 4, s2cnn_amd.so3_equatorial_grid(max_beta=0, max_gamma=0, n_alpha=32, n_beta=1, n_gamma=1)).cuda()

    def phi(t):
        return c2(torch.relu(c1(t)))

    def rot(t, n):
        return torch.cat([t[:, :, :, n:], t[:, :, :, :n]], dim=3)

    with torch.no_grad():
        x = torch.randn(1, 3, 32, 32, device="cuda")
        y = phi(x)
        rel = (rot(phi(x), 2) - phi(rot(x, 8))).std() / y.std()     # a quarter turn: 8 of 32 input samples, 2 of 8 output samples
    assert rel.item() < 1e-4


def test_so3_rotation(hip):
    """s2cnn/soft/so3_rotation.py of the reference: parity with the oracle, the group law, and the
    arbitrary-rotation equivariance of a layer (examples/equivariance_plot/main.py:74-78 of the reference)."""
    b = 6
    x = rnd((2, 3, 2 * b, 2 * b, 2 * b), 90)
    a, bt, g = 0.3, 1.1, -0.7
    got = s2cnn_amd.so3_rotation(x.cuda(), a, bt, g)
    close(got, O.so3_rotation(x.double(), a, bt, g), "so3_rotation")
    # rotating by the z-axis angle 2 pi k / 2b is a roll of the alpha axis (band-limited part of x)
    xb = PSO3.so3_rifft(PSO3.so3_rfft(x.cuda()))
    rolled = s2cnn_amd.so3_rotation(xb, 2 * 3.141592653589793 * 2 / (2 * b), 0.0, 0.0)
    assert (rolled - torch.roll(xb, 2, dims=-2)).abs().max().item() < 1e-4 * xb.abs().max().item() or \
           (rolled - torch.roll(xb, -2, dims=-2)).abs().max().item() < 1e-4 * xb.abs().max().item()
    # equivariance of an SO(3) convolution under an arbitrary rotation
    torch.manual_seed(5)
    conv = s2cnn_amd.SO3Convolution(3, 2, b, b, s2cnn_amd.so3_near_identity_grid(n_alpha=4, n_beta=2, n_gamma=3)).cuda()
    with torch.no_grad():
        y1 = s2cnn_amd.so3_rotation(conv(xb), a, bt, g)
        y2 = conv(s2cnn_amd.so3_rotation(xb, a, bt, g))
    rel = ((y1 - y2).std() / y1.std()).item()
    print("rotation equivariance residual", rel, flush=True)
    assert rel < 1e-3


def test_so3_shortcut(hip):
    sc = s2cnn_amd.SO3Shortcut(3, 3, 4, 4)
    x = rnd((2, 3, 8, 8, 8), 91).cuda()
    assert sc(x) is x
    sc2 = s2cnn_amd.SO3Shortcut(3, 5, 4, 3).cuda()
    want = O.so3_conv(x.cpu().double(), sc2.conv.kernel.detach().cpu().double(), sc2.conv.bias.detach().cpu().double(), 4, 3, ((0, 0, 0),))
    close(sc2(x), want, "shortcut conv")


def test_size_independent_properties_at_config_sizes(hip):
    """Config 2 (b = 32) at a reduced batch: fft -> ifft -> fft reproduces the spectrum (projector),
    linearity, and the Hermitian symmetry of the spectrum of a real signal."""
    b = 32
    x = rnd((8, 2 * b, 2 * b, 2 * b), 70).cuda()
    s = PSO3.so3_rfft(x)
    assert s.shape == (43680, 8, 2)
    s2 = PSO3.so3_rfft(PSO3.so3_rifft(s))
    assert (s2 - s).abs().max().item() < 1e-4 * s.abs().mean().item() * 10
    x2 = rnd((8, 2 * b, 2 * b, 2 * b), 71).cuda()
    lin = PSO3.so3_rfft(2 * x - 3 * x2) - (2 * s - 3 * PSO3.so3_rfft(x2))
    assert lin.abs().max().item() < 1e-4 * s.abs().mean().item() * 10
    l, m, n = 17, 5, -9
    i1 = O.nspec_so3(l) + (l + m) * (2 * l + 1) + (l + n)
    i2 = O.nspec_so3(l) + (l - m) * (2 * l + 1) + (l - n)
    sign = (-1) ** (m - n)
    assert torch.allclose(s[i2, :, 0], sign * s[i1, :, 0]) and torch.allclose(s[i2, :, 1], -sign * s[i1, :, 1])


def test_so3_mm_at_config3_features_linearity(hip):
    """Config 3 feature sizes (batch 16, 64 -> 64) at nl = 16: bilinearity and agreement with a
    per-degree complex einsum on the GPU in float64."""
    nl, B, F = 16, 16, 64
    ns = O.nspec_so3(nl)
    x = rnd((ns, B, F, 2), 80).cuda()
    y = (rnd((ns, F, F, 2), 81) * 0.125).cuda()
    z = s2cnn_amd.so3_mm(x, y)
    xc = torch.view_as_complex(x.double())
    yc = torch.view_as_complex(y.double())
    for l in (0, 1, 7, 15):
        L = 2 * l + 1
        lo = O.nspec_so3(l)
        want = torch.einsum("mpik,npkj->mnij", xc[lo:lo + L * L].view(L, L, B, F), yc[lo:lo + L * L].view(L, L, F, F).conj())
        got = torch.view_as_complex(z[lo:lo + L * L].double()).view(L, L, B, F)
        assert (got - want).abs().max().item() < 1e-4 * want.abs().std().item(), l
    z2 = s2cnn_amd.so3_mm(2 * x, y) - 2 * z
    assert z2.abs().max().item() < 1e-4 * z.std().item()


@pytest.mark.parametrize("b_grid,b_spec,nz", [(22, 22, 2), (22, 7, 5), (40, 8, 1), (5, 5, 60), (1, 1, 300),
                                              # more than 32 frequencies or degrees: the Wigner stage runs in parts
                                              (36, 36, 3), (34, 40, 2), (40, 34, 17), (32, 37, 2), (50, 33, 1)])
def test_so3_real_transforms_on_other_grids(hip, b_grid, b_spec, nz):
    """Real signals on grids other than 64^3: the folded plane transform takes several planes per workgroup
    (ragged last workgroup included) or one large plane; analysis truncates, synthesis zero-extends."""
    print(f"so3 real transforms b_grid={b_grid} b_spec={b_spec} nz={nz}", flush=True)
    x = rnd((nz, 2 * b_grid, 2 * b_grid, 2 * b_grid), 70)
    for for_grad in (False, True):
        close(PSO3.so3_rfft(x.cuda(), for_grad, b_spec), O.so3_rfft(x.double(), for_grad, b_spec), "so3_rfft")
        s = rnd((O.nspec_so3(b_spec), nz, 2), 71)
        close(PSO3.so3_rifft(s.cuda(), for_grad, b_grid), O.so3_rifft(s.double(), for_grad, b_grid), "so3_rifft")


@pytest.mark.parametrize("b_spec,b_grid", [(5, 7), (7, 22), (12, 32), (3, 2)])
def test_so3_synthesis_with_bias(hip, b_spec, b_grid):
    """The bias argument of so3_rifft / SO3_ifft_real (the "+ self.bias" of s2_conv.py:53 and so3_conv.py:56 inside the
    transform): same values as the separate addition, and the gradients autograd gives for that addition."""
    print(f"so3 synthesis with bias b_spec={b_spec} b_grid={b_grid}", flush=True)
    from s2cnn_amd.soft.so3_fft import SO3_ifft_real
    s = rnd((O.nspec_so3(b_spec), 3, 4, 2), 80).cuda().requires_grad_()
    bias = rnd((1, 4, 1, 1, 1), 81).cuda().requires_grad_()
    w = rnd((3, 4, 2 * b_grid, 2 * b_grid, 2 * b_grid), 82).cuda()
    out = SO3_ifft_real.apply(s, b_grid, bias)
    (out * w).sum().backward()
    got = (out.detach(), s.grad.clone(), bias.grad.clone())
    s.grad = bias.grad = None
    ref = SO3_ifft_real.apply(s, b_grid) + bias
    (ref * w).sum().backward()
    for name, a, c in zip(("out", "grad spectrum", "grad bias"), got, (ref.detach(), s.grad, bias.grad)):
        close(a, c.double().cpu(), name)


def test_network_forward_replays_from_a_hip_graph(hip):
    """Nothing on the path allocates through HIP, synchronises or clears memory with a memset node, so a forward pass
    captures into a HIP graph (the launch-bound small configurations gain from it).  Each replay, with eager work and
    synchronisations between the replays, must reproduce the eager result bit for bit."""
    pi = 3.141592653589793
    g1 = s2cnn_amd.s2_near_identity_grid(max_beta=pi / 8, n_alpha=8, n_beta=3)
    g2 = s2cnn_amd.so3_near_identity_grid(max_beta=pi / 8, max_gamma=2 * pi, n_alpha=8, n_beta=3, n_gamma=8)
    torch.manual_seed(3)
    c1 = s2cnn_amd.S2Convolution(1, 20, 30, 10, g1).cuda()
    c2 = s2cnn_amd.SO3Convolution(20, 40, 10, 6, g2).cuda()

    def net(x):
        return s2cnn_amd.so3_integrate(torch.relu(c2(torch.relu(c1(x)))))

    gen = torch.Generator().manual_seed(4)
    xs = [torch.rand(8, 1, 60, 60, generator=gen).cuda() for _ in range(3)]
    static_x = xs[0].clone()
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                net(static_x)                      # tables, workspaces and allocator pools exist before the capture
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_y = net(static_x)
        for i, x in enumerate(xs):
            static_x.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            want = net(x)                          # eager work between the replays
            torch.cuda.synchronize()
            assert torch.equal(static_y, want), f"replay {i} differs from the eager pass"


def test_training_step_replays_from_a_hip_graph(hip):
    """Forward, backward and an SGD update of the MNIST-shaped network (layers with the activation inside) captured
    into one HIP graph: after the same inputs, every replayed step must leave the weights of an eager twin, bit for bit,
    with eager work and synchronisations between the replays."""
    pi = 3.141592653589793
    g1 = s2cnn_amd.s2_near_identity_grid(max_beta=pi / 8, n_alpha=8, n_beta=3)
    g2 = s2cnn_amd.so3_near_identity_grid(max_beta=pi / 8, max_gamma=2 * pi, n_alpha=8, n_beta=3, n_gamma=8)

    def build():
        torch.manual_seed(5)
        c1 = s2cnn_amd.S2Convolution(1, 20, 30, 10, g1, activation="relu").cuda()
        c2 = s2cnn_amd.SO3Convolution(20, 40, 10, 6, g2, activation="relu").cuda()
        head = torch.nn.Linear(40, 10).cuda()
        params = [*c1.parameters(), *c2.parameters(), *head.parameters()]
        return (lambda x: head(s2cnn_amd.so3_integrate(c2(c1(x))))), params, torch.optim.SGD(params, lr=0.05)

    net_g, params_g, opt_g = build()
    net_e, params_e, opt_e = build()
    gen = torch.Generator().manual_seed(6)
    batches = [(torch.rand(8, 1, 60, 60, generator=gen).cuda(), torch.randint(0, 10, (8,), generator=gen).cuda()) for _ in range(3)]
    static_x, static_t = batches[0][0].clone(), batches[0][1].clone()
    start = [q.detach().clone() for q in params_g]

    def step(net, opt, x, t):
        opt.zero_grad(set_to_none=True)
        loss = torch.nn.functional.cross_entropy(net(x), t)
        loss.backward()
        opt.step()
        return loss

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step(net_g, opt_g, static_x, static_t)      # tables, workspaces and allocator pools exist before the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    with torch.no_grad():
        for q, q0 in zip(params_g, start):
            q.copy_(q0)                                 # back to the weights the eager twin starts from
    graph = torch.cuda.CUDAGraph()
    opt_g.zero_grad(set_to_none=True)
    with torch.cuda.graph(graph):
        static_loss = step(net_g, opt_g, static_x, static_t)
    with torch.no_grad():
        for q, q0 in zip(params_g, start):
            q.copy_(q0)                                 # the capture itself ran nothing, but keep the state explicit
    for i, (x, t) in enumerate(batches):
        static_x.copy_(x)
        static_t.copy_(t)
        graph.replay()
        torch.cuda.synchronize()
        loss_e = step(net_e, opt_e, x, t)               # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(static_loss, loss_e), f"replay {i}: loss differs"
        for k, (a, b) in enumerate(zip(params_g, params_e)):
            assert torch.equal(a, b), f"replay {i}: parameter {k} differs from the eager step"


@pytest.mark.parametrize("b,nz", [(48, 2), (64, 3), (33, 17)])
def test_so3_projector_on_a_large_grid(hip, b, nz):
    """b = 48 (96^3 grid, 147 440 coefficients), 64 (every part of the Wigner stage full: 64 frequencies, 64 degrees,
    128 betas) and 33 (parts of one column / one degree): planes with more register blocks than 256 threads hold and
    degrees beyond one part of the tiled Wigner kernels.  No oracle at these sizes: synthesis followed by analysis is
    the identity on spectra of real signals, analysis followed by synthesis a projector, and truncation commutes with both."""
    g = torch.Generator().manual_seed(90)
    x = torch.randn(nz, 2 * b, 2 * b, 2 * b, generator=g).cuda()
    s = PSO3.so3_rfft(x)                                   # spectrum of a real signal
    y = PSO3.so3_rifft(s)                                  # its band-limited projection
    s2 = PSO3.so3_rfft(y)
    rel = ((s2 - s).norm() / s.norm()).item()
    print(f"analysis(synthesis(s)) - s: rel L2 {rel:.2e}", flush=True)
    assert rel < TOL
    y2 = PSO3.so3_rifft(s2)
    rel = ((y2 - y).norm() / y.norm()).item()
    print(f"projector twice: rel L2 {rel:.2e}", flush=True)
    assert rel < TOL
    lo = PSO3.so3_rfft(y, b_out=12)                        # truncation: the first nspec(12) coefficients, nothing else
    n12 = O.nspec_so3(12)
    rel = ((lo - s[:n12]).norm() / s[:n12].norm()).item()
    print(f"truncated analysis: rel L2 {rel:.2e}", flush=True)
    assert rel < TOL
    up = PSO3.so3_rifft(lo, b_out=b)                       # zero-extension on the way back
    sz = torch.zeros_like(s)
    sz[:n12] = lo
    rel = ((up - PSO3.so3_rifft(sz)).norm() / up.norm()).item()
    print(f"zero-extended synthesis: rel L2 {rel:.2e}", flush=True)
    assert rel < TOL


@pytest.mark.parametrize("factorised", [True, False])
def test_so3_rft_kernel_spectrum(hip, factorised, monkeypatch):
    """so3_rft (so3_ft.py:4-25) through the factorised real-basis transform and through the dense product:
    values and the gradient with respect to the kernel, against the oracle."""
    monkeypatch.setattr(s2cnn_amd.so3_rft, "factorised", factorised)
    b = 7
    grid = s2cnn_amd.so3_near_identity_grid(n_alpha=6, n_beta=2, n_gamma=4)
    k = rnd((4, 3, len(grid)), 95)
    w = rnd((O.nspec_so3(b), 4, 3, 2), 96)
    kg = k.cuda().requires_grad_()
    y = s2cnn_amd.so3_rft(kg, b, grid)
    (y * w.cuda()).sum().backward()
    ko = k.double().requires_grad_()
    yo = O.so3_rft(ko, b, grid)
    (yo * w.double()).sum().backward()
    close(y, yo, "so3_rft")
    close(kg.grad, ko.grad, "so3_rft grad")


@pytest.mark.parametrize("shape", [(30, 50), (4, 3), (32, 33 * 4), (1, 1024), (2, 514)])
def test_so3_rft_complex_expansion_equals_dense_product(hip, shape, monkeypatch):
    """so3_rft of a real kernel (so3_ft.py:8-24): the factorised transform writes its expansion as complex pairs, a
    thread's columns in two pairs half a tile (512 columns) apart; column counts that end inside either half of a tile,
    against the dense product with the matrix of Wigner-D samples, values and gradient."""
    b = 6
    grid = s2cnn_amd.so3_near_identity_grid(n_alpha=6, n_beta=3, n_gamma=4)
    k = rnd((*shape, len(grid)), 97).cuda()
    w = rnd((O.nspec_so3(b), *shape, 2), 98).cuda()
    out = {}
    for factorised in (True, False):
        monkeypatch.setattr(s2cnn_amd.so3_rft, "factorised", factorised)
        kg = k.clone().requires_grad_()
        y = s2cnn_amd.so3_rft(kg, b, grid)
        (y * w).sum().backward()
        out[factorised] = (y.detach(), kg.grad)
    close(out[True][0], out[False][0].cpu(), f"so3_rft {shape}")
    close(out[True][1], out[False][1].cpu(), f"so3_rft grad {shape}")


@pytest.mark.parametrize("b,nz", [(32, 8200), (22, 25300)])
def test_so3_transforms_beyond_32_bit_offsets(hip, b, nz):
    """Batches whose tensors pass 2^31 elements (and 2^33 bytes): the last volumes must get the bits they get in a batch of
    their own, for the complex-pair and the real-basis spectra (per-volume kernels of the 64^3 and 44^3 grids).  The small
    batches are 200 volumes: below 129 the analysis gives a volume to several workgroups, which adds the
    beta sum up in another order (the same numbers to rounding, not to the bit)."""
    if torch.cuda.mem_get_info()[0] < 60 * 2 ** 30:
        pytest.skip("needs 60 GiB of free device memory")
    n = 2 * b
    assert nz * n ** 3 > 2 ** 31
    print(f"large batch b={b} nz={nz}", flush=True)
    g = torch.Generator(device="cuda").manual_seed(b)
    x = torch.randn(nz, n, n, n, device="cuda", generator=g)
    last = x[-200:].clone()
    s = PSO3.so3_rfft(x)
    assert torch.equal(s[:, -200:], PSO3.so3_rfft(last))
    assert torch.equal(s[:, 5:205], PSO3.so3_rfft(x[5:205].clone()))
    close(s[:, -3:], PSO3.so3_rfft(x[-3:].clone()).double().cpu(), "three volumes alone")
    r = PSO3.so3_rfft_real_basis(x)
    assert torch.equal(r[:, -200:], PSO3.so3_rfft_real_basis(last))
    del x, last
    y = PSO3.so3_rifft(s)
    assert torch.equal(y[-3:], PSO3.so3_rifft(s[:, -3:].contiguous()))
    assert torch.equal(y[5:8], PSO3.so3_rifft(s[:, 5:8].contiguous()))
    del y, s
    y = PSO3.so3_rifft_real_basis(r)
    assert torch.equal(y[-3:], PSO3.so3_rifft_real_basis(r[:, -3:].contiguous()))
    del y, r
    torch.cuda.empty_cache()


@pytest.mark.parametrize("b,nz", [(16, 2100), (10, 8400), (22, 800), (32, 260)])
def test_so3_streamed_batches_equal_cached_ones(hip, b, nz):
    """Signals of 256 MB or more are loaded and stored with the non-temporal hint (instantiations of their own of the
    per-volume kernels); the hint changes no arithmetic: 200 volumes of such a batch get the bits they get in a batch of
    their own, which takes the plain instantiations, in both directions and with a second tensor in the loads."""
    n = 2 * b
    assert nz * n ** 3 * 4 >= 256 << 20 and 200 * n ** 3 * 4 < 256 << 20
    print(f"streamed batch b={b} nz={nz}", flush=True)
    g = torch.Generator(device="cuda").manual_seed(7 * b)
    x = torch.randn(nz, n, n, n, device="cuda", generator=g)
    m = torch.randn(nz, n, n, n, device="cuda", generator=g)
    for lo in (0, nz - 200):
        sl = slice(lo, lo + 200)
        r = PSO3.so3_rfft_real_basis(x)
        assert torch.equal(r[:, sl], PSO3.so3_rfft_real_basis(x[sl].contiguous()))
        rm = PSO3.so3_rfft_real_basis(x, mask=m)
        assert torch.equal(rm[:, sl], PSO3.so3_rfft_real_basis(x[sl].contiguous(), mask=m[sl].contiguous()))
        y = PSO3.so3_rifft_real_basis(r)
        assert torch.equal(y[sl], PSO3.so3_rifft_real_basis(r[:, sl].contiguous()))
        del r, rm, y


def test_s2_transforms_and_integral_beyond_32_bit_offsets(hip):
    """The same property for the S^2 transforms ([33 000, 256, 256] -> b 32 and back) and for so3_integrate."""
    if torch.cuda.mem_get_info()[0] < 60 * 2 ** 30:
        pytest.skip("needs 60 GiB of free device memory")
    g = torch.Generator(device="cuda").manual_seed(128)
    x = torch.randn(33000, 256, 256, device="cuda", generator=g)
    assert x.numel() > 2 ** 31
    s = PS2.s2_rfft(x, b_out=32)
    assert torch.equal(s[:, -3:], PS2.s2_rfft(x[-3:].clone(), b_out=32))
    del x
    y = PS2.s2_rifft(s, for_grad=True, b_out=128)
    assert y.numel() > 2 ** 31
    assert torch.equal(y[-3:], PS2.s2_rifft(s[:, -3:].contiguous(), for_grad=True, b_out=128))
    del y, s
    x = torch.randn(8200, 64, 64, 64, device="cuda", generator=g)
    v = s2cnn_amd.so3_integrate(x)
    assert torch.equal(v[-3:], s2cnn_amd.so3_integrate(x[-3:].clone()))
    del x
    torch.cuda.empty_cache()


def test_so3_round_trip_at_the_benchmark_size(hip):
    """[256, 64, 64, 64] (the transform benchmark): every volume of the batch gets the bits it gets in another batch
    that is split the same way (the result of a volume does not depend on the workgroup that takes it; 128 volumes
    or fewer are split along beta over several workgroups, whose partial sums are added in another order, so a volume
    alone agrees to rounding only), and analysis o synthesis is the identity on spectra."""
    g = torch.Generator(device="cuda").manual_seed(33)
    x = torch.randn(256, 64, 64, 64, device="cuda", generator=g)
    s = PSO3.so3_rfft(x)
    y = PSO3.so3_rifft(s)
    for i in (0, 126):
        assert torch.equal(PSO3.so3_rfft(x[i:i + 130].contiguous()), s[:, i:i + 130]), i
        assert torch.equal(PSO3.so3_rifft(s[:, i:i + 130].contiguous()), y[i:i + 130]), i
    for i in (0, 7, 100, 255):
        close(PSO3.so3_rfft(x[i:i + 1].contiguous())[:, 0], s[:, i].cpu(), f"rfft of volume {i} alone")
        assert torch.equal(PSO3.so3_rifft(s[:, i:i + 1].contiguous())[0], y[i]), i      # the synthesis adds nothing across workgroups
    s2 = PSO3.so3_rfft(y)
    rel = ((s2 - s).norm() / s.norm()).item()
    print(f"analysis(synthesis(s)) - s: rel L2 {rel:.2e}", flush=True)
    assert rel < TOL
