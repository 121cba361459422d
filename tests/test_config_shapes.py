"""Parity at the shapes of the benchmark configurations themselves (batch 1 where the CPU oracle is the checker, full size
where a float64 einsum on the device is): the complex block product of config 3, the three layers of config 5 and the
layer of config 4 with all their gradients against the float64 oracle, and the S^2 twin of the identity the reference's
own test script asserts for so3_rft (tests/so3_fft.py:8-24 of the reference)."""
import math

import pytest
import torch

import s2cnn_amd
from oracle import cpu_path as O
from s2cnn_amd.soft import s2_fft as PS2

from test_gpu_parity import _conv_case, close

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("b_in,b_out", [(6, 6), (12, 5), (32, 32)])
def test_s2_rft_equals_s2_fft_on_the_soft_grid(hip, b_in, b_out):
    """S2_fft_real(x, b_out) = (b_in / b_out) s2_rft(w * x, b_out, s2_soft_grid(b_in)): the transform's table carries
    2 b_in w_beta (s2cnn/soft/s2_fft.py:124), the kernel transform's matrix 2 b_out (s2cnn/s2_ft.py:38-45).  Two disjoint
    routes of the product (HIP transform kernels against the dense matrix of s2_ft.py), one of which the oracle pins."""
    g = torch.Generator().manual_seed(40 + b_in)
    x = torch.randn(3, 2 * b_in, 2 * b_in, generator=g)
    w = O.quadrature_weights(b_in, torch.float64)
    fft = PS2.S2_fft_real.apply(x.cuda(), b_out)                                        # [b_out^2, 3, 2]
    xw = (x.double() * w.view(1, -1, 1)).float().reshape(3, -1)
    rft = s2cnn_amd.s2_rft(xw.cuda(), b_out, s2cnn_amd.s2_soft_grid(b_in)) * (b_in / b_out)
    close(rft, fft.double().cpu(), f"s2_rft on the soft grid b {b_in}->{b_out}")
    if b_in <= 12:                                                                      # and both against the oracle's s2_rft
        want = O.s2_rft(xw.double(), b_out, O.s2_soft_grid(b_in)) * (b_in / b_out)
        close(fft, want, "S2_fft_real against the oracle's s2_rft")


def test_so3_mm_complex_at_the_benchmark_size(hip):
    """Benchmark config 3: x [43680, 16, 64, 2], y [43680, 64, 64, 2], entries N(0, 1/64); forward and both gradients of the
    complex product against float64 complex einsums per degree on the same device (so3_mm.py:31-61, :96-122)."""
    nl, B, Fi, Fo = 32, 16, 64, 64
    ns = O.nspec_so3(nl)
    g = torch.Generator(device="cuda").manual_seed(3)
    x = (torch.randn(ns, B, Fi, 2, device="cuda", generator=g) * 0.125).requires_grad_()
    y = (torch.randn(ns, Fi, Fo, 2, device="cuda", generator=g) * 0.125).requires_grad_()
    gz = torch.randn(ns, B, Fo, 2, device="cuda", generator=g)
    z = s2cnn_amd.so3_mm(x, y)
    gx, gy = torch.autograd.grad(z, (x, y), gz)
    worst = 0.0
    pos = 0
    for l in range(nl):
        L = 2 * l + 1
        sl = slice(pos, pos + L * L)
        xa = torch.view_as_complex(x.detach()[sl].double().contiguous()).reshape(L, L, B, Fi)
        ya = torch.view_as_complex(y.detach()[sl].double().contiguous()).reshape(L, L, Fi, Fo)
        ga = torch.view_as_complex(gz[sl].double().contiguous()).reshape(L, L, B, Fo)
        for got, want in ((z.detach()[sl], torch.einsum("mpik,npkj->mnij", xa, ya.conj())),
                          (gx[sl], torch.einsum("mnij,npkj->mpik", ga, ya)),
                          (gy[sl], torch.einsum("mnij,mpik->npkj", ga.conj(), xa))):
            want = torch.view_as_real(want.reshape(L * L, *got.shape[1:-1]))
            worst = max(worst, ((got.double() - want).abs().max() / want.std()).item())
        pos += L * L
    print(f"complex product, worst max|d|/std over degrees and the three products: {worst:.2e}", flush=True)
    assert worst < 1e-4


def _config5_grids():
    g1 = s2cnn_amd.s2_near_identity_grid(max_beta=math.pi / 8 * 30 / 128, n_alpha=8, n_beta=3)
    g2 = s2cnn_amd.so3_near_identity_grid(max_beta=math.pi / 8 * 30 / 32, max_gamma=2 * math.pi, n_alpha=8, n_beta=3, n_gamma=8)
    g3 = s2cnn_amd.so3_near_identity_grid(max_beta=math.pi / 8 * 30 / 22, max_gamma=2 * math.pi, n_alpha=8, n_beta=3, n_gamma=8)
    return g1, g2, g3


@pytest.mark.parametrize("layer", [0, 1, 2])
def test_config5_layers_with_gradients(hip, layer):
    """The three layers of benchmark config 5 at their own shapes, batch 1: output and the gradients with respect to the
    input, the kernel and the bias against the float64 oracle (S2Conv 6->100 b 128->32; SO3Conv 100->100 b 32->22;
    SO3Conv 100->55 b 22->7; grids of examples/shrec17/model_original.py:12-40 scaled by the bandwidth ratio)."""
    grids = _config5_grids()
    case = [("s2", 1, 6, 100, 128, 32), ("so3", 1, 100, 100, 32, 22), ("so3", 1, 100, 55, 22, 7)][layer]
    _conv_case(*case, grids[layer], 500 + 10 * layer)


def test_config4_layer_at_batch_one(hip):
    """The layer of the headline benchmark (64 -> 64 features, b_in = b_out = 32, 192-point near-identity grid) on one
    sample: output and all gradients against the float64 oracle."""
    _conv_case("so3", 1, 64, 64, 32, 32, s2cnn_amd.so3_near_identity_grid(), 600)
