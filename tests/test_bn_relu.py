"""Batch normalisation + ReLU between two layers evaluated inside the layers' transforms (s2cnn_amd/soft/bn_relu.py)
against the modules they replace: nn.BatchNorm3d and nn.ReLU of torch between this package's layers, as the reference's
shape networks are written (examples/shrec17/model.py:17-38).  The pieces through the C ABI first: the two sums per
volume, the analysis that applies max(a y + b, 0) in its loads and the one that forms the gradient of the pair in its
loads, each against the same arithmetic as torch tensor expressions followed by the plain analysis."""
import pytest
import torch
from torch import nn

import s2cnn_amd
from s2cnn_amd import harness
from s2cnn_amd.soft import bn_relu
from s2cnn_amd.soft import so3_fft as P

pytestmark = pytest.mark.gpu

PAIRS = [(32, 32), (32, 22), (22, 22), (22, 7), (22, 18), (16, 16), (16, 10), (12, 12), (10, 10), (10, 6), (6, 6), (7, 7), (3, 3)]


def _rel(got, want):
    return (got - want).abs().max().item() / max(want.abs().max().item(), 1e-30)


def _sum_and_squared_deviations(v):
    """[parts, samples] float64 -> [parts, 2]: (sum v, sum (v - mean of the part)^2), what the library's sums of a
    normalisation's input are."""
    return torch.stack([v.sum(-1), ((v - v.mean(-1, keepdim=True)) ** 2).sum(-1)], -1)


def test_volume_moments(hip):
    g = torch.Generator().manual_seed(1)
    for n2, nvol in ((64, 6), (44, 4), (14, 9), (6, 5)):
        x = (torch.randn(nvol, n2, n2, n2, generator=g) + 0.5).cuda()
        got = bn_relu._moments("s2cnn_volume_moments", n2 ** 3, x).double()
        want = _sum_and_squared_deviations(x.double().view(nvol, -1))
        assert _rel(got, want) < 2e-6, n2
        # the sums of the backward pass: sum g m and sum g m y with m = (a y + b > 0), feature = volume % 3
        y = torch.randn(nvol // 3 * 3, n2, n2, n2, generator=g).cuda()
        gr = torch.randn(y.shape, generator=g).cuda()
        ab = torch.tensor([[0.7, -1.3, 2.0], [0.1, 0.4, -0.5]]).cuda()
        a = ab[0].repeat(y.size(0) // 3).view(-1, 1, 1, 1)
        b = ab[1].repeat(y.size(0) // 3).view(-1, 1, 1, 1)
        m = (a * y + b > 0)
        got = bn_relu._moments("s2cnn_bn_relu_grad_moments", n2 ** 3, gr, y, ab, 3).double()
        gm = (gr * m).double()
        want = torch.stack([gm.sum((1, 2, 3)), (gm * y.double()).sum((1, 2, 3))], 1)
        assert (got - want).abs().max().item() < 2e-5 * want.abs().max().item(), n2    # a sample at the threshold may fall either way


@pytest.mark.parametrize("b_in,b_out", [(32, 32), (22, 32), (26, 32), (16, 16), (10, 16), (20, 16), (22, 22), (7, 22), (18, 22), (10, 10), (6, 10), (12, 12), (6, 6)])
def test_sums_formed_by_the_synthesis(hip, b_in, b_out):
    """(sum y, sum (y - mean)^2) per volume (64^3, 44^3 and 32^3 grids) or per plane (two-stage path) written by the synthesis that
    produces y, against float64 sums of that y; y itself bit for bit the output of the synthesis without the sums."""
    parts = P.synthesis_moment_parts(b_in, b_out)
    assert parts == (1 if b_out in (32, 22, 16, 10) else 2 * b_out)
    g = torch.Generator().manual_seed(b_in * 100 + b_out)
    nspec = b_in * (4 * b_in ** 2 - 1) // 3
    r = torch.randn(nspec, 2, 3, generator=g).cuda()
    r[0] += 3.0                                                  # a mean well away from zero
    bias = torch.tensor([0.5, -1.0, 2.0]).cuda()
    mom = torch.full((6 * parts, 2), float("nan")).cuda()
    y = P.so3_rifft_real_basis(r, b_out=b_out, bias=bias, moments=(mom, None, None))
    assert torch.equal(y, P.so3_rifft_real_basis(r, b_out=b_out, bias=bias))
    yd = y.double().view(6 * parts, -1)
    want = _sum_and_squared_deviations(yd)
    # the mean each part's sum stands for, against the spread of the part (what a normalisation divides by), and the spread itself
    mean_err = ((mom.double()[:, 0] - want[:, 0]) / yd.size(1)).abs() / yd.std(-1)
    assert mean_err.max().item() < 1e-6 and _rel(mom.double()[:, 1], want[:, 1]) < 2e-5


@pytest.mark.parametrize("b_in,b_out", [(16, 16), (9, 16), (22, 22), (10, 10), (12, 12)])
def test_sums_formed_by_the_synthesis_of_a_complex_spectrum(hip, b_in, b_out):
    """The same sums from s2cnn_so3_synthesis_real_moments (complex spectrum): per plane on the two-stage path, per volume
    from the per-volume kernels of the 32^3 grid; both kinds of sums, against float64 sums of the output."""
    from s2cnn_amd.soft import so3_fft as F
    parts = F._hip.lib().s2cnn_so3_synthesis_moment_parts(b_in, b_out)
    assert parts == (1 if b_out in (22, 16, 10) else 2 * b_out)
    gen = torch.Generator().manual_seed(b_in * 100 + b_out + 3)
    nspec = b_in * (4 * b_in ** 2 - 1) // 3
    xh = torch.randn(nspec, 2, 3, 2, generator=gen).cuda()
    bias = torch.tensor([0.5, -1.0, 2.0]).cuda()
    mom = torch.full((6 * parts, 2), float("nan")).cuda()
    y = F.so3_rifft(xh, b_out=b_out, bias=bias, moments=(mom, None, None))
    assert torch.equal(y, F.so3_rifft(xh, b_out=b_out, bias=bias))
    yd = y.double().view(6 * parts, -1)
    want = _sum_and_squared_deviations(yd)
    mean_err = ((mom.double()[:, 0] - want[:, 0]) / yd.size(1)).abs() / yd.std(-1)
    assert mean_err.max().item() < 1e-6 and _rel(mom.double()[:, 1], want[:, 1]) < 2e-5
    w = torch.randn(2, 3, 2 * b_out, 2 * b_out, 2 * b_out, generator=gen).cuda()
    ab = torch.tensor([[0.7, 1.3, 2.0], [0.1, 0.4, -0.5]]).cuda()
    mom = torch.full((6 * parts, 2), float("nan")).cuda()
    g = F.so3_rifft(xh, for_grad=True, b_out=b_out, moments=(mom, w, ab))
    assert torch.equal(g, F.so3_rifft(xh, for_grad=True, b_out=b_out))
    m = ab[0].view(1, 3, 1, 1, 1) * w + ab[1].view(1, 3, 1, 1, 1) > 0
    gm = (g * m).double().view(6, parts, -1)
    want = torch.stack([gm.sum(-1), (gm * w.double().view(6, parts, -1)).sum(-1)], -1).view(-1, 2)
    assert (mom.double() - want).abs().max().item() < 2e-5 * want.abs().max().item()


@pytest.mark.parametrize("ratio", [100.0, 1000.0])
@pytest.mark.parametrize("b_in,b_out", [(32, 32), (16, 16), (22, 22), (10, 10), (12, 12), (6, 6)])
def test_statistics_of_a_signal_with_a_large_mean(hip, b_in, b_out, ratio):
    """A mean `ratio` times the standard deviation: the batch variance that the normalisation forms from the library's sums
    (the synthesis's own, and s2cnn_volume_moments) must keep its digits, as nn.BatchNorm3d's does; E[y^2] - mean^2 from
    float32 sums would be off by 10 % at a ratio of 1000."""
    g = torch.Generator().manual_seed(int(ratio) + b_in)
    nspec = b_in * (4 * b_in ** 2 - 1) // 3
    nb, nf = 2, 3
    r = torch.randn(nspec, nb, nf, generator=g).cuda()
    y0 = P.so3_rifft_real_basis(r, b_out=b_out)
    bias = (ratio * y0.std()).item() * torch.tensor([1.0, -1.0, 0.5]).cuda()      # the layer's bias carries the mean
    parts = P.synthesis_moment_parts(b_in, b_out)
    nvox = (2 * b_out) ** 3
    mom = torch.full((nb * nf * parts, 2), float("nan")).cuda()
    y = P.so3_rifft_real_basis(r, b_out=b_out, bias=bias, moments=(mom, None, None))
    want_var = y.double().transpose(0, 1).reshape(nf, -1).var(1, unbiased=False)
    for sums, nparts in ((mom, parts), (bn_relu._moments("s2cnn_volume_moments", nvox, y), 1)):
        ab, stats = torch.empty(2, nf).cuda(), torch.empty(4, nf).cuda()
        from s2cnn_amd import _hip
        _hip.call("s2cnn_bn_forward_from_moments", _hip.ptr(sums), nb, nf, nparts, float(nb * nvox), None, None, None, None, 1e-5, 0.1, 1,
                  _hip.ptr(ab), _hip.ptr(stats), _hip.stream_ptr())
        got_var = stats[1].double()
        assert _rel(got_var, want_var) < 1e-3, (nparts, got_var, want_var)


@pytest.mark.parametrize("b_in,b_out", [(22, 32), (26, 32), (28, 32), (16, 16), (10, 16), (22, 22), (7, 22), (18, 22), (10, 10), (6, 10), (12, 12), (6, 6)])
def test_gradient_sums_formed_by_the_synthesis(hip, b_in, b_out):
    """(sum g m, sum g m y), m = (a y + b > 0), with g the output of the synthesis and y a second tensor, per volume or per
    plane, against float64 sums; none on the 64^3 grid for a spectrum of all 32 degrees."""
    assert P.synthesis_moment_parts(32, 32, grad=True) == 0
    parts = P.synthesis_moment_parts(b_in, b_out, grad=True)
    assert parts == (1 if b_out in (32, 22, 16, 10) else 2 * b_out)
    gen = torch.Generator().manual_seed(b_in * 100 + b_out + 7)
    nspec = b_in * (4 * b_in ** 2 - 1) // 3
    r = torch.randn(nspec, 2, 3, generator=gen).cuda()
    y = torch.randn(2, 3, 2 * b_out, 2 * b_out, 2 * b_out, generator=gen).cuda()
    ab = torch.tensor([[0.7, 1.3, 2.0], [0.1, 0.4, -0.5]]).cuda()
    mom = torch.full((6 * parts, 2), float("nan")).cuda()
    g = P.so3_rifft_real_basis(r, for_grad=True, b_out=b_out, moments=(mom, y, ab))
    assert torch.equal(g, P.so3_rifft_real_basis(r, for_grad=True, b_out=b_out))
    m = ab[0].view(1, 3, 1, 1, 1) * y + ab[1].view(1, 3, 1, 1, 1) > 0
    gm = (g * m).double().view(6, parts, -1)
    want = torch.stack([gm.sum(-1), (gm * y.double().view(6, parts, -1)).sum(-1)], -1).view(-1, 2)
    assert (mom.double() - want).abs().max().item() < 2e-5 * want.abs().max().item()      # a sample at the threshold may fall either way


@pytest.mark.parametrize("b_in,b_out", PAIRS)
def test_analysis_with_the_normalisation_in_its_loads(hip, b_in, b_out):
    """max(a y + b, 0) and a (a y + b > 0 ? g : 0) + p + q y formed by the loads of the analysis against the same
    functions as tensor expressions followed by the plain analysis; complex and real-basis spectra, both tables."""
    assert P.analysis_prologue_available(b_in, b_out)
    print(f"normalisation in the loads b_in={b_in} b_out={b_out}", flush=True)
    nb, nf = 2, 3
    g = torch.Generator().manual_seed(100 * b_in + b_out)
    y = torch.randn(nb, nf, 2 * b_in, 2 * b_in, 2 * b_in, generator=g).cuda()
    gr = torch.randn(y.shape, generator=g).cuda()
    par = torch.tensor([[0.7, -1.3, 2.0], [0.1, 0.4, -0.5], [0.02, -0.01, 0.03], [-0.05, 0.04, 0.01]]).cuda()
    a, b, p, q = (par[i].view(1, nf, 1, 1, 1) for i in range(4))
    u = torch.relu(a * y + b)
    v = a * gr * (a * y + b > 0) + p + q * y
    for for_grad in (False, True):
        for ana in (P.so3_rfft, P.so3_rfft_real_basis):
            want = ana(u, for_grad=for_grad, b_out=b_out)
            got = ana(y, for_grad=for_grad, b_out=b_out, mask=P.LoadAffineReLU(par[:2].contiguous()))
            assert _rel(got, want) < 2e-5, ("affine relu", for_grad, ana.__name__, _rel(got, want))
            want = ana(v, for_grad=for_grad, b_out=b_out)
            got = ana(gr, for_grad=for_grad, b_out=b_out, mask=P.LoadBNReLUGrad(y, par))
            assert _rel(got, want) < 2e-5, ("bn relu grad", for_grad, ana.__name__, _rel(got, want))


class _Norm64(nn.Module):
    """nn.BatchNorm3d evaluated in float64 on float32 activations: the checker's normalisation (the float32 kernels of
    the library behind torch's module lose digits of the statistics at 10^6 samples per feature)."""

    def __init__(self, n, **kwargs):
        super().__init__()
        self.bn = nn.BatchNorm3d(n, dtype=torch.float64, **kwargs)

    def forward(self, x):  # pylint: disable=W0221
        return self.bn(x.double()).float()


def _as_checker(seq):
    """The same sequence with every BatchNorm3d replaced by its float64 twin (same parameters and buffers)."""
    mods = []
    for m in seq:
        if isinstance(m, nn.BatchNorm3d):
            twin = _Norm64(m.num_features, affine=m.affine, momentum=m.momentum, eps=m.eps, track_running_stats=m.track_running_stats).cuda()
            twin.bn.load_state_dict({k: (v.double() if v.is_floating_point() else v) for k, v in m.state_dict().items()})
            mods.append(twin)
        else:
            mods.append(m)
    return nn.Sequential(*mods)


def _sequence(sizes, feats, seed, **bn_kwargs):
    """S2Conv, then (BatchNorm3d, ReLU, SO3Conv) per further bandwidth, then BatchNorm3d, ReLU: the reference's pattern."""
    torch.manual_seed(seed)
    mods = [s2cnn_amd.S2Convolution(feats[0], feats[1], sizes[0], sizes[1], s2cnn_amd.s2_near_identity_grid())]
    for i in range(1, len(sizes) - 1):
        mods += [nn.BatchNorm3d(feats[i], **bn_kwargs), nn.ReLU(),
                 s2cnn_amd.SO3Convolution(feats[i], feats[i + 1], sizes[i], sizes[i + 1], s2cnn_amd.so3_near_identity_grid())]
    mods += [nn.BatchNorm3d(feats[-1], **bn_kwargs), nn.ReLU()]
    seq = nn.Sequential(*mods)
    with torch.no_grad():
        for m in seq:
            if isinstance(m, nn.BatchNorm3d) and m.affine:
                m.weight.uniform_(0.5, 1.5)
                m.bias.normal_(0, 0.3)
            elif hasattr(m, "kernel"):
                m.bias.normal_(0, 0.3)
    return seq


@pytest.mark.parametrize("head", [None, "integrate", "max"])       # what follows the sequence, with the last pair inside it
@pytest.mark.parametrize("sizes,feats,bn_kwargs", [
    ((12, 8, 6, 4), (2, 4, 5, 3), {}),                                       # small grids: folded plane kernels
    ((40, 32, 22, 7), (2, 3, 4, 3), {}),                                     # 64^3 and 44^3: per-volume kernels, truncated spectra
    ((12, 8, 6, 4), (2, 4, 5, 3), {"affine": False, "momentum": None}),      # no weights, cumulative running averages
    ((10, 8, 6), (2, 4, 5), {"track_running_stats": False})])                # batch statistics in evaluation mode as well
def test_sequence_with_fused_normalisation(hip, sizes, feats, bn_kwargs, head):
    import copy
    fus = _sequence(sizes, feats, 5, **bn_kwargs).cuda()
    ref = _as_checker(copy.deepcopy(fus))
    # One sample of 10^6 whose normalised value lies within rounding of the threshold of the ReLU may pass in one
    # evaluation and not in the other, which moves a spectral gradient by 10^-3 of its size: the comparison is made on an
    # input for which the checker sees no such sample (three evaluations: two training steps and one in evaluation mode).
    closest = []
    hooks = [m.register_forward_hook(lambda _m, _i, out: closest.append(out.abs().min().item())) for m in ref if isinstance(m, _Norm64)]
    for seed in range(6, 36):
        x = torch.randn(3, feats[0], 2 * sizes[0], 2 * sizes[0], generator=torch.Generator().manual_seed(seed)).cuda()
        probe = copy.deepcopy(ref)
        phooks = [m.register_forward_hook(lambda _m, _i, out: closest.append(out.abs().min().item())) for m in probe if isinstance(m, _Norm64)]
        del closest[:]
        with torch.no_grad():
            probe.train(); probe(x); probe(x); probe.eval(); probe(x)
        if min(closest) > 5e-7:                 # the two evaluations of a normalised value differ by 1.5e-7 at most
            break
    else:
        pytest.skip("no input without a sample at the threshold among thirty seeds")
    for h in hooks + phooks:
        h.remove()
    print(f"input seed {seed}: closest normalised value to the threshold {min(closest):.1e}", flush=True)
    for mode in ("train", "train", "eval"):                 # two training steps (running averages move twice), then evaluation
        ref.train(mode == "train")
        fus.train(mode == "train")
        xa, xb = x.clone().requires_grad_(), x.clone().requires_grad_()
        if head == "integrate":
            ya, yb = s2cnn_amd.so3_integrate(ref(xa)), bn_relu.run_sequence(fus, xb, head=head)
        elif head == "max":
            out = ref(xa)
            ya, yb = out.view(out.size(0), out.size(1), -1).max(-1)[0], bn_relu.run_sequence(fus, xb, head=head)
        else:
            ya, yb = ref(xa), bn_relu.run_sequence(fus, xb)
        assert _rel(yb, ya) < 1e-4, (mode, _rel(yb, ya))
        w = torch.randn(ya.shape, generator=torch.Generator().manual_seed(7)).cuda()
        for net in (ref, fus):
            net.zero_grad(set_to_none=True)
        (ya * w).sum().backward()
        (yb * w).sum().backward()
        assert _rel(xb.grad, xa.grad) < 2e-4, (mode, "input", _rel(xb.grad, xa.grad))
        # a bias in front of a normalisation with batch statistics has gradient zero (rounding noise on either side):
        # differences are measured against the largest gradient of the network where a parameter's own is smaller
        scale = max(q.grad.abs().max().item() for q in ref.parameters())
        for (name, pa), (_, pb) in zip(ref.named_parameters(), fus.named_parameters()):
            err = (pb.grad - pa.grad.float()).abs().max().item() / max(pa.grad.abs().max().item(), 0.1 * scale)
            assert err < 2e-4, (mode, name, err)
        for (name, ba), (_, bb) in zip(ref.named_buffers(), fus.named_buffers()):
            assert _rel(bb.double(), ba.double()) < 1e-5, (mode, name)
        print(f"{sizes} {mode}: output {_rel(yb, ya):.1e}, input gradient {_rel(xb.grad, xa.grad):.1e}", flush=True)


def test_shape_network_with_fused_normalisation(hip):
    """The SHREC17 network of the harness with the normalisations inside the transforms: the same losses over training
    steps as the plain module sequence, from the same initial weights."""
    torch.manual_seed(0)
    plain = harness.Shrec17Model(55)
    torch.manual_seed(0)
    fused = harness.Shrec17Model(55, fused_norm=True)
    _, la, _ = harness.train_steps("shrec17", batch=4, steps=4, warmup=0, lr=0.02, model=plain)
    _, lb, _ = harness.train_steps("shrec17", batch=4, steps=4, warmup=0, lr=0.02, model=fused)
    print("plain", ["%.5f" % l for l in la], "fused", ["%.5f" % l for l in lb], flush=True)
    assert max(abs(a - b) for a, b in zip(la, lb)) < 2e-4 * abs(la[0])
