"""The reference's example networks against the float64 oracle at their own shapes and grids.

The SHREC17 models of the reference put ONE ring of 2 b_in points on the equator under every layer
(examples/shrec17/model.py:17-31, model_original.py:17-31): `s2_equatorial_grid(max_beta=0, n_alpha=2 b_in, n_beta=1)`
and `so3_equatorial_grid(max_beta=0, max_gamma=0, n_alpha=2 b_in, n_beta=1, n_gamma=1)`, i.e. 64 to 256 points that all
share one beta.  Each layer is run on one sample with output and all gradients compared (the `_conv_case` of the other
parity tests), then the whole Shrec17Model in evaluation mode against the oracle's layers chained with float64 batch
normalisation, and benchmark config 1 (the digit network of examples/mnist/run.py:55-98) at its batch of 32."""
import pytest
import torch
import torch.nn.functional as F

import s2cnn_amd
from oracle import cpu_path as O
from s2cnn_amd import harness

from test_gpu_parity import _conv_case, close

pytestmark = pytest.mark.gpu

# (kind, features in, features out, b_in, b_out) of the layers of examples/shrec17/model.py:12-13 ...
SHREC17_LAYERS = [("s2", 6, 100, 64, 16), ("so3", 100, 100, 16, 10)]
# ... and of examples/shrec17/model_original.py:12-13
SHREC17_ORIGINAL_LAYERS = [("s2", 6, 50, 128, 32), ("so3", 50, 70, 32, 22), ("so3", 70, 350, 22, 7)]


def _ring(kind, b_in):
    if kind == "s2":
        return s2cnn_amd.s2_equatorial_grid(max_beta=0, n_alpha=2 * b_in, n_beta=1)
    return s2cnn_amd.so3_equatorial_grid(max_beta=0, max_gamma=0, n_alpha=2 * b_in, n_beta=1, n_gamma=1)


@pytest.mark.parametrize("kind,f_in,f_out,b_in,b_out", SHREC17_LAYERS + SHREC17_ORIGINAL_LAYERS)
def test_shrec17_layers_on_their_equatorial_rings(hip, kind, f_in, f_out, b_in, b_out):
    """One sample through each layer of the two SHREC17 models at the model's own feature counts, bandwidths and
    equatorial ring: output and the gradients with respect to input, kernel and bias against the float64 oracle."""
    grid = _ring(kind, b_in)
    assert len(grid) == 2 * b_in and len({p[0] for p in grid}) == 1      # one ring: every point has beta = pi / 2
    print(f"{kind} layer {f_in}->{f_out}, b {b_in}->{b_out}, ring of {len(grid)} points", flush=True)
    _conv_case(kind, 1, f_in, f_out, b_in, b_out, grid, 900 + b_in + f_out)


def _oracle_batch_norm_eval(x, bn):
    """nn.BatchNorm3d in evaluation mode, in float64: (x - running_mean) / sqrt(running_var + eps) * weight + bias."""
    shape = (1, -1, 1, 1, 1)
    mean, var = bn.running_mean.double().view(shape), bn.running_var.double().view(shape)
    return (x - mean) / torch.sqrt(var + bn.eps) * bn.weight.detach().double().view(shape) + bn.bias.detach().double().view(shape)


@pytest.mark.parametrize("fused_norm", [False, True])
def test_shrec17_model_forward_against_the_oracle_chain(hip, fused_norm):
    """Shrec17Model (examples/shrec17/model.py:7-48) in evaluation mode, batch 2: log-probabilities against the oracle's
    layers chained with float64 batch normalisation, ReLU, the Haar integral and the linear layer.  The normalisation
    layers get non-trivial running statistics and affine parameters first.  fused_norm: the same modules with the
    normalisations evaluated inside the neighbouring transforms."""
    torch.manual_seed(21)
    model = harness.Shrec17Model(55, fused_norm=fused_norm)
    g = torch.Generator().manual_seed(22)
    for m in model.sequential:
        if isinstance(m, torch.nn.BatchNorm3d):
            with torch.no_grad():
                m.running_mean.copy_(torch.randn(m.num_features, generator=g) * 0.2)
                m.running_var.copy_(torch.rand(m.num_features, generator=g) + 0.5)
                m.weight.copy_(torch.rand(m.num_features, generator=g) + 0.5)
                m.bias.copy_(torch.randn(m.num_features, generator=g) * 0.3)
        elif hasattr(m, "bias"):
            with torch.no_grad():
                m.bias.copy_(torch.randn(m.bias.shape, generator=g) * 0.1)
    model.eval()
    x = torch.rand(2, 6, 128, 128, generator=g)

    y = x.double()
    for m in model.sequential:
        if isinstance(m, s2cnn_amd.S2Convolution):
            y = O.s2_conv(y, m.kernel.detach().double(), m.bias.detach().double(), m.b_in, m.b_out, m.grid)
        elif isinstance(m, s2cnn_amd.SO3Convolution):
            y = O.so3_conv(y, m.kernel.detach().double(), m.bias.detach().double(), m.b_in, m.b_out, m.grid)
        elif isinstance(m, torch.nn.BatchNorm3d):
            y = _oracle_batch_norm_eval(y, m)
        else:
            assert isinstance(m, torch.nn.ReLU)
            y = torch.relu(y)
    feat = O.so3_integrate(y)
    lin = model.out_layer
    want = F.log_softmax(feat @ lin.weight.detach().double().t() + lin.bias.detach().double(), dim=1)

    model = model.cuda()
    with torch.no_grad():
        got = model(x.cuda())
    close(got, want, "Shrec17Model log-probabilities (fused_norm=%s)" % fused_norm)


def test_config1_network_at_batch_32(hip):
    """Benchmark config 1 as it is stated: input [32, 1, 60, 60] with 70 % zeros, S2Conv 1->20 (b 30->10), ReLU, SO3Conv
    20->40 (b 10->6), ReLU, so3_integrate, Linear 40->10, forward only; the network is the harness's S2ConvNet_original
    (examples/mnist/run.py:55-98), checked against the oracle's layers chained in float64."""
    g = torch.Generator().manual_seed(1)
    x = torch.rand(32, 1, 60, 60, generator=g) * (torch.rand(32, 1, 60, 60, generator=g) < 0.3)
    torch.manual_seed(0)
    for fused in (False, True):
        net = harness.S2ConvNet_original(fused_activation=fused)
        c1, c2, lin = net.conv1, net.conv2, net.out_layer
        y = O.s2_conv(x.double(), c1.kernel.detach().double(), c1.bias.detach().double(), 30, 10, c1.grid)
        y = O.so3_conv(torch.relu(y), c2.kernel.detach().double(), c2.bias.detach().double(), 10, 6, c2.grid)
        feat = O.so3_integrate(torch.relu(y))
        want = feat @ lin.weight.detach().double().t() + lin.bias.detach().double()
        net = net.cuda()
        with torch.no_grad():
            got = net(x.cuda())
        close(got, want, "config-1 logits at batch 32 (fused_activation=%s)" % fused)
