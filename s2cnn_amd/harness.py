"""The reference's example networks on this package's layers, and a training step on synthetic data.

The module and parameter names are those of the reference's scripts, so a state dict saved by either loads into the
other (examples/shrec17/train.py:123 saves `model.state_dict()`, examples/shrec17/test.py:49 loads it):

  S2ConvNet_original   examples/mnist/run.py:55-98          S2Conv 1->20 (b 30->10), ReLU, SO3Conv 20->40 (b 10->6), ReLU,
                                                            so3_integrate, Linear 40->10; near-identity grids
  Shrec17Model         examples/shrec17/model.py:7-48       S2Conv 6->100 (b 64->16), [BatchNorm3d, ReLU, SO3Conv 100->100
                                                            (b 16->10)], BatchNorm3d, ReLU, so3_integrate, Linear, log_softmax;
                                                            equatorial grids with 2 b_in points on one ring
  Shrec17ModelOriginal examples/shrec17/model_original.py   features 6, 50, 70, 350, bandwidths 128, 32, 22, 7, maximum over the
                                                            grid instead of the integral, BatchNorm1d in the output layer

Data sets, loaders and logging of the reference's scripts are not reproduced: `train_steps` feeds a fixed synthetic batch.
"""
import time

import torch
import torch.nn.functional as F
from torch import nn

from .soft.bn_relu import run_sequence
from . import (S2Convolution, SO3Convolution, s2_equatorial_grid, s2_near_identity_grid, so3_equatorial_grid, so3_integrate,
               so3_near_identity_grid)


class S2ConvNet_original(nn.Module):
    """examples/mnist/run.py:55-98.  fused_activation: the two ReLUs inside the layers' last transforms (same function)."""

    def __init__(self, fused_activation=False):
        super().__init__()
        f1, f2, f_output = 20, 40, 10
        b_in, b_l1, b_l2 = 30, 10, 6
        act = "relu" if fused_activation else None
        self.fused_activation = fused_activation
        self.conv1 = S2Convolution(nfeature_in=1, nfeature_out=f1, b_in=b_in, b_out=b_l1, grid=s2_near_identity_grid(), activation=act)
        self.conv2 = SO3Convolution(nfeature_in=f1, nfeature_out=f2, b_in=b_l1, b_out=b_l2, grid=so3_near_identity_grid(), activation=act)
        self.out_layer = nn.Linear(f2, f_output)

    def forward(self, x):  # pylint: disable=W0221
        x = self.conv1(x)
        if not self.fused_activation:
            x = F.relu(x)
        x = self.conv2(x)
        if not self.fused_activation:
            x = F.relu(x)
        x = so3_integrate(x)
        return self.out_layer(x)


def _shrec17_sequence(features, bandwidths):
    """S2 layer, then (BatchNorm3d, ReLU, SO3 layer) per further bandwidth, then BatchNorm3d, ReLU
    (examples/shrec17/model.py:17-38, model_original.py:17-38)."""
    assert len(bandwidths) == len(features) - 1
    sequence = []
    grid = s2_equatorial_grid(max_beta=0, n_alpha=2 * bandwidths[0], n_beta=1)
    sequence.append(S2Convolution(features[0], features[1], bandwidths[0], bandwidths[1], grid))
    for l in range(1, len(features) - 2):
        b_in, b_out = bandwidths[l], bandwidths[l + 1]
        sequence.append(nn.BatchNorm3d(features[l], affine=True))
        sequence.append(nn.ReLU())
        grid = so3_equatorial_grid(max_beta=0, max_gamma=0, n_alpha=2 * b_in, n_beta=1, n_gamma=1)
        sequence.append(SO3Convolution(features[l], features[l + 1], b_in, b_out, grid))
    sequence.append(nn.BatchNorm3d(features[-2], affine=True))
    sequence.append(nn.ReLU())
    return nn.Sequential(*sequence)


class Shrec17Model(nn.Module):
    """examples/shrec17/model.py:7-48.  fused_norm: the BatchNorm3d + ReLU pairs between two layers are evaluated inside
    the layers' transforms (s2cnn_amd/soft/bn_relu.py): same modules, parameters and buffers, same function."""

    def __init__(self, nclasses, fused_norm=False):
        super().__init__()
        self.fused_norm = fused_norm
        self.features = [6, 100, 100, nclasses]
        self.bandwidths = [64, 16, 10]
        self.sequential = _shrec17_sequence(self.features, self.bandwidths)
        self.out_layer = nn.Linear(self.features[-2], self.features[-1])

    def forward(self, x):  # pylint: disable=W0221
        if self.fused_norm:
            x = run_sequence(self.sequential, x, head="integrate")    # [batch, feature]
        else:
            x = so3_integrate(self.sequential(x))                     # [batch, feature, beta, alpha, gamma] -> [batch, feature]
        return F.log_softmax(self.out_layer(x), dim=1)


class Shrec17ModelOriginal(nn.Module):
    """examples/shrec17/model_original.py:7-50.  fused_norm: as in Shrec17Model."""

    def __init__(self, nclasses, fused_norm=False):
        super().__init__()
        self.fused_norm = fused_norm
        self.features = [6, 50, 70, 350, nclasses]
        self.bandwidths = [128, 32, 22, 7]
        self.sequential = _shrec17_sequence(self.features, self.bandwidths)
        self.out_layer = nn.Sequential(nn.BatchNorm1d(self.features[-2], affine=False), nn.Linear(self.features[-2], self.features[-1]))

    def forward(self, x):  # pylint: disable=W0221
        if self.fused_norm:
            x = run_sequence(self.sequential, x, head="max")          # [batch, feature]
        else:
            x = self.sequential(x)
            x = x.view(x.size(0), x.size(1), -1).max(-1)[0]
        return F.log_softmax(self.out_layer(x), dim=1)


NETWORKS = {
    # name: (constructor, input shape without the batch, number of classes, loss on the network's output)
    "mnist": (S2ConvNet_original, (1, 60, 60), 10, F.cross_entropy),                       # examples/mnist/run.py:211-223
    "shrec17": (lambda: Shrec17Model(55), (6, 128, 128), 55, F.nll_loss),                  # examples/shrec17/train.py:70-82
    "shrec17_original": (lambda: Shrec17ModelOriginal(55), (6, 256, 256), 55, F.nll_loss),
}


def synthetic_batch(name, batch, device, seed=0):
    """A fixed batch of the network's input shape: uniform values with 70 % of the samples zero for the digit network
    (projected digits are sparse), uniform values for the six ray-cast channels of the shape networks; random labels."""
    _, shape, nclasses, _ = NETWORKS[name]
    g = torch.Generator().manual_seed(seed)
    x = torch.rand(batch, *shape, generator=g)
    if name == "mnist":
        x = x * (torch.rand(batch, *shape, generator=g) < 0.3)
    y = torch.randint(0, nclasses, (batch,), generator=g)
    return x.to(device), y.to(device)


def smooth_spherical_batch(batch, channels, b, device, seed=0, lmax=16, noise=0.1):
    """Signals on the 2b x 2b grid of the sphere with smooth low-bandwidth structure: the synthesis of a random spectrum of
    degrees l < lmax (amplitudes falling like 1 / (l + 1)), rescaled per signal to [0, 1 - noise], plus uniform noise in
    [0, noise): the ray-cast depth / normal look of the inputs of the shape networks, values in [0, 1)."""
    from .soft.s2_fft import S2_ifft_real
    g = torch.Generator().manual_seed(seed)
    spec = torch.randn(lmax * lmax, batch * channels, 2, generator=g)
    falloff = torch.cat([torch.full((2 * l + 1,), 1.0 / (l + 1)) for l in range(lmax)])
    y = S2_ifft_real.apply((spec * falloff.view(-1, 1, 1)).to(device), b)          # [batch * channels, 2b, 2b]
    flat = y.reshape(y.size(0), -1)
    lo, hi = flat.min(1, keepdim=True)[0], flat.max(1, keepdim=True)[0]
    flat = (flat - lo) / (hi - lo).clamp_min(1e-12) * (1.0 - noise)
    flat = flat + noise * torch.rand(flat.shape, generator=g).to(device)
    return flat.clamp_(0.0, 1.0 - 1e-7).view(batch, channels, 2 * b, 2 * b)


def train_steps(name, batch=32, steps=10, warmup=2, lr=0.05, device="cuda:0", seed=0, model=None):
    """`warmup + steps` SGD steps (momentum 0.9, as examples/shrec17/train.py:66) on one synthetic batch.
    Returns (model, losses of all steps, milliseconds per timed step)."""
    ctor, _, _, loss_fn = NETWORKS[name]
    torch.manual_seed(seed)
    if model is None:
        model = ctor()
    model = model.to(device)
    model.train()
    x, y = synthetic_batch(name, batch, device, seed)
    opt = torch.optim.SGD(model.parameters(), lr=lr, momentum=0.9)
    losses = []

    def step():
        opt.zero_grad(set_to_none=True)
        loss = loss_fn(model(x), y)
        loss.backward()
        opt.step()
        losses.append(loss.detach())

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / max(steps, 1) * 1e3
    return model, [float(l) for l in losses], ms


def train_steps_replayed(name, batch=32, steps=10, warmup=3, lr=0.05, device="cuda:0", seed=0, model=None):
    """The step of `train_steps` captured once into a HIP graph (torch.cuda.graph) and replayed `steps` times: nothing on
    the path allocates through HIP, synchronises or records a memset, so the whole step (forward, loss, backward, SGD
    update) is one graph launch; for the small networks, whose step is bound by launches, that is most of the time.
    Returns (model, losses of the replayed steps, milliseconds per replayed step)."""
    ctor, _, _, loss_fn = NETWORKS[name]
    torch.manual_seed(seed)
    if model is None:
        model = ctor()
    model = model.to(device)
    model.train()
    x, y = synthetic_batch(name, batch, device, seed)
    opt = torch.optim.SGD(model.parameters(), lr=lr, momentum=0.9)

    def step():
        opt.zero_grad(set_to_none=True)
        loss = loss_fn(model(x), y)
        loss.backward()
        opt.step()
        return loss

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(max(warmup, 3)):     # tables, workspaces, momentum buffers and allocator pools exist before the capture
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    opt.zero_grad(set_to_none=True)
    with torch.cuda.graph(graph):
        static_loss = step()
    losses = []
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        graph.replay()
        losses.append(static_loss.detach().clone())
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / max(steps, 1) * 1e3
    return model, [float(l) for l in losses], ms
