"""State and input checks shared by the two convolution layers."""
import math

import torch
from torch import nn


class SpectralConvolution(nn.Module):
    """A convolution evaluated in the spectral domain: learnable kernel samples on a grid of group elements,
    a fixed normalisation, one bias per output feature.

    Parameter names and shapes are those of the reference's layers (`kernel` [feature_in, feature_out, len(grid)],
    `bias` [1, feature_out, 1, 1, 1]), so state dicts load either way."""

    # Signal and kernel are real, so their spectra, and every product and gradient formed from them, obey the
    # conjugate symmetry of a real signal; on real-basis spectra the products need a quarter (SO(3)) or half (S^2) of
    # the work of the complex ones.  False selects the complex operators of the reference literally.
    real_basis = True

    def __init__(self, nfeature_in, nfeature_out, b_in, b_out, grid, variance_per_sample, activation=None):
        super().__init__()
        # None: the layer of the reference.  "relu": max(., 0) applied where the output is written, and its gradient
        # where the backward transform reads the incoming gradient: the same function as F.relu(layer(x)) without
        # the passes of the activation over the output.
        assert activation in (None, "relu"), activation
        self.activation = activation
        self.nfeature_in, self.nfeature_out = nfeature_in, nfeature_out
        self.b_in, self.b_out = b_in, b_out
        self.grid = grid
        self.kernel = nn.Parameter(torch.empty(nfeature_in, nfeature_out, len(grid)).uniform_(-1, 1))
        self.bias = nn.Parameter(torch.zeros(1, nfeature_out, 1, 1, 1))
        # kept outside the parameter: activations of order one for kernel entries of order one
        self.scaling = 1.0 / math.sqrt(len(grid) * nfeature_in * variance_per_sample)

    @property
    def fused_relu(self):
        return self.activation == "relu"

    def scaled_kernel(self):
        return self.kernel * self.scaling

    def check_input(self, x, n_grid_dims):
        want = (self.nfeature_in,) + (2 * self.b_in,) * n_grid_dims
        assert tuple(x.shape[1:]) == want, f"expected [batch, {', '.join(map(str, want))}], got {tuple(x.shape)}"
