"""SO(3) convolution layer: mirrors s2cnn/soft/so3_conv.py of the reference (same constructor,
attributes, parameter names and shapes, so state dicts are interchangeable)."""
import math

import torch
from torch.nn.modules import Module
from torch.nn.parameter import Parameter

from ..so3_ft import so3_rft
from ..so3_mm import so3_mm
from ..so3_real import so3_mm_real, so3_rft_real
from .so3_fft import SO3_fft_real, SO3_fft_real_basis, SO3_ifft_real, SO3_ifft_real_basis


class SO3Convolution(Module):
    # Signal and kernel are real, so their spectra - and every product and gradient formed from them - obey
    # X[l,-m,-n] = (-1)^(m-n) conj(X[l,m,n]); in the real basis the block product needs a quarter of the
    # multiply-adds of the complex one.  False selects the complex product of the reference literally.
    real_basis = True

    def __init__(self, nfeature_in, nfeature_out, b_in, b_out, grid):
        '''
        :param nfeature_in: number of input fearures
        :param nfeature_out: number of output features
        :param b_in: input bandwidth (precision of the input SOFT grid)
        :param b_out: output bandwidth
        :param grid: points of the SO(3) group defining the kernel, tuple of (beta, alpha, gamma)'s
        '''
        super().__init__()
        self.nfeature_in = nfeature_in
        self.nfeature_out = nfeature_out
        self.b_in = b_in
        self.b_out = b_out
        self.grid = grid
        self.kernel = Parameter(torch.empty(nfeature_in, nfeature_out, len(grid)).uniform_(-1, 1))
        self.bias = Parameter(torch.zeros(1, nfeature_out, 1, 1, 1))
        # the scaling that keeps activations of order one lives outside the parameter
        # (s2cnn/soft/so3_conv.py:30-34)
        self.scaling = 1. / math.sqrt(len(self.grid) * self.nfeature_in * (self.b_out ** 3.) / (self.b_in ** 3.))

    def forward(self, x):  # pylint: disable=W
        '''
        :x:      [batch, feature_in,  beta, alpha, gamma]
        :return: [batch, feature_out, beta, alpha, gamma]
        '''
        assert x.size(1) == self.nfeature_in
        assert x.size(2) == 2 * self.b_in
        assert x.size(3) == 2 * self.b_in
        assert x.size(4) == 2 * self.b_in

        if self.real_basis:
            x = SO3_fft_real_basis.apply(x, self.b_out)  # [l * m * n, batch, feature_in]
            y = so3_rft_real(self.kernel * self.scaling, self.b_out, self.grid)  # [l * m * n, feature_in, feature_out]
            assert x.size(0) == y.size(0)
            assert x.size(2) == y.size(1)
            z = so3_mm_real(x, y)  # [l * m * n, batch, feature_out]
            return SO3_ifft_real_basis.apply(z, None, self.bias)  # [batch, feature_out, beta, alpha, gamma], bias added
        x = SO3_fft_real.apply(x, self.b_out)  # [l * m * n, batch, feature_in, complex]
        y = so3_rft(self.kernel * self.scaling, self.b_out, self.grid)  # [l * m * n, feature_in, feature_out, complex]
        assert x.size(0) == y.size(0)
        assert x.size(2) == y.size(1)
        z = so3_mm(x, y)  # [l * m * n, batch, feature_out, complex]
        assert z.size(0) == x.size(0)
        assert z.size(1) == x.size(1)
        assert z.size(2) == y.size(2)
        return SO3_ifft_real.apply(z, None, self.bias)  # [batch, feature_out, beta, alpha, gamma], bias added in the transform


class SO3Shortcut(Module):
    '''
    Useful for ResNet
    '''

    def __init__(self, nfeature_in, nfeature_out, b_in, b_out):
        super().__init__()
        assert b_out <= b_in
        if (nfeature_in != nfeature_out) or (b_in != b_out):
            self.conv = SO3Convolution(nfeature_in=nfeature_in, nfeature_out=nfeature_out, b_in=b_in, b_out=b_out,
                                       grid=((0, 0, 0),))
        else:
            self.conv = None

    def forward(self, x):  # pylint: disable=W
        '''
        :x:      [batch, feature_in,  beta, alpha, gamma]
        :return: [batch, feature_out, beta, alpha, gamma]
        '''
        return x if self.conv is None else self.conv(x)
