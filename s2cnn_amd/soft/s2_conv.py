"""S^2 convolution layer: mirrors s2cnn/soft/s2_conv.py of the reference."""
import math

import torch
from torch.nn.modules import Module
from torch.nn.parameter import Parameter

from ..s2_ft import s2_rft
from ..s2_mm import s2_mm
from ..s2_real import s2_mm_real, s2_rft_real, s2_spectrum_to_real
from .s2_fft import S2_fft_real
from .so3_fft import SO3_ifft_real, SO3_ifft_real_basis


class S2Convolution(Module):
    def __init__(self, nfeature_in, nfeature_out, b_in, b_out, grid):
        '''
        :param nfeature_in: number of input fearures
        :param nfeature_out: number of output features
        :param b_in: input bandwidth (precision of the input SOFT grid)
        :param b_out: output bandwidth
        :param grid: points of the sphere defining the kernel, tuple of (beta, alpha)'s
        '''
        super().__init__()
        self.nfeature_in = nfeature_in
        self.nfeature_out = nfeature_out
        self.b_in = b_in
        self.b_out = b_out
        self.grid = grid
        self.kernel = Parameter(torch.empty(nfeature_in, nfeature_out, len(grid)).uniform_(-1, 1))
        self.scaling = 1. / math.sqrt(len(self.grid) * self.nfeature_in * (self.b_out ** 4.) / (self.b_in ** 2.))
        self.bias = Parameter(torch.zeros(1, nfeature_out, 1, 1, 1))
        # Signal and kernel are real, so their spectra obey x[l,-m] = (-1)^m conj(x[l,m]): the product and the
        # synthesis run on real-basis spectra (half the bytes, same result).  False: the reference's complex path.
        self.real_basis = True

    def forward(self, x):  # pylint: disable=W
        '''
        :x:      [batch, feature_in,  beta, alpha]
        :return: [batch, feature_out, beta, alpha, gamma]
        '''
        assert x.size(1) == self.nfeature_in
        assert x.size(2) == 2 * self.b_in
        assert x.size(3) == 2 * self.b_in
        x = S2_fft_real.apply(x, self.b_out)  # [l * m, batch, feature_in, complex]
        if self.real_basis:
            x = s2_spectrum_to_real(x)  # [l * m, batch, feature_in]
            y = s2_rft_real(self.kernel * self.scaling, self.b_out, self.grid)  # [l * m, feature_in, feature_out]
            z = s2_mm_real(x, y)  # [l * m * n, batch, feature_out]
            return SO3_ifft_real_basis.apply(z, None, self.bias)  # [batch, feature_out, beta, alpha, gamma], bias added
        y = s2_rft(self.kernel * self.scaling, self.b_out, self.grid)  # [l * m, feature_in, feature_out, complex]
        z = s2_mm(x, y)  # [l * m * n, batch, feature_out, complex]
        return SO3_ifft_real.apply(z, None, self.bias)  # [batch, feature_out, beta, alpha, gamma], bias added in the transform
