"""SO3Convolution and SO3Shortcut (the layers of s2cnn/soft/so3_conv.py)."""
from torch import nn

from ..so3_ft import so3_rft
from ..so3_mm import so3_mm
from ..so3_real import so3_mm_real, so3_rft_real
from ._spectral_conv import SpectralConvolution
from .so3_fft import SO3_fft_real, SO3_fft_real_basis, SO3_ifft_real, SO3_ifft_real_basis


class SO3Convolution(SpectralConvolution):
    def __init__(self, nfeature_in, nfeature_out, b_in, b_out, grid, *, activation=None):
        """
        nfeature_in, nfeature_out: feature counts; b_in: bandwidth of the input (a (2 b_in)^3 SOFT grid);
        b_out: bandwidth of the output; grid: the rotations that carry the kernel, a tuple of
        (beta, alpha, gamma) triples (s2cnn/soft/so3_conv.py:13-34, normalisation :31).
        activation (not in the reference): None, or "relu" for F.relu(layer(x)) computed inside the layer.
        """
        super().__init__(nfeature_in, nfeature_out, b_in, b_out, grid, b_out ** 3.0 / b_in ** 3.0, activation)

    def forward(self, x):  # pylint: disable=W
        """[batch, feature_in, beta, alpha, gamma] -> [batch, feature_out, beta, alpha, gamma]"""
        self.check_input(x, 3)
        if self.real_basis:
            return self.from_spectrum(self.product_spectrum(x))
        xh = SO3_fft_real.apply(x, self.b_out)                                 # [l m n, batch, feature_in, complex]
        yh = so3_rft(self.scaled_kernel(), self.b_out, self.grid)              # [l m n, feature_in, feature_out, complex]
        return SO3_ifft_real.apply(so3_mm(xh, yh), None, self.bias, self.fused_relu)


    # The two halves of the real-basis forward pass, for callers that put something else between the layers' transforms
    # (s2cnn_amd/soft/bn_relu.py): the spectrum of the output before the last transform, and that transform.
    def product_spectrum(self, x, xh=None):
        """[l m n, batch, feature_out] in the real basis, from the input x or from its spectrum xh [l m n, batch, feature_in]."""
        if xh is None:
            self.check_input(x, 3)
            xh = SO3_fft_real_basis.apply(x, self.b_out)                       # [l m n, batch, feature_in]
        yh = so3_rft_real(self.scaled_kernel(), self.b_out, self.grid)         # [l m n, feature_in, feature_out]
        return so3_mm_real(xh, yh)

    def from_spectrum(self, zh):
        return SO3_ifft_real_basis.apply(zh, None, self.bias, self.fused_relu)  # bias added inside the transform


class SO3Shortcut(nn.Module):
    """Identity when neither the feature count nor the bandwidth changes, otherwise a convolution with the one-point
    kernel at the identity rotation: the skip branch of residual blocks (s2cnn/soft/so3_conv.py:59-79)."""

    def __init__(self, nfeature_in, nfeature_out, b_in, b_out):
        super().__init__()
        assert b_out <= b_in
        same = nfeature_in == nfeature_out and b_in == b_out
        self.conv = None if same else SO3Convolution(nfeature_in, nfeature_out, b_in, b_out, grid=((0, 0, 0),))

    def forward(self, x):  # pylint: disable=W
        """[batch, feature_in, beta, alpha, gamma] -> [batch, feature_out, beta, alpha, gamma]"""
        return x if self.conv is None else self.conv(x)
