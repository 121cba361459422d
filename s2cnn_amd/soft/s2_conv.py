"""S2Convolution: signal on the sphere in, signal on SO(3) out (the layer of s2cnn/soft/s2_conv.py)."""
from ..s2_ft import s2_rft
from ..s2_mm import s2_mm
from ..s2_real import s2_mm_real, s2_rft_real, s2_spectrum_to_real
from ._spectral_conv import SpectralConvolution
from .s2_fft import S2_fft_real
from .so3_fft import SO3_ifft_real, SO3_ifft_real_basis


class S2Convolution(SpectralConvolution):
    def __init__(self, nfeature_in, nfeature_out, b_in, b_out, grid, *, activation=None):
        """
        nfeature_in, nfeature_out: feature counts; b_in: bandwidth of the input (a 2 b_in x 2 b_in SOFT grid);
        b_out: bandwidth of the output; grid: the points of the sphere that carry the kernel, a tuple of
        (beta, alpha) pairs (s2cnn/soft/s2_conv.py:14-30, normalisation :27).
        activation (not in the reference): None, or "relu" for F.relu(layer(x)) computed inside the layer.
        """
        super().__init__(nfeature_in, nfeature_out, b_in, b_out, grid, b_out ** 4.0 / b_in ** 2.0, activation)

    def forward(self, x):  # pylint: disable=W
        """[batch, feature_in, beta, alpha] -> [batch, feature_out, beta, alpha, gamma]"""
        self.check_input(x, 2)
        if self.real_basis:
            return self.from_spectrum(self.product_spectrum(x))
        xh = S2_fft_real.apply(x, self.b_out)                                  # [l m, batch, feature_in, complex]
        yh = s2_rft(self.scaled_kernel(), self.b_out, self.grid)               # [l m, feature_in, feature_out, complex]
        zh = s2_mm(xh, yh)                                                     # [l m n, batch, feature_out, complex]
        return SO3_ifft_real.apply(zh, None, self.bias, self.fused_relu)

    # The two halves of the real-basis forward pass (see SO3Convolution.product_spectrum).
    def product_spectrum(self, x, xh=None):
        """[l m n, batch, feature_out] in the real basis, from the input x (xh: its complex S^2 spectrum, if at hand)."""
        if xh is None:
            self.check_input(x, 2)
            xh = S2_fft_real.apply(x, self.b_out)                              # [l m, batch, feature_in, complex]
        yh = s2_rft_real(self.scaled_kernel(), self.b_out, self.grid)          # [l m, feature_in, feature_out]
        return s2_mm_real(s2_spectrum_to_real(xh), yh)                         # [l m n, batch, feature_out]

    def from_spectrum(self, zh):
        return SO3_ifft_real_basis.apply(zh, None, self.bias, self.fused_relu)  # bias added inside the transform
