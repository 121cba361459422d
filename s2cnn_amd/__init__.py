"""MI355X-native spectral path of spherical CNNs, behind the Python API of s2cnn
(same exported names as s2cnn/__init__.py of the reference)."""
from .s2_ft import s2_rft
from .so3_ft import so3_rft
from .s2_grid import s2_near_identity_grid, s2_equatorial_grid, s2_soft_grid
from .so3_grid import so3_near_identity_grid, so3_equatorial_grid, so3_soft_grid
from .s2_mm import s2_mm
from .so3_mm import so3_mm
from .so3_real import so3_mm_real, so3_rft_real, so3_spectrum_to_complex, so3_spectrum_to_real
from .s2_real import s2_mm_real, s2_rft_real, s2_spectrum_to_real
from .soft import *  # noqa: F401,F403
from .soft import S2Convolution, SO3Convolution, SO3Shortcut, so3_integrate, so3_rotation
