"""MI355X-native spectral path of spherical CNNs.  The package exports the names of the reference's `s2cnn`
package (layers, operators, kernel transforms, grids) plus the real-basis operators the layers use internally."""
from . import s2_grid as _s2_grid, so3_grid as _so3_grid
from .soft import S2Convolution, SO3Convolution, SO3Shortcut, so3_integrate, so3_rotation
from .so3_mm import so3_mm
from .s2_mm import s2_mm
from .so3_ft import so3_rft
from .s2_ft import s2_rft
from .so3_real import so3_mm_real, so3_rft_real, so3_spectrum_to_complex, so3_spectrum_to_real
from .s2_real import s2_mm_real, s2_rft_real, s2_spectrum_to_real

s2_near_identity_grid, s2_equatorial_grid, s2_soft_grid = (
    _s2_grid.s2_near_identity_grid, _s2_grid.s2_equatorial_grid, _s2_grid.s2_soft_grid)
so3_near_identity_grid, so3_equatorial_grid, so3_soft_grid = (
    _so3_grid.so3_near_identity_grid, _so3_grid.so3_equatorial_grid, _so3_grid.so3_soft_grid)
