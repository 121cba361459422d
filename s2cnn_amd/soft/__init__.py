"""Layers and grid-domain operators on the SOFT grid."""
from .so3_integrate import so3_integrate
from .so3_rotation import so3_rotation
from .so3_conv import SO3Convolution, SO3Shortcut
from .s2_conv import S2Convolution

__all__ = ["S2Convolution", "SO3Convolution", "SO3Shortcut", "so3_integrate", "so3_rotation"]
