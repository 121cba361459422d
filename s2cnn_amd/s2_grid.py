"""Kernel grids on the sphere: tuples of (beta, alpha) points (same functions, defaults and point order as
s2cnn/s2_grid.py)."""
import numpy as np

from . import _grid_util as G


def s2_near_identity_grid(max_beta=np.pi / 8, n_alpha=8, n_beta=3):
    """n_beta rings of n_alpha points around the north pole, out to colatitude max_beta."""
    return G.points(*G.mesh(G.polar_rings(max_beta, n_beta), G.circle(n_alpha)))


def s2_equatorial_grid(max_beta=0, n_alpha=32, n_beta=1):
    """n_beta rings of n_alpha points in the band of half-width max_beta around the equator."""
    return G.points(*G.mesh(G.band(np.pi / 2, max_beta, n_beta), G.circle(n_alpha)))


def s2_soft_grid(b):
    """Every point of the 2b x 2b SOFT grid."""
    return G.points(*G.mesh(G.soft_colatitudes(b), G.circle(2 * b)))
