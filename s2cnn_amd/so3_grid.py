"""Kernel grids on SO(3): tuples of (beta, alpha, gamma) Euler-angle points (same functions, defaults and point
order as s2cnn/so3_grid.py)."""
import warnings

import numpy as np

from . import _grid_util as G


def _checked(beta, alpha, gamma):
    pts = G.points(beta, alpha, gamma)
    if sum(1 for p in pts if p[0] == 0) > 1:     # at beta = 0 only alpha + gamma matters: such points may coincide
        warnings.warn("Gimbal lock: beta take value 0 in the grid")
    return pts


def so3_near_identity_grid(max_beta=np.pi / 8, max_gamma=2 * np.pi, n_alpha=8, n_beta=3, n_gamma=None):
    """Rotations close to the identity: n_beta rings (every rotation of a ring is equally far from the identity) of
    n_alpha directions, and n_gamma (default n_alpha) in-plane angles with alpha + gamma in [-max_gamma, max_gamma]."""
    n_gamma = n_alpha if n_gamma is None else n_gamma
    beta, alpha, twist = G.mesh(G.polar_rings(max_beta, n_beta), G.circle(n_alpha), G.band(0.0, max_gamma, n_gamma))
    return _checked(beta, alpha, twist - alpha)


def so3_equatorial_grid(max_beta=0, max_gamma=np.pi / 8, n_alpha=32, n_beta=1, n_gamma=2):
    """Rotations that take the north pole into the band of half-width max_beta around the equator, with
    n_gamma in-plane angles in [-max_gamma, max_gamma]."""
    return _checked(*G.mesh(G.band(np.pi / 2, max_beta, n_beta), G.circle(n_alpha), G.band(0.0, max_gamma, n_gamma)))


def so3_soft_grid(b):
    """Every point of the (2b)^3 SOFT grid."""
    return G.points(*G.mesh(G.soft_colatitudes(b), G.circle(2 * b), G.circle(2 * b)))
