"""Angle axes and point lists shared by the kernel grids of s2_grid.py and so3_grid.py."""
import numpy as np

TWO_PI = 2.0 * np.pi


def circle(n):
    """n equally spaced angles in [0, 2 pi)."""
    return TWO_PI * np.arange(n) / n


def polar_rings(max_beta, n):
    """n colatitudes max_beta / n, 2 max_beta / n, ..., max_beta (the pole itself is left out)."""
    return max_beta * np.arange(1, n + 1, dtype=float) / n


def band(centre, half_width, n):
    """n angles from centre - half_width to centre + half_width, both ends included."""
    return np.linspace(centre - half_width, centre + half_width, n)


def soft_colatitudes(b):
    """The 2b colatitudes of the SOFT grid: pi (2j + 1) / (4b)."""
    return np.pi * (2.0 * np.arange(2 * b) + 1.0) / (4.0 * b)


def points(*coords):
    """Flattened coordinate arrays -> tuple of tuples of Python floats (hashable: grids key caches)."""
    cols = np.stack([np.asarray(c, dtype=float).reshape(-1) for c in coords], axis=1)
    return tuple(tuple(float(v) for v in row) for row in cols)


def mesh(*axes):
    """Cartesian product of the axes, first axis slowest."""
    return np.meshgrid(*axes, indexing="ij")
