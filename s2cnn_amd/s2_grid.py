"""Sampling grids on the sphere for convolution kernels: mirrors s2cnn/s2_grid.py of the reference.
Every grid is a tuple of (beta, alpha) tuples of Python floats."""
import numpy as np


def _pack(B, A):
    grid = np.stack((B.flatten(), A.flatten()), axis=1)
    return tuple(tuple(float(v) for v in ba) for ba in grid)


def s2_near_identity_grid(max_beta=np.pi / 8, n_alpha=8, n_beta=3):
    '''
    :return: rings around the north pole
    size of the kernel = n_alpha * n_beta
    '''
    beta = np.arange(start=1, stop=n_beta + 1, dtype=float) * max_beta / n_beta
    alpha = np.linspace(start=0, stop=2 * np.pi, num=n_alpha, endpoint=False)
    return _pack(*np.meshgrid(beta, alpha, indexing='ij'))


def s2_equatorial_grid(max_beta=0, n_alpha=32, n_beta=1):
    '''
    :return: rings around the equator
    size of the kernel = n_alpha * n_beta
    '''
    beta = np.linspace(start=np.pi / 2 - max_beta, stop=np.pi / 2 + max_beta, num=n_beta, endpoint=True)
    alpha = np.linspace(start=0, stop=2 * np.pi, num=n_alpha, endpoint=False)
    return _pack(*np.meshgrid(beta, alpha, indexing='ij'))


def s2_soft_grid(b):
    beta = (np.arange(2 * b) + 0.5) / (2 * b) * np.pi
    alpha = np.linspace(start=0, stop=2 * np.pi, num=2 * b, endpoint=False)
    return _pack(*np.meshgrid(beta, alpha, indexing='ij'))
