"""The package is a drop-in for the reference's `s2cnn`: the names it exports and the leading parameters (names and
defaults) of every public callable are those of s2cnn/__init__.py:2-8, s2cnn/soft/__init__.py:2-5 and the definitions
they point to; anything this package adds comes after them or is keyword-only."""
import inspect
import math

import pytest

import s2cnn_amd
from s2cnn_amd.soft import s2_conv, s2_fft, so3_conv, so3_fft

REQ = inspect.Parameter.empty
PI = math.pi

# (owner, name, [(parameter, default)] as the reference declares them; file:line of the reference definition)
SIGNATURES = [
    (s2cnn_amd, "s2_near_identity_grid", [("max_beta", PI / 8), ("n_alpha", 8), ("n_beta", 3)]),                       # s2_grid.py:5
    (s2cnn_amd, "s2_equatorial_grid", [("max_beta", 0), ("n_alpha", 32), ("n_beta", 1)]),                              # s2_grid.py:19
    (s2cnn_amd, "s2_soft_grid", [("b", REQ)]),                                                                         # s2_grid.py:33
    (s2cnn_amd, "so3_near_identity_grid", [("max_beta", PI / 8), ("max_gamma", 2 * PI), ("n_alpha", 8), ("n_beta", 3), ("n_gamma", None)]),  # so3_grid.py:6
    (s2cnn_amd, "so3_equatorial_grid", [("max_beta", 0), ("max_gamma", PI / 8), ("n_alpha", 32), ("n_beta", 1), ("n_gamma", 2)]),          # so3_grid.py:28
    (s2cnn_amd, "so3_soft_grid", [("b", REQ)]),                                                                        # so3_grid.py:46
    (s2cnn_amd, "s2_rft", [("x", REQ), ("b", REQ), ("grid", REQ)]),                                                    # s2_ft.py:8
    (s2cnn_amd, "so3_rft", [("x", REQ), ("b", REQ), ("grid", REQ)]),                                                   # so3_ft.py:8
    (s2cnn_amd, "s2_mm", [("x", REQ), ("y", REQ)]),                                                                    # s2_mm.py:10
    (s2cnn_amd, "so3_mm", [("x", REQ), ("y", REQ)]),                                                                   # so3_mm.py:8
    (s2cnn_amd, "so3_integrate", [("x", REQ)]),                                                                        # soft/so3_integrate.py:7
    (s2cnn_amd, "so3_rotation", [("x", REQ), ("alpha", REQ), ("beta", REQ), ("gamma", REQ)]),                          # soft/so3_rotation.py:11
    (so3_fft, "so3_fft", [("x", REQ), ("for_grad", False), ("b_out", None)]),                                          # soft/so3_fft.py:12
    (so3_fft, "so3_rfft", [("x", REQ), ("for_grad", False), ("b_out", None)]),                                         # soft/so3_fft.py:64
    (so3_fft, "so3_ifft", [("x", REQ), ("for_grad", False), ("b_out", None)]),                                         # soft/so3_fft.py:115
    (so3_fft, "so3_rifft", [("x", REQ), ("for_grad", False), ("b_out", None)]),                                        # soft/so3_fft.py:158
    (s2_fft, "s2_fft", [("x", REQ), ("for_grad", False), ("b_out", None)]),                                            # soft/s2_fft.py:13
    (s2_fft, "s2_ifft", [("x", REQ), ("for_grad", False), ("b_out", None)]),                                           # soft/s2_fft.py:61
]
LAYER = [("nfeature_in", REQ), ("nfeature_out", REQ), ("b_in", REQ), ("b_out", REQ), ("grid", REQ)]
CLASSES = [
    (s2cnn_amd, "S2Convolution", LAYER),            # soft/s2_conv.py:14
    (s2cnn_amd, "SO3Convolution", LAYER),           # soft/so3_conv.py:13
    (so3_conv, "SO3Shortcut", LAYER[:4]),           # soft/so3_conv.py:66
    (s2_conv, "S2Convolution", LAYER),
]
FUNCTIONS = [(so3_fft, "SO3_fft_real"), (so3_fft, "SO3_ifft_real"), (s2_fft, "S2_fft_real"), (s2_fft, "S2_ifft_real")]   # forward(ctx, x, b_out=None)


def _check(params, want, what):
    params = list(params)
    assert len(params) >= len(want), what
    for p, (name, default) in zip(params, want):
        assert p.name == name, (what, p.name, name)
        assert p.kind in (p.POSITIONAL_OR_KEYWORD,), (what, name)
        if default is REQ:
            assert p.default is REQ, (what, name)
        elif isinstance(default, float):
            assert p.default == pytest.approx(default), (what, name)
        else:
            assert p.default == default and type(p.default) is type(default), (what, name, p.default)
    for p in params[len(want):]:       # additions must not disturb a positional call written for the reference
        assert p.default is not REQ or p.kind == p.KEYWORD_ONLY, (what, p.name)


@pytest.mark.parametrize("owner,name,want", SIGNATURES, ids=[s[1] for s in SIGNATURES])
def test_function_signatures(owner, name, want):
    _check(inspect.signature(getattr(owner, name)).parameters.values(), want, name)


@pytest.mark.parametrize("owner,name,want", CLASSES, ids=[f"{c[0].__name__.split('.')[-1]}.{c[1]}" for c in CLASSES])
def test_layer_constructors(owner, name, want):
    cls = getattr(owner, name)
    _check(list(inspect.signature(cls.__init__).parameters.values())[1:], want, name)
    assert [p.name for p in list(inspect.signature(cls.forward).parameters.values())[1:]] == ["x"]


@pytest.mark.parametrize("owner,name", FUNCTIONS, ids=[f[1] for f in FUNCTIONS])
def test_autograd_functions(owner, name):
    fn = getattr(owner, name)
    _check(list(inspect.signature(fn.forward).parameters.values())[1:], [("x", REQ), ("b_out", None)], name)
    assert callable(fn.apply)


def test_layer_state_matches_the_reference():
    """Parameter names, shapes and the value of `scaling` (s2cnn/soft/so3_conv.py:22-34, s2_conv.py:23-29): state dicts
    written by either implementation load into the other."""
    g3, g2 = s2cnn_amd.so3_near_identity_grid(), s2cnn_amd.s2_near_identity_grid()
    assert len(g3) == 192 and len(g2) == 24
    c = s2cnn_amd.SO3Convolution(5, 7, 8, 6, g3)
    assert {k: tuple(v.shape) for k, v in c.state_dict().items()} == {"kernel": (5, 7, 192), "bias": (1, 7, 1, 1, 1)}
    assert c.scaling == pytest.approx(1.0 / math.sqrt(192 * 5 * 6 ** 3 / 8 ** 3))
    assert (c.nfeature_in, c.nfeature_out, c.b_in, c.b_out, c.grid) == (5, 7, 8, 6, g3)
    c = s2cnn_amd.S2Convolution(3, 4, 10, 6, g2)
    assert {k: tuple(v.shape) for k, v in c.state_dict().items()} == {"kernel": (3, 4, 24), "bias": (1, 4, 1, 1, 1)}
    assert c.scaling == pytest.approx(1.0 / math.sqrt(24 * 3 * 6 ** 4 / 10 ** 2))
    assert float(c.kernel.detach().abs().max()) <= 1.0 and float(c.bias.detach().abs().max()) == 0.0
    s = so3_conv.SO3Shortcut(4, 4, 6, 6)
    assert list(s.state_dict()) == []                                       # identity: no parameters
    s = so3_conv.SO3Shortcut(4, 6, 6, 4)
    assert {k: tuple(v.shape) for k, v in s.state_dict().items()} == {"conv.kernel": (4, 6, 1), "conv.bias": (1, 6, 1, 1, 1)}


def test_shape_errors_are_assertion_errors():
    """As in the reference (asserts at s2cnn/so3_mm.py:17-26, s2_mm.py:17-27, soft/so3_fft.py:17-21, soft/s2_fft.py:24,71,
    soft/so3_conv.py:41-42): a call with inconsistent shapes fails with AssertionError before anything touches a device."""
    import torch
    z = torch.zeros
    with pytest.raises(AssertionError):
        s2cnn_amd.so3_mm(z(10, 2, 3, 2), z(10, 4, 5, 2))            # feature counts differ
    with pytest.raises(AssertionError):
        s2cnn_amd.so3_mm(z(11, 2, 3, 2), z(11, 3, 5, 2))            # 11 is no nspec(b)
    with pytest.raises(AssertionError):
        s2cnn_amd.s2_mm(z(9, 2, 3, 2), z(4, 3, 5, 2))               # spectra of different bandwidth
    with pytest.raises(AssertionError):
        s2cnn_amd.s2_mm(z(8, 2, 3, 2), z(8, 3, 5, 2))               # 8 is no b^2
    with pytest.raises(AssertionError):
        s2_fft.s2_fft(z(2, 8, 8, 2), b_out=5)                       # b_out > b_in
    with pytest.raises(AssertionError):
        s2_fft.s2_ifft(z(16, 2, 2), b_out=3)                        # b_out < b_in
    with pytest.raises(AssertionError):
        so3_fft.so3_rfft(z(2, 8, 8, 6))                             # not a cube
    with pytest.raises(AssertionError):
        so3_fft.so3_rifft(z(11, 2, 2))                              # 11 is no nspec(b)
    with pytest.raises(AssertionError):
        s2cnn_amd.SO3Convolution(2, 3, 4, 4, s2cnn_amd.so3_near_identity_grid())(z(1, 2, 8, 8, 6))
    with pytest.raises(AssertionError):
        s2cnn_amd.S2Convolution(2, 3, 4, 4, s2cnn_amd.s2_near_identity_grid())(z(1, 3, 8, 8))
