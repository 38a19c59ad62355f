"""The e3nn-convention wrapper (reference: sphericart-torch/python/sphericart/torch/e3nn.py and
its test sphericart-torch/python/tests/test_e3nn.py, which compares with e3nn itself; e3nn is
not installed here, so the conventions are pinned by what they are defined to be: degree one
in "component" scale is sqrt(3) (x, y, z) / r, "norm" makes every degree a unit vector on the
sphere, "integral" is orthonormal, and a rotation about z mixes (l, m) with (l, -m) only)."""

import math
import types

import numpy as np
import pytest
import torch

from gpu_utils import announce


def _points(n, seed):
    rng = np.random.default_rng(seed)
    return torch.from_numpy(rng.normal(size=(n, 3))).cuda()


@pytest.mark.gpu
def test_degree_one_and_scales():
    from sphericart_amd.torch import e3nn_spherical_harmonics as sh
    announce("e3nn conventions")
    x = _points(500, 0)
    unit = x / x.norm(dim=1, keepdim=True)
    # component: sqrt(3) * direction, in e3nn's (x, y, z) order
    got = sh(1, x, normalize=True, normalization="component")
    torch.testing.assert_close(got, math.sqrt(3.0) * unit, rtol=0, atol=1e-12)
    # solid harmonics of degree one are the vector itself, up to the scale
    got = sh([1], x, normalize=False, normalization="norm")
    torch.testing.assert_close(got, x, rtol=0, atol=1e-12)
    # norm: every degree a unit vector; component: squared norm 2l + 1; integral: (2l + 1) / 4 pi
    degrees = [0, 1, 2, 3, 5, 8]
    for scale, want in (("norm", lambda l: 1.0), ("component", lambda l: 2 * l + 1.0),
                        ("integral", lambda l: (2 * l + 1) / (4 * math.pi))):
        out = sh(degrees, x, normalize=True, normalization=scale)
        at = 0
        for l in degrees:
            block = out[:, at:at + 2 * l + 1]
            at += 2 * l + 1
            torch.testing.assert_close((block ** 2).sum(dim=1), torch.full((500,), want(l), dtype=x.dtype, device="cuda"),
                                       rtol=1e-11, atol=0)
        assert at == out.shape[1]


@pytest.mark.gpu
def test_selection_order_and_full_range():
    from sphericart_amd.torch import SphericalHarmonics, e3nn_spherical_harmonics as sh
    announce("e3nn selection")
    x = _points(200, 1)
    full = sh(list(range(5)), x, normalize=True)
    torch.testing.assert_close(full, SphericalHarmonics(4)(x[:, [2, 0, 1]]), rtol=0, atol=0)
    torch.testing.assert_close(sh(4, x, normalize=True), full[:, 16:25], rtol=0, atol=0)
    picked = sh([3, 1], x, normalize=True)
    torch.testing.assert_close(picked, torch.cat([full[:, 9:16], full[:, 1:4]], dim=1), rtol=0, atol=0)
    with pytest.raises(ValueError):
        sh([2], x, normalization="other")
    with pytest.raises(ValueError):
        sh([], x)


@pytest.mark.gpu
def test_gradients_flow():
    from sphericart_amd.torch import e3nn_spherical_harmonics as sh
    announce("e3nn autograd")
    x = _points(50, 2).requires_grad_(True)
    out = sh([0, 2, 3], x, normalize=True, normalization="norm")
    (out ** 2).sum().backward()
    # every block has unit norm whatever the point: the gradient of the sum of squares vanishes
    assert x.grad is not None and x.grad.abs().max() < 1e-10
    torch.autograd.gradcheck(lambda t: sh([1, 2], t, normalize=False, normalization="component"),
                             (_points(7, 3).requires_grad_(True),), eps=1e-6, atol=1e-6)


def test_patch_and_unpatch():
    from sphericart_amd.torch import e3nn_spherical_harmonics, patch_e3nn, unpatch_e3nn
    original = object()
    fake = types.SimpleNamespace(o3=types.SimpleNamespace(spherical_harmonics=original))
    with pytest.raises(RuntimeError):
        unpatch_e3nn(fake)
    patch_e3nn(fake)
    assert fake.o3.spherical_harmonics is e3nn_spherical_harmonics
    with pytest.raises(RuntimeError):
        patch_e3nn(fake)
    unpatch_e3nn(fake)
    assert fake.o3.spherical_harmonics is original
