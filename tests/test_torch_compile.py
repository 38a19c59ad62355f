"""The modules under torch.jit.script, torch.compile and functorch transforms, after the
reference's sphericart-torch/python/tests/test_script.py, test_compile.py and test_nn.py.
torch.compile runs with the "aot_eager" backend: what is tested is that tracing, the fake-tensor
rules and the autograd registration of the operators hold with no graph break; code generation
for the surrounding torch operations is not this package's concern."""

import pytest
import torch

import sphericart_amd.torch
from gpu_utils import announce

pytestmark = pytest.mark.gpu


class SHModule(torch.nn.Module):
    def __init__(self, l_max, normalized=False):
        super().__init__()
        cls = sphericart_amd.torch.SphericalHarmonics if normalized else sphericart_amd.torch.SolidHarmonics
        self._sph = cls(l_max)

    def forward(self, xyz):
        return self._sph.compute(xyz)


def _xyz(n=100, seed=0):
    torch.manual_seed(seed)
    return (6 * torch.randn(n, 3, dtype=torch.float64)).cuda()


@pytest.mark.parametrize("normalized", [True, False])
def test_script(normalized, tmp_path):
    announce("script", normalized)
    module = SHModule(10, normalized)
    a = _xyz().requires_grad_()
    b = _xyz().requires_grad_()
    module(a).sum().backward()
    script = torch.jit.script(module)
    out = script(b)
    out.sum().backward()
    torch.testing.assert_close(out, module(a), rtol=0, atol=0)
    torch.testing.assert_close(b.grad, a.grad, rtol=0, atol=0)
    # the scripted module survives a round trip through a file in this process
    path = str(tmp_path / "sh.pt")
    script.save(path)
    again = torch.jit.load(path)
    torch.testing.assert_close(again(_xyz()), module(_xyz()), rtol=0, atol=0)


def test_script_with_derivative_arrays():
    announce("script, derivative arrays")

    class Both(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self._sph = sphericart_amd.torch.SphericalHarmonics(5)

        def forward(self, xyz):
            sph, dsph, ddsph = self._sph.compute_with_hessians(xyz)
            return sph.sum() + dsph.sum() + ddsph.sum()

    module = Both()
    torch.testing.assert_close(torch.jit.script(module)(_xyz()), module(_xyz()), rtol=0, atol=0)


@pytest.mark.parametrize("normalized", [True, False])
def test_compile_without_graph_breaks(normalized):
    announce("compile", normalized)
    module = SHModule(10, normalized)
    a = _xyz().requires_grad_()
    b = _xyz().requires_grad_()
    eager = module(a)
    eager.sum().backward()
    compiled = torch.compile(module, fullgraph=True, backend="aot_eager")
    out = compiled(b)
    out.sum().backward()
    torch.testing.assert_close(out, eager, rtol=0, atol=0)
    torch.testing.assert_close(b.grad, a.grad, rtol=0, atol=0)
    explanation = torch._dynamo.explain(module)(_xyz())
    assert explanation.graph_count == 1 and explanation.graph_break_count == 0


@pytest.mark.parametrize("normalized", [True, False])
def test_compile_of_vmap(normalized):
    """vmap, also over an expanded, non-contiguous batch, eager and under torch.compile.
    (Forward-mode differentiation, jacfwd, is not offered: torch gives operators whose
    derivative is registered as a backward formula zero tangents, for the reference's as for
    these, so nothing is asserted about it.)"""
    announce("compile of vmap", normalized)
    module = SHModule(4, normalized)

    def single(point):
        return module(point.unsqueeze(0)).squeeze(0)

    x = _xyz(10, 7)
    eager = torch.func.vmap(single)(x)
    compiled = torch.compile(torch.func.vmap(single), fullgraph=True, backend="aot_eager")(x)
    torch.testing.assert_close(compiled, eager, rtol=0, atol=0)
    batch = _xyz(1, 8)[0].expand(5, -1)
    torch.testing.assert_close(torch.func.vmap(single)(batch), module(batch.contiguous()), rtol=0, atol=0)


@pytest.mark.parametrize("normalized", [True, False])
def test_vmap_and_jacobians(normalized):
    announce("vmap, jacobian", normalized)
    module = SHModule(4, normalized)
    x = _xyz(12, 2)

    def single(point):
        return module(point.unsqueeze(0)).squeeze(0)

    batched = torch.vmap(single)(x)
    torch.testing.assert_close(batched, module(x), rtol=0, atol=0)
    jac = torch.autograd.functional.jacobian(lambda t: module(t).sum(dim=0), x)   # [25, 12, 3]
    _, dsph = module._sph.compute_with_gradients(x)                               # [12, 3, 25]
    torch.testing.assert_close(jac, dsph.permute(2, 0, 1), rtol=1e-12, atol=1e-12)


def test_inside_a_training_loop():
    """After test_nn.py: the harmonics feed a small network and an optimiser moves the points."""
    announce("training loop")
    torch.manual_seed(4)
    sph = sphericart_amd.torch.SphericalHarmonics(3)
    net = torch.nn.Linear(16, 1, dtype=torch.float64).cuda()
    x = _xyz(64, 5).requires_grad_()
    opt = torch.optim.SGD(list(net.parameters()) + [x], lr=1e-2)
    losses = []
    for _ in range(20):
        opt.zero_grad()
        loss = (net(sph(x)) ** 2).mean()
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    assert losses[-1] < losses[0]


class ReferenceNames(torch.nn.Module):
    """Names the operators as the reference registers them (sphericart-torch/src/torch.cpp:367-385)."""

    def forward(self, xyz):
        sph = torch.ops.sphericart_torch.spherical_harmonics(xyz, 8)
        solid, dsolid = torch.ops.sphericart_torch.solid_harmonics_with_gradients(xyz, 4)
        return sph, solid, dsolid


def test_reference_namespace_resolves(oracle, tmp_path):
    """A module written against `torch.ops.sphericart_torch.*`: eager, scripted, saved and loaded;
    forward equal to the oracle number for number, xyz.grad equal to the oracle's gradients
    contracted in float64 to rounding; the two *_omp_num_threads operators exist."""
    import numpy as np

    from sphericart_amd.torch import ops

    assert ops.reference_namespace_defined
    announce("reference namespace")
    assert torch.ops.sphericart_torch.spherical_harmonics_omp_num_threads(8) == 1
    assert torch.ops.sphericart_torch.solid_harmonics_omp_num_threads(4) == 1
    assert sphericart_amd.torch.SolidHarmonics(4).omp_num_threads() == 1
    xyz_host = _xyz(257, seed=3).cpu().numpy()
    want_sph, want_dsph, _ = oracle.compute(xyz_host, 8, True, "gradients")
    want_solid, want_dsolid, _ = oracle.compute(xyz_host, 4, False, "gradients")
    script = torch.jit.script(ReferenceNames())
    path = str(tmp_path / "reference_names.pt")
    script.save(path)
    for module in (ReferenceNames(), script, torch.jit.load(path)):
        xyz = torch.from_numpy(xyz_host).cuda().requires_grad_()
        sph, solid, dsolid = module(xyz)
        np.testing.assert_array_equal(sph.detach().cpu().numpy(), want_sph)
        np.testing.assert_array_equal(solid.detach().cpu().numpy(), want_solid)
        np.testing.assert_array_equal(dsolid.detach().cpu().numpy(), want_dsolid)
        (sph.sum() + solid.sum()).backward()
        want_grad = want_dsph.sum(axis=2) + want_dsolid.sum(axis=2)
        scale = np.abs(want_dsph).sum(axis=2) + np.abs(want_dsolid).sum(axis=2)
        assert (np.abs(xyz.grad.cpu().numpy() - want_grad) <= 1e-12 * scale).all()
    with pytest.raises(RuntimeError, match="GPU"):
        torch.ops.sphericart_torch.spherical_harmonics(torch.zeros(2, 3), 3)
