"""The torch operators' C++ side, libsphericart_amd_torch.so (csrc/sphx_torch.cpp), after the reference's extension
(sphericart-torch/src/torch.cpp:237-294, 367-385): it is what `sphericart_amd.torch` loads when it has been built,
the Python implementations over ctypes remain behind SPHERICART_AMD_PYTHON_OPERATORS=1, both give the same
numbers, and a scripted module written against `torch.ops.sphericart_torch.*` loads and runs in a process that has
loaded nothing but that library."""

import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from gpu_utils import announce

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(code, **env):
    return subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, cwd=ROOT,
                          env=dict(os.environ, **env), timeout=300)


def test_the_library_is_built_and_is_what_the_package_loads():
    from sphericart_amd.torch import ops

    assert os.path.exists(ops.TORCH_LIBRARY_PATH), "python -m sphericart_amd.build makes it where torch is importable"
    assert ops.cpp_operators and ops.reference_namespace_defined
    for name in ("spherical_harmonics", "solid_harmonics_with_hessians", "spherical_harmonics_vjp", "contract_hessians"):
        assert hasattr(torch.ops.sphericart_amd, name)
    assert torch.ops.sphericart_torch.solid_harmonics_omp_num_threads(4) == 1
    with pytest.raises(RuntimeError, match="GPU"):
        torch.ops.sphericart_amd.solid_harmonics_with_gradients(torch.zeros(2, 3), 3)


def test_the_python_operators_remain_behind_a_switch():
    done = _run("import torch, sphericart_amd.torch.ops as o; print(o.cpp_operators, o.reference_namespace_defined, "
                "torch.ops.sphericart_amd.spherical_harmonics_with_gradients(torch.zeros(4, 3, device='meta'), 2)[1].shape)",
                SPHERICART_AMD_PYTHON_OPERATORS="1")
    assert done.returncode == 0, done.stderr
    assert done.stdout.split()[:2] == ["False", "True"] and "[4, 3, 9]" in done.stdout


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_same_numbers_as_the_python_operators_and_the_same_errors(dtype):
    from sphericart_amd.torch import ops

    assert ops.cpp_operators
    torch.manual_seed(5)
    for n, l_max, normalized in ((257, 8, True), (33, 3, False), (1000, 14, True), (0, 5, True)):
        announce("C++ operators", dtype, n, l_max, normalized)
        xyz = (3 * torch.randn(n, 3, dtype=torch.float64)).to(dtype).cuda()
        prefix = "spherical_harmonics" if normalized else "solid_harmonics"
        sph, dsph, ddsph = getattr(torch.ops.sphericart_amd, prefix + "_with_hessians")(xyz, l_max)
        want = ops._forward(xyz, l_max, normalized, 2)
        for got, expected in zip((sph, dsph, ddsph), want):
            assert got.shape == expected.shape and torch.equal(got.nan_to_num(), expected.nan_to_num())
        assert torch.equal(getattr(torch.ops.sphericart_amd, prefix)(xyz, l_max), ops._forward(xyz, l_max, normalized, 0)[0])
        both = getattr(torch.ops.sphericart_amd, prefix + "_with_gradients")(xyz, l_max)
        for got, expected in zip(both, ops._forward(xyz, l_max, normalized, 1)):
            assert torch.equal(got, expected)
        upstream = torch.randn_like(sph)
        assert torch.equal(getattr(torch.ops.sphericart_amd, prefix + "_vjp")(xyz, upstream, l_max),
                           ops._vjp(xyz, upstream, l_max, normalized))
        assert torch.equal(torch.ops.sphericart_amd.contract_gradients(dsph, upstream),
                           ops._contract("sphx_backward", dsph, upstream))
        upstream2 = torch.randn_like(dsph)
        assert torch.equal(torch.ops.sphericart_amd.contract_hessians(ddsph, upstream2),
                           ops._contract("sphx_backward_second", ddsph, upstream2))
    xyz = torch.zeros(5, 3, dtype=dtype, device="cuda")
    with pytest.raises(ValueError, match="n_samples x 3"):
        torch.ops.sphericart_amd.spherical_harmonics(xyz[:, :2], 3)
    with pytest.raises(ValueError, match="non-negative"):
        torch.ops.sphericart_amd.spherical_harmonics(xyz, -1)
    with pytest.raises(TypeError, match="float32 and float64"):
        torch.ops.sphericart_amd.spherical_harmonics(xyz.to(torch.float16), 3)
    with pytest.raises(ValueError, match="sph_grad must have shape"):
        torch.ops.sphericart_amd.spherical_harmonics_vjp(xyz, torch.zeros(5, 15, dtype=dtype, device="cuda"), 3)
    with pytest.raises(ValueError, match="do not contract"):
        torch.ops.sphericart_amd.contract_gradients(torch.zeros(5, 3, 16, dtype=dtype, device="cuda"),
                                                    torch.zeros(5, 15, dtype=dtype, device="cuda"))
    with pytest.raises(RuntimeError, match="prefactor tables"):
        torch.ops.sphericart_amd.spherical_harmonics(xyz, 65)
    # a stream other than the default one is the one the launch goes to
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        xyz = torch.randn(300, 3, dtype=dtype, device="cuda")
        got = torch.ops.sphericart_amd.solid_harmonics(xyz, 9)
    side.synchronize()
    assert torch.equal(got, ops._forward(xyz, 9, False, 0)[0])


class _ReferenceNames(torch.nn.Module):
    def forward(self, xyz):
        sph = torch.ops.sphericart_torch.spherical_harmonics(xyz, 8)
        solid, dsolid = torch.ops.sphericart_torch.solid_harmonics_with_gradients(xyz, 4)
        return sph, solid, dsolid


@pytest.mark.gpu
def test_a_saved_module_runs_with_nothing_but_the_library_loaded(oracle, tmp_path):
    import sphericart_amd.torch  # noqa: F401 (defines the operators the module is scripted against)
    from sphericart_amd.torch import ops

    announce("saved module, library alone")
    path = str(tmp_path / "reference_names.pt")
    torch.jit.script(_ReferenceNames()).save(path)
    rng = np.random.default_rng(3)
    xyz = rng.uniform(-2, 2, size=(257, 3))
    np.save(str(tmp_path / "xyz.npy"), xyz)
    code = (
        "import sys, numpy as np, torch\n"
        f"torch.ops.load_library({ops.TORCH_LIBRARY_PATH!r})\n"
        "assert 'sphericart_amd' not in sys.modules\n"
        f"module = torch.jit.load({path!r})\n"
        f"xyz = torch.from_numpy(np.load({str(tmp_path / 'xyz.npy')!r})).cuda()\n"
        "sph, solid, dsolid = module(xyz)\n"
        f"np.savez({str(tmp_path / 'out.npz')!r}, sph=sph.cpu().numpy(), solid=solid.cpu().numpy(), dsolid=dsolid.cpu().numpy())\n"
        "print(torch.ops.sphericart_torch.spherical_harmonics_omp_num_threads(8), torch.ops.sphericart_amd.owns_reference_namespace())\n"
    )
    done = _run(code)
    assert done.returncode == 0, done.stderr
    assert done.stdout.split() == ["1", "True"]
    out = np.load(str(tmp_path / "out.npz"))
    want_sph, _, _ = oracle.compute(xyz, 8, True, "values")
    want_solid, want_dsolid, _ = oracle.compute(xyz, 4, False, "gradients")
    np.testing.assert_array_equal(out["sph"], want_sph)
    np.testing.assert_array_equal(out["solid"], want_solid)
    np.testing.assert_array_equal(out["dsolid"], want_dsolid)
