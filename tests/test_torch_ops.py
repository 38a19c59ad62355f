"""Torch operators: registration, shapes and error behaviour (no GPU needed), and on the GPU the
behaviours the reference's torch tests pin (sphericart-torch/python/tests/test_autograd.py,
test_cuda.py, test_cuda_stream.py, test_no_points.py), with the CPU checker as the other side."""

import numpy as np
import pytest
import torch

import sphericart_amd.torch as sphx_torch
from gpu_utils import announce

OPS = [
    f"{kind}_harmonics{suffix}"
    for kind in ("spherical", "solid")
    for suffix in ("", "_with_gradients", "_with_hessians")
]


def test_operators_are_registered_with_the_reference_schemas():
    for name in OPS:
        schema = str(getattr(torch.ops.sphericart_amd, name).default._schema)
        assert "(Tensor xyz, int l_max)" in schema, schema
    assert hasattr(torch.ops.sphericart_amd, "contract_gradients")
    assert hasattr(torch.ops.sphericart_amd, "contract_hessians")


def test_shapes_through_fake_tensors():
    from torch._subclasses.fake_tensor import FakeTensorMode

    with FakeTensorMode():
        xyz = torch.empty(7, 3, device="cuda", dtype=torch.float64)
        sph, dsph, ddsph = sphx_torch.SolidHarmonics(5).compute_with_hessians(xyz)
        assert sph.shape == (7, 36) and dsph.shape == (7, 3, 36) and ddsph.shape == (7, 3, 3, 36)
        assert sphx_torch.SphericalHarmonics(0).compute(xyz).shape == (7, 1)
        assert torch.ops.sphericart_amd.contract_gradients(dsph, sph).shape == (7, 3)
        assert torch.ops.sphericart_amd.contract_hessians(ddsph, dsph).shape == (7, 3)


def test_cpu_tensors_are_refused_loudly():
    with pytest.raises(RuntimeError, match="GPU"):
        sphx_torch.SphericalHarmonics(3).compute(torch.zeros(4, 3))
    with pytest.raises(ValueError):
        sphx_torch.SphericalHarmonics(-1)
    assert sphx_torch.SolidHarmonics(6).l_max() == 6


# ---- GPU ---------------------------------------------------------------------

def _points(n, dtype, seed=0):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal((n, 3)) * 1.5 + 0.1).astype(dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("normalized", [True, False])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("l_max", [0, 3, 6, 9])
def test_forward_equals_checker(oracle, normalized, dtype, l_max):
    announce("torch forward", normalized, dtype.__name__, l_max)
    cls = sphx_torch.SphericalHarmonics if normalized else sphx_torch.SolidHarmonics
    xyz = _points(333, dtype)
    got = cls(l_max).compute_with_hessians(torch.from_numpy(xyz).cuda())
    want = oracle.compute(xyz, l_max, normalized, "hessians")
    for g, w in zip(got, want):
        np.testing.assert_array_equal(g.cpu().numpy(), w)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(np.float32, 1e-5), (np.float64, 1e-12)])
@pytest.mark.parametrize("n_total", [1, 4, 16, 49, 81, 289, 1089])
def test_contractions_equal_checker(oracle, dtype, tol, n_total):
    """Tolerance relative to the sum of absolute terms: the device adds in another order."""
    announce("contractions", dtype.__name__, n_total)
    rng = np.random.default_rng(n_total)
    for n in (1, 63, 1000):
        dsph = rng.standard_normal((n, 3, n_total)).astype(dtype)
        ddsph = rng.standard_normal((n, 3, 3, n_total)).astype(dtype)
        g1 = rng.standard_normal((n, n_total)).astype(dtype)
        g2 = rng.standard_normal((n, 3, n_total)).astype(dtype)
        got1 = torch.ops.sphericart_amd.contract_gradients(torch.from_numpy(dsph).cuda(), torch.from_numpy(g1).cuda())
        got2 = torch.ops.sphericart_amd.contract_hessians(torch.from_numpy(ddsph).cuda(), torch.from_numpy(g2).cuda())
        scale1 = np.einsum("iak,ik->ia", np.abs(dsph), np.abs(g1)) + 1
        scale2 = np.einsum("iabk,iak->ib", np.abs(ddsph), np.abs(g2)) + 1
        assert np.max(np.abs(got1.cpu().numpy() - oracle.backward(dsph, g1)) / scale1) <= tol
        assert np.max(np.abs(got2.cpu().numpy() - oracle.backward_second(ddsph, g2)) / scale2) <= tol


@pytest.mark.gpu
@pytest.mark.parametrize("normalized", [True, False])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_fused_vjp_equals_checker_number_for_number(library, oracle, normalized, dtype):
    """sphx_vjp_* sums over k in index order with one rounding per operation, as the checker's
    contraction of the checker's gradients does: the results are identical, not merely close."""
    rng = np.random.default_rng(11)
    fn = library.sphx_vjp_f32 if dtype == np.float32 else library.sphx_vjp_f64
    stream = torch.cuda.current_stream().cuda_stream
    for l_max in range(7):
        for n in (1, 63, 64, 65, 1000, 4099):
            announce("fused vjp", normalized, np.dtype(dtype).name, l_max, n)
            xyz = _points(n, dtype, seed=l_max * 10 + n)
            weights = rng.standard_normal((n, (l_max + 1) ** 2)).astype(dtype)
            _, dsph, _ = oracle.compute(xyz, l_max, normalized, "gradients")
            want = oracle.backward(dsph, weights)
            d_xyz, d_w = torch.from_numpy(xyz).cuda(), torch.from_numpy(weights).cuda()
            out = torch.full((n, 3), float("nan"), dtype=d_xyz.dtype, device="cuda")
            status = fn(d_xyz.data_ptr(), d_w.data_ptr(), n, l_max, int(normalized), out.data_ptr(), 0, stream)
            assert status == 0, library.sphx_last_error()
            np.testing.assert_array_equal(out.cpu().numpy(), want)
            # accumulate: adds to what is there
            start = rng.standard_normal((n, 3)).astype(dtype)
            out = torch.from_numpy(start).cuda()
            assert fn(d_xyz.data_ptr(), d_w.data_ptr(), n, l_max, int(normalized), out.data_ptr(), 1, stream) == 0
            np.testing.assert_array_equal(out.cpu().numpy(), want + start)
    assert fn(d_xyz.data_ptr(), d_w.data_ptr(), 0, 3, 1, None, 0, None) == 0


@pytest.mark.gpu
@pytest.mark.parametrize("route", ["lanes", "rows"])
@pytest.mark.parametrize("normalized", [True, False])
@pytest.mark.parametrize("dtype,tol", [(np.float32, 1e-5), (np.float64, 1e-12)])
def test_fused_vjp_beyond_the_closed_forms(library, oracle, normalized, dtype, tol, route, switches):
    """l_max > 6, two routes: one point per lane with the entries kept in registers ("lanes", the
    default wherever a tile of 8 points or more fits in LDS), or the recursion kernel contracting
    its staged rows ("rows"). Either adds the terms in another order than the checker's loop,
    so the comparison is relative to the sum of absolute terms."""
    if route == "rows":
        switches("SPHX_VJP_LANES", "0")
    rng = np.random.default_rng(12)
    fn = library.sphx_vjp_f32 if dtype == np.float32 else library.sphx_vjp_f64
    stream = torch.cuda.current_stream().cuda_stream
    # (14-25: shapes where the lanes kernel has a CU to itself, with eight to sixteen waves)
    # (31, 35, 36: float32 shapes with sixteen waves, or tiles of 28 and 24 points)
    for l_max in (7, 8, 11, 14, 16, 17, 19, 21, 24, 31, 32, 35, 36):
        for n in (1, 17, 1000, 5003):
            if l_max >= 31 and n > 1000:
                continue
            announce("fused vjp", route, normalized, np.dtype(dtype).name, l_max, n)
            xyz = _points(n, dtype, seed=l_max * 10 + n)
            weights = rng.standard_normal((n, (l_max + 1) ** 2)).astype(dtype)
            _, dsph, _ = oracle.compute(xyz, l_max, normalized, "gradients")
            overflows = l_max >= 29 and dtype == np.float32
            if overflows:
                # float32 arithmetic leaves the range of the type from l = 29 (NaN and inf in the reference,
                # too): a component of a point's product is then NaN where a term of its sum is not finite,
                # and the sum of the finite terms elsewhere
                with np.errstate(invalid="ignore", over="ignore"):
                    lost = ~np.isfinite(dsph * weights[:, None, :]).all(axis=2)
                dsph = np.where(np.isfinite(dsph), dsph, 0).astype(dtype)
            want = oracle.backward(dsph, weights)
            scale = np.einsum("iak,ik->ia", np.abs(dsph), np.abs(weights)) + 1
            # the weights once aligned, once starting one element into a 16-byte vector
            holder = torch.zeros(weights.size + 1, dtype=torch.from_numpy(weights).dtype, device="cuda")
            d_xyz = torch.from_numpy(xyz).cuda()
            for shift in (0, 1):
                d_w = holder[shift:shift + weights.size].view(weights.shape)
                d_w.copy_(torch.from_numpy(weights))
                for accumulate in (0, 1):
                    start = rng.standard_normal((n, 3)).astype(dtype)
                    out = torch.from_numpy(start).cuda()
                    status = fn(d_xyz.data_ptr(), d_w.data_ptr(), n, l_max, int(normalized), out.data_ptr(),
                                accumulate, stream)
                    assert status == 0, library.sphx_last_error()
                    expect = want + start if accumulate else want
                    got = out.cpu().numpy()
                    if overflows:
                        assert (~np.isfinite(got) == lost).all(), (l_max, n, accumulate, shift)
                        got, expect = np.where(lost, 0, got), np.where(lost, 0, expect)
                    assert np.max(np.abs(got - expect) / scale) <= tol, (l_max, n, accumulate, shift)


@pytest.mark.gpu
def test_contraction_accumulates_on_request(library, oracle):
    announce("contraction accumulate flag")
    rng = np.random.default_rng(5)
    dsph = rng.standard_normal((100, 3, 49))
    grad = rng.standard_normal((100, 49))
    start = rng.standard_normal((100, 3))
    d, g, out = (torch.from_numpy(a).cuda() for a in (dsph, grad, start))
    status = library.sphx_backward_f64(d.data_ptr(), g.data_ptr(), 100, 49, out.data_ptr(), 1,
                                       torch.cuda.current_stream().cuda_stream)
    assert status == 0
    np.testing.assert_allclose(out.cpu().numpy(), start + oracle.backward(dsph, grad), rtol=0, atol=1e-12)
    assert library.sphx_backward_f64(d.data_ptr(), g.data_ptr(), 0, 49, None, 0, None) == 0
    assert library.sphx_backward_f64(d.data_ptr(), None, 100, 49, out.data_ptr(), 0, None) == 1


@pytest.mark.gpu
@pytest.mark.parametrize("normalized", [True, False])
@pytest.mark.parametrize("dtype,tol", [(np.float32, 1e-5), (np.float64, 1e-12)])
@pytest.mark.parametrize("l_max", [2, 6, 10])
def test_backward_equals_checker(oracle, normalized, dtype, tol, l_max):
    """xyz.grad of sum(w * sph) is the checker's contraction of the checker's gradients with w."""
    announce("torch backward", normalized, dtype.__name__, l_max)
    cls = sphx_torch.SphericalHarmonics if normalized else sphx_torch.SolidHarmonics
    xyz = _points(257, dtype, seed=l_max)
    weights = np.random.default_rng(1).standard_normal((257, (l_max + 1) ** 2)).astype(dtype)
    device_xyz = torch.from_numpy(xyz).cuda().requires_grad_(True)
    sph = cls(l_max).compute(device_xyz)
    (sph * torch.from_numpy(weights).cuda()).sum().backward()
    _, dsph, _ = oracle.compute(xyz, l_max, normalized, "gradients")
    want = oracle.backward(dsph, weights)
    scale = np.einsum("iak,ik->ia", np.abs(dsph), np.abs(weights)) + 1
    assert np.max(np.abs(device_xyz.grad.cpu().numpy() - want) / scale) <= tol


@pytest.mark.gpu
@pytest.mark.parametrize("normalized", [True, False])
def test_gradcheck_and_gradgradcheck(normalized):
    """As sphericart-torch/python/tests/test_autograd.py:16-47, on the device."""
    announce("gradcheck", normalized)
    cls = sphx_torch.SphericalHarmonics if normalized else sphx_torch.SolidHarmonics
    calculator = cls(l_max=4)
    torch.manual_seed(0)
    xyz = (6 * torch.randn(20, 3, dtype=torch.float64)).cuda().requires_grad_(True)

    def compute(xyz_in):
        sph = calculator.compute(xyz_in)
        assert torch.linalg.norm(sph) != 0.0
        return sph

    assert torch.autograd.gradcheck(compute, xyz, fast_mode=True)
    assert torch.autograd.gradgradcheck(compute, xyz, fast_mode=True)
    # the operators that return derivatives are differentiable as well
    assert torch.autograd.gradcheck(lambda x: calculator.compute_with_gradients(x)[1], xyz, fast_mode=True)
    assert torch.autograd.gradcheck(lambda x: calculator.compute_with_hessians(x)[1], xyz, fast_mode=True)


@pytest.mark.gpu
def test_autograd_hessian_of_a_scalar_function():
    """sphericart-torch/python/tests/test_autograd.py:50-85: sph[0..3] are proportional to 1, y, z, x."""
    announce("torch.autograd.functional.hessian")
    calculator = sphx_torch.SolidHarmonics(l_max=1)
    xyz = torch.tensor([[0.67, 0.53, -0.22]], device="cuda", requires_grad=True)

    def f(xyz):
        sph = calculator.compute(xyz)[0]
        return (sph[1] ** 2 + sph[2] + 0.20 * sph[1] * sph[3] + sph[2] ** 2
                + 0.42 * sph[1] * sph[2] + sph[0] ** 12)

    hessian = torch.autograd.functional.hessian(f, xyz)[0, :, 0, :].cpu()
    analytical = torch.tensor([[0.0, 0.2, 0.0], [0.2, 2.0, 0.42], [0.0, 0.42, 2.0]])
    factor = analytical[2, 2] / hessian[2, 2]
    assert torch.allclose(analytical, hessian * factor)


@pytest.mark.gpu
def test_third_derivatives_are_refused():
    announce("third derivatives")
    xyz = torch.randn(5, 3, device="cuda", dtype=torch.float64, requires_grad=True)
    ddsph = sphx_torch.SphericalHarmonics(3).compute_with_hessians(xyz)[2]
    with pytest.raises(RuntimeError, match="Third derivatives"):
        ddsph.sum().backward()


@pytest.mark.gpu
@pytest.mark.parametrize("normalized", [True, False])
def test_noncontiguous_input(normalized):
    """sphericart-torch/python/tests/test_autograd.py:88-124."""
    announce("noncontiguous", normalized)
    cls = sphx_torch.SphericalHarmonics if normalized else sphx_torch.SolidHarmonics
    calculator = cls(l_max=4)
    base = torch.randn(20, 6, dtype=torch.float64, device="cuda")
    xyz = base[:, ::2].detach().requires_grad_(True)
    xyz_ref = xyz.detach().clone().contiguous().requires_grad_(True)
    value, value_ref = calculator.compute(xyz), calculator.compute(xyz_ref)
    assert torch.equal(value, value_ref)
    value.sum().backward()
    value_ref.sum().backward()
    assert torch.equal(xyz.grad, xyz_ref.grad)
    for got, want in zip(calculator.compute_with_hessians(xyz), calculator.compute_with_hessians(xyz_ref)):
        assert torch.equal(got, want)


@pytest.mark.gpu
def test_no_points():
    """sphericart-torch/python/tests/test_no_points.py:32-45: empty input, empty outputs, empty gradient."""
    announce("no points")
    calculator = sphx_torch.SphericalHarmonics(l_max=5)
    xyz = torch.empty(0, 3, device="cuda", dtype=torch.float64, requires_grad=True)
    sph, dsph, ddsph = calculator.compute_with_hessians(xyz)
    assert sph.shape == (0, 36) and dsph.shape == (0, 3, 36) and ddsph.shape == (0, 3, 3, 36)
    calculator.compute(xyz).sum().backward()
    assert xyz.grad.shape == (0, 3)


@pytest.mark.gpu
def test_side_stream(oracle):
    """sphericart-torch/python/tests/test_cuda_stream.py:15-29: work goes to the current stream."""
    announce("torch side stream")
    xyz = _points(5000, np.float64, seed=3)
    device_xyz = torch.from_numpy(xyz).cuda().requires_grad_(True)
    calculator = sphx_torch.SolidHarmonics(l_max=8)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        sph = calculator.compute(device_xyz)
        sph.sum().backward()
    stream.synchronize()
    want_sph, want_dsph, _ = oracle.compute(xyz, 8, False, "gradients")
    np.testing.assert_array_equal(sph.detach().cpu().numpy(), want_sph)
    np.testing.assert_allclose(device_xyz.grad.cpu().numpy(), want_dsph.sum(axis=2), rtol=1e-11, atol=1e-9)


@pytest.mark.gpu
def test_vmap_over_a_leading_batch():
    announce("vmap")
    calculator = sphx_torch.SphericalHarmonics(l_max=3)
    xyz = torch.randn(4, 10, 3, device="cuda")
    batched = torch.vmap(calculator.compute)(xyz)
    assert batched.shape == (4, 10, 16)
    assert torch.equal(batched[2], calculator.compute(xyz[2]))
