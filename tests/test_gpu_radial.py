"""`radial_linear`: the matrix-core kernel of the radial network's last layer against the same
product in float64 (tolerance: float32 sums of `inner` terms)."""

import pytest
import torch

from e3j_amd import _lib
from e3j_amd.radial import radial_linear

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("inner", [8, 16, 32, 64, 128])
@pytest.mark.parametrize("edges,n", [(1, 32), (31, 64), (256, 1472), (257, 2944), (1000, 96)])
def test_forward_matches_the_float64_product(inner, edges, n):
    g = torch.Generator(device="cuda").manual_seed(inner * 1000 + edges)
    h = torch.randn(edges, inner, device="cuda", generator=g)
    w = torch.randn(inner, n, device="cuda", generator=g)
    s = radial_linear(h, w)
    want = h.double() @ w.double()
    bound = 1e-6 + 1e-5 * want.abs() + 8 * 2.0 ** -24 * (h.double().abs() @ w.double().abs())
    assert s.shape == (edges, n) and s.dtype == torch.float32
    assert bool(((s.double() - want).abs() <= bound).all())


@pytest.mark.parametrize("inner", [32, 64, 128])
def test_every_row_and_column_lands_in_its_place(inner):
    """h = one-hot rows, w = distinct integers: s[e, :] must be row (e mod inner) of w exactly
    (also on the kernels that split their operands three ways: integers below 2^24 split exactly)."""
    edges, n = 333, 160
    h = torch.zeros(edges, inner, device="cuda")
    h[torch.arange(edges), torch.arange(edges) % inner] = 1.0
    w = torch.arange(inner * n, device="cuda", dtype=torch.float32).reshape(inner, n)
    assert torch.equal(radial_linear(h, w), w[torch.arange(edges, device="cuda") % inner])


def test_gradients_and_errors():
    g = torch.Generator(device="cuda").manual_seed(5)
    h = torch.randn(100, 32, device="cuda", generator=g, requires_grad=True)
    w = torch.randn(32, 64, device="cuda", generator=g, requires_grad=True)
    ds = torch.randn(100, 64, device="cuda", generator=g)
    dh, dw = torch.autograd.grad(radial_linear(h, w), (h, w), ds)
    torch.testing.assert_close(dh, ds @ w.detach().t(), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(dw, h.detach().t() @ ds, rtol=1e-5, atol=1e-5)
    assert radial_linear(h[:0], w).shape == (0, 64)
    with pytest.raises(ValueError, match="multiple of 32"):
        radial_linear(h, w[:, :40])
    with pytest.raises(ValueError):
        radial_linear(h[:, :24], w[:24])
    lib = _lib.load()
    assert lib.e3j_amd_radial_linear_fwd(None, None, None, 4, 24, 64, None) == _lib.UNIMPLEMENTED
    assert lib.e3j_amd_radial_linear_fwd(None, None, None, 4, 32, 64, None) == _lib.INVALID_ARGUMENT


@pytest.mark.parametrize("inner", [8, 16, 32, 64, 128])
@pytest.mark.parametrize("edges,n", [(1, 32), (70, 128), (4099, 1472), (20001, 96)])
def test_weight_gradient_matches_the_float64_product_and_repeats(inner, edges, n):
    g = torch.Generator(device="cuda").manual_seed(inner * 31 + edges)
    h = torch.randn(edges, inner, device="cuda", generator=g)
    w = torch.randn(inner, n, device="cuda", generator=g, requires_grad=True)
    ds = torch.randn(edges, n, device="cuda", generator=g)
    (dw,) = torch.autograd.grad(radial_linear(h, w), (w,), ds)
    want = h.double().t() @ ds.double()
    bound = 1e-6 + 1e-5 * want.abs() + 16 * 2.0 ** -24 * (h.double().abs().t() @ ds.double().abs())
    assert dw.shape == (inner, n)
    assert bool(((dw.double() - want).abs() <= bound).all())
    (again,) = torch.autograd.grad(radial_linear(h, w), (w,), ds)
    assert torch.equal(dw, again)   # fixed summation order over the edges


def test_second_derivative_goes_through_the_library_products():
    g = torch.Generator(device="cuda").manual_seed(9)
    h = torch.randn(50, 16, device="cuda", generator=g, requires_grad=True)
    w = torch.randn(16, 64, device="cuda", generator=g, requires_grad=True)
    ds = torch.randn(50, 64, device="cuda", generator=g, requires_grad=True)
    dh, dw = torch.autograd.grad(radial_linear(h, w), (h, w), ds, create_graph=True)
    (dds,) = torch.autograd.grad((dh.sum() + dw.sum()), (ds,))
    want = (torch.ones_like(dh) @ w + h @ torch.ones_like(dw)).detach()
    torch.testing.assert_close(dds, want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("inner", [32, 64, 128])
@pytest.mark.parametrize("edges,n", [(1, 32), (33, 64), (257, 1472), (1000, 2944)])
def test_input_gradient_matches_the_float64_product(inner, edges, n):
    g = torch.Generator(device="cuda").manual_seed(inner * 77 + edges)
    h = torch.randn(edges, inner, device="cuda", generator=g, requires_grad=True)
    w = torch.randn(inner, n, device="cuda", generator=g)
    ds = torch.randn(edges, n, device="cuda", generator=g)
    (dh,) = torch.autograd.grad(radial_linear(h, w), (h,), ds)
    want = ds.double() @ w.double().t()
    bound = 1e-6 + 1e-5 * want.abs() + 16 * 2.0 ** -24 * (ds.double().abs() @ w.double().abs().t())
    assert dh.shape == (edges, inner)
    assert bool(((dh.double() - want).abs() <= bound).all())
    # one-hot cotangent rows pick rows of w^T exactly (integers split exactly)
    wi = torch.arange(inner * n, device="cuda", dtype=torch.float32).reshape(inner, n) % 4093
    pick = torch.zeros(edges, n, device="cuda")
    pick[torch.arange(edges), (torch.arange(edges) * 7) % n] = 1.0
    (picked,) = torch.autograd.grad(radial_linear(h, wi), (h,), pick)
    assert torch.equal(picked, wi.t()[(torch.arange(edges, device="cuda") * 7) % n])
