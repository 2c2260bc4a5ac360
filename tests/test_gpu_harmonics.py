"""The spherical-harmonics kernels against the CPU checker `oracle/sh_oracle.py` (values from
scipy's harmonics and, to degree 3, the textbook polynomials; cotangents from float64 central
differences), and against the package's tensor-operation form of the same functions."""

import numpy as np
import pytest
import torch

from e3j_amd import _lib
from e3j_amd.harmonics import Harmonics
from oracle import sh_oracle

pytestmark = pytest.mark.gpu


def _vectors(n, dtype, seed=0):
    v = np.random.default_rng(seed).standard_normal((n, 3)) * 1.7
    return torch.from_numpy(v).to(dtype).cuda()


@pytest.mark.parametrize("dtype, tol", [(torch.float64, 1e-11), (torch.float32, 2e-6)])
@pytest.mark.parametrize("normalize", [False, True])
@pytest.mark.parametrize("normalization", ["component", "integral", "norm"])
def test_kernel_matches_checker(normalization, normalize, dtype, tol):
    """`e3j_amd_harmonics` against the scipy-based checker (and the polynomial table to degree 3);
    `e3j_amd_harmonics_bwd` against float64 central differences of the checker."""
    for l_max in range(7):
        h = Harmonics(l_max, normalize=normalize, normalization=normalization)
        v = _vectors(400, dtype, seed=10 + l_max).requires_grad_(True)
        got = h(v)
        host = v.detach().cpu().numpy().astype(np.float64)
        want = sh_oracle.harmonics_scipy(host, l_max, normalize, normalization)
        scale = np.abs(want).max()
        assert np.abs(got.detach().cpu().numpy() - want).max() <= tol * scale, (l_max, "values")
        if l_max <= 3:
            table = sh_oracle.harmonics_polynomial(host, l_max, normalize, normalization)
            assert np.abs(got.detach().cpu().numpy() - table).max() <= tol * scale, (l_max, "polynomial table")
        dout = np.random.default_rng(11).standard_normal(want.shape)
        (g,) = torch.autograd.grad(got, v, torch.from_numpy(dout).to(dtype).cuda())
        fd = sh_oracle.harmonics_vjp_fd(host, dout, l_max, normalize, normalization)
        bound = max(4 * tol, 2e-6) * (np.abs(fd).max() + 1e-30)   # the differences carry 1e-6 of their own
        assert np.abs(g.cpu().numpy() - fd).max() <= bound, (l_max, "gradient")


@pytest.mark.parametrize("dtype, tol", [(torch.float64, 1e-12), (torch.float32, 2e-6)])
@pytest.mark.parametrize("normalize", [False, True])
@pytest.mark.parametrize("normalization", ["component", "integral", "norm"])
def test_kernel_matches_tensor_form(normalization, normalize, dtype, tol):
    for l_max in range(7):
        h = Harmonics(l_max, normalize=normalize, normalization=normalization)
        v = _vectors(1000, dtype, seed=l_max).requires_grad_(True)
        got = h(v)
        want = h._evaluate(v)
        assert got.shape == want.shape == (1000, (l_max + 1) ** 2)
        scale = float(want.detach().abs().max())
        assert float((got - want).detach().abs().max()) <= tol * scale, (l_max, "values")
        dout = torch.from_numpy(np.random.default_rng(9).standard_normal(tuple(want.shape))).to(dtype).cuda()
        (g,) = torch.autograd.grad(got, v, dout)
        if l_max == 0:                                   # a constant: no gradient
            assert not g.any()
            continue
        (gw,) = torch.autograd.grad(want, v, dout)
        assert float((g - gw).abs().max()) <= 4 * tol * float(gw.abs().max() + 1e-30), (l_max, "gradient")


def test_batched_shapes_zero_vectors_and_fallbacks():
    h = Harmonics(3, normalize=True)
    v = _vectors(24, torch.float32).reshape(2, 3, 4, 3).clone()
    v[0, 0, 0] = 0.0                                   # projected on the sphere: left at the origin
    out = h(v.requires_grad_(True))
    assert out.shape == (2, 3, 4, 16) and torch.isfinite(out).all()
    (g,) = torch.autograd.grad(out.sum(), v)
    assert torch.isfinite(g).all()
    assert torch.allclose(out[0, 0, 0, 1:], torch.zeros(15, device="cuda"))
    # targets that are not 0..l_max, and host tensors, take the tensor-operation form
    partial = Harmonics("0e+2e")
    assert partial(_vectors(5, torch.float32)).shape == (5, 6)
    assert Harmonics(2)(_vectors(5, torch.float32).cpu()).shape == (5, 9)


def test_second_derivative_goes_through_the_tensor_form():
    h = Harmonics(3, normalize=True)
    v = _vectors(50, torch.float64, seed=4).requires_grad_(True)
    w = v.detach().clone().requires_grad_(True)
    weights = torch.from_numpy(np.random.default_rng(5).standard_normal((50, 16))).cuda()

    def curvature(out, vec):
        (g,) = torch.autograd.grad((out * weights).sum(), vec, create_graph=True)
        (gg,) = torch.autograd.grad((g ** 2).sum(), vec)
        return gg

    torch.testing.assert_close(curvature(h(v), v), curvature(h._evaluate(w), w), rtol=1e-10, atol=1e-10)


def test_abi_errors():
    lib = _lib.load()
    v = _vectors(4, torch.float32)
    out = torch.empty(4, 64, device="cuda")
    assert lib.e3j_amd_harmonics(v.data_ptr(), 4, 7, 0, 1, _lib.F32, out.data_ptr(), None) == _lib.UNIMPLEMENTED
    assert lib.e3j_amd_harmonics(v.data_ptr(), 4, 2, 0, 5, _lib.F32, out.data_ptr(), None) == _lib.INVALID_ARGUMENT
    assert lib.e3j_amd_harmonics(None, 4, 2, 0, 1, _lib.F32, out.data_ptr(), None) == _lib.INVALID_ARGUMENT
    assert lib.e3j_amd_harmonics(None, 0, 2, 0, 1, _lib.F32, None, None) == _lib.OK


def test_torch_func_transforms():
    """vmap over a batch of vector lists and second derivatives through `torch.func`."""
    from torch.func import grad, vmap
    from e3j_amd.harmonics import Harmonics
    h = Harmonics(3, normalize=True)
    g = torch.Generator().manual_seed(3)
    r = torch.randn(4, 11, 3, generator=g, dtype=torch.float64).cuda()
    torch.testing.assert_close(vmap(h)(r), torch.stack([h._evaluate(r[b]) for b in range(4)]))
    w = torch.randn(11, 16, generator=g, dtype=torch.float64).cuda()
    energy = lambda fn: (lambda v: (fn(v) * w).sum())  # noqa: E731
    torch.testing.assert_close(grad(energy(h))(r[0]), grad(energy(h._evaluate))(r[0]))
    second = lambda fn: grad(lambda v: (grad(energy(fn))(v) ** 2).sum())  # noqa: E731
    torch.testing.assert_close(second(h)(r[0]), second(h._evaluate)(r[0]))
    torch.testing.assert_close(vmap(grad(energy(h)))(r), vmap(grad(energy(h._evaluate)))(r))
