"""Pins `oracle/sh_oracle.py` by what the mathematics fixes, and the package's host form of the
harmonics against it."""

import math

import numpy as np
import pytest
import torch

from e3j_amd.harmonics import Harmonics
from oracle import sh_oracle as S


def _sphere(n, seed):
    v = np.random.default_rng(seed).standard_normal((n, 3))
    return v / np.linalg.norm(v, axis=1, keepdims=True)


def test_closed_forms_of_degrees_0_to_2():
    """e3nn's published low degrees in the component normalisation: 1; sqrt(3) (x, y, z);
    sqrt(15) xz, sqrt(15) xy, sqrt(5) (y^2 - (x^2 + z^2) / 2), sqrt(15) yz, sqrt(15)/2 (z^2 - x^2)."""
    v = np.random.default_rng(0).standard_normal((64, 3))
    x, y, z = v.T
    want = np.stack([np.ones_like(x), math.sqrt(3) * x, math.sqrt(3) * y, math.sqrt(3) * z,
                     math.sqrt(15) * x * z, math.sqrt(15) * x * y, math.sqrt(5) * (y * y - 0.5 * (x * x + z * z)),
                     math.sqrt(15) * y * z, 0.5 * math.sqrt(15) * (z * z - x * x)], axis=1)
    for fn in (S.harmonics_polynomial, S.harmonics_scipy):
        np.testing.assert_allclose(fn(v, 2, False, "component"), want, rtol=1e-12, atol=1e-12)


def test_two_constructions_agree_to_degree_3():
    v = np.random.default_rng(1).standard_normal((200, 3)) * 1.3
    for normalize in (False, True):
        for normalization in ("integral", "component", "norm"):
            a = S.harmonics_polynomial(v, 3, normalize, normalization)
            b = S.harmonics_scipy(v, 3, normalize, normalization)
            np.testing.assert_allclose(a, b, rtol=1e-11, atol=1e-11)


@pytest.mark.parametrize("l_max", [3, 6])
def test_addition_theorem(l_max):
    """sum_m Y_lm(a) Y_lm(b) = (2l + 1) / (4 pi) P_l(a . b) on the sphere (integral normalisation)."""
    a, b = _sphere(50, 2), _sphere(50, 3)
    fn = S.harmonics_scipy if l_max > 3 else S.harmonics_polynomial
    ya, yb = fn(a, l_max, False, "integral"), fn(b, l_max, False, "integral")
    cos = (a * b).sum(axis=1)
    for l in range(l_max + 1):
        sl = slice(l * l, (l + 1) ** 2)
        legendre = np.polynomial.legendre.legval(cos, [0] * l + [1])
        np.testing.assert_allclose((ya[:, sl] * yb[:, sl]).sum(axis=1), (2 * l + 1) / (4 * math.pi) * legendre,
                                   rtol=1e-10, atol=1e-12)


def test_unit_norm_and_orthogonality_on_the_sphere():
    """The reference's sphere expectation (`tests/test_harmonics.py:162-176`), here by an exact
    quadrature (Gauss-Legendre in cos(theta) x uniform in phi): the Gram matrix of the integral-
    normalised functions is the identity."""
    l_max = 6
    nodes, weights = np.polynomial.legendre.leggauss(16)
    phi = 2 * math.pi * (np.arange(32) + 0.5) / 32
    ct, ph = np.meshgrid(nodes, phi, indexing="ij")
    st = np.sqrt(1 - ct * ct)
    X, Y, Z = st * np.cos(ph), st * np.sin(ph), ct
    vec = np.stack([Y, Z, X], axis=-1).reshape(-1, 3)          # input components (x, y, z) = (Y, Z, X)
    w = (weights[:, None] * np.full_like(ph, 2 * math.pi / 32)).reshape(-1)
    vals = S.harmonics_scipy(vec, l_max, False, "integral")
    gram = (vals * w[:, None]).T @ vals
    np.testing.assert_allclose(gram, np.eye((l_max + 1) ** 2), atol=1e-10)
    comp = S.harmonics_scipy(vec, l_max, False, "component")
    for l in range(l_max + 1):      # "component": |Y^l|^2 = 2l + 1 at every point; "norm": |Y^l| = 1
        np.testing.assert_allclose((comp[:, l * l:(l + 1) ** 2] ** 2).sum(axis=1), 2 * l + 1, rtol=1e-10)
    nrm = S.harmonics_scipy(vec, l_max, False, "norm")
    np.testing.assert_allclose((nrm[:, 9:16] ** 2).sum(axis=1), 1.0, rtol=1e-10)


def test_homogeneity_and_the_zero_vector():
    v = np.random.default_rng(4).standard_normal((20, 3))
    base = S.harmonics_scipy(v, 6)
    scaled = S.harmonics_scipy(2.5 * v, 6)
    for l in range(7):
        np.testing.assert_allclose(scaled[:, l * l:(l + 1) ** 2], 2.5 ** l * base[:, l * l:(l + 1) ** 2], rtol=1e-10)
    zero = S.harmonics_scipy(np.zeros((1, 3)), 4, True)
    assert abs(zero[0, 0] - 1.0) < 1e-15 and not zero[0, 1:].any()


def test_equivariance_of_degree_1_and_invariance_of_block_norms():
    """Rotating the input rotates the degree-1 block the same way (it is sqrt(3) (x, y, z)) and
    leaves the norm of every block unchanged (`tests/test_harmonics.py:207-216` without Wigner-D)."""
    rng = np.random.default_rng(5)
    q, _ = np.linalg.qr(rng.standard_normal((3, 3)))
    if np.linalg.det(q) < 0:
        q[:, 0] = -q[:, 0]
    v = rng.standard_normal((30, 3))
    a, b = S.harmonics_scipy(v, 6), S.harmonics_scipy(v @ q, 6)
    np.testing.assert_allclose(b[:, 1:4], a[:, 1:4] @ q, atol=1e-12)
    for l in range(7):
        sl = slice(l * l, (l + 1) ** 2)
        np.testing.assert_allclose((a[:, sl] ** 2).sum(1), (b[:, sl] ** 2).sum(1), rtol=1e-10)


@pytest.mark.parametrize("normalize", [False, True])
@pytest.mark.parametrize("normalization", ["integral", "component", "norm"])
def test_package_host_form_matches_the_checker(normalization, normalize):
    v = np.random.default_rng(6).standard_normal((100, 3)) * 1.4
    for l_max in range(7):
        got = Harmonics(l_max, normalize=normalize, normalization=normalization)._evaluate(torch.from_numpy(v)).numpy()
        want = S.harmonics_scipy(v, l_max, normalize, normalization)
        np.testing.assert_allclose(got, want, rtol=1e-10, atol=1e-10)
    got = Harmonics("0e+2e", normalize=normalize, normalization=normalization)._evaluate(torch.from_numpy(v)).numpy()
    want = S.harmonics_scipy(v, 2, normalize, normalization)
    np.testing.assert_allclose(got, np.concatenate([want[:, :1], want[:, 4:9]], axis=1), rtol=1e-10, atol=1e-10)


def test_central_differences_agree_with_autograd_of_the_host_form():
    v = np.random.default_rng(7).standard_normal((40, 3)) * 1.2
    dout = np.random.default_rng(8).standard_normal((40, 49))
    for normalize in (False, True):
        t = torch.from_numpy(v).requires_grad_(True)
        out = Harmonics(6, normalize=normalize)._evaluate(t)
        (g,) = torch.autograd.grad(out, t, torch.from_numpy(dout))
        fd = S.harmonics_vjp_fd(v, dout, 6, normalize)
        np.testing.assert_allclose(g.numpy(), fd, rtol=2e-6, atol=2e-6 * np.abs(fd).max())
