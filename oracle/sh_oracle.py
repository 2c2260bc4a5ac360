"""CPU checker of the real spherical harmonics of edge vectors.  TEST INFRASTRUCTURE ONLY:
nothing under `e3j_amd/` imports this module.

Restates the conventions of the reference's `Harmonics` module without its ladder-operator
construction:

* frame: the physical axes `(X, Y, Z)` of the textbook definition are the input components
  `(z, x, y)` (`src/e3j/utils/spherical_harmonics.py:33-38`), so the degree-1 block is
  proportional to `(x, y, z)`;
* real harmonics in the standard sign convention, ordered `m = -l..l`
  (`src/e3j/utils/spherical_harmonics.py:66-75`; with the complex harmonics of that file,
  `Y(l, l) = +(X + iY)^l / norm` stepped down by `J_`, the signs `(-1)^(l+m)` / `(-1)^(l+1)` of
  `:68` reduce to `sqrt(2) N_lm P_l^m(cos t) cos(m p)` for `m > 0` and `... sin(|m| p)` for
  `m < 0`, with `P_l^m` taken without the Condon-Shortley phase);
* homogeneous polynomials of degree `l` (a vector of length `r` gives `r^l` times the value on
  the sphere) unless `normalize` projects the vectors on the sphere first
  (`src/e3j/core/harmonics.py:92-101`);
* block scalings `integral` (unit L2 norm on the sphere), `component` (times `sqrt(4 pi)`),
  `norm` (times `sqrt(4 pi / (2 l + 1))`) (`src/e3j/core/harmonics.py:25-42`).

Two constructions that share no code: `harmonics_polynomial` (the explicit Cartesian polynomials of
degrees 0..3 from the textbook table of real harmonics) and `harmonics_scipy` (degrees 0..6+
from scipy's complex harmonics).  `tests/test_sh_oracle.py` pins them against each other, the
closed forms of degrees 0..2, the addition theorem and the unit L2 norm on the sphere of the
reference's own test (`tests/test_harmonics.py:162-176`).  What stays unpinned is agreement with
the third-party e3nn_jax values, which the reference checks at run time only
(`tests/test_harmonics.py:178-182`).
"""

from __future__ import annotations

import math

import numpy as np


def block_scale(l: int, normalization: str) -> float:
    if normalization == "integral":
        return 1.0
    if normalization == "component":
        return math.sqrt(4.0 * math.pi)
    if normalization == "norm":
        return math.sqrt(4.0 * math.pi / (2 * l + 1))
    raise ValueError(normalization)


def _prepare(vec, normalize):
    v = np.asarray(vec, dtype=np.float64)
    if normalize:
        n = np.linalg.norm(v, axis=-1, keepdims=True)
        v = v / np.where(n > 0, n, 1.0)
    return v


def harmonics_polynomial(vec, l_max: int, normalize: bool = False, normalization: str = "component"):
    """Degrees 0..l_max (l_max <= 3) as explicit polynomials; `(..., (l_max + 1)^2)` float64."""
    if l_max > 3:
        raise ValueError("the polynomial table stops at degree 3")
    v = _prepare(vec, normalize)
    X, Y, Z = v[..., 2], v[..., 0], v[..., 1]   # harmonic frame: (X, Y, Z) = (z, x, y) of the input
    r2 = X * X + Y * Y + Z * Z
    pi = math.pi
    table = [
        [0.5 * math.sqrt(1 / pi) * np.ones_like(X)],
        [math.sqrt(3 / (4 * pi)) * Y, math.sqrt(3 / (4 * pi)) * Z, math.sqrt(3 / (4 * pi)) * X],
        [0.5 * math.sqrt(15 / pi) * X * Y, 0.5 * math.sqrt(15 / pi) * Y * Z,
         0.25 * math.sqrt(5 / pi) * (3 * Z * Z - r2), 0.5 * math.sqrt(15 / pi) * X * Z,
         0.25 * math.sqrt(15 / pi) * (X * X - Y * Y)],
        [0.25 * math.sqrt(35 / (2 * pi)) * Y * (3 * X * X - Y * Y), 0.5 * math.sqrt(105 / pi) * X * Y * Z,
         0.25 * math.sqrt(21 / (2 * pi)) * Y * (5 * Z * Z - r2), 0.25 * math.sqrt(7 / pi) * (5 * Z ** 3 - 3 * Z * r2),
         0.25 * math.sqrt(21 / (2 * pi)) * X * (5 * Z * Z - r2), 0.25 * math.sqrt(105 / pi) * (X * X - Y * Y) * Z,
         0.25 * math.sqrt(35 / (2 * pi)) * X * (X * X - 3 * Y * Y)],
    ]
    blocks = [block_scale(l, normalization) * np.stack(table[l], axis=-1) for l in range(l_max + 1)]
    return np.concatenate(blocks, axis=-1)


def harmonics_scipy(vec, l_max: int, normalize: bool = False, normalization: str = "component"):
    """Degrees 0..l_max from scipy's complex harmonics; `(..., (l_max + 1)^2)` float64."""
    from scipy.special import sph_harm_y
    v = _prepare(vec, normalize)
    X, Y, Z = v[..., 2], v[..., 0], v[..., 1]
    r = np.sqrt(X * X + Y * Y + Z * Z)
    safe = np.where(r > 0, r, 1.0)
    theta = np.arccos(np.clip(np.where(r > 0, Z / safe, 1.0), -1.0, 1.0))   # polar angle from Z
    phi = np.arctan2(Y, X)
    blocks = []
    for l in range(l_max + 1):
        comps = []
        for m in range(-l, l + 1):
            ylm = sph_harm_y(l, abs(m), theta, phi)    # Condon-Shortley phase included
            if m == 0:
                val = ylm.real
            elif m > 0:
                val = (-1) ** m * math.sqrt(2.0) * ylm.real
            else:
                val = (-1) ** m * math.sqrt(2.0) * ylm.imag
            comps.append(val * r ** l)                 # homogeneous of degree l
        blocks.append(block_scale(l, normalization) * np.stack(comps, axis=-1))
    out = np.concatenate(blocks, axis=-1)
    if l_max > 0:                                      # the zero vector: every degree above 0 vanishes
        out[..., 1:] = np.where((r > 0)[..., None], out[..., 1:], 0.0)
    return out


def harmonics_vjp_fd(vec, dout, l_max: int, normalize: bool = False, normalization: str = "component",
                     step: float = 1e-6):
    """Vector-Jacobian product by float64 central differences of `harmonics_scipy`."""
    v = np.asarray(vec, dtype=np.float64)
    dout = np.asarray(dout, dtype=np.float64)
    grad = np.zeros_like(v)
    for a in range(3):
        e = np.zeros(3)
        e[a] = step
        up = harmonics_scipy(v + e, l_max, normalize, normalization)
        dn = harmonics_scipy(v - e, l_max, normalize, normalization)
        grad[..., a] = ((up - dn) / (2 * step) * dout).sum(axis=-1)
    return grad
