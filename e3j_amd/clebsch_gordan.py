"""Real-basis Clebsch-Gordan tensors of SO(3).

The reference takes these values from a third-party package that is not part
of its source tree: `e3nn_jax.clebsch_gordan` (e3nn-jax 0.21.0, the single
numeric call site is `src/e3j/core/tensor_product.py:238`).  This module
restates that package's published construction:

1. complex (Condon-Shortley) coefficients `<j1 m1 j2 m2 | j3 m3>` from Racah's
   closed form, evaluated in exact rational arithmetic;
2. change of basis from complex to real harmonics, `Q_l`, with the extra
   `(-i)^l` phase that makes every coupling tensor real;
3. `C[a, b, c] = sum Q1[i, a] Q2[k, b] conj(Q3)[c, n] C_su2[i, k, n]`;
4. scaling to unit Frobenius norm.

The only value of that package held by the reference's own files is
`|C(0; 1, 1)| = delta_ij / sqrt(3)` (`tests/test_power_expansion.py:157-158`);
it and the closed-form special cases (identity, dot product, cross product),
orthogonality and equivariance are what the tests of this module check.  The
per-path sign and basis phase beyond those are a restated convention and
cannot be compared with the third-party package here.
"""

from __future__ import annotations

import functools
from fractions import Fraction
from math import factorial, sqrt

import numpy as np


def _su2_coefficient(j1: int, m1: int, j2: int, m2: int, j3: int, m3: int) -> float:
    """`<j1 m1 j2 m2 | j3 m3>` for integer spins, Condon-Shortley phase."""
    if m3 != m1 + m2 or not abs(j1 - j2) <= j3 <= j1 + j2:
        return 0.0
    if abs(m1) > j1 or abs(m2) > j2 or abs(m3) > j3:
        return 0.0
    prefactor = Fraction(
        (2 * j3 + 1)
        * factorial(j3 + j1 - j2) * factorial(j3 - j1 + j2) * factorial(j1 + j2 - j3),
        factorial(j1 + j2 + j3 + 1),
    ) * (
        factorial(j3 + m3) * factorial(j3 - m3)
        * factorial(j1 - m1) * factorial(j1 + m1)
        * factorial(j2 - m2) * factorial(j2 + m2)
    )
    total = Fraction(0)
    for k in range(0, j1 + j2 - j3 + 1):
        denominators = (
            k, j1 + j2 - j3 - k, j1 - m1 - k, j2 + m2 - k,
            j3 - j2 + m1 + k, j3 - j1 - m2 + k,
        )
        if min(denominators) < 0:
            continue
        term = Fraction(1)
        for d in denominators:
            term /= factorial(d)
        total += term if k % 2 == 0 else -term
    return float(total) * sqrt(float(prefactor))


def su2_clebsch_gordan(j1: int, j2: int, j3: int) -> np.ndarray:
    """Dense `(2j1+1, 2j2+1, 2j3+1)` array indexed by `m + j`."""
    out = np.zeros((2 * j1 + 1, 2 * j2 + 1, 2 * j3 + 1), dtype=np.float64)
    for m1 in range(-j1, j1 + 1):
        for m2 in range(-j2, j2 + 1):
            m3 = m1 + m2
            if abs(m3) <= j3:
                out[j1 + m1, j2 + m2, j3 + m3] = _su2_coefficient(j1, m1, j2, m2, j3, m3)
    return out


def change_basis_real_to_complex(l: int) -> np.ndarray:
    """`Q_l` with complex harmonics on the rows and real harmonics on the columns.

    Real components are ordered `m = -l..l` (sine-like, zonal, cosine-like),
    which for `l = 1` is `(y, z, x)` of the standard frame.
    """
    q = np.zeros((2 * l + 1, 2 * l + 1), dtype=np.complex128)
    inv_sqrt2 = 1.0 / sqrt(2.0)
    for m in range(-l, 0):
        q[l + m, l + abs(m)] = inv_sqrt2
        q[l + m, l - abs(m)] = -1j * inv_sqrt2
    q[l, l] = 1.0
    for m in range(1, l + 1):
        q[l + m, l + abs(m)] = (-1) ** m * inv_sqrt2
        q[l + m, l - abs(m)] = 1j * (-1) ** m * inv_sqrt2
    return (-1j) ** l * q


@functools.lru_cache(maxsize=None)
def _clebsch_gordan_cached(l1: int, l2: int, l3: int) -> np.ndarray:
    if not abs(l2 - l3) <= l1 <= l2 + l3:
        raise ValueError(f"({l1}, {l2}, {l3}) violates the triangle inequality")
    c = su2_clebsch_gordan(l1, l2, l3).astype(np.complex128)
    q1 = change_basis_real_to_complex(l1)
    q2 = change_basis_real_to_complex(l2)
    q3 = change_basis_real_to_complex(l3)
    c = np.einsum("ij,kl,mn,ikn->jlm", q1, q2, np.conj(q3.T), c)
    if np.abs(c.imag).max() > 1e-9:
        raise AssertionError("real-basis coupling tensor has an imaginary part")
    c = np.ascontiguousarray(c.real)
    c[np.abs(c) < 1e-14] = 0.0
    c /= np.linalg.norm(c)
    c.setflags(write=False)
    return c


def clebsch_gordan(l1: int, l2: int, l3: int) -> np.ndarray:
    """Real coupling tensor `C[m1, m2, m3]` of degrees `(l1, l2, l3)`, unit Frobenius norm.

    The index order is the argument order; the reference calls it as
    `(l_out, l_x, l_y)` (`src/e3j/core/tensor_product.py:238`).
    """
    return _clebsch_gordan_cached(int(l1), int(l2), int(l3))
