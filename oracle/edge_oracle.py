"""CPU restatement (numpy, float64) of the steps around the convolution in the energy model.

TEST INFRASTRUCTURE ONLY: the checker for `e3j_amd_edge_features_fwd/bwd` and `e3j_amd_rows_regroup`
(+ the mixing products).  Nothing in the `e3j_amd` package imports it.

The reference has no module for these steps: its callers bring `edge_features` (harmonics of the edge
directions, `src/e3j/core/harmonics.py:45-101`) and `edge_scalars` (`src/e3j/core/convolution.py:342-350`)
ready-made, and mix channels per degree with `Linear` (`src/e3j/core/linear.py:125-243`).  The formulas
restated here are the published ones of the radial featurisation that message-passing models of this
family use: Bessel functions `sqrt(2 / rc) sin(n pi r / rc) / r` (the normalised zeroth spherical Bessel
functions on a ball of radius rc), the polynomial cutoff envelope of degree 5, a hidden layer with the
SiLU activation.  Pinned by (`tests/test_edge_oracle.py`): scipy's `spherical_jn` and the orthonormality
of the basis on the ball (quadrature); the envelope's values and derivatives at 0 and 1; float64 central
differences for every derivative; `sh_oracle` (itself pinned) for the harmonics; a literal loop for the mixing.
"""

from __future__ import annotations

import numpy as np

from oracle import sh_oracle


def envelope(t):
    """Cutoff envelope `1 - 10 t^3 + 15 t^4 - 6 t^5` on [0, 1], zero beyond: value 1 at 0, value and
    first two derivatives 0 at 1."""
    t = np.minimum(np.asarray(t, dtype=np.float64), 1.0)
    return 1.0 - 10.0 * t ** 3 + 15.0 * t ** 4 - 6.0 * t ** 5


def envelope_dt(t):
    t = np.asarray(t, dtype=np.float64)
    return np.where(t < 1.0, -30.0 * t ** 2 + 60.0 * t ** 3 - 30.0 * t ** 4, 0.0)


def bessel(r, cutoff: float, num_basis: int):
    """`(..., num_basis)`: `sqrt(2 / rc) sin(n pi r / rc) / r`, n = 1..num_basis (no envelope)."""
    r = np.asarray(r, dtype=np.float64)[..., None]
    n = np.arange(1, num_basis + 1, dtype=np.float64)
    return np.sqrt(2.0 / cutoff) * np.sin(n * np.pi * r / cutoff) / r


def bessel_dr(r, cutoff: float, num_basis: int):
    r = np.asarray(r, dtype=np.float64)[..., None]
    n = np.arange(1, num_basis + 1, dtype=np.float64)
    k = n * np.pi / cutoff
    return np.sqrt(2.0 / cutoff) * (k * np.cos(k * r) / r - np.sin(k * r) / r ** 2)


def radial_basis(r, cutoff: float, num_basis: int):
    r = np.asarray(r, dtype=np.float64)
    return bessel(r, cutoff, num_basis) * envelope(r / cutoff)[..., None]


def radial_basis_dr(r, cutoff: float, num_basis: int):
    r = np.asarray(r, dtype=np.float64)
    t = r / cutoff
    return (bessel_dr(r, cutoff, num_basis) * envelope(t)[..., None]
            + bessel(r, cutoff, num_basis) * (envelope_dt(t) / cutoff)[..., None])


def silu(v):
    return v / (1.0 + np.exp(-v))


def silu_dv(v):
    sg = 1.0 / (1.0 + np.exp(-v))
    return sg * (1.0 + v * (1.0 - sg))


def _edge_vectors(positions, sender, receiver, shift):
    positions = np.asarray(positions, dtype=np.float64)
    n = positions.shape[0]
    sender, receiver = np.asarray(sender, dtype=np.int64), np.asarray(receiver, dtype=np.int64)
    live = (sender >= 0) & (sender < n) & (receiver >= 0) & (receiver < n)
    vec = np.zeros((sender.shape[0], 3))
    vec[live] = positions[sender[live]] - positions[receiver[live]]
    if shift is not None:
        vec[live] += np.asarray(shift, dtype=np.float64)[live]
    r = np.linalg.norm(vec, axis=1)
    live &= r > 0
    return vec, r, live


def edge_features(positions, sender, receiver, shift, w1, l_max: int, cutoff: float,
                  normalization: str = "component"):
    """`(y (E, (l_max+1)^2), basis (E, B), h (layers, E, hidden))` in float64; edges with an endpoint
    outside the node range or of zero length get zeros."""
    w1 = np.asarray(w1, dtype=np.float64)
    vec, r, live = _edge_vectors(positions, sender, receiver, shift)
    edges = vec.shape[0]
    y = np.zeros((edges, (l_max + 1) ** 2))
    basis = np.zeros((edges, w1.shape[1]))
    h = np.zeros((w1.shape[0], edges, w1.shape[2]))
    if live.any():
        y[live] = sh_oracle.harmonics_scipy(vec[live], l_max, normalize=True, normalization=normalization)
        basis[live] = radial_basis(r[live], cutoff, w1.shape[1])
        for layer in range(w1.shape[0]):
            h[layer, live] = silu(basis[live] @ w1[layer])
    return y, basis, h


def edge_features_vjp(positions, sender, receiver, shift, w1, l_max: int, cutoff: float, dy, dh,
                      normalization: str = "component", dbasis=None):
    """Cotangent of the positions `(N, 3)` for cotangents of y, h (and optionally the basis)."""
    positions = np.asarray(positions, dtype=np.float64)
    w1 = np.asarray(w1, dtype=np.float64)
    vec, r, live = _edge_vectors(positions, sender, receiver, shift)
    dvec = np.zeros_like(vec)
    if live.any():
        v, rr = vec[live], r[live]
        u = v / rr[:, None]
        if dy is not None:
            dvec[live] += sh_oracle.harmonics_vjp_fd(v, np.asarray(dy, dtype=np.float64)[live], l_max, normalize=True,
                                                     normalization=normalization)
        basis = radial_basis(rr, cutoff, w1.shape[1])
        db = np.zeros_like(basis) if dbasis is None else np.asarray(dbasis, dtype=np.float64)[live].copy()
        if dh is not None:
            for layer in range(w1.shape[0]):
                pre = basis @ w1[layer]
                db += (np.asarray(dh, dtype=np.float64)[layer, live] * silu_dv(pre)) @ w1[layer].T
        dr = (db * radial_basis_dr(rr, cutoff, w1.shape[1])).sum(axis=1)
        dvec[live] += dr[:, None] * u
    dpos = np.zeros_like(positions)
    s, t = np.asarray(sender, dtype=np.int64)[live], np.asarray(receiver, dtype=np.int64)[live]
    np.add.at(dpos, s, dvec[live])
    np.add.at(dpos, t, -dvec[live])
    return dpos


def channel_mix(out, blocks, weights):
    """`x'[n, off_l + m, c] = sum_{u, k} out[n, base_l + u dim_l + m, k] w_l[u, k, c]`; `blocks`:
    (mul, dim) per degree in row order, `weights[l] (mul, K, K)`."""
    out = np.asarray(out, dtype=np.float64)
    n, _, channels = out.shape
    rows_out = sum(d for _, d in blocks)
    x = np.zeros((n, rows_out, channels))
    base = off = 0
    for (mul, dim), w in zip(blocks, weights):
        w = np.asarray(w, dtype=np.float64)
        for u in range(mul):
            for m in range(dim):
                x[:, off + m, :] += out[:, base + u * dim + m, :] @ w[u]
        base += mul * dim
        off += dim
    return x


def channel_mix_vjp(dx, blocks, weights):
    """Cotangent of `out` for the cotangent `dx` of `channel_mix`."""
    dx = np.asarray(dx, dtype=np.float64)
    n, _, channels = dx.shape
    rows_in = sum(m * d for m, d in blocks)
    dout = np.zeros((n, rows_in, channels))
    base = off = 0
    for (mul, dim), w in zip(blocks, weights):
        w = np.asarray(w, dtype=np.float64)
        for u in range(mul):
            for m in range(dim):
                dout[:, base + u * dim + m, :] = dx[:, off + m, :] @ w[u].T
        base += mul * dim
        off += dim
    return dout
