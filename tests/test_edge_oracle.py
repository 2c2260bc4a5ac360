"""Pins `oracle/edge_oracle.py` (edge featurisation and channel mixing on the CPU) by what the
mathematics fixes, and checks that the tensor-operation form of `EnergyModel` computes the same."""

import numpy as np
import pytest
import torch

from oracle import edge_oracle as E


def test_bessel_functions_are_the_normalised_spherical_bessel_functions():
    """`sqrt(2/rc) sin(n pi r/rc)/r = sqrt(2/rc) (n pi/rc) j0(n pi r/rc)` with scipy's j0, and the
    functions are orthonormal on the ball of radius rc with the weight r^2."""
    from scipy.integrate import quad
    from scipy.special import spherical_jn
    rc, nb = 5.0, 8
    r = np.linspace(0.05, rc, 97)
    k = np.arange(1, nb + 1) * np.pi / rc
    want = np.sqrt(2.0 / rc) * k * spherical_jn(0, k * r[:, None])
    np.testing.assert_allclose(E.bessel(r, rc, nb), want, rtol=1e-12, atol=1e-12)
    for a in range(nb):
        for b in range(a, nb):
            val, _ = quad(lambda x: E.bessel(x, rc, nb)[a] * E.bessel(x, rc, nb)[b] * x * x, 0.0, rc, limit=200)
            assert abs(val - (1.0 if a == b else 0.0)) < 1e-9, (a, b, val)
    # the limit at the origin of every function: sqrt(2/rc) n pi / rc
    np.testing.assert_allclose(E.bessel(1e-9, rc, nb), np.sqrt(2.0 / rc) * k, rtol=1e-9)


def test_envelope_is_the_smooth_cutoff():
    assert E.envelope(0.0) == 1.0 and abs(E.envelope(1.0)) < 1e-15 and E.envelope(1.7) == E.envelope(1.0)
    eps = 1e-4
    d1 = (E.envelope(1.0 - eps) - E.envelope(1.0)) / -eps      # first derivative at 1 from the left
    d2 = (E.envelope(1.0 - 2 * eps) - 2 * E.envelope(1.0 - eps) + E.envelope(1.0)) / eps ** 2
    assert abs(d1) < 1e-6 and abs(d2) < 1e-2                   # both vanish (third-order contact)
    t = np.linspace(0.0, 1.0, 51)
    assert (np.diff(E.envelope(t)) <= 0).all()                 # monotone
    h = 1e-6
    np.testing.assert_allclose(E.envelope_dt(t[1:-1]), (E.envelope(t[1:-1] + h) - E.envelope(t[1:-1] - h)) / (2 * h),
                               atol=1e-8)
    assert E.envelope_dt(1.3) == 0.0


def test_radial_derivatives_by_central_differences():
    rc, nb = 5.0, 8
    r = np.linspace(0.3, 5.6, 41)   # on both sides of the cutoff
    h = 1e-6
    fd = (E.radial_basis(r + h, rc, nb) - E.radial_basis(r - h, rc, nb)) / (2 * h)
    np.testing.assert_allclose(E.radial_basis_dr(r, rc, nb), fd, atol=2e-8)
    assert not E.radial_basis(r[r >= rc], rc, nb).any()
    v = np.linspace(-6, 6, 25)
    np.testing.assert_allclose(E.silu_dv(v), (E.silu(v + h) - E.silu(v - h)) / (2 * h), atol=1e-8)


def _problem(rng, n=12, edges=60, layers=2, nb=8, hidden=6):
    pos = rng.uniform(0.0, 4.0, size=(n, 3))
    snd = rng.integers(0, n, size=edges).astype(np.int32)
    rcv = (snd + rng.integers(1, n, size=edges)).astype(np.int32) % n      # no self edges
    shift = rng.normal(size=(edges, 3)) * 0.3
    w1 = rng.normal(size=(layers, nb, hidden)) / np.sqrt(nb)
    return pos, snd, rcv, shift, w1


def test_edge_features_vjp_by_central_differences():
    rng = np.random.default_rng(3)
    pos, snd, rcv, shift, w1 = _problem(rng)
    snd[5] = np.iinfo(np.int32).max          # a padding edge
    l_max, rc = 3, 5.0
    y, basis, hid = E.edge_features(pos, snd, rcv, shift, w1, l_max, rc)
    assert not y[5].any() and not basis[5].any() and not hid[:, 5].any()
    dy, dh, db = rng.normal(size=y.shape), rng.normal(size=hid.shape), rng.normal(size=basis.shape)

    def loss(p):
        a, b, c = E.edge_features(p, snd, rcv, shift, w1, l_max, rc)
        return (a * dy).sum() + (b * db).sum() + (c * dh).sum()

    got = E.edge_features_vjp(pos, snd, rcv, shift, w1, l_max, rc, dy, dh, dbasis=db)
    want = np.zeros_like(pos)
    h = 1e-6
    for i in range(pos.shape[0]):
        for d in range(3):
            up, dn = pos.copy(), pos.copy()
            up[i, d] += h
            dn[i, d] -= h
            want[i, d] = (loss(up) - loss(dn)) / (2 * h)
    np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-6)
    # a rigid translation changes nothing: the cotangents of the positions sum to zero
    assert np.abs(got.sum(axis=0)).max() < 1e-10


def test_channel_mix_is_the_einsum_and_its_vjp_the_transpose():
    rng = np.random.default_rng(4)
    blocks, K, n = [(4, 1), (6, 3), (7, 5), (6, 7)], 8, 5
    Z = sum(m * d for m, d in blocks)
    out = rng.normal(size=(n, Z, K))
    weights = [rng.normal(size=(m, K, K)) for m, _ in blocks]
    x = E.channel_mix(out, blocks, weights)
    rows, parts = 0, []
    for (mul, dim), w in zip(blocks, weights):
        parts.append(np.einsum("numk,ukc->nmc", out[:, rows:rows + mul * dim].reshape(n, mul, dim, K), w))
        rows += mul * dim
    np.testing.assert_allclose(x, np.concatenate(parts, axis=1), rtol=1e-13, atol=1e-13)
    dx = rng.normal(size=x.shape)
    dout = E.channel_mix_vjp(dx, blocks, weights)
    assert abs((dout * out).sum() - (dx * x).sum()) < 1e-9 * abs((dx * x).sum())   # <A^T dx, out> = <dx, A out>


def test_energy_model_tensor_form_matches_the_oracle_chain():
    """The tensor-operation form of the model's edge inputs and mixing (what the GPU kernels are also
    compared with through the end-to-end tests) against the oracle, float64 on the host."""
    from e3j_amd import workloads as W
    w = W.config5(0.01)
    model = w.model
    d = w.to("cpu", torch.float64)
    y, basis = model.edge_inputs(d.positions, d.sender, d.receiver, d.shift)
    w1 = np.stack([a for a, _ in model.mlp])
    oy, ob, oh = E.edge_features(w.positions.numpy(), w.sender.numpy(), w.receiver.numpy(), w.shift.numpy(), w1,
                                 max(model.harmonics.degrees), model.cutoff)
    np.testing.assert_allclose(y.numpy(), oy, rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(basis.numpy(), ob, rtol=1e-10, atol=1e-12)
    hid = torch.nn.functional.silu(basis @ torch.as_tensor(w1[1]))
    np.testing.assert_allclose(hid.numpy(), oh[1], rtol=1e-10, atol=1e-12)
