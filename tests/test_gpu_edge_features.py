"""The producer chain of the convolution's operands and the mixing after it as kernels:
`edge_features` (positions -> harmonics and hidden radial layers, one launch each way) and
`ChannelMix` (row regrouping around the per-degree products) against `oracle/edge_oracle.py`."""

import numpy as np
import pytest
import torch

from e3j_amd import ChannelMix, edge_features
from oracle import edge_oracle as E

pytestmark = pytest.mark.gpu


def _problem(seed, n=200, edges=3000, layers=2, nb=8, hidden=32, padding=True, shift=True):
    rng = np.random.default_rng(seed)
    pos = rng.uniform(0.0, 9.0, size=(n, 3))
    snd = rng.integers(0, n, size=edges).astype(np.int32)
    rcv = ((snd + rng.integers(1, n, size=edges)) % n).astype(np.int32)
    if padding:
        snd[::97] = np.iinfo(np.int32).max
        rcv[13::101] = np.iinfo(np.int32).max
        rcv[7] = snd[7]                                 # a self edge of zero length (no shift on it)
    sh = rng.normal(size=(edges, 3)) * 0.5 if shift else None
    if sh is not None and padding:
        sh[7] = 0.0
    w1 = rng.normal(size=(layers, nb, hidden)) / np.sqrt(nb)
    return pos, snd, rcv, sh, w1


def _dev(a, dtype):
    return None if a is None else torch.as_tensor(a).to("cuda", dtype if a.dtype.kind == "f" else None)


@pytest.mark.parametrize("dtype,l_max,shift", [(torch.float32, 3, True), (torch.float64, 3, True),
                                               (torch.float32, 2, False), (torch.float64, 6, True),
                                               (torch.float32, 0, True)])
def test_edge_features_forward_and_backward_match_the_oracle(dtype, l_max, shift):
    pos, snd, rcv, sh, w1 = _problem(1 + l_max, shift=shift)
    rc = 5.0
    oy, _, oh = E.edge_features(pos, snd, rcv, sh, w1, l_max, rc)
    p = _dev(pos, dtype).requires_grad_(True)
    y, h = edge_features(p, _dev(snd, None), _dev(rcv, None), _dev(sh, dtype), _dev(w1, dtype), l_max, rc)
    assert y.dtype == dtype and h.shape == (w1.shape[0], snd.shape[0], w1.shape[2])
    # float32: 1e-5 relative, and absolutely 1e-5 = a few roundings of the largest terms of the sums
    # (degree-3 harmonics in the component normalisation add terms of magnitude up to about 10)
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(y.detach().cpu().numpy(), oy, **tol)
    np.testing.assert_allclose(h.detach().cpu().numpy(), oh, **tol)
    dead = (snd >= pos.shape[0]) | (rcv >= pos.shape[0]) | (np.arange(len(snd)) == 7) & (snd == rcv)
    assert dead.any() and not y.detach()[torch.as_tensor(dead).cuda()].any()      # exact zeros
    rng = np.random.default_rng(9)
    dy, dh = rng.normal(size=oy.shape), rng.normal(size=oh.shape)
    (got,) = torch.autograd.grad((y * _dev(dy, dtype)).sum() + (h * _dev(dh, dtype)).sum(), p, retain_graph=True)
    want = E.edge_features_vjp(pos, snd, rcv, sh, w1, l_max, rc, dy, dh)
    scale = np.abs(want).max()
    err = np.abs(got.cpu().numpy() - want).max()
    assert err <= (2e-5 if dtype == torch.float32 else 1e-7) * scale, (err, scale)   # (oracle's harmonics VJP: central differences)
    # only one of the two cotangents
    (gy,) = torch.autograd.grad((y * _dev(dy, dtype)).sum(), p)
    want_y = E.edge_features_vjp(pos, snd, rcv, sh, w1, l_max, rc, dy, None)
    assert np.abs(gy.cpu().numpy() - want_y).max() <= (2e-5 if dtype == torch.float32 else 1e-7) * max(np.abs(want_y).max(), 1e-30)


def test_edge_features_on_an_empty_edge_list_and_errors():
    pos = torch.rand(5, 3, device="cuda", requires_grad=True)
    none = torch.zeros(0, dtype=torch.int32, device="cuda")
    w1 = torch.rand(2, 8, 16, device="cuda")
    y, h = edge_features(pos, none, none, None, w1, 3, 5.0)
    assert y.shape == (0, 16) and h.shape == (2, 0, 16)
    (g,) = torch.autograd.grad(y.sum() + h.sum(), pos)
    assert not g.any()
    with pytest.raises(ValueError):
        edge_features(pos.cpu(), none.cpu(), none.cpu(), None, w1.cpu(), 3, 5.0)
    with pytest.raises(ValueError):
        edge_features(pos, none, none, None, torch.rand(1, 17, 4, device="cuda"), 3, 5.0)


@pytest.mark.parametrize("dtype,K", [(torch.float32, 64), (torch.float32, 128), (torch.float32, 32),
                                     (torch.float64, 64)])
def test_channel_mix_matches_the_oracle(dtype, K):
    """float32 at 64 and 128 channels: the matrix-core kernel, one launch each way; 32 channels and
    float64: row regrouping around library products.  37 nodes: a whole tile of 32 and a partial one."""
    rng = np.random.default_rng(5)
    blocks, n = [(4, 1), (6, 3), (7, 5), (6, 7)], 37
    Z = sum(m * d for m, d in blocks)
    out = rng.normal(size=(n, Z, K))
    weights = [rng.normal(size=(m, K, K)) / np.sqrt(m * K) for m, _ in blocks]
    mixer = ChannelMix(blocks, K, weights)
    o = torch.as_tensor(out).to("cuda", dtype).requires_grad_(True)
    x = mixer(o)
    want = E.channel_mix(out, blocks, weights)
    tol = 2e-5 if dtype == torch.float32 else 1e-12
    assert np.abs(x.detach().cpu().numpy() - want).max() <= tol * np.abs(want).max()
    dx = rng.normal(size=want.shape)
    (g,) = torch.autograd.grad(x, o, torch.as_tensor(dx).to("cuda", dtype))
    want_g = E.channel_mix_vjp(dx, blocks, weights)
    assert np.abs(g.cpu().numpy() - want_g).max() <= tol * np.abs(want_g).max()
    # a second size through the same object (row tables are per node count)
    o2 = torch.as_tensor(out[:3]).to("cuda", dtype)
    assert np.abs(mixer(o2).cpu().numpy() - want[:3]).max() <= tol * np.abs(want).max()
    with pytest.raises(ValueError):
        mixer(o2[:, :-1])
