"""Shared builders and the parity criterion of the test-suite."""

from __future__ import annotations


import collections
import hashlib

import numpy as np

from oracle import conv_oracle as O

EPS32 = float(np.finfo(np.float32).eps)


# ---------------------------------------------------------------------------
# problem builders
# ---------------------------------------------------------------------------
def random_table(rng, nnz, num_x, num_y, num_out, num_scalars):
    """Random sparse table covering every out/x/y coordinate, sorted by output index.

    Construction of the reference's op tests (tests/test_ops/test_convolution_op.py:102-131).
    Returns idx (nnz, 3), val (nnz,), mix_idx (num_out,).
    """
    def make(dim):
        extra = rng.integers(0, max(dim - 1, 1), size=max(nnz - dim, 0))
        return np.concatenate([np.arange(dim), extra])[:max(nnz, dim)]
    n = max(nnz, num_x, num_y, num_out)
    cols = []
    for dim in (num_out, num_x, num_y):
        c = make(dim)
        if c.shape[0] < n:
            c = np.concatenate([c, rng.integers(0, dim, size=n - c.shape[0])])
        cols.append(c[:n])
    order = np.argsort(cols[0], kind="stable")
    idx = np.stack(cols, axis=-1)[order]
    val = rng.normal(size=n).astype(np.float32)
    mix = np.sort(np.concatenate([np.arange(num_scalars),
                                  rng.integers(0, num_scalars, size=num_out - num_scalars)]))
    return idx, val, mix


def random_graph(rng, num_nodes, num_edges, sort_by="receiver"):
    sender = rng.integers(0, num_nodes, size=num_edges).astype(np.int32)
    receiver = rng.integers(0, num_nodes, size=num_edges).astype(np.int32)
    if sort_by == "receiver":
        order = np.argsort(receiver, kind="stable")
    elif sort_by == "sender":
        order = np.argsort(sender, kind="stable")
    else:
        order = np.arange(num_edges)
    return sender[order], receiver[order]


def random_operands(rng, num_nodes, num_edges, num_x, num_y, num_scalars, channels, num_out,
                    dtype=np.float32):
    x = rng.normal(size=(num_nodes, num_x, channels)).astype(dtype)
    y = rng.normal(size=(num_edges, num_y)).astype(dtype)
    s = rng.normal(size=(num_edges, num_scalars, channels)).astype(dtype)
    dm = rng.normal(size=(num_nodes, num_out, channels)).astype(dtype)
    return x, y, s, dm


def pack_table(idx, val, mix_idx, val_dtype=np.float32, idx_dtype=None):
    from e3j_amd.coef import Coef4D
    from e3j_amd.sparse import narrow_index_dtype
    idx = np.asarray(idx)
    idx4 = np.concatenate([idx, np.asarray(mix_idx)[idx[:, 0]][:, None]], axis=1)
    if idx_dtype is None:
        idx_dtype = narrow_index_dtype((int(idx4.max()) + 1,) if idx4.size else (1,))
    return Coef4D(np.asarray(val), idx4, val_dtype=val_dtype, idx_dtype=idx_dtype).pack()


# ---------------------------------------------------------------------------
# parity criterion
# ---------------------------------------------------------------------------
# The float64 references of a test are remembered by the content of their operands: tests that
# run one workload through several launch shapes, layouts or tile sizes compute them once.
_REFERENCES: "collections.OrderedDict[bytes, tuple]" = collections.OrderedDict()
_REFERENCE_BUDGET = 3 << 30  # bytes of results kept


def _nbytes(v):
    return sum(_nbytes(t) for t in v) if isinstance(v, tuple) else int(np.asarray(v).nbytes)


def _remembered(tag, arrays, extra, compute):
    h = hashlib.blake2b(repr((tag, extra)).encode(), digest_size=16)
    for a in arrays:
        a = np.ascontiguousarray(a)
        h.update(repr((a.dtype.str, a.shape)).encode())
        h.update(a.view(np.uint8).reshape(-1).data)
    key = h.digest()
    if key in _REFERENCES:
        _REFERENCES.move_to_end(key)
        return _REFERENCES[key]
    value = compute()
    _REFERENCES[key] = value
    while len(_REFERENCES) > 1 and sum(_nbytes(v) for v in _REFERENCES.values()) > _REFERENCE_BUDGET:
        _REFERENCES.popitem(last=False)
    return value


def forward_reference(idx, val, mix, x, y, s, snd, rcv, num_out, leading=False):
    """float64 value and the sum of absolute terms of every output element (read-only arrays)."""
    def compute():
        ref = O.convolution_unfused(idx, val, mix, x, y, s, snd, rcv, num_out, leading=leading,
                                    dtype=np.float64)
        mag = O.convolution_unfused(idx, np.abs(val), mix, np.abs(x), np.abs(y), np.abs(s), snd, rcv,
                                    num_out, leading=leading, dtype=np.float64)
        for a in (ref, mag):
            a.setflags(write=False)
        return ref, mag
    return _remembered("forward", (idx, val, mix, x, y, s, snd, rcv), (int(num_out), bool(leading)), compute)


def backward_reference(idx, val, mix, x, y, s, snd, rcv, dm, leading=False):
    def compute():
        ref = O.convolution_vjp(idx, val, mix, x, y, s, snd, rcv, dm, leading=leading, dtype=np.float64)
        mag = O.convolution_vjp(idx, np.abs(val), mix, np.abs(x), np.abs(y), np.abs(s), snd, rcv,
                                np.abs(dm), leading=leading, dtype=np.float64)
        for a in tuple(ref) + tuple(mag):
            a.setflags(write=False)
        return tuple(ref), tuple(mag)
    return _remembered("backward", (idx, val, mix, x, y, s, snd, rcv, dm), (bool(leading),), compute)


def assert_parity(result, ref64, mag64, what="", rtol=1e-5, atol=1e-6, ulps=16.0):
    """|result - ref| <= atol + rtol*|ref| elementwise (1e-5 relative / 1e-6 absolute);
    an element outside that must lie within `ulps` float32 roundings of the sum of the
    absolute values of its terms - the float32 summation-order allowance.
    Returns the share of the elements that needed that allowance."""
    result = np.asarray(result, dtype=np.float64)
    assert result.shape == ref64.shape, f"{what}: shape {result.shape} != {ref64.shape}"
    assert np.isfinite(result).all(), f"{what}: non-finite values"
    err = np.abs(result - ref64)
    in_band = err <= atol + rtol * np.abs(ref64)
    ok = in_band | (err <= ulps * EPS32 * mag64)
    if not ok.all():
        bad = np.argwhere(~ok)[0]
        t = tuple(bad)
        raise AssertionError(
            f"{what}: {int((~ok).sum())} of {ok.size} elements out of tolerance; first at {t}: "
            f"got {result[t]!r}, want {ref64[t]!r}, err {err[t]:.3e}, term magnitude {mag64[t]:.3e}")
    return 1.0 - float(in_band.mean()) if in_band.size else 0.0


def float32_noise_bound(ref64, mag64, rtol=1e-5, atol=1e-6, ulps=16.0):
    return np.maximum(atol + rtol * np.abs(ref64), ulps * EPS32 * mag64)


def dense_convolve(model):
    """The operator of an `EnergyModel` as a dense einsum with index_add, differentiable by torch
    on the host: the independent form the end-to-end energy and forces are checked against."""
    import torch

    def convolve(layer, x, y, s, sender, receiver):
        m = model.layers[layer]
        c = m.coef
        idx = np.asarray(c.idx, dtype=np.int64)
        Z, X, Y = m.params.num_out, x.shape[1], y.shape[1]
        dense = torch.zeros((Z, X, Y), dtype=x.dtype)
        dense.index_put_(tuple(torch.as_tensor(idx[:, :3].T)), torch.as_tensor(np.asarray(c.val), dtype=x.dtype),
                         accumulate=True)
        mix = torch.as_tensor(m._mix.mix_indices, dtype=torch.long)
        weights = torch.einsum("ijk,ek->eij", dense, y)
        msg = torch.einsum("eij,ejc->eic", weights, x[sender.long()]) * s[:, mix, :]
        return torch.zeros((x.shape[0], Z, x.shape[2]), dtype=x.dtype).index_add(0, receiver.long(), msg)
    return convolve
