"""Seeded random graphs that stress the row walk of the compile-time-unrolled kernels: empty rows,
single hubs, one sender for every edge, padding inside and after the edge list, unsorted edges,
one-node graphs; every built-in table, both layouts, the atomic and the atomic-free backward,
against the numpy checker."""

import numpy as np
import pytest
import torch

import e3j_amd
from e3j_amd import DUMMY_INDEX, Convolution
from tests import helpers as H

pytestmark = pytest.mark.gpu

TABLES = [(("0e+1o", "0e+1o+2e"), "0e+1o+2e", (32, 64, 128)),
          (("0e+1o+2e", "0e+1o+2e+3o"), "0e+1o+2e", (32, 64, 128)),
          (("0e+1o+2e", "0e+1o+2e+3o"), "0e+1o+2e+3o", (64, 128)),
          (("0e+1o+2e+3o", "0e+1o+2e+3o"), "0e+1o+2e+3o", (32, 64, 128, 256)),
          (("0e", "0e+1o+2e+3o"), "0e+1o+2e+3o", (64, 128, 256))]


def _degrees(rng, kind, n):
    if kind == 0:
        return rng.integers(0, 4, n)
    if kind == 1:   # a few hubs among nearly empty rows
        return np.where(rng.random(n) < 0.1, rng.integers(50, 200, n), rng.integers(0, 3, n))
    if kind == 2:   # every edge in one row
        deg = np.zeros(n, dtype=np.int64)
        deg[rng.integers(0, n)] = int(rng.integers(1, 300))
        return deg
    if kind == 3:
        return rng.poisson(8, n)
    return rng.integers(0, 2, n)


@pytest.mark.parametrize("case", range(50))
def test_odd_graph(case):
    rng = np.random.default_rng(7000 + case)
    src, tgt, channel_counts = TABLES[case % len(TABLES)]
    K = int(rng.choice(channel_counts))
    ordering = ("RECEIVER", "NONE")[case % 2]
    layout = ("TRAILING_CHANNELS", "LEADING_CHANNELS")[(case // 2) % 2]
    m = Convolution(src, tgt, graph_ordering=ordering, layout=layout)
    N = int(rng.integers(1, 70))
    rcv = np.repeat(np.arange(N), _degrees(rng, case % 5, N)).astype(np.int32)
    snd = rng.integers(0, N, rcv.size).astype(np.int32)
    if rcv.size and rng.random() < 0.5:
        snd[rng.random(rcv.size) < 0.2] = DUMMY_INDEX            # padding inside the list
    if rcv.size and rng.random() < 0.3:
        snd[:] = 0 if snd[0] == DUMMY_INDEX else snd[0]           # one sender for every edge
    pad = int(rng.integers(0, 5))
    snd = np.concatenate([snd, np.full(pad, DUMMY_INDEX, np.int32)])
    rcv = np.concatenate([rcv, np.full(pad, DUMMY_INDEX, np.int32)])
    E = rcv.size
    if ordering == "NONE" and E:
        shuffle = rng.permutation(E)
        snd, rcv = snd[shuffle], rcv[shuffle]
    X, Y, Z, S = m.source[0].dim, m.source[1].dim, m.target.dim, m.params.num_scalars
    x, y, s, dm = H.random_operands(rng, N, E, X, Y, S, K, Z)
    leading = layout == "LEADING_CHANNELS"
    put = (lambda a: np.ascontiguousarray(a.transpose(0, 2, 1))) if leading else (lambda a: a)
    back = (lambda g: g.transpose(1, 2)) if leading else (lambda g: g)

    def dev(a):
        return torch.from_numpy(np.ascontiguousarray(a)).cuda()

    coef = m._packed_coef("float32")
    args = (dev(put(x)), dev(y), dev(put(s)), dev(snd), dev(rcv))
    out = e3j_amd.convolution(coef, *args, m.params, ordering, layout=layout)
    atomics = e3j_amd.convolution_bwd(coef, *args, dev(put(dm)), m.params, ordering, layout=layout)
    with e3j_amd.config.use(deterministic=True):
        ordered = e3j_amd.convolution_bwd(coef, *args, dev(put(dm)), m.params, ordering, layout=layout)
    idx = np.asarray(m.coef.idx, dtype=np.int64)[:, :3]
    val, mix = np.asarray(m.coef.val, dtype=np.float32), m._mix.mix_indices
    ref, mag = H.forward_reference(idx, val, mix, x, y, s, snd, rcv, Z)
    H.assert_parity(back(out).cpu().numpy(), ref, mag, "out")
    refs, mags = H.backward_reference(idx, val, mix, x, y, s, snd, rcv, dm)
    for grads in (atomics, ordered):
        for got, r, g, name in zip(grads, refs, mags, ("dx", "dy", "ds")):
            got = back(got) if got.dim() == 3 else got
            H.assert_parity(got.cpu().numpy(), r, g, name, ulps=32.0)


@pytest.mark.parametrize("dtype", ["float64", "float16"])
@pytest.mark.parametrize("case", range(20))
def test_odd_graph_in_float64_and_float16(case, dtype):
    """The same graphs on the float64 and float16 unrolled kernels (trailing layout, whole waves of
    channels), with NaN in the operands of the padding edges: a padding edge contributes nothing
    and its dy / ds rows are exact zeros, a row without edges is an exact zero row."""
    rng = np.random.default_rng(9000 + case)
    src, tgt, channel_counts = TABLES[case % len(TABLES)]
    K = int(rng.choice([k for k in channel_counts if k % 64 == 0]))
    ordering = ("RECEIVER", "NONE")[case % 2]
    m = Convolution(src, tgt, graph_ordering=ordering, layout="TRAILING_CHANNELS", avg_num_neighbors=16.0)
    N = int(rng.integers(1, 70))
    rcv = np.repeat(np.arange(N), _degrees(rng, case % 5, N)).astype(np.int32)
    snd = rng.integers(0, N, rcv.size).astype(np.int32)
    if rcv.size and rng.random() < 0.6:
        snd[rng.random(rcv.size) < 0.2] = DUMMY_INDEX
    pad = int(rng.integers(0, 5))
    snd = np.concatenate([snd, np.full(pad, DUMMY_INDEX, np.int32)])
    rcv = np.concatenate([rcv, np.full(pad, DUMMY_INDEX, np.int32)])
    E = rcv.size
    if ordering == "NONE" and E:
        shuffle = rng.permutation(E)
        snd, rcv = snd[shuffle], rcv[shuffle]
    X, Y, Z, S = m.source[0].dim, m.source[1].dim, m.target.dim, m.params.num_scalars
    np_dtype = np.float64 if dtype == "float64" else np.float16
    x, y, s, dm = ((0.5 * a).astype(np_dtype) for a in H.random_operands(rng, N, E, X, Y, S, K, Z))
    padding = (snd == DUMMY_INDEX) | (rcv == DUMMY_INDEX)
    y_dev, s_dev = y.copy(), s.copy()
    y_dev[padding] = np.nan          # what a padding edge holds is never used
    s_dev[padding] = np.nan

    def dev(a):
        return torch.from_numpy(np.ascontiguousarray(a)).cuda()

    coef = m._packed_coef(dtype)
    args = (dev(x), dev(y_dev), dev(s_dev), dev(snd), dev(rcv))
    out = e3j_amd.convolution(coef, *args, m.params, ordering, layout="TRAILING_CHANNELS")
    dx, dy, ds = e3j_amd.convolution_bwd(coef, *args, dev(dm), m.params, ordering, layout="TRAILING_CHANNELS")
    torch.cuda.synchronize()
    idx = np.asarray(m.coef.idx, dtype=np.int64)[:, :3]
    val = np.asarray(m.coef.val).astype(np_dtype).astype(np.float64)
    mix = m._mix.mix_indices
    f64 = [a.astype(np.float64) for a in (x, y, s, dm)]
    from oracle import conv_oracle as O
    ref = O.convolution_unfused(idx, val, mix, f64[0], f64[1], f64[2], snd, rcv, Z, dtype=np.float64)
    mag = O.convolution_unfused(idx, np.abs(val), mix, *(np.abs(a) for a in f64[:3]), snd, rcv, Z, dtype=np.float64)
    refs = O.convolution_vjp(idx, val, mix, f64[0], f64[1], f64[2], snd, rcv, f64[3], dtype=np.float64)
    mags = O.convolution_vjp(idx, np.abs(val), mix, *(np.abs(a) for a in f64[:3]), snd, rcv, np.abs(f64[3]),
                             dtype=np.float64)
    for got, r, g, name, sums in zip((out, dx, dy, ds), (ref,) + tuple(refs), (mag,) + tuple(mags),
                                     ("out", "dx", "dy", "ds"), (1.0, 8.0, 2.0, 1.0)):
        got = got.double().cpu().numpy()
        assert np.isfinite(got).all(), f"{name}: a padding edge's NaN reached the result"
        bound = 64 * 2.0 ** -52 * g + 1e-300 if dtype == "float64" else 6 * sums * 2.0 ** -10 * g + 1e-3
        assert (np.abs(got - r) <= bound).all(), f"{name}: worst error {np.abs(got - r).max():.3e}"
    assert not dy[torch.as_tensor(padding).cuda()].any() and not ds[torch.as_tensor(padding).cuda()].any()
    no_edges = np.setdiff1d(np.arange(N), rcv[~padding])
    assert not out[torch.as_tensor(no_edges).cuda()].any()
