"""The backward over tiles of receivers (`e3j_amd_convolution_bwd_tiled`) through the C ABI:
the schedule against a numpy restatement, the cotangents against the CPU oracle and against
the one-wave-per-receiver backward, for tile sizes and work-piece lengths that cut tiles and
sender runs in every way (one row per tile, tiles past the last node, pieces of a few edges),
on graphs with padding edges, empty rows, hubs and an edge permutation."""

import ctypes
import zlib

import numpy as np
import pytest
import torch

from e3j_amd import _lib, workloads as W
from e3j_amd.graph import TileSchedule, csr_row_ptr, locality_order, sort_edges
from e3j_amd.ops import _Table
from tests import helpers as H

pytestmark = pytest.mark.gpu

DUMMY = int(np.iinfo(np.int32).max)


def _signature_of(w):
    packed = w.module._packed_coef("float32")
    dims = (int(w.x.shape[1]), int(w.y.shape[1]), w.module.params.num_out, int(w.s.shape[1]))
    return _Table.get(packed, np.float32).signature(dims, w.channels, w.module.layout), dims


def _params(w, sig, scale, dims, order):
    table = _Table.get(w.module._packed_coef("float32"), np.float32)
    return _lib.ConvParams(
        num_nodes=w.num_nodes, num_edges=w.num_edges, num_coef=table.num_coef, num_x=dims[0], num_y=dims[1],
        num_out=dims[2], num_scalars=dims[3], channels=w.channels, layout=_lib.LAYOUT_TRAILING,
        val_dtype=_lib.F32, coef_idx_bytes=table.idx_bytes, signature=sig, coef_scale=scale, debug=0,
        y_flip=0, row_order=order.data_ptr() if order is not None else None)


def _run_tiled(d, p, other, ptr, perm, schedule):
    dx, dy, ds = torch.empty_like(d.x), torch.empty_like(d.y), torch.empty_like(d.s)
    # poison: every element must be written (or zero-filled) by the call
    dx.fill_(float("nan")); dy.fill_(float("nan")); ds.fill_(float("nan"))
    _lib.check(_lib.load().e3j_amd_convolution_bwd_tiled(
        ctypes.byref(p), d.x.data_ptr(), d.y.data_ptr(), d.s.data_ptr(), d.dm.data_ptr(), other.data_ptr(),
        ptr.data_ptr(), perm.data_ptr() if perm is not None else None, ctypes.byref(schedule.struct),
        dx.data_ptr(), dy.data_ptr(), ds.data_ptr(), int(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    return dx, dy, ds


def _run_receiver(d, p, other, ptr, perm):
    dx, dy, ds = torch.empty_like(d.x), torch.empty_like(d.y), torch.empty_like(d.s)
    _lib.check(_lib.load().e3j_amd_convolution_bwd_receiver(
        ctypes.byref(p), None, d.x.data_ptr(), d.y.data_ptr(), d.s.data_ptr(), d.dm.data_ptr(),
        other.data_ptr(), ptr.data_ptr(), perm.data_ptr() if perm is not None else None,
        dx.data_ptr(), dy.data_ptr(), ds.data_ptr(), int(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    return dx, dy, ds


def _check_schedule(sch, other, ptr, perm, order, n, tile_rows, max_work):
    """The schedule is what a host restatement builds: per tile the positions sorted by
    (sender, position), padding senders last (tiles of more than 512 positions: live positions
    in tile order, then the padding ones); descriptors tile every tile's list."""
    other, ptr = other.cpu().numpy(), ptr.cpu().numpy().astype(np.int64)
    order = np.arange(n) if order is None else order.cpu().numpy()
    perm = None if perm is None else perm.cpu().numpy()
    snd, edge, loc = sch.sender.cpu().numpy(), sch.edge.cpu().numpy(), sch.local.cpu().numpy()
    work = sch.work.cpu().numpy()[:sch.num_work]
    used = int(work[0, 3])
    assert (n + tile_rows - 1) // tile_rows <= used <= sch.num_work
    work = work[:used]          # the entries behind the used ones are not written
    at, covered = 0, []
    for t in range((n + tile_rows - 1) // tile_rows):
        rows = order[t * tile_rows:(t + 1) * tile_rows]
        pos = np.concatenate([np.arange(ptr[r], ptr[r + 1]) for r in rows] + [np.zeros(0, np.int64)])
        local = np.concatenate([np.full(ptr[r + 1] - ptr[r], i) for i, r in enumerate(rows)] + [np.zeros(0, np.int64)])
        s = other[pos].astype(np.int64)
        key = np.where((s >= 0) & (s < n), s, n)
        m = len(pos)
        if m <= 512:
            o = np.lexsort((pos, key))
        else:   # a long tile: live positions in tile order, padding positions behind them
            o = np.concatenate([np.nonzero(key < n)[0], np.nonzero(key == n)[0]])
        want_snd = np.where(key[o] == n, -1, key[o])
        assert np.array_equal(snd[at:at + m], want_snd), f"tile {t}: senders"
        assert np.array_equal(edge[at:at + m], pos[o] if perm is None else perm[pos[o]]), f"tile {t}: edge rows"
        assert np.array_equal(loc[at:at + m], local[o]), f"tile {t}: local receivers"
        mine = work[(work[:, 0] == t) & (work[:, 2] > work[:, 1])]
        pieces = sorted((int(b), int(e)) for _, b, e, _ in mine)
        if m:
            assert pieces[0][0] == at and pieces[-1][1] == at + m, f"tile {t}: descriptors {pieces}"
            assert all(a[1] == b[0] for a, b in zip(pieces, pieces[1:]))
            assert all(e - b <= max_work for b, e in pieces)
        else:
            assert not pieces
        covered.append(m)
        at += m
    assert at == ptr[n]
    live = work[work[:, 2] > work[:, 1]]
    assert (live[:, 2] - live[:, 1]).sum() == at


def _odd_graph(rng, n, kind):
    if kind == "hubs":       # two receivers take most of the edges, many rows are empty
        receiver = np.concatenate([np.full(700, 3), np.full(400, n - 2), rng.integers(0, n, 300)])
    elif kind == "one_sender":
        receiver = rng.integers(0, n, 600)
    else:
        receiver = rng.integers(0, n, 900)
    e = len(receiver)
    sender = np.zeros(e, np.int64) + 5 if kind == "one_sender" else rng.integers(0, n, e)
    if kind == "padding":    # padding edges inside the rows and behind the last row
        sender[rng.random(e) < 0.15] = DUMMY
        receiver[-40:] = DUMMY
    order = np.argsort(receiver, kind="stable")
    return sender[order].astype(np.int32), receiver[order].astype(np.int32)


@pytest.mark.parametrize("tile_rows,max_work", [(16, 2048), (1, 2048), (5, 7), (16, 64), (3, 1)])
@pytest.mark.parametrize("kind", ["cfg3", "cfg3_k64", "cfg2_k256ish", "hubs", "padding", "one_sender", "unsorted"])
def test_tiled_backward_matches_oracle(kind, tile_rows, max_work):
    # (the large cases keep one problem for every tile shape: their float64 reference is computed once)
    rng = np.random.default_rng(zlib.crc32((kind if kind == "unsorted" else f"{kind}/{tile_rows}").encode()))
    if kind == "cfg3":
        w = W.config3(0.006)
    elif kind == "cfg3_k64":
        w = W.config3(0.006, channels=64)
    elif kind == "cfg2_k256ish":
        w = W.config3(0.003, channels=256)
    else:
        w = W.config3(0.004)
        n = w.num_nodes
        if kind == "unsorted":
            p = rng.permutation(w.num_edges)
            snd, rcv = w.sender.numpy()[p], w.receiver.numpy()[p]
        else:
            snd, rcv = _odd_graph(rng, n, kind)
        e = len(snd)
        y = torch.as_tensor(rng.normal(size=(e, w.y.shape[1])).astype(np.float32))
        s = torch.as_tensor(rng.normal(size=(e,) + tuple(w.s.shape[1:])).astype(np.float32))
        w = W.Workload(kind, w.module, w.x, y, s, w.dm, torch.as_tensor(snd), torch.as_tensor(rcv), w.positions, 0.0)
    (sig, scale, flip), dims = _signature_of(w)
    assert sig >= 0 and flip == 0
    lib = _lib.load()
    limit = int(lib.e3j_amd_tile_rows(sig))
    assert limit >= 4, "the signatures of the benchmark have a tiled backward"
    tile_rows = min(tile_rows, limit)
    d = w.to("cuda")
    n = w.num_nodes
    if kind == "unsorted":
        perm, other, ptr = sort_edges(d.receiver, d.sender, n)
    else:
        perm, other, ptr = None, d.sender.contiguous(), csr_row_ptr(d.receiver, n)
    order = locality_order(other, ptr, n, 2) if kind != "hubs" else None
    sch = TileSchedule(other, ptr, perm, order, n, tile_rows, max_work)
    torch.cuda.synchronize()
    _check_schedule(sch, other, ptr, perm, order, n, tile_rows, max_work)

    p = _params(w, sig, scale, dims, order)
    dx, dy, ds = _run_tiled(d, p, other, ptr, perm, sch)
    idx, val, mix = w.table()
    a = w.numpy()
    (rx, ry, rs), (mx, my, ms) = H.backward_reference(idx, val, mix, a["x"], a["y"], a["s"], a["sender"],
                                                      a["receiver"], a["dm"])
    H.assert_parity(dx.cpu().numpy(), rx, mx, f"{kind} dx")
    H.assert_parity(dy.cpu().numpy(), ry, my, f"{kind} dy")
    H.assert_parity(ds.cpu().numpy(), rs, ms, f"{kind} ds")
    # padding edges: exact zeros
    pad = (a["sender"] == DUMMY) | (a["receiver"] == DUMMY)
    if pad.any():
        assert not dy.cpu().numpy()[pad].any() and not ds.cpu().numpy()[pad].any()
    # ds belongs to the edge alone: bit-identical to the one-wave-per-receiver backward
    bx, by, bs = _run_receiver(d, p, other, ptr, perm)
    assert torch.equal(ds, bs)
    scale_x = float(bx.abs().max())
    assert float((dx - bx).abs().max()) <= 2e-5 * scale_x


def test_tile_rows_beyond_the_lds_is_refused():
    w = W.config3(0.003)
    (sig, scale, _), dims = _signature_of(w)
    d = w.to("cuda")
    n = w.num_nodes
    other, ptr = d.sender.contiguous(), csr_row_ptr(d.receiver, n)
    limit = int(_lib.load().e3j_amd_tile_rows(sig))
    sch = TileSchedule(other, ptr, None, None, n, limit + 1)
    with pytest.raises(_lib.E3jAmdError, match="LDS"):
        _run_tiled(d, _params(w, sig, scale, dims, None), other, ptr, None, sch)


def test_signature_without_tiled_kernel_is_unimplemented():
    w = W.config3(0.003, channels=32)
    (sig, scale, _), dims = _signature_of(w)
    assert sig >= 0 and int(_lib.load().e3j_amd_tile_rows(sig)) == 0
    d = w.to("cuda")
    n = w.num_nodes
    other, ptr = d.sender.contiguous(), csr_row_ptr(d.receiver, n)
    sch = TileSchedule(other, ptr, None, None, n, 4)
    with pytest.raises(_lib.E3jAmdError) as err:
        _run_tiled(d, _params(w, sig, scale, dims, None), other, ptr, None, sch)
    assert err.value.code == _lib.UNIMPLEMENTED
