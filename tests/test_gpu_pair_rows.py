"""`e3j_amd_pair_rows`: the reordered list is a permutation, pairs sit on positions 2q, 2q + 1 and
share senders, rows without edges or with too many stay unpaired in their old order, and the tiles
of two receivers issue fewer distinct (tile, sender) pairs than before."""

import numpy as np
import pytest
import torch

from e3j_amd import workloads as W
from e3j_amd.graph import csr_row_ptr, locality_order, pair_rows

pytestmark = pytest.mark.gpu


def _requests(order, sender, receiver, n, tile=2):
    rank = np.empty(n, np.int64)
    rank[order] = np.arange(n)
    live = (sender >= 0) & (sender < n) & (receiver >= 0) & (receiver < n)
    return len(np.unique((rank[receiver[live]] // tile) * n + sender[live]))


def test_pairs_share_senders_on_a_radius_graph():
    w = W.config3(0.1)
    n = w.num_nodes
    snd, rcv = w.sender.cuda(), w.receiver.cuda()
    ptr = csr_row_ptr(rcv, n)
    base = locality_order(snd, ptr, n, 2)
    paired = pair_rows(snd, ptr, n, base)
    torch.cuda.synchronize()
    o = paired.cpu().numpy()
    assert np.array_equal(np.sort(o), np.arange(n))
    s, r = w.sender.numpy().astype(np.int64), w.receiver.numpy().astype(np.int64)
    before, after = _requests(base.cpu().numpy(), s, r, n), _requests(o, s, r, n)
    assert after < 0.9 * before, (before, after)
    # the leading positions hold pairs: rows that have an edge from each other and common senders
    rows = [set(s[r == i]) for i in range(n)]
    shared = [len(rows[o[2 * q]] & rows[o[2 * q + 1]]) for q in range(n // 4)]
    assert np.mean(shared) > 0.5 * len(s) / n
    # without an input order the index order is the base
    plain = pair_rows(snd, ptr, n).cpu().numpy()
    assert np.array_equal(np.sort(plain), np.arange(n))
    assert _requests(plain, s, r, n) < 0.9 * _requests(np.arange(n), s, r, n)


def test_rows_without_partner_keep_their_order():
    """Empty rows, a hub above the degree limit, padding edges and an asymmetric graph."""
    rng = np.random.default_rng(5)
    n = 300
    receiver = np.concatenate([np.full(400, 7), rng.integers(20, n, 2000)])   # rows 0..19 but 7 are empty
    sender = rng.integers(0, n, receiver.shape[0])
    sender[rng.random(sender.shape[0]) < 0.1] = np.iinfo(np.int32).max
    keep = np.argsort(receiver, kind="stable")
    receiver, sender = receiver[keep].astype(np.int32), sender[keep].astype(np.int32)
    ptr = csr_row_ptr(torch.as_tensor(receiver).cuda(), n)
    order = pair_rows(torch.as_tensor(sender).cuda(), ptr, n).cpu().numpy()
    assert np.array_equal(np.sort(order), np.arange(n))
    unpaired = [int(i) for i in order if i < 20]   # the hub and the empty rows: no partner, index order kept
    assert unpaired == list(range(20))
    first = int(np.nonzero(order == 0)[0][0])      # and they come after every pair
    assert first % 2 == 0 and first > 0
