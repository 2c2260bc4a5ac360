"""Device graph preparation (CSR row pointers, stable edge sort) against numpy."""

import numpy as np
import pytest
import torch

from e3j_amd.graph import (DUMMY_INDEX, GraphCSR, csr_row_ptr, fold_endpoints, locality_order, sort_edges,
                           wrap_global_index)
from oracle import conv_oracle as O

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("num_nodes, num_edges", [(4, 9), (1000, 30000), (32000, 200000), (5, 0)])
def test_row_ptr_and_sort(num_nodes, num_edges):
    rng = np.random.default_rng(num_edges)
    key = rng.integers(0, num_nodes, num_edges).astype(np.int32)
    other = rng.integers(0, num_nodes, num_edges).astype(np.int32)
    if num_edges:
        key[rng.integers(0, num_edges, max(1, num_edges // 50))] = DUMMY_INDEX
        key[rng.integers(0, num_edges, 2)] = -3          # negative keys are padding too
    ptr = csr_row_ptr(dev(key), num_nodes)
    assert ptr.dtype == torch.int32
    np.testing.assert_array_equal(ptr.cpu().numpy(), O.receiver_ptr(key, num_nodes))
    perm, other_sorted, ptr2 = sort_edges(dev(key), dev(other), num_nodes)
    np.testing.assert_array_equal(ptr2.cpu().numpy(), O.receiver_ptr(key, num_nodes))
    want = np.argsort(key.view(np.uint32), kind="stable")
    np.testing.assert_array_equal(perm.cpu().numpy(), want)
    np.testing.assert_array_equal(other_sorted.cpu().numpy(), other[want])


def test_graph_csr_with_dummy_edges():
    """tests/test_graph.py:86-141."""
    sender = np.array([1, 2, 0, 1, 3, 2] + [DUMMY_INDEX] * 3, dtype=np.int32)
    receiver = np.array([0, 1, 1, 2, 2, 3] + [DUMMY_INDEX] * 3, dtype=np.int32)
    s_l, r_l = wrap_global_index(dev(sender), 4), wrap_global_index(dev(receiver), 4)
    graph = GraphCSR(4, s_l, r_l)
    assert graph.receiver_ptr.tolist() == [0, 1, 3, 5, 6]
    assert graph.num_neighbors.tolist() == [1, 2, 2, 1]
    perm, graph_t, inverse = graph.transpose()
    assert graph_t.receiver_ptr.tolist() == [0, 1, 3, 5, 6]
    assert perm[inverse.long()].tolist() == list(range(9))
    assert graph_t.sender.tolist()[:6] == receiver[perm.cpu().numpy()][:6].tolist()
    # folding two graphs keeps the grouping key non-decreasing and counts every edge
    r_f, s_f = fold_endpoints(dev(np.stack([receiver, receiver])).long(), dev(np.stack([sender, sender])).long(), 2, 4)
    assert bool((r_f[1:] >= r_f[:-1]).all())
    assert int(csr_row_ptr(r_f, 8)[-1]) == 18
    assert int((s_f == DUMMY_INDEX).sum()) == 6
    masked_s, masked_r = GraphCSR.mask_edges(dev(sender[:6]), dev(receiver[:6]), dev(np.arange(4) < 3))
    assert ((masked_s == DUMMY_INDEX) | (masked_r == DUMMY_INDEX)).tolist() == [False, False, False, False, True, True]


def test_cpu_tensors_are_rejected():
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        csr_row_ptr(torch.zeros(4, dtype=torch.int32), 4)


@pytest.mark.parametrize("rounds", [0, 1, 3])
def test_locality_order_is_a_permutation_that_groups_neighbours(rounds):
    from e3j_amd import workloads as W
    w = W.config2(0.2)
    n = w.num_nodes
    ptr = csr_row_ptr(w.receiver.cuda(), n)
    order = locality_order(w.sender.cuda(), ptr, n, rounds).cpu().numpy()
    assert sorted(order.tolist()) == list(range(n))
    if rounds == 0:
        assert order.tolist() == list(range(n))
        return
    # neighbours in the graph end up closer in the order than in a random numbering
    position = np.empty(n, dtype=np.int64)
    position[order] = np.arange(n)
    snd, rcv = w.sender.numpy(), w.receiver.numpy()
    window = 64
    close = (np.abs(position[snd] - position[rcv]) <= window).mean()
    close_before = (np.abs(snd.astype(np.int64) - rcv) <= window).mean()
    assert close > 3.0 * close_before, (close, close_before)
    # padding endpoints are ignored
    snd2 = snd.copy()
    snd2[::7] = DUMMY_INDEX
    order2 = locality_order(dev(snd2), ptr, n, rounds).cpu().numpy()
    assert sorted(order2.tolist()) == list(range(n))


@pytest.mark.parametrize("num_nodes", [5, 64, 1003])
def test_long_rows_are_dealt_to_the_fronts_of_the_eighths_of_the_row_list(num_nodes):
    """Rows with more than twice the mean number of edges start first on every XCD: eighth p of
    the list holds the p-th eighth of the long rows, then the p-th eighth of the others."""
    rng = np.random.default_rng(num_nodes)
    degree = np.where(rng.random(num_nodes) < 0.1, 40, 4)
    degree[0] = 40
    receiver = np.repeat(np.arange(num_nodes), degree).astype(np.int32)
    sender = rng.integers(0, num_nodes, receiver.size).astype(np.int32)
    ptr = csr_row_ptr(dev(receiver), num_nodes)
    order = locality_order(dev(sender), ptr, num_nodes, 0).cpu().numpy()   # no sweeps: index order, then the deal
    assert sorted(order.tolist()) == list(range(num_nodes))
    long_row = degree * num_nodes > 2 * degree.sum()
    longs, shorts = np.flatnonzero(long_row), np.flatnonzero(~long_row)
    want = []
    for p in range(8):
        want += longs[p * len(longs) // 8:(p + 1) * len(longs) // 8].tolist()
        want += shorts[p * len(shorts) // 8:(p + 1) * len(shorts) // 8].tolist()
    assert order.tolist() == want
    # a graph without long rows keeps its list
    even = np.repeat(np.arange(num_nodes), 3).astype(np.int32)
    same = locality_order(dev(sender[:even.size] % num_nodes), csr_row_ptr(dev(even), num_nodes), num_nodes, 0)
    assert same.cpu().tolist() == list(range(num_nodes))


@pytest.mark.parametrize("num_nodes", [1, 7, 1000])
def test_wrap_global_index_matches_the_tensor_arithmetic(num_nodes):
    """Global ids of a sharded graph modulo the shard size, sentinel kept
    (`src/e3j/ops/convolution.py:39-51`); the int32 device path against int64 host arithmetic."""
    rng = np.random.default_rng(num_nodes)
    index = rng.integers(0, 5 * num_nodes, size=4099).astype(np.int32)
    index[rng.random(index.size) < 0.1] = DUMMY_INDEX
    index[:3] = [0, num_nodes - 1, num_nodes]
    want = np.where(index == DUMMY_INDEX, index, index % num_nodes)
    got = wrap_global_index(torch.from_numpy(index).cuda(), num_nodes)
    assert got.dtype == torch.int32
    np.testing.assert_array_equal(got.cpu().numpy(), want)
    # wide indices take the tensor-arithmetic route and agree
    got64 = wrap_global_index(torch.from_numpy(index.astype(np.int64)).cuda(), num_nodes)
    np.testing.assert_array_equal(got64.cpu().numpy(), want)
    assert wrap_global_index(torch.empty(0, dtype=torch.int32, device="cuda"), num_nodes).numel() == 0
