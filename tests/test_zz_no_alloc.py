"""The allocation-free row-pointer entry point (`e3j_amd_csr_row_ptr_static`, its scan storage in
a device array inside the library) against the entry point that takes a workspace, through the C
ABI: two calls in a row, the second on a smaller input, bit-exact; sizes beyond the built-in
scratch are refused."""

import numpy as np
import pytest
import torch

from e3j_amd import _lib

pytestmark = pytest.mark.gpu


def _with_workspace(key, num_nodes):
    lib = _lib.load()
    row_ptr = torch.empty(num_nodes + 1, dtype=torch.int32, device=key.device)
    ws = torch.empty(max(int(lib.e3j_amd_csr_workspace_bytes(num_nodes, key.numel())), 256), dtype=torch.uint8,
                     device=key.device)
    _lib.check(lib.e3j_amd_csr_row_ptr(key.data_ptr(), key.numel(), num_nodes, row_ptr.data_ptr(), ws.data_ptr(),
                                       int(torch.cuda.current_stream().cuda_stream)))
    return row_ptr


def _static(key, num_nodes, row_ptr):
    _lib.check(_lib.load().e3j_amd_csr_row_ptr_static(key.data_ptr(), key.numel(), num_nodes, row_ptr.data_ptr(),
                                                      int(torch.cuda.current_stream().cuda_stream)))


def test_static_row_ptr_matches_workspace_version_twice():
    rng = np.random.default_rng(7)
    outputs = []
    # results are allocated before the calls under test: those allocate nothing themselves
    cases = [(200_000, 3_000_000), (1_000, 4_000)]
    keys, results = [], []
    for n, e in cases:
        k = np.sort(rng.integers(0, n, size=e)).astype(np.int32)
        k[rng.random(e) < 0.01] = np.iinfo(np.int32).max  # padding edges drop out
        keys.append(torch.as_tensor(k, device="cuda"))
        results.append(torch.full((n + 1,), -1, dtype=torch.int32, device="cuda"))
    for (n, _), key, out in zip(cases, keys, results):   # the second call reuses the scratch of the first
        _static(key, n, out)
    torch.cuda.synchronize()
    for (n, e), key, out in zip(cases, keys, results):
        want = _with_workspace(key, n)
        torch.cuda.synchronize()
        assert torch.equal(out, want)
        k = key.cpu().numpy()
        ref = np.concatenate([[0], np.cumsum(np.bincount(k[k < n], minlength=n))])
        assert np.array_equal(out.cpu().numpy(), ref)
        outputs.append(out)


def test_static_row_ptr_allocates_nothing_and_replays_from_a_graph():
    """What the entry point is for: the two calls are recorded into a HIP graph (a capture fails on
    any allocation or synchronisation inside the recorded calls) and the graph is replayed on rewritten
    inputs, with eager work between the replays; the device's free memory does not move across
    the eager calls either."""
    rng = np.random.default_rng(11)
    cases = [(50_000, 600_000), (700, 2_000)]
    keys = [torch.empty(e, dtype=torch.int32, device="cuda") for _, e in cases]
    outs = [torch.empty(n + 1, dtype=torch.int32, device="cuda") for n, _ in cases]

    def fresh_keys():
        host = []
        for (n, e), key in zip(cases, keys):
            k = np.sort(rng.integers(0, n, size=e)).astype(np.int32)
            k[rng.random(e) < 0.02] = np.iinfo(np.int32).max
            key.copy_(torch.as_tensor(k))
            host.append(k)
        return host

    def expected(host):
        return [np.concatenate([[0], np.cumsum(np.bincount(k[k < n], minlength=n))]) for (n, _), k in zip(cases, host)]

    host = fresh_keys()
    for (n, _), key, out in zip(cases, keys, outs):   # warm-up: looks up the scratch address once
        _static(key, n, out)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for (n, _), key, out in zip(cases, keys, outs):
        _static(key, n, out)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the static entry point changed the device's free memory"
    for out, want in zip(outs, expected(host)):
        assert np.array_equal(out.cpu().numpy(), want)

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for (n, _), key, out in zip(cases, keys, outs):
            _static(key, n, out)
    for _ in range(3):
        host = fresh_keys()
        for out in outs:
            out.fill_(-7)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for out, want in zip(outs, expected(host)):
            assert np.array_equal(out.cpu().numpy(), want)


def test_static_row_ptr_refuses_bad_node_counts():
    key = torch.zeros(4, dtype=torch.int32, device="cuda")
    out = torch.empty(8, dtype=torch.int32, device="cuda")
    with pytest.raises(_lib.E3jAmdError, match="bad sizes"):
        _static(key, np.iinfo(np.int32).max, out)


def test_static_row_ptr_refuses_sizes_beyond_its_scratch():
    lib = _lib.load()
    limit = int(lib.e3j_amd_csr_row_ptr_static_max_nodes())
    assert limit >= 1_000_000
    if limit >= np.iinfo(np.int32).max - 2:
        pytest.skip("the scan's storage never outgrows the scratch")
    key = torch.zeros(4, dtype=torch.int32, device="cuda")
    out = torch.empty(8, dtype=torch.int32, device="cuda")  # never written: the call must fail first
    with pytest.raises(_lib.E3jAmdError, match="scratch"):
        _static(key, limit + 1, out)
