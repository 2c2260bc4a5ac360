"""Parity of the table-driven HIP kernels against the CPU oracle, through the C ABI."""

import ctypes

import numpy as np
import pytest
import torch

from e3j_amd import _lib
from oracle import conv_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _params(n, e, nnz, X, Y, Z, S, K, layout, val, idx_bytes, debug=1):
    return _lib.ConvParams(num_nodes=n, num_edges=e, num_coef=nnz, num_x=X, num_y=Y, num_out=Z,
                           num_scalars=S, channels=K, layout=layout, val_dtype=val,
                           coef_idx_bytes=idx_bytes, signature=-1, coef_scale=1.0, debug=debug)


def run_abi(idx, val, mix, x, y, s, dm, snd, rcv, Z, *, leading=False, dtype=np.float32,
            idx_dtype=None, grouping="receiver", perm=None, plan=None):
    """Forward and backward through the C ABI on receiver-sorted (or permuted) edges.

    `plan`: None, the calls plan their table themselves; "ready", the plan is built once by the status
    call and the calls are told so; "none", the calls are told not to plan."""
    lib = _lib.load()
    n, e = x.shape[0], y.shape[0]
    X, S = (x.shape[2], s.shape[2]) if leading else (x.shape[1], s.shape[1])
    K = x.shape[1] if leading else x.shape[2]
    packed = H.pack_table(idx, val, mix, val_dtype=dtype, idx_dtype=idx_dtype)
    coef_d = _dev(packed.view(np.uint8).reshape(-1))
    xd, yd, sd, dmd = _dev(x), _dev(y), _dev(s), _dev(dm)
    if perm is None:
        ptr = O.receiver_ptr(rcv, n)
        other, perm_d = _dev(snd.astype(np.int32)), None
    else:
        ptr = O.receiver_ptr(rcv[perm], n)
        other, perm_d = _dev(snd[perm].astype(np.int32)), _dev(perm.astype(np.int32))
    ptr_d = _dev(ptr)
    p = _params(n, e, len(val), X, y.shape[1], Z, S, K, 0 if leading else 1,
                _lib.F32 if dtype == np.float32 else _lib.F64, packed.dtype.itemsize)
    out = torch.full((n,) + ((K, Z) if leading else (Z, K)), float("nan"),
                     dtype=xd.dtype, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    if plan == "ready":
        plan_d = torch.empty(max(int(lib.e3j_amd_table_plan_bytes(ctypes.byref(p))), 4) // 4, dtype=torch.int32,
                             device="cuda")
        p.table_plan = plan_d.data_ptr()
        status = (ctypes.c_int32 * 4)()
        _lib.check(lib.e3j_amd_table_plan_status(ctypes.byref(p), coef_d.data_ptr(), 0, status, stream))
        assert status[0] == 1, "the planned kernels do not take this table"
        p.table_plan_state = _lib.PLAN_READY
    elif plan == "none":
        p.table_plan_state = _lib.PLAN_NONE
    _lib.check(lib.e3j_amd_convolution_fwd(ctypes.byref(p), coef_d.data_ptr(), xd.data_ptr(),
                                           yd.data_ptr(), sd.data_ptr(), other.data_ptr(),
                                           ptr_d.data_ptr(),
                                           perm_d.data_ptr() if perm_d is not None else None,
                                           out.data_ptr(), stream))
    dx = torch.full_like(xd, float("nan"))
    dy = torch.full_like(yd, float("nan"))
    ds = torch.full_like(sd, float("nan"))
    if grouping == "receiver":
        _lib.check(lib.e3j_amd_convolution_bwd_receiver(
            ctypes.byref(p), coef_d.data_ptr(), xd.data_ptr(), yd.data_ptr(), sd.data_ptr(),
            dmd.data_ptr(), other.data_ptr(), ptr_d.data_ptr(),
            perm_d.data_ptr() if perm_d is not None else None,
            dx.data_ptr(), dy.data_ptr(), ds.data_ptr(), stream))
    else:
        perm_t, recv_t, sptr = O.transpose_graph(snd, rcv, n)
        recv_t_d, sptr_d, perm_t_d = _dev(recv_t.astype(np.int32)), _dev(sptr), _dev(perm_t)
        _lib.check(lib.e3j_amd_convolution_bwd_sender(
            ctypes.byref(p), coef_d.data_ptr(), xd.data_ptr(), yd.data_ptr(), sd.data_ptr(),
            dmd.data_ptr(), recv_t_d.data_ptr(), sptr_d.data_ptr(), perm_t_d.data_ptr(),
            dx.data_ptr(), dy.data_ptr(), ds.data_ptr(), stream))
    torch.cuda.synchronize()
    return out.cpu().numpy(), dx.cpu().numpy(), dy.cpu().numpy(), ds.cpu().numpy()


def check_all(idx, val, mix, x, y, s, dm, snd, rcv, Z, results, leading=False, tag=""):
    out, dx, dy, ds = results
    ref, mag = H.forward_reference(idx, val, mix, x, y, s, snd, rcv, Z, leading=leading)
    H.assert_parity(out, ref, mag, f"{tag} out")
    (rx, ry, rs), (mx, my, ms) = H.backward_reference(idx, val, mix, x, y, s, snd, rcv, dm, leading=leading)
    H.assert_parity(dx, rx, mx, f"{tag} dx")
    H.assert_parity(dy, ry, my, f"{tag} dy")
    H.assert_parity(ds, rs, ms, f"{tag} ds")


@pytest.mark.parametrize("scale_s", [False, True])
@pytest.mark.parametrize("channels", [32, 64, 96, 128])
@pytest.mark.parametrize("idx_dtype", [np.int32, np.uint8])
def test_strip_case_bit_exact(channels, scale_s, idx_dtype):
    """Known-answer case of the reference's C++ test, required bit-exact
    (lib/e3j_ops/tests/test_convolution.cpp:288-290,316-384)."""
    c = O.strip_case(3, channels, scale_s)
    dm = np.ones((4, c["num_out"], channels), dtype=np.float32)
    out, *_ = run_abi(c["idx"], c["val"], c["mix_idx"], c["x"], c["y"], c["s"], dm, c["sender"],
                      c["receiver"], c["num_out"], idx_dtype=idx_dtype)
    assert np.array_equal(out, c["expect"])


# channel counts of the reference's op tests (tests/test_ops/test_convolution_op.py:209-282)
@pytest.mark.parametrize("channels", [1, 2, 4, 8, 16, 32, 128, 256])
@pytest.mark.parametrize("grouping", ["receiver", "sender"])
def test_random_table_fwd_bwd(channels, grouping):
    rng = np.random.default_rng(100 + channels)
    N, E, X, Y, Z, S, nnz = 8, 24, 9, 16, 9, 3, 200
    idx, val, mix = H.random_table(rng, nnz, X, Y, Z, S)
    snd, rcv = H.random_graph(rng, N, E)
    x, y, s, dm = H.random_operands(rng, N, E, X, Y, S, channels, Z)
    res = run_abi(idx, val, mix, x, y, s, dm, snd, rcv, Z, grouping=grouping)
    check_all(idx, val, mix, x, y, s, dm, snd, rcv, Z, res, tag=f"K={channels} {grouping}")


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("grouping", ["receiver", "sender"])
def test_more_than_64_harmonics_components(dtype, grouping):
    """Up to 64 y components travel in one register of the wave; longer rows (here 81, the
    harmonics up to l = 8) are read from memory, and a table longer than one 64-entry load."""
    rng = np.random.default_rng(81)
    N, E, X, Y, Z, S, K, nnz = 7, 30, 4, 81, 12, 5, 40, 300
    idx, val, mix = H.random_table(rng, nnz, X, Y, Z, S)
    assert idx[:, 2].max() >= 64
    snd, rcv = H.random_graph(rng, N, E)
    x, y, s, dm = H.random_operands(rng, N, E, X, Y, S, K, Z, dtype=dtype)
    out, dx, dy, ds = run_abi(idx, val, mix, x, y, s, dm, snd, rcv, Z, dtype=dtype, grouping=grouping)
    ref, mag = H.forward_reference(idx, val, mix, x, y, s, snd, rcv, Z)
    (rx, ry, rs), (mx, my, ms) = H.backward_reference(idx, val, mix, x, y, s, snd, rcv, dm)
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == np.float32 else dict(rtol=1e-12, atol=1e-12, ulps=0.0)
    for got, r, m, name in ((out, ref, mag, "out"), (dx, rx, mx, "dx"), (dy, ry, my, "dy"), (ds, rs, ms, "ds")):
        H.assert_parity(got, r, m, f"{name} Y=81 {np.dtype(dtype).name} {grouping}", **tol)


# ---------------------------------------------------------------------------
# layouts, dtypes, index widths
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("leading", [False, True])
@pytest.mark.parametrize("idx_dtype", [np.uint8, np.int32])
def test_layout_dtype_grid(dtype, leading, idx_dtype):
    rng = np.random.default_rng(7)
    N, E, X, Y, Z, S, K, nnz = 9, 40, 5, 7, 6, 4, 24, 60
    idx, val, mix = H.random_table(rng, nnz, X, Y, Z, S)
    snd, rcv = H.random_graph(rng, N, E)
    x, y, s, dm = H.random_operands(rng, N, E, X, Y, S, K, Z, dtype=dtype)
    args = [a.swapaxes(1, 2).copy() if leading else a for a in (x, s, dm)]
    out, dx, dy, ds = run_abi(idx, val, mix, args[0], y, args[1], args[2], snd, rcv, Z, leading=leading,
                              dtype=dtype, idx_dtype=idx_dtype)
    ref, mag = H.forward_reference(idx, val, mix, args[0], y, args[1], snd, rcv, Z, leading=leading)
    (rx, ry, rs), (mx, my, ms) = H.backward_reference(idx, val, mix, args[0], y, args[1], snd, rcv,
                                                      args[2], leading=leading)
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == np.float32 else dict(rtol=1e-12, atol=1e-12, ulps=0.0)
    for got, r, m, name in ((out, ref, mag, "out"), (dx, rx, mx, "dx"), (dy, ry, my, "dy"), (ds, rs, ms, "ds")):
        H.assert_parity(got, r, m, f"{name} leading={leading} {np.dtype(dtype).name}", **tol)


# scalar irreps at 4096 / vector edges at 8192 channels (tests/test_ops/test_convolution_op.py:257-301)
@pytest.mark.parametrize("X, Y, Z, S, nnz, K", [(1, 1, 1, 1, 1, 4096), (1, 4, 4, 1, 4, 8192)])
def test_wide_channels(X, Y, Z, S, nnz, K):
    rng = np.random.default_rng(K)
    idx, val, mix = H.random_table(rng, nnz, X, Y, Z, S)
    snd, rcv = H.random_graph(rng, 8, 24)
    x, y, s, dm = H.random_operands(rng, 8, 24, X, Y, S, K, Z)
    res = run_abi(idx, val, mix, x, y, s, dm, snd, rcv, Z)
    check_all(idx, val, mix, x, y, s, dm, snd, rcv, Z, res, tag=f"K={K}")


# ---------------------------------------------------------------------------
# padding, empty rows, gaps (each rule has a reference test, see include/e3j_amd.h)
# ---------------------------------------------------------------------------
def _padded_problem(rng, K=16):
    N, X, Y, Z, S, nnz = 6, 4, 5, 6, 3, 40
    idx, val, mix = H.random_table(rng, nnz, X, Y, Z, S)
    # node 2 has no incoming edge; 3 trailing padding edges; 1 sender-only padding edge inside node 4's row
    snd = np.array([1, 3, 0, 5, 4, 0, O.DUMMY_INDEX, 2, 1, O.DUMMY_INDEX, O.DUMMY_INDEX, O.DUMMY_INDEX], dtype=np.int32)
    rcv = np.array([0, 0, 1, 1, 3, 4, 4, 4, 5, O.DUMMY_INDEX, O.DUMMY_INDEX, O.DUMMY_INDEX], dtype=np.int32)
    x, y, s, dm = H.random_operands(rng, N, len(snd), X, Y, S, K, Z)
    dead = (snd == O.DUMMY_INDEX) | (rcv == O.DUMMY_INDEX)
    y[dead] = np.nan          # features of padding edges may hold anything
    s[dead] = np.inf
    return idx, val, mix, x, y, s, dm, snd, rcv, Z, dead


@pytest.mark.parametrize("grouping", ["receiver", "sender"])
def test_padding_edges_and_empty_rows(grouping):
    """Zero rows for nodes without live edges, NaN/Inf on padding edges never read, dy/ds of
    padding edges written as exact zeros over poisoned memory
    (tests/test_ops/test_convolution_jax_transforms.py:229-306)."""
    idx, val, mix, x, y, s, dm, snd, rcv, Z, dead = _padded_problem(np.random.default_rng(3))
    out, dx, dy, ds = run_abi(idx, val, mix, x, y, s, dm, snd, rcv, Z, grouping=grouping)
    assert not out[2].any() and np.isfinite(out).all()
    assert not dy[dead].any() and not ds[dead].any()
    live = ~dead
    ref, mag = H.forward_reference(idx, val, mix, x, y[live], s[live], snd[live], rcv[live], Z)
    H.assert_parity(out, ref, mag, "out")
    (rx, ry, rs), (mx, my, ms) = H.backward_reference(idx, val, mix, x, y[live], s[live], snd[live],
                                                      rcv[live], dm)
    H.assert_parity(dx, rx, mx, "dx")
    H.assert_parity(dy[live], ry, my, "dy")
    H.assert_parity(ds[live], rs, ms, "ds")


def test_no_edges():
    """E = 0: all-zero out and dx (tests/test_pallas_mosaic_gpu_convolution.py:1566-1589)."""
    rng = np.random.default_rng(4)
    idx, val, mix = H.random_table(rng, 20, 3, 3, 4, 2)
    x, y, s, dm = H.random_operands(rng, 5, 0, 3, 3, 2, 8, 4)
    empty = np.zeros((0,), dtype=np.int32)
    out, dx, dy, ds = run_abi(idx, val, mix, x, y, s, dm, empty, empty, 4)
    assert not out.any() and not dx.any() and dy.shape == (0, 3) and ds.shape == (0, 2, 8)


@pytest.mark.parametrize("grouping", ["receiver", "sender"])
def test_gap_rows_are_zero(grouping):
    """Coordinates no coefficient touches yield zeros, not garbage (tests/test_ops/test_zero_gap_rows.py:15-26)."""
    rng = np.random.default_rng(5)
    X, Y, Z, S, K = 6, 5, 7, 4, 8
    idx = np.array([[0, 0, 0], [0, 2, 1], [3, 2, 4], [6, 5, 1]])   # out rows 1,2,4,5; x rows 1,3,4; y 2,3; scalar 2 untouched
    val = rng.normal(size=4).astype(np.float32)
    mix = np.array([0, 0, 1, 1, 2, 2, 3])
    snd, rcv = H.random_graph(rng, 5, 14)
    x, y, s, dm = H.random_operands(rng, 5, 14, X, Y, S, K, Z)
    out, dx, dy, ds = run_abi(idx, val, mix, x, y, s, dm, snd, rcv, Z, grouping=grouping)
    assert not out[:, [1, 2, 4, 5]].any() and not dx[:, [1, 3, 4]].any()
    assert not dy[:, [2, 3]].any() and not ds[:, 2].any()
    check_all(idx, val, mix, x, y, s, dm, snd, rcv, Z, (out, dx, dy, ds), tag="gaps")


def test_unsorted_edges_through_permutation():
    """Edges in any order: CSR positions refer to y/s rows through edge_perm."""
    rng = np.random.default_rng(6)
    N, E, X, Y, Z, S, K, nnz = 10, 60, 4, 6, 5, 3, 32, 50
    idx, val, mix = H.random_table(rng, nnz, X, Y, Z, S)
    snd, rcv = H.random_graph(rng, N, E, sort_by=None)
    x, y, s, dm = H.random_operands(rng, N, E, X, Y, S, K, Z)
    perm = np.argsort(rcv, kind="stable").astype(np.int32)
    res = run_abi(idx, val, mix, x, y, s, dm, snd, rcv, Z, perm=perm)
    check_all(idx, val, mix, x, y, s, dm, snd, rcv, Z, res, tag="perm")


def test_repeated_senders_accumulate():
    """Several edges from one sender (tests/test_pallas_mosaic_gpu_convolution.py:325-350)."""
    rng = np.random.default_rng(8)
    idx, val, mix = H.random_table(rng, 30, 3, 4, 4, 2)
    snd = np.zeros(12, dtype=np.int32)
    rcv = np.sort(rng.integers(0, 4, 12)).astype(np.int32)
    x, y, s, dm = H.random_operands(rng, 4, 12, 3, 4, 2, 16, 4)
    res = run_abi(idx, val, mix, x, y, s, dm, snd, rcv, 4)
    check_all(idx, val, mix, x, y, s, dm, snd, rcv, 4, res, tag="repeated")
    assert not res[1][1:].any()


def test_sorted_path_is_bit_reproducible():
    """Forward and the sender-grouped backward give identical bits run to run
    (tests/test_ops/test_convolution_op.py:322-342)."""
    rng = np.random.default_rng(9)
    N, E, X, Y, Z, S, K, nnz = 128, 4096, 16, 16, 4, 4, 32, 64
    idx, val, mix = H.random_table(rng, nnz, X, Y, Z, S)
    snd, rcv = H.random_graph(rng, N, E)
    x, y, s, dm = H.random_operands(rng, N, E, X, Y, S, K, Z)
    base = run_abi(idx, val, mix, x, y, s, dm, snd, rcv, Z, grouping="sender")
    for _ in range(5):
        again = run_abi(idx, val, mix, x, y, s, dm, snd, rcv, Z, grouping="sender")
        for a, b in zip(base, again):
            assert np.array_equal(a, b)
