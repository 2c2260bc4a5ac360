"""Pins the CPU oracle before anything is compared against it.

Checks, chosen so that a dropped term, a wrong sign/index or a transposed operand
fails at least one of them:
  * the reference's own known-answer case (closed form, bit-exact);
  * literal restatements of the reference's C++ CPU loops on random inputs;
  * an independent torch restatement differentiated by torch.autograd;
  * float64 central differences;
  * Euler's identity of a trilinear form;
  * the reference's expected CSR arrays with padding edges.
"""

import numpy as np
import pytest
import torch

from oracle import c_oracle, conv_oracle as O
from tests import helpers as H


def _case(seed, N=7, E=22, X=5, Y=4, S=3, Z=6, K=3, nnz=30, dtype=np.float32):
    rng = np.random.default_rng(seed)
    idx, val, mix = H.random_table(rng, nnz, X, Y, Z, S)
    snd, rcv = H.random_graph(rng, N, E)
    x, y, s, dm = H.random_operands(rng, N, E, X, Y, S, K, Z, dtype=dtype)
    return idx, val, mix, x, y, s, dm, snd, rcv, Z


# --- known answers ---------------------------------------------------------
@pytest.mark.parametrize("scale_s", [False, True])
@pytest.mark.parametrize("channels", [32, 96])
def test_strip_case_closed_form(channels, scale_s):
    """lib/e3j_ops/tests/test_convolution.cpp:122-207,288-290: equality must be exact."""
    c = O.strip_case(3, channels, scale_s)
    out = O.convolution_unfused(c["idx"], c["val"], c["mix_idx"], c["x"], c["y"], c["s"],
                                c["sender"], c["receiver"], c["num_out"])
    assert np.array_equal(out, c["expect"])
    out_c = c_oracle.convolution(c["idx"], c["val"], c["mix_idx"], c["x"], c["y"], c["s"],
                                 c["sender"], c["receiver"], c["num_out"])
    assert np.array_equal(out_c, c["expect"])


def test_strip_case_hand_value():
    """One entry by hand: node 0 receives edges 0, 1; strip 1, a = 1, s = (e+1)(t+1):
    out = 2 * (3+4+5) * (1*2 + 2*2) = 144."""
    c = O.strip_case(3, 4, True)
    assert c["expect"][0, 3, 0] == 144.0
    out = O.convolution_loops(np.concatenate([c["idx"], c["mix_idx"][c["idx"][:, 0]][:, None]], 1),
                              c["val"], c["x"], c["y"], c["s"], c["sender"], c["ptr"], c["num_out"])
    assert np.array_equal(out, c["expect"])


# --- restatement vs literal loops -------------------------------------------
@pytest.mark.parametrize("seed", [0, 1])
def test_forward_matches_reference_loops(seed):
    idx, val, mix, x, y, s, dm, snd, rcv, Z = _case(seed)
    idx4 = np.concatenate([idx, mix[idx[:, 0]][:, None]], axis=1)
    ptr = O.receiver_ptr(rcv, x.shape[0])
    loops = O.convolution_loops(idx4, val, x, y, s, snd, ptr, Z)
    ref, mag = H.forward_reference(idx, val, mix, x, y, s, snd, rcv, Z)
    H.assert_parity(loops, ref, mag, "loops")
    H.assert_parity(O.convolution_unfused(idx, val, mix, x, y, s, snd, rcv, Z), ref, mag, "numpy f32")
    H.assert_parity(c_oracle.convolution(idx, val, mix, x, y, s, snd, rcv, Z), ref, mag, "C f32")


@pytest.mark.parametrize("seed", [2, 3])
def test_vjp_matches_reference_loops(seed):
    idx, val, mix, x, y, s, dm, snd, rcv, Z = _case(seed)
    ptr = O.receiver_ptr(rcv, x.shape[0])
    loops = O.convolution_vjp_loops(idx, val, mix, x, y, s, dm, snd, ptr)
    ref, mag = H.backward_reference(idx, val, mix, x, y, s, snd, rcv, dm)
    got_np = O.convolution_vjp(idx, val, mix, x, y, s, snd, rcv, dm)
    got_c = c_oracle.convolution_vjp(idx, val, mix, x, y, s, snd, rcv, dm)
    for name, l, n, c, r, m in zip(("dx", "dy", "ds"), loops, got_np, got_c, ref, mag):
        H.assert_parity(l, r, m, f"loops {name}")
        H.assert_parity(n, r, m, f"numpy {name}")
        H.assert_parity(c, r, m, f"C {name}")


# --- independent derivations -------------------------------------------------
def _torch_forward(idx, val, mix, x, y, s, snd, rcv, Z):
    """Dense einsum restatement (different algorithm): c_ijk as a dense tensor."""
    N, X, K = x.shape
    dense = torch.zeros((Z, X, y.shape[1]), dtype=x.dtype)
    dense.index_put_(tuple(torch.as_tensor(idx.T, dtype=torch.long)), torch.as_tensor(val, dtype=x.dtype),
                     accumulate=True)
    msg = torch.einsum("ijk,ejc,ek->eic", dense, x[torch.as_tensor(snd, dtype=torch.long)], y)
    msg = msg * s[:, torch.as_tensor(mix, dtype=torch.long), :]
    out = torch.zeros((N, Z, K), dtype=x.dtype)
    return out.index_add(0, torch.as_tensor(rcv, dtype=torch.long), msg)


def test_vjp_matches_autograd_of_dense_einsum():
    idx, val, mix, x, y, s, dm, snd, rcv, Z = _case(4, dtype=np.float64)
    xt, yt, st = (torch.tensor(a, requires_grad=True) for a in (x, y, s))
    out = _torch_forward(idx, val.astype(np.float64), mix, xt, yt, st, snd, rcv, Z)
    ref = O.convolution_unfused(idx, val, mix, x, y, s, snd, rcv, Z, dtype=np.float64)
    np.testing.assert_allclose(out.detach().numpy(), ref, rtol=1e-12, atol=1e-12)
    gx, gy, gs = torch.autograd.grad(out, (xt, yt, st), torch.tensor(dm))
    dx, dy, ds = O.convolution_vjp(idx, val, mix, x, y, s, snd, rcv, dm, dtype=np.float64)
    np.testing.assert_allclose(dx, gx.numpy(), rtol=1e-11, atol=1e-11)
    np.testing.assert_allclose(dy, gy.numpy(), rtol=1e-11, atol=1e-11)
    np.testing.assert_allclose(ds, gs.numpy(), rtol=1e-11, atol=1e-11)


def test_vjp_matches_central_differences():
    idx, val, mix, x, y, s, dm, snd, rcv, Z = _case(5, N=4, E=9, K=2, dtype=np.float64)
    dx, dy, ds = O.convolution_vjp(idx, val, mix, x, y, s, snd, rcv, dm, dtype=np.float64)

    def f(x_, y_, s_):
        return float((O.convolution_unfused(idx, val, mix, x_, y_, s_, snd, rcv, Z,
                                            dtype=np.float64) * dm).sum())
    rng = np.random.default_rng(0)
    h = 1e-6
    for arr, grad, pos in ((x, dx, 0), (y, dy, 1), (s, ds, 2)):
        for _ in range(6):
            at = tuple(rng.integers(0, n) for n in arr.shape)
            plus, minus = arr.copy(), arr.copy()
            plus[at] += h
            minus[at] -= h
            args_p = [x, y, s]
            args_m = [x, y, s]
            args_p[pos], args_m[pos] = plus, minus
            fd = (f(*args_p) - f(*args_m)) / (2 * h)
            assert abs(fd - grad[at]) <= 1e-6 * max(1.0, abs(fd))


def test_euler_identity():
    """<x, dx> = <y, dy> = <s, ds> = <out, dm> for a form linear in each of x, y, s."""
    idx, val, mix, x, y, s, dm, snd, rcv, Z = _case(6, dtype=np.float64)
    out = O.convolution_unfused(idx, val, mix, x, y, s, snd, rcv, Z, dtype=np.float64)
    dx, dy, ds = O.convolution_vjp(idx, val, mix, x, y, s, snd, rcv, dm, dtype=np.float64)
    total = (out * dm).sum()
    for a, g in ((x, dx), (y, dy), (s, ds)):
        assert abs((a * g).sum() - total) <= 1e-10 * abs(total)


def test_leading_layout_is_swapaxes_of_trailing():
    """tests/test_tensor_product.py:211-239, tests/test_scalar_mixing.py:93-137."""
    idx, val, mix, x, y, s, dm, snd, rcv, Z = _case(7)
    out_t = O.convolution_unfused(idx, val, mix, x, y, s, snd, rcv, Z)
    out_l = O.convolution_unfused(idx, val, mix, x.swapaxes(1, 2).copy(), y, s.swapaxes(1, 2).copy(),
                                  snd, rcv, Z, leading=True)
    assert np.array_equal(out_l, out_t.swapaxes(1, 2))
    g_t = O.convolution_vjp(idx, val, mix, x, y, s, snd, rcv, dm)
    g_l = O.convolution_vjp(idx, val, mix, x.swapaxes(1, 2).copy(), y, s.swapaxes(1, 2).copy(),
                            snd, rcv, dm.swapaxes(1, 2).copy(), leading=True)
    assert np.array_equal(g_l[0], g_t[0].swapaxes(1, 2))
    assert np.array_equal(g_l[1], g_t[1])
    assert np.array_equal(g_l[2], g_t[2].swapaxes(1, 2))


# --- padding and CSR semantics (tests/test_graph.py:30-141) -------------------
SENDER_REAL = np.array([1, 2, 0, 1, 3, 2], dtype=np.int32)
RECEIVER_REAL = np.array([0, 1, 1, 2, 2, 3], dtype=np.int32)
NUM_NODES = 4


def _padded():
    dummy = np.full(3, O.DUMMY_INDEX, dtype=np.int32)
    return np.concatenate([SENDER_REAL, dummy]), np.concatenate([RECEIVER_REAL, dummy])


def test_csr_drops_dummies():
    sender, receiver = _padded()
    ptr = O.receiver_ptr(O.wrap_global_index(receiver, NUM_NODES), NUM_NODES)
    assert ptr.tolist() == [0, 1, 3, 5, 6] and ptr.dtype == np.int32
    perm, recv_t, sptr = O.transpose_graph(O.wrap_global_index(sender, NUM_NODES),
                                           O.wrap_global_index(receiver, NUM_NODES), NUM_NODES)
    assert sptr.tolist() == [0, 1, 3, 5, 6]
    assert sorted(perm.tolist()) == list(range(9))


def test_wrap_global_index():
    wrapped = O.wrap_global_index(np.array([0, 3, O.DUMMY_INDEX], dtype=np.int32), NUM_NODES)
    assert int(wrapped[-1]) == int(O.DUMMY_INDEX)
    assert O.wrap_global_index(np.array([4, 5]), NUM_NODES).tolist() == [0, 1]


@pytest.mark.parametrize("real", range(NUM_NODES + 1))
def test_mask_edges_matches_endpoint_gather(real):
    node_mask = np.arange(NUM_NODES) < real
    expected = node_mask[SENDER_REAL] & node_mask[RECEIVER_REAL]
    s, r = O.mask_edges(SENDER_REAL, RECEIVER_REAL, node_mask)
    assert np.array_equal((s == O.DUMMY_INDEX) | (r == O.DUMMY_INDEX), ~expected)


def test_fold_keeps_csr_contiguous():
    sender, receiver = _padded()
    n2 = 2 * NUM_NODES
    recv_f, send_f = O.fold_endpoints(np.stack([receiver, receiver]), np.stack([sender, sender]), 2,
                                      NUM_NODES)
    assert np.all(np.diff(recv_f) >= 0)
    ptr = O.receiver_ptr(recv_f, n2)
    assert int(ptr[-1]) == 2 * 9
    assert int((send_f == O.DUMMY_INDEX).sum()) == 6


def test_padded_graph_matches_unpadded():
    """Dummy edges carrying arbitrary data are no-ops, forward and backward; their dy/ds are zero."""
    rng = np.random.default_rng(8)
    X, Y, S, Z, K, nnz = 4, 4, 2, 5, 4, 20
    idx, val, mix = H.random_table(rng, nnz, X, Y, Z, S)
    x, y, s, dm = H.random_operands(rng, NUM_NODES, 6, X, Y, S, K, Z)
    ref = O.convolution_unfused(idx, val, mix, x, y, s, SENDER_REAL, RECEIVER_REAL, Z)
    sender, receiver = _padded()
    y_pad = np.concatenate([y, rng.normal(size=(3, Y)).astype(np.float32)])
    s_pad = np.concatenate([s, np.full((3, S, K), np.nan, dtype=np.float32)])
    out = O.convolution_unfused(idx, val, mix, x, y_pad, s_pad, sender, receiver, Z)
    assert np.array_equal(out, ref)
    assert np.array_equal(c_oracle.convolution(idx, val, mix, x, y_pad, s_pad, sender, receiver, Z),
                          c_oracle.convolution(idx, val, mix, x, y, s, SENDER_REAL, RECEIVER_REAL, Z))
    for impl in (O.convolution_vjp, c_oracle.convolution_vjp):
        dx, dy, ds = impl(idx, val, mix, x, y_pad, s_pad, sender, receiver, dm)
        dx0, dy0, ds0 = impl(idx, val, mix, x, y, s, SENDER_REAL, RECEIVER_REAL, dm)
        assert np.array_equal(dx, dx0)
        assert np.array_equal(dy[:6], dy0) and not dy[6:].any()
        assert np.array_equal(ds[:6], ds0) and not ds[6:].any()


def test_c_oracle_handles_unsorted_edges():
    idx, val, mix, x, y, s, dm, snd, rcv, Z = _case(9)
    order = np.random.default_rng(1).permutation(len(snd))
    a = c_oracle.convolution(idx, val, mix, x, y[order], s[order], snd[order], rcv[order], Z)
    ref, mag = H.forward_reference(idx, val, mix, x, y, s, snd, rcv, Z)
    H.assert_parity(a, ref, mag, "unsorted")


def test_c_checker_in_float64_is_the_numpy_restatement():
    """The C loops compiled for double (the exact reference of the full-size GPU tests) against the
    numpy restatement in float64, forward and VJP, with padding edges and an unsorted edge list."""
    from oracle import c_oracle
    rng = np.random.default_rng(21)
    idx, val, mix = H.random_table(rng, 60, 6, 5, 11, 4)
    snd, rcv = H.random_graph(rng, 30, 200, sort_by=None)
    snd[::17] = np.iinfo(np.int32).max
    rcv[5::23] = np.iinfo(np.int32).max
    x, y, s, dm = H.random_operands(rng, 30, 200, 6, 5, 4, 12, 11)
    got = c_oracle.convolution(idx, val, mix, x, y, s, snd, rcv, 11, dtype=np.float64)
    want = O.convolution_unfused(idx, val, mix, x, y, s, snd, rcv, 11, dtype=np.float64)
    assert got.dtype == np.float64
    np.testing.assert_allclose(got, want, rtol=1e-13, atol=1e-13)
    grads = c_oracle.convolution_vjp(idx, val, mix, x, y, s, snd, rcv, dm, dtype=np.float64)
    wants = O.convolution_vjp(idx, val, mix, x, y, s, snd, rcv, dm, dtype=np.float64)
    for g, w_ in zip(grads, wants):
        np.testing.assert_allclose(g, w_, rtol=1e-13, atol=1e-12)
    # and the float32 build differs from it by float32 rounding only
    low = c_oracle.convolution(idx, val, mix, x, y, s, snd, rcv, 11)
    assert low.dtype == np.float32 and np.abs(low - want).max() <= 1e-5 * np.abs(want).max()
