"""CPU restatement of the reference's unfused message-passing convolution.

TEST INFRASTRUCTURE ONLY.  Nothing in the `e3j_amd` package imports this
module; it is the checker for the HIP kernels (used by `tests/`, by
`__graft_entry__.smoke()` and by the `cpu_baseline` leg of `bench.py`).

What is restated, and from where:

* `convolution_unfused`  - `Convolution._unfused_eval`
  (`src/e3j/core/convolution.py:172-191`): gather `x[senders]`; sparse
  tensor product `(x_j * y_k) * c_ijk` scatter-added over output coordinates
  (`src/e3j/core/tensor_product.py:300-319`, `src/e3j/utils/sparse.py:251-268`);
  scalar mixing `s[:, mix_idx] * messages` (`src/e3j/core/scalar_mixing.py:69-91`);
  scatter-add over receivers.  Same operation order, same dtype, both layouts.
  Identical to `convolution_reference` of the reference's op tests
  (`tests/test_ops/test_convolution_op.py:56-70`).
* `convolution_vjp`      - the three transposed trilinear forms the reference
  hands to its backward kernel (`src/e3j/ops/convolution.py:361-369`), written
  as explicit sums (same sums as the CPU loop of
  `lib/e3j_ops/tests/test_convolution_bwd.cpp:111-182`).
* `convolution_loops` / `convolution_vjp_loops` - literal pure-Python loops of
  `lib/e3j_ops/tests/test_convolution.cpp:63-106` and
  `test_convolution_bwd.cpp:111-182`, for tiny cases only.
* `strip_case`           - the hand-built known-answer case of
  `lib/e3j_ops/tests/test_convolution.cpp:122-207`.
* `receiver_ptr`, `transpose_graph`, `mask_edges`, `fold_endpoints` - CSR and
  padding semantics of `src/e3j/data/graph.py:49-91` and
  `src/e3j/ops/convolution.py:39-78`.

Padding: an edge whose sender or receiver lies outside `[0, num_nodes)`
contributes nothing and receives zero `dy`/`ds` (out-of-bounds scatter is
dropped in the unfused path; `lib/e3j_ops/cuda/convolution/fwd.cuh:368`,
`bwd.cuh:225-226,308-319` for the fused one).

Pinning status.  `convolution_unfused` and `convolution_vjp` are pinned by:
the strip case's closed-form answers (required bit-exact by the reference,
`test_convolution.cpp:288-290`), the literal loops on small random cases,
`torch.autograd` of an independent torch restatement, central differences in
float64, and the Euler identities of a trilinear form.  The graph helpers are
pinned by the expected arrays of `tests/test_graph.py:86-141`.
"""

from __future__ import annotations

import numpy as np

DUMMY_INDEX = np.int32(np.iinfo(np.int32).max)


# ---------------------------------------------------------------------------
# graph helpers
# ---------------------------------------------------------------------------
def receiver_ptr(receivers, num_nodes: int) -> np.ndarray:
    """`[0] + cumsum(bincount(receivers, length=num_nodes))`, int32; out-of-range keys drop out."""
    receivers = np.asarray(receivers, dtype=np.int64)
    live = receivers[(receivers >= 0) & (receivers < num_nodes)]
    counts = np.bincount(live, minlength=num_nodes)[:num_nodes]
    return np.concatenate(([0], np.cumsum(counts))).astype(np.int32)


def transpose_graph(senders, receivers, num_nodes: int):
    """Sort edges by sender: `(perm, receiver_t, sender_ptr)` with `receiver_t = receivers[perm]`."""
    senders = np.asarray(senders)
    perm = np.argsort(senders, kind="stable").astype(np.int32)
    return perm, np.asarray(receivers)[perm], receiver_ptr(senders[perm], num_nodes)


def mask_edges(senders, receivers, node_mask):
    """Edges touching a node at or past `count_nonzero(node_mask)` get `DUMMY_INDEX` on both ends."""
    real = int(np.count_nonzero(node_mask))
    senders, receivers = np.asarray(senders), np.asarray(receivers)
    keep = (senders < real) & (receivers < real)
    return (np.where(keep, senders, DUMMY_INDEX).astype(np.int32),
            np.where(keep, receivers, DUMMY_INDEX).astype(np.int32))


def wrap_global_index(index, num_nodes: int) -> np.ndarray:
    """`index % num_nodes`, keeping the `DUMMY_INDEX` sentinel."""
    index = np.asarray(index)
    return np.where(index == DUMMY_INDEX, index, index % num_nodes).astype(np.int32)


def fold_endpoints(group, guard, axis_size: int, num_nodes: int):
    """Fold `axis_size` graphs of `(axis_size, E)` endpoints into one disjoint graph.

    Grouping endpoints of padding edges move to their graph's last node, guard
    endpoints keep the sentinel (`src/e3j/ops/convolution.py:54-78`).
    """
    group, guard = np.asarray(group), np.asarray(guard)
    offsets = (np.arange(axis_size, dtype=group.dtype) * num_nodes)[:, None]
    last = offsets + (num_nodes - 1)
    group = np.where(group == DUMMY_INDEX, last, group + offsets)
    guard = np.where(guard == DUMMY_INDEX, guard, guard + offsets)
    return group.reshape(-1).astype(np.int32), guard.reshape(-1).astype(np.int32)


# ---------------------------------------------------------------------------
# layout helpers: everything below computes in (rows, dim, channels)
# ---------------------------------------------------------------------------
def _to_trailing(a, leading: bool):
    a = np.asarray(a)
    return np.swapaxes(a, -1, -2) if (leading and a.ndim == 3) else a


def _live_edges(senders, receivers, num_nodes):
    senders = np.asarray(senders, dtype=np.int64)
    receivers = np.asarray(receivers, dtype=np.int64)
    return (senders >= 0) & (senders < num_nodes) & (receivers >= 0) & (receivers < num_nodes)


# ---------------------------------------------------------------------------
# forward
# ---------------------------------------------------------------------------
def convolution_unfused(idx, val, mix_idx, x, y, s, senders, receivers, num_out: int,
                        leading: bool = False, dtype=np.float32, chunk: int = 4096) -> np.ndarray:
    """out[r, i, c] = sum_{e: recv(e)=r} s[e, mix[i], c] * sum_{(v;i,j,k)} (x[send(e), j, c] * y[e, k]) * v.

    idx: (nnz, 3) = (i, j, k); val: (nnz,); mix_idx: (num_out,).
    x: (N, X, K) [leading: (N, K, X)]; y: (E, Y); s: (E, S, K) [leading: (E, K, S)].
    Edges are processed in chunks of `chunk` so the (E, nnz, K) intermediate stays small;
    chunking does not change any summation order.
    """
    idx = np.asarray(idx, dtype=np.int64)
    val = np.asarray(val).astype(dtype)
    mix_idx = np.asarray(mix_idx, dtype=np.int64)
    x = _to_trailing(x, leading).astype(dtype, copy=False)
    s = _to_trailing(s, leading).astype(dtype, copy=False)
    y = np.asarray(y).astype(dtype, copy=False)
    if y.ndim == 3:
        y = y[..., 0]
    num_nodes, _, channels = x.shape
    senders = np.asarray(senders, dtype=np.int64)
    receivers = np.asarray(receivers, dtype=np.int64)
    live = np.nonzero(_live_edges(senders, receivers, num_nodes))[0]
    out = np.zeros((num_nodes, num_out, channels), dtype=dtype)
    for start in range(0, live.shape[0], chunk):
        e = live[start:start + chunk]
        x_e = x[senders[e]]                                     # gather
        cxy = (x_e[:, idx[:, 1], :] * y[e][:, idx[:, 2], None]) * val[None, :, None]
        msg = np.zeros((e.shape[0], num_out, channels), dtype=dtype)
        np.add.at(msg, (slice(None), idx[:, 0]), cxy)           # aggregate over output coords
        msg = s[e][:, mix_idx, :] * msg                         # scalar mixing
        np.add.at(out, receivers[e], msg)                       # scatter-add over receivers
    return np.swapaxes(out, -1, -2) if leading else out


def convolution_loops(idx4, val, x, y, s, sender, ptr, num_out: int) -> np.ndarray:
    """Literal loops of `cpu_convolution` (`lib/e3j_ops/tests/test_convolution.cpp:63-106`), float32.

    idx4: (nnz, 4) = (i, j, k, l); CSR adjacency `(sender, ptr)`; trailing layout.
    """
    f = np.float32
    num_nodes, _, channels = x.shape
    out = np.zeros((num_nodes, num_out, channels), dtype=f)
    for r in range(num_nodes):
        for e in range(int(ptr[r]), int(ptr[r + 1])):
            for u in range(channels):
                message = np.zeros(num_out, dtype=f)
                for n in range(len(val)):
                    i, j, k, l = (int(t) for t in idx4[n])
                    message[i] = f(message[i] + f(f(f(f(val[n]) * x[sender[e], j, u]) * y[e, k]) * s[e, l, u]))
                for i in range(num_out):
                    out[r, i, u] = f(out[r, i, u] + message[i])
    return out


# ---------------------------------------------------------------------------
# backward
# ---------------------------------------------------------------------------
def convolution_vjp(idx, val, mix_idx, x, y, s, senders, receivers, dm,
                    leading: bool = False, dtype=np.float32, chunk: int = 4096):
    """Cotangents `(dx, dy, ds)` of `convolution_unfused` for the output cotangent `dm`.

    dx[n,j,c] = sum_{e: send(e)=n} sum v * dm[recv(e),i,c] * y[e,k] * s[e,l(i),c]
    dy[e,k]   = sum_c sum v * dm[recv(e),i,c] * x[send(e),j,c] * s[e,l(i),c]
    ds[e,l,c] = sum_{l(i)=l} v * dm[recv(e),i,c] * x[send(e),j,c] * y[e,k]
    Padding edges get zero `dy` and `ds`.
    """
    idx = np.asarray(idx, dtype=np.int64)
    val = np.asarray(val).astype(dtype)
    mix_idx = np.asarray(mix_idx, dtype=np.int64)
    x_t = _to_trailing(x, leading).astype(dtype, copy=False)
    s_t = _to_trailing(s, leading).astype(dtype, copy=False)
    dm_t = _to_trailing(dm, leading).astype(dtype, copy=False)
    y2 = np.asarray(y).astype(dtype, copy=False)
    y_shape = y2.shape
    if y2.ndim == 3:
        y2 = y2[..., 0]
    num_nodes = x_t.shape[0]
    senders = np.asarray(senders, dtype=np.int64)
    receivers = np.asarray(receivers, dtype=np.int64)
    live = np.nonzero(_live_edges(senders, receivers, num_nodes))[0]
    i_idx, j_idx, k_idx = idx[:, 0], idx[:, 1], idx[:, 2]
    l_idx = mix_idx[i_idx]
    dx = np.zeros_like(x_t)
    dy = np.zeros_like(y2)
    ds = np.zeros_like(s_t)
    for start in range(0, live.shape[0], chunk):
        e = live[start:start + chunk]
        x_e = x_t[senders[e]][:, j_idx, :]           # (e, nnz, K)
        g_e = dm_t[receivers[e]][:, i_idx, :]        # (e, nnz, K)
        s_e = s_t[e][:, l_idx, :]                    # (e, nnz, K)
        y_e = y2[e][:, k_idx, None]                  # (e, nnz, 1)
        v = val[None, :, None]
        gs = g_e * s_e
        # dx: scatter over (sender, j)
        t = (gs * y_e) * v
        dxe = np.zeros((e.shape[0],) + x_t.shape[1:], dtype=dtype)
        np.add.at(dxe, (slice(None), j_idx), t)
        np.add.at(dx, senders[e], dxe)
        # dy: reduce over channels, scatter over k
        t = ((gs * x_e) * v).sum(axis=-1)
        dye = np.zeros((e.shape[0], y2.shape[1]), dtype=dtype)
        np.add.at(dye, (slice(None), k_idx), t)
        dy[e] = dye
        # ds: scatter over l
        t = ((g_e * x_e) * y_e) * v
        dse = np.zeros((e.shape[0],) + s_t.shape[1:], dtype=dtype)
        np.add.at(dse, (slice(None), l_idx), t)
        ds[e] = dse
    if leading:
        dx, ds = np.swapaxes(dx, -1, -2), np.swapaxes(ds, -1, -2)
    return dx, dy.reshape(y_shape), ds


def convolution_vjp_loops(idx, val, mix_idx, x, y, s, dz, sender, ptr):
    """Literal loops of `cpu_convolution_bwd` (`lib/e3j_ops/tests/test_convolution_bwd.cpp:111-182`)."""
    f = np.float32
    num_nodes, _, channels = x.shape
    num_out = dz.shape[1]
    dx = np.zeros_like(x, dtype=f)
    dy = np.zeros_like(y, dtype=f)
    ds = np.zeros_like(s, dtype=f)
    for recv in range(num_nodes):
        for e in range(int(ptr[recv]), int(ptr[recv + 1])):
            send = int(sender[e])
            for ch in range(channels):
                for n in range(len(val)):
                    i, j, k = (int(t) for t in idx[n])
                    ds[e, mix_idx[i], ch] += f(f(f(f(val[n]) * x[send, j, ch]) * y[e, k]) * dz[recv, i, ch])
                g = np.array([f(s[e, mix_idx[i], ch] * dz[recv, i, ch]) for i in range(num_out)], dtype=f)
                for n in range(len(val)):
                    i, j, k = (int(t) for t in idx[n])
                    dx[send, j, ch] += f(f(f(val[n]) * g[i]) * y[e, k])
                    dy[e, k] += f(f(f(val[n]) * g[i]) * x[send, j, ch])
    return dx, dy, ds


# ---------------------------------------------------------------------------
# known-answer case of the reference's C++ forward test
# ---------------------------------------------------------------------------
def strip_case(num_strips: int = 3, channels: int = 32, scale_s: bool = False):
    """Inputs of `prepareHostArgs` (`lib/e3j_ops/tests/test_convolution.cpp:122-207`).

    Per strip t: outputs (2t, 2t+1), x coords (2t, 2t+1), y coords (3t..3t+2),
    one scalar t; all six coefficients are 1: out[2t+a] = x[2t+a] * (y0+y1+y2).
    x = (1, 2) per strip on every node, y = (3, 4, 5) per strip on every edge,
    s = 1 or (edge+1)*(strip+1).  4 nodes, 6 edges:
    node 0 <- {1, 2}, node 1 <- {0, 3}, node 2 <- {0}, node 3 <- {1}.
    Closed form: out[r, 2t+a, c] = (a+1) * 12 * sum_{e in row r} s[e, t].
    """
    n_nodes, n_edges = 4, 6
    i = np.tile([0, 0, 0, 1, 1, 1], num_strips) + np.repeat(np.arange(num_strips), 6) * 2
    j = i.copy()
    k = np.tile([0, 1, 2, 0, 1, 2], num_strips) + np.repeat(np.arange(num_strips), 6) * 3
    idx = np.stack([i, j, k], axis=-1)
    val = np.ones(6 * num_strips, dtype=np.float32)
    mix_idx = np.repeat(np.arange(num_strips), 2)
    x = np.tile(np.repeat(np.tile([1.0, 2.0], num_strips), channels).reshape(2 * num_strips, channels),
                (n_nodes, 1, 1)).astype(np.float32)
    y = np.tile(np.tile([3.0, 4.0, 5.0], num_strips), (n_edges, 1)).astype(np.float32)
    if scale_s:
        s = ((np.arange(n_edges) + 1)[:, None, None] * (np.arange(num_strips) + 1)[None, :, None]
             * np.ones((1, 1, channels))).astype(np.float32)
    else:
        s = np.ones((n_edges, num_strips, channels), dtype=np.float32)
    sender = np.array([1, 2, 0, 3, 0, 1], dtype=np.int32)
    ptr = np.array([0, 2, 4, 5, 6], dtype=np.int32)
    receiver = np.repeat(np.arange(n_nodes), np.diff(ptr)).astype(np.int32)
    # closed-form expectation, exact in float32 (small integers)
    expect = np.zeros((n_nodes, 2 * num_strips, channels), dtype=np.float32)
    for r in range(n_nodes):
        for t in range(num_strips):
            s_sum = s[ptr[r]:ptr[r + 1], t, :].sum(axis=0)
            for a in range(2):
                expect[r, 2 * t + a, :] = (a + 1) * 12.0 * s_sum
    return dict(idx=idx, val=val, mix_idx=mix_idx, x=x, y=y, s=s, sender=sender,
                receiver=receiver, ptr=ptr, num_out=2 * num_strips, expect=expect)
