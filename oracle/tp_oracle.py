"""CPU restatement of the reference's row-wise sparse tensor product.

TEST INFRASTRUCTURE ONLY.  Nothing in the `e3j_amd` package imports this module; it is the
checker for the HIP tensor-product kernels (used by `tests/` only).

What is restated, and from where:

* `tensor_product_unfused` - `TensorProduct._sparse_eval`
  (`src/e3j/core/tensor_product.py:300-319`): gather `x[..., j]`, `y[..., k]`, multiply with
  the coefficients, scatter-add over output coordinates (`src/e3j/utils/sparse.py:251-268`),
  with the channel modes of `tensor_product_reference` of the reference's op tests
  (`tests/test_ops/test_tensor_product_op.py:86-147`): OUTER broadcasts or crosses the channel
  axes, INNER sums the shared channel axis after the product, MAP keeps it.
* `tensor_product_vjp`     - the two transposed bilinear forms the reference hands to its
  backward kernel (`src/e3j/ops/tensor_product.py:331-338,503-560`), written as explicit sums.
* `tensor_product_loops`   - literal pure-Python loops, for tiny cases only.

All functions work in the leading-channels form `(rows, channels, dim)` internally; the
trailing layout `(rows, dim, channels)` is a transpose of the last two axes on the way in and
out, as in the reference's test helper (`test_tensor_product_op.py:91-98`).

Pinning status.  `tensor_product_unfused` is pinned by the dense contraction
`einsum("ijk,...j,...k->...i")` of `TensorProduct._dense_eval`
(`src/e3j/core/tensor_product.py:276-278`) on Clebsch-Gordan tables and random tables, by the
literal loops, and by closed forms (1o x 1o -> 0e is the dot product over sqrt(3), 1o x 1o -> 1e
the cross product over sqrt(6)); `tensor_product_vjp` by central differences in float64 and by
the Euler identity of a bilinear form (<dx, x> = <dy, y> = <dz, z>).
"""

from __future__ import annotations

import numpy as np

OUTER, INNER, MAP = "OUTER", "INNER", "MAP"


def _to_leading(a: np.ndarray, layout: str) -> np.ndarray:
    if a.ndim == 3 and layout == "TRAILING_CHANNELS":
        return np.swapaxes(a, 1, 2)
    return a


def _from_leading(a: np.ndarray, layout: str) -> np.ndarray:
    if layout != "TRAILING_CHANNELS" or a.ndim < 3:
        return a
    return np.ascontiguousarray(np.moveaxis(a, -1, 1))


def _scatter_last(terms: np.ndarray, i: np.ndarray, num_out: int) -> np.ndarray:
    """Sum `terms[..., n]` into `out[..., i[n]]`, in table order."""
    out = np.zeros(terms.shape[:-1] + (num_out,), dtype=terms.dtype)
    np.add.at(out, (..., i), terms)
    return out


def tensor_product_unfused(idx, val, x, y, num_out, mode=OUTER, layout="LEADING_CHANNELS"):
    """`z[..., i] += val * x[..., j] * y[..., k]` with the channel mode applied.

    idx: (nnz, 3) columns (i, j, k); val: (nnz,).  x: (R, X) or (R, Cx, X) [trailing (R, X, Cx)],
    y likewise.  Returns (R, Z), (R, C, Z) or (R, Cx, Cy, Z) [trailing (R, Z, ...)].
    """
    idx = np.asarray(idx).astype(np.int64)
    x, y = _to_leading(np.asarray(x), layout), _to_leading(np.asarray(y), layout)
    val = np.asarray(val).astype(x.dtype)
    i, j, k = idx[:, 0], idx[:, 1], idx[:, 2]
    has_cx, has_cy = x.ndim > 2, y.ndim > 2
    if mode in (MAP, INNER):
        assert has_cx and has_cy and x.shape[1] == y.shape[1]
        terms = (x[..., j] * y[..., k]) * val
        if mode == INNER:
            terms = terms.sum(axis=-2)
    elif has_cx and has_cy:
        terms = (x[:, :, None, j] * y[:, None, :, k]) * val
    elif has_cx:
        terms = (x[..., j] * y[:, None, k]) * val
    elif has_cy:
        terms = (x[:, None, j] * y[..., k]) * val
    else:
        terms = (x[..., j] * y[..., k]) * val
    return _from_leading(_scatter_last(terms, i, num_out), layout)


def tensor_product_vjp(idx, val, x, y, dz, mode=OUTER, layout="LEADING_CHANNELS"):
    """`(dx, dy)` with `dx[..., j] += val * dz[..., i] * y[..., k]` and
    `dy[..., k] += val * dz[..., i] * x[..., j]`, summed over whatever axis the forward mode
    broadcast or crossed."""
    idx = np.asarray(idx).astype(np.int64)
    x_in, y_in = np.asarray(x), np.asarray(y)
    x, y = _to_leading(x_in, layout), _to_leading(y_in, layout)
    dz = np.asarray(dz)
    if layout == "TRAILING_CHANNELS" and dz.ndim > 2:
        dz = np.moveaxis(dz, 1, -1)
    val = np.asarray(val).astype(x.dtype)
    i, j, k = idx[:, 0], idx[:, 1], idx[:, 2]
    has_cx, has_cy = x.ndim > 2, y.ndim > 2
    X, Y = x.shape[-1], y.shape[-1]
    g = dz[..., i] * val                                  # (..., nnz)
    if mode == MAP:
        tx, ty = g * y[..., k], g * x[..., j]
    elif mode == INNER:
        tx, ty = g[:, None, :] * y[..., k], g[:, None, :] * x[..., j]
    elif has_cx and has_cy:
        tx = (g * y[:, None, :, k]).sum(axis=2)
        ty = (g * x[:, :, None, j]).sum(axis=1)
    elif has_cx:
        tx = g * y[:, None, k]
        ty = (g * x[..., j]).sum(axis=1)
    elif has_cy:
        tx = (g * y[..., k]).sum(axis=1)
        ty = g * x[:, None, j]
    else:
        tx, ty = g * y[..., k], g * x[..., j]
    dx = _scatter_last(tx, j, X)
    dy = _scatter_last(ty, k, Y)
    if layout == "TRAILING_CHANNELS":
        dx = np.ascontiguousarray(np.swapaxes(dx, 1, 2)) if dx.ndim == 3 else dx
        dy = np.ascontiguousarray(np.swapaxes(dy, 1, 2)) if dy.ndim == 3 else dy
    return dx, dy


def tensor_product_loops(idx, val, x, y, num_out, mode=OUTER):
    """Pure-Python loops, leading layout: x (R, Cx, X) or (R, X); y likewise."""
    x, y = np.asarray(x), np.asarray(y)
    rows = x.shape[0]
    has_cx, has_cy = x.ndim > 2, y.ndim > 2
    cx = x.shape[1] if has_cx else 1
    cy = y.shape[1] if has_cy else 1
    x3 = x.reshape(rows, cx, -1)
    y3 = y.reshape(rows, cy, -1)
    if mode == OUTER:
        z = np.zeros((rows, cx, cy, num_out), dtype=x.dtype)
        for r in range(rows):
            for a in range(cx):
                for b in range(cy):
                    for (i, j, k), c in zip(idx, val):
                        z[r, a, b, i] += c * x3[r, a, j] * y3[r, b, k]
        shape = (rows,) + ((cx,) if has_cx else ()) + ((cy,) if has_cy else ()) + (num_out,)
        return z.reshape(shape)
    z = np.zeros((rows, cx, num_out), dtype=x.dtype)
    for r in range(rows):
        for a in range(cx):
            for (i, j, k), c in zip(idx, val):
                z[r, a, i] += c * x3[r, a, j] * y3[r, a, k]
    return z.sum(axis=1) if mode == INNER else z
