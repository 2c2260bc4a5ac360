"""The CPU checker of the row-wise tensor product against what the mathematics fixes, and the
host logic of the operator (no GPU)."""

import numpy as np
import pytest
import torch

import e3j_amd
from e3j_amd import TensorProduct
from e3j_amd.coef import Coef
from e3j_amd.tp_ops import TensorProductParams, _Table
from oracle import tp_oracle as T
from tests import helpers as H

MODES = ("OUTER", "INNER", "MAP")
LAYOUTS = ("LEADING_CHANNELS", "TRAILING_CHANNELS")


def _dense(idx, val, shape):
    d = np.zeros(shape)
    np.add.at(d, tuple(np.asarray(idx).T.astype(np.int64)), np.asarray(val, dtype=np.float64))
    return d


def _dense_eval(dense, x, y, mode, has_cx=True, has_cy=True):
    """Leading layout, the contraction of `TensorProduct._dense_eval`
    (src/e3j/core/tensor_product.py:276-278) with explicit channel letters."""
    if mode == "MAP":
        return np.einsum("ijk,rcj,rck->rci", dense, x, y)
    if mode == "INNER":
        return np.einsum("ijk,rcj,rck->ri", dense, x, y)
    sx = "raj" if has_cx else "rj"
    sy = "rbk" if has_cy else "rk"
    so = "r" + ("a" if has_cx else "") + ("b" if has_cy else "") + "i"
    return np.einsum(f"ijk,{sx},{sy}->{so}", dense, x, y)


def _cg_table():
    tp = TensorProduct(("0e+1o+2e", "0e+1o+2e"), None)
    return np.asarray(tp.indices, dtype=np.int64), np.asarray(tp.values, dtype=np.float64), tp.shape


def _random_table(rng, nnz=120, dims=(11, 7, 5)):
    idx, val, _ = H.random_table(rng, nnz, dims[1], dims[2], dims[0], 3)
    return idx, val, dims


@pytest.mark.parametrize("table", ["cg", "random"])
@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("layout", LAYOUTS)
def test_unfused_matches_dense_contraction(table, mode, layout):
    rng = np.random.default_rng(0)
    idx, val, shape = _cg_table() if table == "cg" else _random_table(rng)
    Z, X, Y = shape
    x = rng.normal(size=(6, 4, X))
    y = rng.normal(size=(6, 4, Y))
    want = _dense_eval(_dense(idx, val, shape), x, y, mode)
    tr = layout == "TRAILING_CHANNELS"
    xin, yin = (np.swapaxes(x, 1, 2), np.swapaxes(y, 1, 2)) if tr else (x, y)
    got = T.tensor_product_unfused(idx, val, xin, yin, Z, mode, layout)
    if tr and got.ndim > 2:
        got = np.moveaxis(got, 1, -1)
    assert got.shape == want.shape
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("has_cx,has_cy", [(True, False), (False, True), (False, False), (True, True)])
@pytest.mark.parametrize("layout", LAYOUTS)
def test_outer_mode_channel_axes(has_cx, has_cy, layout):
    rng = np.random.default_rng(1)
    idx, val, shape = _random_table(rng)
    Z, X, Y = shape
    x = rng.normal(size=(5, 3, X) if has_cx else (5, X))
    y = rng.normal(size=(5, 2, Y) if has_cy else (5, Y))
    want = _dense_eval(_dense(idx, val, shape), x, y, "OUTER", has_cx, has_cy)
    tr = layout == "TRAILING_CHANNELS"
    xin = np.swapaxes(x, 1, 2) if tr and has_cx else x
    yin = np.swapaxes(y, 1, 2) if tr and has_cy else y
    got = T.tensor_product_unfused(idx, val, xin, yin, Z, "OUTER", layout)
    if tr and got.ndim > 2:
        got = np.moveaxis(got, 1, -1)
    assert got.shape == want.shape
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("mode", MODES)
def test_unfused_matches_literal_loops(mode):
    rng = np.random.default_rng(2)
    idx, val, (Z, X, Y) = _random_table(rng, nnz=40, dims=(6, 4, 3))
    x, y = rng.normal(size=(3, 2, X)), rng.normal(size=(3, 2, Y))
    np.testing.assert_allclose(T.tensor_product_unfused(idx, val, x, y, Z, mode),
                               T.tensor_product_loops(idx, val, x, y, Z, mode), rtol=1e-13, atol=1e-13)


def test_closed_forms_of_vector_products():
    """1o x 1o -> 0e is the dot product over sqrt(3); -> 1e the cross product over sqrt(6) (the
    blocks have unit Frobenius norm: 3 entries of 1/sqrt(3), 6 entries of 1/sqrt(6); up to
    the sign and axis convention fixed by the table: checked through norms and the Lagrange
    identity; the table holds float32 values, hence 1e-6)."""
    rng = np.random.default_rng(3)
    a, b = rng.normal(size=(7, 3)), rng.normal(size=(7, 3))
    tp0 = TensorProduct(("1o", "1o"), "0e")
    z0 = T.tensor_product_unfused(tp0.indices, tp0.values, a, b, 1)
    np.testing.assert_allclose(np.abs(z0[:, 0]), np.abs((a * b).sum(1)) / np.sqrt(3), rtol=1e-6)
    tp1 = TensorProduct(("1o", "1o"), "1e")
    z1 = T.tensor_product_unfused(tp1.indices, tp1.values, a, b, 3)
    np.testing.assert_allclose(np.linalg.norm(z1, axis=1), np.linalg.norm(np.cross(a, b), axis=1) / np.sqrt(6),
                               rtol=1e-6)
    np.testing.assert_allclose((z1 * z1).sum(1) * 6 + ((a * b).sum(1)) ** 2,
                               (a * a).sum(1) * (b * b).sum(1), rtol=1e-6)   # Lagrange identity


@pytest.mark.parametrize("mode,has_cx,has_cy", [("MAP", True, True), ("INNER", True, True),
                                                ("OUTER", True, False), ("OUTER", False, True),
                                                ("OUTER", False, False), ("OUTER", True, True)])
@pytest.mark.parametrize("layout", LAYOUTS)
def test_vjp_against_central_differences_and_euler(mode, has_cx, has_cy, layout):
    rng = np.random.default_rng(4)
    idx, val, (Z, X, Y) = _random_table(rng, nnz=60, dims=(7, 5, 4))
    tr = layout == "TRAILING_CHANNELS"
    C = 3
    x = rng.normal(size=((4, X, C) if tr else (4, C, X)) if has_cx else (4, X))
    y = rng.normal(size=((4, Y, C) if tr else (4, C, Y)) if has_cy else (4, Y))
    f = lambda a, b: T.tensor_product_unfused(idx, val, a, b, Z, mode, layout)  # noqa: E731
    z = f(x, y)
    dz = rng.normal(size=z.shape)
    dx, dy = T.tensor_product_vjp(idx, val, x, y, dz, mode, layout)
    assert dx.shape == x.shape and dy.shape == y.shape
    # bilinear: <dx, x> = <dy, y> = <dz, z>
    np.testing.assert_allclose((dx * x).sum(), (dz * z).sum(), rtol=1e-11)
    np.testing.assert_allclose((dy * y).sum(), (dz * z).sum(), rtol=1e-11)
    h = 1e-6
    for arr, grad, which in ((x, dx, 0), (y, dy, 1)):
        for _ in range(5):
            pos = tuple(rng.integers(0, n) for n in arr.shape)
            e = np.zeros_like(arr)
            e[pos] = h
            args_p = (x + e, y) if which == 0 else (x, y + e)
            args_m = (x - e, y) if which == 0 else (x, y - e)
            fd = ((f(*args_p) - f(*args_m)) * dz).sum() / (2 * h)
            np.testing.assert_allclose(grad[pos], fd, rtol=1e-6, atol=1e-8)


def test_backward_tables_are_sorted_transposes():
    rng = np.random.default_rng(5)
    idx, val, _ = _random_table(rng)
    shuffle = rng.permutation(len(val))
    packed = Coef(val[shuffle], idx[shuffle], "float32", "int32").pack()
    t = _Table.get(packed, np.float32)
    assert not t.sorted
    for half, cols in enumerate(((1, 0, 2), (2, 0, 1))):
        c = Coef.unpack(t.packed_bwd[half], np.float32)
        assert np.all(np.diff(c.idx[:, 0].astype(np.int64)) >= 0)
        want = sorted(zip(idx[:, cols[0]], idx[:, cols[1]], idx[:, cols[2]], val.astype(np.float32)))
        got = sorted(zip(c.idx[:, 0], c.idx[:, 1], c.idx[:, 2], c.val))
        assert [tuple(map(float, a)) for a in got] == [tuple(map(float, a)) for a in want]
    assert _Table.get(Coef(val, idx, "float32", "uint8").pack(), np.float32).sorted


def test_operator_argument_errors_need_no_gpu():
    idx, val, (Z, X, Y) = _random_table(np.random.default_rng(6))
    coef = Coef(val, idx, "float32", "int32").pack()
    p = TensorProductParams(num_out=Z, mode="MAP", layout="TRAILING_CHANNELS")
    x, y = torch.zeros(3, X, 4), torch.zeros(3, Y, 4)
    with pytest.raises(ValueError, match="no CPU path"):
        e3j_amd.tensor_product(coef, x, y, p)
    with pytest.raises(ValueError, match="rank 2 or 3"):
        e3j_amd.tensor_product(coef, torch.zeros(3), y, p)
    with pytest.raises(TypeError, match="share a dtype"):
        e3j_amd.tensor_product(coef, x.double(), y, p)
    with pytest.raises(NotImplementedError, match="float16, float32 or float64"):
        e3j_amd.tensor_product(coef, x.bfloat16(), y.bfloat16(), p)
    assert e3j_amd.CUDATensorProductParams is TensorProductParams
    assert e3j_amd.MixingMode.parse("map") is e3j_amd.MixingMode.MAP
    assert [m.value for m in e3j_amd.MixingMode] == [0, 1, 2]   # the integers the FFI carries
