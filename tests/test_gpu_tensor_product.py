"""Row-wise tensor product on the GPU against the CPU checker: the grid of the reference's op
tests (`tests/test_ops/test_tensor_product_op.py`: modes x channel counts x layouts, random
table of 530 entries over 42 x 25 coordinates) plus dtypes, index widths, unsorted tables,
uncovered coordinates, autograd to second order and the module-level call."""

import ctypes

import numpy as np
import pytest
import torch

import e3j_amd
from e3j_amd import TensorProduct, _lib
from e3j_amd.coef import Coef
from e3j_amd.tp_ops import TensorProductParams
from oracle import tp_oracle as T
from tests import helpers as H

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
MODES = ("OUTER", "INNER", "MAP")
LAYOUTS = ("LEADING_CHANNELS", "TRAILING_CHANNELS")
NUM_X, NUM_Y, NUM_OUT, NNZ = 42, 25, 30, 530


def _table(seed=1234, nnz=NNZ, dims=(NUM_OUT, NUM_X, NUM_Y)):
    idx, val, _ = H.random_table(np.random.default_rng(seed), nnz, dims[1], dims[2], dims[0], 3)
    return idx, val.astype(np.float64)


def _operands(rng, mode, layout, channels, rows=100, dims=(NUM_X, NUM_Y), dtype=np.float32, has=(True, True)):
    tr = layout == "TRAILING_CHANNELS"
    def make(dim, has_c):
        if not has_c:
            return rng.normal(size=(rows, dim)).astype(dtype)
        return rng.normal(size=(rows, dim, channels) if tr else (rows, channels, dim)).astype(dtype)
    if mode != "OUTER":
        has = (True, True)
    return make(dims[0], has[0]), make(dims[1], has[1])


def _check_forward(idx, val, x, y, num_out, mode, layout, idx_dtype="int32", what=""):
    coef = Coef(val, idx, str(x.dtype), idx_dtype).pack()
    p = TensorProductParams(num_out=num_out, mode=mode, layout=layout)
    z = e3j_amd.tensor_product(coef, torch.from_numpy(x).to(DEV), torch.from_numpy(y).to(DEV), p).cpu().numpy()
    x64, y64 = x.astype(np.float64), y.astype(np.float64)
    val_r = val.astype(x.dtype).astype(np.float64)    # the kernel sees the table rounded to the value dtype
    ref = T.tensor_product_unfused(idx, val_r, x64, y64, num_out, mode, layout)
    mag = T.tensor_product_unfused(idx, np.abs(val_r), np.abs(x64), np.abs(y64), num_out, mode, layout)
    if x.dtype == np.float64:
        np.testing.assert_allclose(z, ref, rtol=1e-12, atol=1e-12 * max(1.0, float(mag.max())))
    else:
        H.assert_parity(z, ref, mag, f"{what} z")
    return z


def _check_backward(idx, val, x, y, num_out, mode, layout, rng, idx_dtype="int32", what=""):
    coef = Coef(val, idx, str(x.dtype), idx_dtype).pack()
    p = TensorProductParams(num_out=num_out, mode=mode, layout=layout)
    xt = torch.from_numpy(x).to(DEV).requires_grad_(True)
    yt = torch.from_numpy(y).to(DEV).requires_grad_(True)
    z = e3j_amd.tensor_product(coef, xt, yt, p)
    dz = rng.normal(size=tuple(z.shape)).astype(x.dtype)
    dx, dy = torch.autograd.grad(z, (xt, yt), torch.from_numpy(dz).to(DEV))
    x64, y64, dz64 = (a.astype(np.float64) for a in (x, y, dz))
    val_r = val.astype(x.dtype).astype(np.float64)
    rdx, rdy = T.tensor_product_vjp(idx, val_r, x64, y64, dz64, mode, layout)
    mdx, mdy = T.tensor_product_vjp(idx, np.abs(val_r), np.abs(x64), np.abs(y64), np.abs(dz64), mode, layout)
    for got, ref, mag, name in ((dx, rdx, mdx, "dx"), (dy, rdy, mdy, "dy")):
        got = got.cpu().numpy()
        if x.dtype == np.float64:
            np.testing.assert_allclose(got, ref, rtol=1e-12, atol=1e-12 * max(1.0, float(mag.max())))
        else:
            H.assert_parity(got, ref, mag, f"{what} {name}", ulps=32.0)


@pytest.mark.parametrize("channels", [1, 2, 16, 32, 64, 128, 512])
@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("layout", LAYOUTS)
def test_forward_and_backward_grid(channels, mode, layout):
    rng = np.random.default_rng(channels)
    idx, val = _table()
    x, y = _operands(rng, mode, layout, channels, has=(True, False))
    _check_forward(idx, val, x, y, NUM_OUT, mode, layout, what=f"{mode} {layout} C={channels}")
    _check_backward(idx, val, x, y, NUM_OUT, mode, layout, rng, what=f"{mode} {layout} C={channels}")


@pytest.mark.parametrize("has", [(False, True), (False, False), (True, True)])
@pytest.mark.parametrize("layout", LAYOUTS)
def test_outer_mode_channel_axes(has, layout):
    rng = np.random.default_rng(7)
    idx, val = _table()
    x, y = _operands(rng, "OUTER", layout, 8, rows=37, has=has)
    if has == (True, True):    # different channel counts on the two sides
        tr = layout == "TRAILING_CHANNELS"
        y = rng.normal(size=(37, NUM_Y, 3) if tr else (37, 3, NUM_Y)).astype(np.float32)
    _check_forward(idx, val, x, y, NUM_OUT, "OUTER", layout, what=f"OUTER {has}")
    if has != (True, True):
        _check_backward(idx, val, x, y, NUM_OUT, "OUTER", layout, rng, what=f"OUTER {has}")
    else:
        coef = Coef(val, idx, "float32", "int32").pack()
        p = TensorProductParams(num_out=NUM_OUT, mode="OUTER", layout=layout)
        xt = torch.from_numpy(x).to(DEV).requires_grad_(True)
        z = e3j_amd.tensor_product(coef, xt, torch.from_numpy(y).to(DEV), p)
        with pytest.raises(NotImplementedError, match="channel axes on both inputs"):
            z.sum().backward()
        with pytest.raises(NotImplementedError, match="one channel"):
            e3j_amd.tensor_product_bwd(coef, xt, torch.from_numpy(y).to(DEV), z.detach(), p)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("idx_dtype", ["uint8", "int32"])
@pytest.mark.parametrize("mode", MODES)
def test_dtypes_and_index_widths(dtype, idx_dtype, mode):
    rng = np.random.default_rng(11)
    idx, val = _table()
    for layout in LAYOUTS:
        x, y = _operands(rng, mode, layout, 24, rows=33, dtype=dtype, has=(True, False))
        _check_forward(idx, val, x, y, NUM_OUT, mode, layout, idx_dtype, what=f"{mode} {dtype.__name__} {idx_dtype}")
        _check_backward(idx, val, x, y, NUM_OUT, mode, layout, rng, idx_dtype)


@pytest.mark.parametrize("mode", MODES)
def test_clebsch_gordan_table_through_the_module(mode):
    """`TensorProduct.__call__` on the full l <= 2 product (nnz 357) against the dense contraction."""
    rng = np.random.default_rng(12)
    for layout in LAYOUTS:
        tp = TensorProduct(("0e+1o+2e", "0e+1o+2e"), None, layout=layout, mode=mode)
        Z, X, Y = tp.shape
        x, y = _operands(rng, mode, layout, 64, rows=50, dims=(X, Y), has=(True, False))
        z = tp(torch.from_numpy(x).to(DEV), torch.from_numpy(y).to(DEV)).cpu().numpy()
        idx, val = np.asarray(tp.indices, dtype=np.int64), np.asarray(tp.values, dtype=np.float64)
        ref = T.tensor_product_unfused(idx, val, x.astype(np.float64), y.astype(np.float64), Z, mode, layout)
        mag = T.tensor_product_unfused(idx, np.abs(val), np.abs(x).astype(np.float64), np.abs(y).astype(np.float64),
                                       Z, mode, layout)
        H.assert_parity(z, ref, mag, f"module {mode} {layout}")


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("layout", LAYOUTS)
def test_unsorted_table_and_uncovered_coordinates(mode, layout):
    """Entries in any order give the same result; output coordinates (and, in the backward pass,
    input coordinates) that no entry touches are exact zeros, never stale memory
    (`tests/test_ops/test_zero_gap_rows.py:15-26`)."""
    rng = np.random.default_rng(13)
    idx, val = _table(nnz=200)
    keep = (idx[:, 0] != 3) & (idx[:, 0] != NUM_OUT - 1) & (idx[:, 1] != 5) & (idx[:, 2] != 0)
    idx, val = idx[keep], val[keep]
    x, y = _operands(rng, mode, layout, 16, rows=21, has=(True, False))
    z_sorted = _check_forward(idx, val, x, y, NUM_OUT, mode, layout, what="gaps")
    tr = layout == "TRAILING_CHANNELS"
    zi = np.moveaxis(z_sorted, 1, -1) if tr and z_sorted.ndim > 2 else z_sorted
    assert np.all(zi[..., 3] == 0) and np.all(zi[..., NUM_OUT - 1] == 0)
    shuffle = rng.permutation(len(val))
    z_any = _check_forward(idx[shuffle], val[shuffle], x, y, NUM_OUT, mode, layout, what="shuffled")
    np.testing.assert_allclose(z_any, z_sorted, rtol=1e-5, atol=1e-5)
    # backward: poison the results first, the gaps must come back as zeros
    coef = Coef(val[shuffle], idx[shuffle], "float32", "int32").pack()
    p = TensorProductParams(num_out=NUM_OUT, mode=mode, layout=layout)
    xt, yt = torch.from_numpy(x).to(DEV), torch.from_numpy(y).to(DEV)
    dz = torch.randn(tuple(z_sorted.shape), device=DEV)
    poison = [torch.full_like(xt, float("nan")), torch.full_like(yt, float("nan"))]
    torch.cuda.synchronize()
    del poison          # the allocator hands these blocks to the results of the next call
    dx, dy = e3j_amd.tensor_product_bwd(coef, xt, yt, dz, p)
    dxi = dx.movedim(1, -1) if tr and dx.ndim > 2 else dx
    dyi = dy.movedim(1, -1) if tr and dy.ndim > 2 else dy
    assert torch.all(dxi[..., 5] == 0) and torch.all(dyi[..., 0] == 0)
    assert torch.isfinite(dx).all() and torch.isfinite(dy).all()
    _check_backward(idx[shuffle], val[shuffle], x, y, NUM_OUT, mode, layout, rng, what="shuffled")


def _dense_torch(idx, val, num_out, dims, mode, layout, has):
    dense = torch.zeros((num_out,) + dims, dtype=torch.float64, device=DEV)
    dense.index_put_(tuple(torch.as_tensor(np.asarray(idx).T.astype(np.int64), device=DEV)),
                     torch.as_tensor(val, dtype=torch.float64, device=DEV), accumulate=True)
    tr = layout == "TRAILING_CHANNELS"

    def f(x, y):
        xl = x.transpose(1, 2) if tr and x.ndim == 3 else x
        yl = y.transpose(1, 2) if tr and y.ndim == 3 else y
        if mode == "MAP":
            z = torch.einsum("ijk,rcj,rck->rci", dense, xl, yl)
        elif mode == "INNER":
            z = torch.einsum("ijk,rcj,rck->ri", dense, xl, yl)
        else:
            sx = "raj" if has[0] else "rj"
            sy = "rbk" if has[1] else "rk"
            so = "r" + ("a" if has[0] else "") + ("b" if has[1] else "") + "i"
            z = torch.einsum(f"ijk,{sx},{sy}->{so}", dense, xl, yl)
        return z.movedim(-1, 1) if tr and z.ndim > 2 else z
    return f


@pytest.mark.parametrize("mode,has", [("MAP", (True, True)), ("INNER", (True, True)), ("OUTER", (True, False)),
                                      ("OUTER", (False, True))])
@pytest.mark.parametrize("layout", LAYOUTS)
def test_second_order_gradients_against_dense_autograd(mode, has, layout):
    rng = np.random.default_rng(14)
    idx, val = _table(nnz=90, dims=(9, 6, 5))
    x, y = _operands(rng, mode, layout, 4, rows=6, dims=(6, 5), dtype=np.float64, has=has)
    coef = Coef(val, idx, "float64", "int32").pack()
    p = TensorProductParams(num_out=9, mode=mode, layout=layout)
    dense = _dense_torch(idx, val, 9, (6, 5), mode, layout, has)

    def run(fn):
        xt = torch.from_numpy(x).to(DEV).requires_grad_(True)
        yt = torch.from_numpy(y).to(DEV).requires_grad_(True)
        z = fn(xt, yt)
        g = torch.Generator(device="cpu").manual_seed(0)
        dz = torch.randn(tuple(z.shape), generator=g, dtype=torch.float64).to(DEV).requires_grad_(True)
        dx, dy = torch.autograd.grad(z, (xt, yt), dz, create_graph=True)
        wx = torch.randn(tuple(dx.shape), generator=g, dtype=torch.float64).to(DEV)
        wy = torch.randn(tuple(dy.shape), generator=g, dtype=torch.float64).to(DEV)
        second = torch.autograd.grad((dx * wx).sum() + (dy * wy).sum(), (xt, yt, dz))
        return [z, dx, dy, *second]

    for a, b in zip(run(lambda u, v: e3j_amd.tensor_product(coef, u, v, p)), run(dense)):
        torch.testing.assert_close(a, b, rtol=1e-11, atol=1e-11)


def test_no_rows_and_repeatability():
    idx, val = _table()
    coef = Coef(val, idx, "float32", "uint8").pack()
    p = TensorProductParams(num_out=NUM_OUT, mode="MAP", layout="TRAILING_CHANNELS")
    z = e3j_amd.tensor_product(coef, torch.zeros(0, NUM_X, 8, device=DEV), torch.zeros(0, NUM_Y, 8, device=DEV), p)
    assert tuple(z.shape) == (0, NUM_OUT, 8)
    x, y = torch.randn(64, NUM_X, 32, device=DEV), torch.randn(64, NUM_Y, 32, device=DEV)
    a = e3j_amd.tensor_product(coef, x, y, p)
    b = e3j_amd.tensor_product(coef, x, y, p)
    assert torch.equal(a, b)


def test_c_abi_errors():
    lib = _lib.load()
    stream = int(torch.cuda.current_stream().cuda_stream)
    buf = torch.zeros(4096, device=DEV)
    def params(**kw):
        base = dict(num_rows=2, num_coef=3, num_x=4, num_y=3, num_out=5, channels_x=8, channels_y=8,
                    mode=_lib.MODE_MAP, layout=_lib.LAYOUT_TRAILING, val_dtype=_lib.F32, coef_idx_bytes=4,
                    coef_sorted=1, debug=0, signature=-1, coef_scale=1.0)
        base.update(kw)
        return _lib.TpParams(**base)
    def fwd(p):
        return lib.e3j_amd_tensor_product_fwd(ctypes.byref(p), buf.data_ptr(), buf.data_ptr(), buf.data_ptr(),
                                              buf.data_ptr(), stream)
    assert lib.e3j_amd_tensor_product_fwd(None, None, None, None, None, None) == _lib.INVALID_ARGUMENT
    assert fwd(params(mode=7)) == _lib.INVALID_ARGUMENT and b"unknown mode" in lib.e3j_amd_last_error()
    assert fwd(params(channels_y=4)) == _lib.INVALID_ARGUMENT and b"same number" in lib.e3j_amd_last_error()
    assert fwd(params(coef_idx_bytes=2)) == _lib.INVALID_ARGUMENT and b"dtype pair" in lib.e3j_amd_last_error()
    assert fwd(params(layout=5)) == _lib.INVALID_ARGUMENT
    assert fwd(params(mode=_lib.MODE_INNER, num_out=400, val_dtype=_lib.F64)) == _lib.UNIMPLEMENTED
    p = params(mode=_lib.MODE_OUTER, channels_y=2)
    rc = lib.e3j_amd_tensor_product_bwd(ctypes.byref(p), *[buf.data_ptr()] * 6, stream)
    assert rc == _lib.UNIMPLEMENTED and b"one channel" in lib.e3j_amd_last_error()
    torch.cuda.synchronize()


# ---------------------------------------------------------------------------
# compile-time-unrolled kernels (built-in Clebsch-Gordan tables, trailing layout)
# ---------------------------------------------------------------------------
KIND = {"MAP": 0, "OUTER": 1, "INNER": 2}
BUILTIN = [("0e+1o+2e", "0e+1o+2e", None), ("0e+1o+2e", "0e+1o+2e+3o", "0e+1o+2e+3o"),
           ("0e+1o+2e+3o", "0e+1o+2e+3o", "0e+1o+2e+3o")]


@pytest.mark.parametrize("spaces,channels", [(BUILTIN[t], k) for t in range(3) for k in (32, 64, 128)
                                             if not (t == 1 and k == 32)],   # (not built in at 32 channels)
                         ids=lambda v: str(v) if isinstance(v, int) else "-".join(str(a) for a in v))
@pytest.mark.parametrize("mode", ["MAP", "OUTER", "INNER"])
def test_unrolled_kernels_against_the_checker(spaces, channels, mode):
    """77 rows: at 32 channels a wave takes two rows side by side and the last wave has one."""
    from e3j_amd.tp_ops import _Table
    rng = np.random.default_rng(21)
    tp = TensorProduct(spaces[:2], spaces[2], layout="TRAILING_CHANNELS", mode=mode)
    Z, X, Y = tp.shape
    idx, val = np.asarray(tp.indices, dtype=np.int64), 1.5 * np.asarray(tp.values, dtype=np.float64)
    table = _Table.get(Coef(val, idx, "float32", "uint8").pack(), np.float32)
    sig, scale = table.signature(X, Y, Z, channels, KIND[mode])
    assert sig >= 0 and abs(scale - 1.5) < 1e-6, "a built-in unrolled kernel must serve this table"
    x, y = _operands(rng, mode, "TRAILING_CHANNELS", channels, rows=77, dims=(X, Y), has=(True, False))
    _check_forward(idx, val, x, y, Z, mode, "TRAILING_CHANNELS", "uint8", what=f"unrolled {mode} K={channels}")
    _check_backward(idx, val, x, y, Z, mode, "TRAILING_CHANNELS", rng, "uint8", what=f"unrolled {mode} K={channels}")


@pytest.mark.parametrize("mode", ["MAP", "OUTER", "INNER"])
def test_unrolled_and_table_driven_kernels_agree_through_the_c_abi(mode):
    lib = _lib.load()
    tp = TensorProduct(("0e+1o+2e+3o", "0e+1o+2e+3o"), "0e+1o+2e+3o", layout="TRAILING_CHANNELS", mode=mode)
    Z, X, Y = tp.shape
    K, R = 128, 301
    packed = tp.packed_coef("float32")
    from e3j_amd.tp_ops import _Table
    table = _Table.get(packed, np.float32)
    uniform = mode == "OUTER"
    sig, scale = table.signature(X, Y, Z, K, KIND[mode])
    assert sig >= 0
    g = torch.Generator(device="cpu").manual_seed(3)
    x = torch.randn(R, X, K, generator=g).to(DEV)
    y = (torch.randn(R, Y, generator=g) if uniform else torch.randn(R, Y, K, generator=g)).to(DEV)
    z_shape = (R, Z) if mode == "INNER" else (R, Z, K)
    dz = torch.randn(z_shape, generator=g).to(DEV)
    stream = int(torch.cuda.current_stream().cuda_stream)
    results = []
    for signature in (sig, -1):
        p = _lib.TpParams(num_rows=R, num_coef=table.num_coef, num_x=X, num_y=Y, num_out=Z, channels_x=K,
                          channels_y=1 if uniform else K,
                          mode={"MAP": _lib.MODE_MAP, "OUTER": _lib.MODE_OUTER, "INNER": _lib.MODE_INNER}[mode],
                          layout=_lib.LAYOUT_TRAILING, val_dtype=_lib.F32, coef_idx_bytes=table.idx_bytes,
                          coef_sorted=1, debug=1, signature=signature, coef_scale=scale)
        z = torch.full(z_shape, float("nan"), device=DEV)
        dx, dy = torch.full_like(x, float("nan")), torch.full_like(y, float("nan"))
        coef = None if signature >= 0 else table.device(x.device).data_ptr()
        coef_bwd = None if signature >= 0 else table.device(x.device, backward=True).data_ptr()
        _lib.check(lib.e3j_amd_tensor_product_fwd(ctypes.byref(p), coef, x.data_ptr(), y.data_ptr(), z.data_ptr(), stream))
        _lib.check(lib.e3j_amd_tensor_product_bwd(ctypes.byref(p), coef_bwd, x.data_ptr(), y.data_ptr(), dz.data_ptr(),
                                                  dx.data_ptr(), dy.data_ptr(), stream))
        results.append((z, dx, dy))
    for a, b, name in zip(results[0], results[1], ("z", "dx", "dy")):
        assert torch.isfinite(a).all(), name
        torch.testing.assert_close(a, b, rtol=2e-5, atol=2e-4 if mode == "INNER" else 2e-5,
                                   msg=lambda m, name=name: f"{name}: {m}")
    # repeatable to the bit (no atomics anywhere)
    z2 = torch.empty_like(results[0][0])
    p.signature = sig
    _lib.check(lib.e3j_amd_tensor_product_fwd(ctypes.byref(p), None, x.data_ptr(), y.data_ptr(), z2.data_ptr(), stream))
    torch.cuda.synchronize()
    assert torch.equal(z2, results[0][0])


@pytest.mark.parametrize("spaces", BUILTIN, ids=["l2_l2_full", "l2_l3_to_l3", "l3_l3_to_l3"])
@pytest.mark.parametrize("mode,channels", [("MAP", 4), ("MAP", 12), ("MAP", 64), ("MAP", 100), ("MAP", 128),
                                           ("OUTER", 64), ("OUTER", 128), ("OUTER", 256),
                                           ("INNER", 64), ("INNER", 128), ("INNER", 256)])
def test_unrolled_leading_kernels_against_the_checker(spaces, mode, channels):
    from e3j_amd.options import Layout
    from e3j_amd.tp_ops import _Table
    rng = np.random.default_rng(22)
    tp = TensorProduct(spaces[:2], spaces[2], layout="LEADING_CHANNELS", mode=mode)
    Z, X, Y = tp.shape
    idx, val = np.asarray(tp.indices, dtype=np.int64), 0.5 * np.asarray(tp.values, dtype=np.float64)
    table = _Table.get(Coef(val, idx, "float32", "uint8").pack(), np.float32)
    sig, scale = table.signature(X, Y, Z, channels, KIND[mode], Layout.LEADING_CHANNELS)
    assert sig >= 0 and abs(scale - 0.5) < 1e-6, "a built-in unrolled kernel must serve this table"
    rows = 77 if channels >= 64 else 53      # 53 * 4 = 212 and 53 * 12 = 636 columns: a moved-back last tile
    x, y = _operands(rng, mode, "LEADING_CHANNELS", channels, rows=rows, dims=(X, Y), has=(True, False))
    _check_forward(idx, val, x, y, Z, mode, "LEADING_CHANNELS", "uint8", what=f"leading {mode} K={channels}")
    _check_backward(idx, val, x, y, Z, mode, "LEADING_CHANNELS", rng, "uint8", what=f"leading {mode} K={channels}")


def test_leading_kernels_fall_back_below_one_tile():
    """Fewer than 64 columns in all: the table-driven kernels serve the call."""
    rng = np.random.default_rng(23)
    tp = TensorProduct(("0e+1o+2e", "0e+1o+2e"), None, layout="LEADING_CHANNELS", mode="MAP")
    Z, X, Y = tp.shape
    idx, val = np.asarray(tp.indices, dtype=np.int64), np.asarray(tp.values, dtype=np.float64)
    x, y = _operands(rng, "MAP", "LEADING_CHANNELS", 4, rows=9, dims=(X, Y))
    _check_forward(idx, val, x, y, Z, "MAP", "LEADING_CHANNELS", "uint8", what="small leading")
    _check_backward(idx, val, x, y, Z, "MAP", "LEADING_CHANNELS", rng, "uint8", what="small leading")


def test_batched_call_folds_the_batch_into_rows():
    rng = np.random.default_rng(24)
    idx, val = _table(nnz=120, dims=(9, 6, 5))
    coef = Coef(val, idx, "float32", "uint8").pack()
    p = TensorProductParams(num_out=9, mode="OUTER", layout="TRAILING_CHANNELS")
    x = torch.from_numpy(rng.normal(size=(3, 17, 6, 8)).astype(np.float32)).to(DEV)
    y = torch.from_numpy(rng.normal(size=(3, 17, 5)).astype(np.float32)).to(DEV)
    z = e3j_amd.tensor_product_batched(coef, x, y, p)
    assert tuple(z.shape) == (3, 17, 9, 8)
    for b in range(3):
        assert torch.equal(z[b], e3j_amd.tensor_product(coef, x[b], y[b], p))
    shared = e3j_amd.tensor_product_batched(coef, x, y[0], p, y_batched=False)   # y broadcast over the batch
    for b in range(3):
        assert torch.equal(shared[b], e3j_amd.tensor_product(coef, x[b], y[0], p))


def test_torch_func_transforms():
    """vmap over either operand, Jacobians and Hessian-vector products through `torch.func`, as the
    reference's transform tests do with jax (`tests/test_ops/test_tensor_product_jax_transforms.py`)."""
    from torch.func import grad, jacrev, vmap
    rng = np.random.default_rng(25)
    idx, val = _table(nnz=90, dims=(9, 6, 5))
    coef = Coef(val, idx, "float64", "int32").pack()
    p = TensorProductParams(num_out=9, mode="MAP", layout="TRAILING_CHANNELS")
    dense = _dense_torch(idx, val, 9, (6, 5), "MAP", "TRAILING_CHANNELS", (True, True))
    f = lambda a, b: e3j_amd.tensor_product(coef, a, b, p)  # noqa: E731
    x = torch.from_numpy(rng.normal(size=(3, 7, 6, 4))).to(DEV)
    y = torch.from_numpy(rng.normal(size=(3, 7, 5, 4))).to(DEV)
    torch.testing.assert_close(vmap(f)(x, y), torch.stack([dense(x[b], y[b]) for b in range(3)]))
    torch.testing.assert_close(vmap(f, in_dims=(0, None))(x, y[0]), torch.stack([dense(x[b], y[0]) for b in range(3)]))
    torch.testing.assert_close(vmap(f, in_dims=(None, 0))(x[0], y), torch.stack([dense(x[0], y[b]) for b in range(3)]))
    # Jacobian of a small product with respect to x (a vmap over the backward operator)
    xs, ys = x[0, :2], y[0, :2]
    torch.testing.assert_close(jacrev(f)(xs, ys), jacrev(dense)(xs, ys))
    # gradient of a scalar of the gradient (second order through the transforms)
    w = torch.from_numpy(rng.normal(size=(7, 9, 4))).to(DEV)
    energy = lambda fn: (lambda a, b: (fn(a, b) * w).sum())  # noqa: E731
    second = lambda fn: grad(lambda a, b: (grad(energy(fn))(a, b) ** 2).sum(), argnums=1)  # noqa: E731
    torch.testing.assert_close(second(f)(x[0], y[0]), second(dense)(x[0], y[0]))
    with pytest.raises(RuntimeError):   # forward-mode differentiation is not defined for the operator
        torch.func.jvp(f, (x[0], y[0]), (x[0], y[0]))


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("idx_dtype", ["uint8", "int32"])
def test_float16_operands(mode, layout, idx_dtype):
    """float16 values run the table-driven kernels in half precision, both layouts (the
    reference serves float16 in the trailing layout only, tests/test_ops/test_dtype.py:136-190):
    parity with the float64 checker on the rounded operands within half-precision rounding."""
    rng = np.random.default_rng(26)
    idx, val = _table(nnz=200)
    val16 = val.astype(np.float16)
    x, y = _operands(rng, mode, layout, 16, rows=40, dtype=np.float16, has=(True, False))
    coef = Coef(val16, idx, "float16", idx_dtype).pack()
    p = TensorProductParams(num_out=NUM_OUT, mode=mode, layout=layout)
    xt, yt = torch.from_numpy(x).to(DEV).requires_grad_(True), torch.from_numpy(y).to(DEV).requires_grad_(True)
    z = e3j_amd.tensor_product(coef, xt, yt, p)
    assert z.dtype == torch.float16
    dz = rng.normal(size=tuple(z.shape)).astype(np.float16)
    dx, dy = torch.autograd.grad(z, (xt, yt), torch.from_numpy(dz).to(DEV))
    f64 = lambda a: a.astype(np.float64)  # noqa: E731
    v = f64(val16)
    ref = T.tensor_product_unfused(idx, v, f64(x), f64(y), NUM_OUT, mode, layout)
    mag = T.tensor_product_unfused(idx, np.abs(v), np.abs(f64(x)), np.abs(f64(y)), NUM_OUT, mode, layout)
    rdx, rdy = T.tensor_product_vjp(idx, v, f64(x), f64(y), f64(dz), mode, layout)
    mdx, mdy = T.tensor_product_vjp(idx, np.abs(v), np.abs(f64(x)), np.abs(f64(y)), np.abs(f64(dz)), mode, layout)
    eps = 2.0 ** -10
    for got, r, m, name in ((z, ref, mag, "z"), (dx, rdx, mdx, "dx"), (dy, rdy, mdy, "dy")):
        err = np.abs(got.detach().float().cpu().numpy().astype(np.float64) - r)
        assert np.all(err <= 8 * eps * m + 1e-3), f"{name}: {err.max()} against magnitude {m.max()}"


# ---------------------------------------------------------------------------
# compile-time-unrolled kernels in float16 and float64 (trailing layout, whole waves of channels)
# ---------------------------------------------------------------------------
def _unrolled_case(spaces, mode, channels, np_dtype, factor, rows=77, seed=31):
    rng = np.random.default_rng(seed)
    tp = TensorProduct(spaces[:2], spaces[2], layout="TRAILING_CHANNELS", mode=mode)
    Z, X, Y = tp.shape
    idx = np.asarray(tp.indices, dtype=np.int64)
    val = (factor * np.asarray(tp.values, dtype=np.float64)).astype(np_dtype)
    x, y = _operands(rng, mode, "TRAILING_CHANNELS", channels, rows=rows, dims=(X, Y), has=(True, False))
    x, y = (0.5 * x).astype(np_dtype), (0.5 * y).astype(np_dtype)
    return tp, idx, val, x, y, rng


@pytest.mark.parametrize("spaces,channels", [(BUILTIN[t], k) for t in range(3) for k in (64, 128)],
                         ids=lambda v: str(v) if isinstance(v, int) else "-".join(str(a) for a in v))
@pytest.mark.parametrize("mode", ["MAP", "OUTER", "INNER"])
@pytest.mark.parametrize("dtype", ["float64", "float16"])
def test_unrolled_kernels_in_float64_and_float16(spaces, channels, mode, dtype):
    """The operator on a built-in table in float64 / float16: an unrolled kernel serves it (the
    look-up says so) and the results match the float64 checker on the table's own values: within
    64 float64 roundings of the sum of magnitudes, or within half-precision rounding (the
    float16 kernels compute in float with the built-in table times one factor, which differs from
    the half-rounded entries by their rounding)."""
    from e3j_amd.tp_ops import _Table
    np_dtype = np.dtype(dtype)
    tp, idx, val, x, y, rng = _unrolled_case(spaces, mode, channels, np_dtype, 1.5)
    Z, X, Y = tp.shape
    packed = Coef(val, idx, dtype, "uint8").pack()
    sig, _ = _Table.get(packed, np_dtype).signature(X, Y, Z, channels, KIND[mode])
    assert sig >= 0, "a built-in unrolled kernel must serve this table"
    p = TensorProductParams(num_out=Z, mode=mode, layout="TRAILING_CHANNELS")
    xt, yt = (torch.from_numpy(a).to(DEV).requires_grad_(True) for a in (x, y))
    z = e3j_amd.tensor_product(packed, xt, yt, p)
    assert z.dtype == getattr(torch, dtype)
    dz = (0.5 * rng.normal(size=tuple(z.shape))).astype(np_dtype)
    dx, dy = torch.autograd.grad(z, (xt, yt), torch.from_numpy(dz).to(DEV))
    f64 = lambda a: a.astype(np.float64)  # noqa: E731
    v = f64(val)
    lay = "TRAILING_CHANNELS"
    ref = T.tensor_product_unfused(idx, v, f64(x), f64(y), Z, mode, lay)
    mag = T.tensor_product_unfused(idx, np.abs(v), np.abs(f64(x)), np.abs(f64(y)), Z, mode, lay)
    rdx, rdy = T.tensor_product_vjp(idx, v, f64(x), f64(y), f64(dz), mode, lay)
    mdx, mdy = T.tensor_product_vjp(idx, np.abs(v), np.abs(f64(x)), np.abs(f64(y)), np.abs(f64(dz)), mode, lay)
    for got, r, m, name in ((z, ref, mag, "z"), (dx, rdx, mdx, "dx"), (dy, rdy, mdy, "dy")):
        err = np.abs(got.detach().double().cpu().numpy() - r)
        bound = 64 * 2.0 ** -52 * m + 1e-300 if dtype == "float64" else 8 * 2.0 ** -10 * m + 1e-3
        assert np.all(err <= bound), f"{name}: {err.max()} against magnitude {m.max()}"


@pytest.mark.parametrize("mode", ["MAP", "OUTER", "INNER"])
def test_float64_classes_serve_exact_and_rounded_tables(mode):
    """The float64 kernels take their coefficients from the caller's table: a table of exact
    double values (what a float64 front end builds) and the same table rounded to float32 both
    find the signature, and each result follows its own table to float64 accuracy."""
    from e3j_amd.tp_ops import _Table
    spaces, K = BUILTIN[2], 64
    tp, idx, _, x, y, rng = _unrolled_case(spaces, mode, K, np.dtype("float64"), 1.0, rows=33)
    Z, X, Y = tp.shape
    rounded = np.asarray(tp.values, dtype=np.float32).astype(np.float64)
    # exact values: what the float32 entries were rounded from, recovered through their squares
    # (squares of the entries of a Clebsch-Gordan table are small rationals)
    from fractions import Fraction
    exact = np.array([np.sign(v) * np.sqrt(float(Fraction(float(v) ** 2).limit_denominator(10000))) for v in rounded])
    assert 0 < np.abs(exact - rounded).max() < 1e-7
    p = TensorProductParams(num_out=Z, mode=mode, layout="TRAILING_CHANNELS")
    xt, yt = torch.from_numpy(x).to(DEV), torch.from_numpy(y).to(DEV)
    outs = []
    for val in (rounded, exact):
        packed = Coef(val, idx, "float64", "uint8").pack()
        sig, classes = _Table.get(packed, np.dtype("float64")).signature(X, Y, Z, K, KIND[mode])
        assert sig >= 0
        z = e3j_amd.tensor_product(packed, xt, yt, p).cpu().numpy()
        ref = T.tensor_product_unfused(idx, val, x, y, Z, mode, "TRAILING_CHANNELS")
        mag = T.tensor_product_unfused(idx, np.abs(val), np.abs(x), np.abs(y), Z, mode, "TRAILING_CHANNELS")
        assert np.all(np.abs(z - ref) <= 64 * 2.0 ** -52 * mag + 1e-300)
        outs.append(z)
    assert np.abs(outs[0] - outs[1]).max() > 1e-10   # (the two tables do differ)
    # a table of another structure is refused: one entry of a class changed
    broken = exact.copy()
    broken[5] *= 1.0 + 1e-9
    packed = Coef(broken, idx, "float64", "uint8").pack()
    assert _Table.get(packed, np.dtype("float64")).signature(X, Y, Z, K, KIND[mode])[0] == -1


@pytest.mark.parametrize("dtype", ["float64", "float16"])
def test_unrolled_float64_float16_through_the_c_abi(dtype):
    """The C ABI with a signature in float64 / float16 against the table-driven kernels of the
    same call (signature -1), MAP mode, 301 rows."""
    lib = _lib.load()
    np_dtype, tdtype = np.dtype(dtype), getattr(torch, dtype)
    tp = TensorProduct(("0e+1o+2e+3o", "0e+1o+2e+3o"), "0e+1o+2e+3o", layout="TRAILING_CHANNELS", mode="MAP")
    Z, X, Y = tp.shape
    K, R = 128, 301
    from e3j_amd.tp_ops import _Table
    table = _Table.get(tp.packed_coef(dtype), np_dtype)
    sig, scale = table.signature(X, Y, Z, K, 0)
    assert sig >= 0
    g = torch.Generator(device="cpu").manual_seed(5)
    x = (0.5 * torch.randn(R, X, K, generator=g)).to(tdtype).to(DEV)
    y = (0.5 * torch.randn(R, Y, K, generator=g)).to(tdtype).to(DEV)
    dz = (0.5 * torch.randn(R, Z, K, generator=g)).to(tdtype).to(DEV)
    stream = int(torch.cuda.current_stream().cuda_stream)
    results = []
    for signature in (sig, -1):
        p = _lib.TpParams(num_rows=R, num_coef=table.num_coef, num_x=X, num_y=Y, num_out=Z, channels_x=K,
                          channels_y=K, mode=_lib.MODE_MAP, layout=_lib.LAYOUT_TRAILING,
                          val_dtype=_lib.F64 if dtype == "float64" else _lib.F16, coef_idx_bytes=table.idx_bytes,
                          coef_sorted=1, debug=1, signature=signature,
                          coef_scale=scale if isinstance(scale, float) else 1.0)
        if signature >= 0 and dtype == "float64":
            p.coef_classes = ctypes.cast(scale, ctypes.c_void_p).value
        z = torch.full((R, Z, K), float("nan"), device=DEV, dtype=tdtype)
        dx, dy = torch.full_like(x, float("nan")), torch.full_like(y, float("nan"))
        coef = None if signature >= 0 else table.device(x.device).data_ptr()
        coef_bwd = None if signature >= 0 else table.device(x.device, backward=True).data_ptr()
        _lib.check(lib.e3j_amd_tensor_product_fwd(ctypes.byref(p), coef, x.data_ptr(), y.data_ptr(), z.data_ptr(), stream))
        _lib.check(lib.e3j_amd_tensor_product_bwd(ctypes.byref(p), coef_bwd, x.data_ptr(), y.data_ptr(), dz.data_ptr(),
                                                  dx.data_ptr(), dy.data_ptr(), stream))
        results.append((z, dx, dy))
    tol = dict(rtol=1e-12, atol=1e-12) if dtype == "float64" else dict(rtol=2e-2, atol=2e-2)
    for a, b, name in zip(results[0], results[1], ("z", "dx", "dy")):
        assert torch.isfinite(a).all(), name
        torch.testing.assert_close(a, b, msg=lambda m, name=name: f"{name}: {m}", **tol)
    # a float64 signature without its classes is refused
    if dtype == "float64":
        p = _lib.TpParams(num_rows=R, num_coef=table.num_coef, num_x=X, num_y=Y, num_out=Z, channels_x=K,
                          channels_y=K, mode=_lib.MODE_MAP, layout=_lib.LAYOUT_TRAILING, val_dtype=_lib.F64,
                          coef_idx_bytes=table.idx_bytes, coef_sorted=1, debug=0, signature=sig, coef_scale=1.0)
        rc = lib.e3j_amd_tensor_product_fwd(ctypes.byref(p), None, x.data_ptr(), y.data_ptr(), results[0][0].data_ptr(),
                                            stream)
        assert rc == _lib.INVALID_ARGUMENT and b"coef_classes" in lib.e3j_amd_last_error()
    torch.cuda.synchronize()
