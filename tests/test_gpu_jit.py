"""Kernels generated and compiled at run time for tables the library was not built for
(`config(jit=True)`), against the CPU oracle."""

import numpy as np
import pytest
import torch

import e3j_amd
from e3j_amd import ConvolutionParams, convolution, convolution_bwd
from e3j_amd.ops import _Table
from tests import helpers as H

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _random_case(seed, N, E, X, Y, Z, S, K, nnz):
    rng = np.random.default_rng(seed)
    idx, val, mix = H.random_table(rng, nnz, X, Y, Z, S)
    snd, rcv = H.random_graph(rng, N, E)
    x, y, s, dm = H.random_operands(rng, N, E, X, Y, S, K, Z)
    return dict(idx=idx, val=val, mix=mix, snd=snd, rcv=rcv, x=x, y=y, s=s, dm=dm,
                coef=H.pack_table(idx, val, mix), params=ConvolutionParams(num_out=Z, num_scalars=S))


@pytest.mark.parametrize("layout", ["TRAILING_CHANNELS", "LEADING_CHANNELS"])
@pytest.mark.parametrize("case", [
    dict(seed=1, N=40, E=600, X=5, Y=6, Z=7, S=4, K=64, nnz=60),     # whole waves
    dict(seed=2, N=30, E=400, X=3, Y=9, Z=10, S=5, K=48, nnz=80),    # idle lanes; leading: table-driven
    dict(seed=3, N=25, E=300, X=6, Y=4, Z=12, S=6, K=128, nnz=100),  # two channels per lane backward
    dict(seed=4, N=20, E=250, X=4, Y=25, Z=9, S=5, K=64, nnz=150),   # harmonics up to l = 4: 25 y components
    dict(seed=5, N=30, E=500, X=5, Y=6, Z=8, S=4, K=32, nnz=70),     # two edges of a row side by side
    dict(seed=6, N=30, E=500, X=5, Y=6, Z=8, S=4, K=16, nnz=70),     # four edges side by side
])
def test_random_tables_run_on_generated_kernels(case, layout):
    p = _random_case(**case)
    leading = layout == "LEADING_CHANNELS"
    t = (lambda a: np.ascontiguousarray(a.transpose(0, 2, 1))) if leading else (lambda a: a)
    back = (lambda g: g.transpose(1, 2)) if leading else (lambda g: g)
    x, y, s, dm = dev(t(p["x"])), dev(p["y"]), dev(t(p["s"])), dev(t(p["dm"]))
    snd, rcv = dev(p["snd"]), dev(p["rcv"])
    dims = (case["X"], case["Y"], case["Z"], case["S"])
    table = _Table.get(p["coef"], np.float32)
    with e3j_amd.config.use(jit=True):  # (a registered table stays registered for the process)
        sig = table.signature(dims, case["K"], e3j_amd.Layout.parse(layout))[0]
        # leading layout: whole waves, or a power-of-two channel count below 64
        assert (sig >= 0) == (not leading or case["K"] % 64 == 0 or case["K"] in (16, 32))
        out = convolution(p["coef"], x, y, s, snd, rcv, p["params"], layout=layout)
        grads = convolution_bwd(p["coef"], x, y, s, snd, rcv, dm, p["params"], layout=layout)
        with e3j_amd.config.use(jit=True, deterministic=True):
            ordered = convolution_bwd(p["coef"], x, y, s, snd, rcv, dm, p["params"], layout=layout)
    ref, mag = H.forward_reference(p["idx"], p["val"], p["mix"], p["x"], p["y"], p["s"], p["snd"], p["rcv"],
                                   case["Z"])
    H.assert_parity(back(out).cpu().numpy(), ref, mag, "out")
    refs, mags = H.backward_reference(p["idx"], p["val"], p["mix"], p["x"], p["y"], p["s"], p["snd"], p["rcv"],
                                      p["dm"])
    for g, o, r, m, name in zip(grads, ordered, refs, mags, ("dx", "dy", "ds")):
        for got in (g, o):
            got = back(got) if got.dim() == 3 else got
            H.assert_parity(got.cpu().numpy(), r, m, name)


def test_module_with_irreps_outside_the_built_in_tables():
    """x = 0e+1o+2e, y up to l = 2, out up to l = 2, 64 channels: generated on first use, then
    the same numbers as the table-driven kernels."""
    m = e3j_amd.Convolution(("0e+1o+2e", "0e+1o+2e"), "0e+1o+2e", graph_ordering="RECEIVER")
    rng = np.random.default_rng(5)
    N, E, K = 50, 900, 64
    snd, rcv = H.random_graph(rng, N, E)
    x = dev(rng.standard_normal((N, m.source[0].dim, K)).astype(np.float32)).requires_grad_(True)
    y = dev(rng.standard_normal((E, m.source[1].dim)).astype(np.float32)).requires_grad_(True)
    s = dev(rng.standard_normal((E, m.params.num_scalars, K)).astype(np.float32)).requires_grad_(True)
    dm = dev(rng.standard_normal((N, m.target.dim, K)).astype(np.float32))

    def run():
        out = m(x, y, s, dev(snd), dev(rcv))
        return (out,) + torch.autograd.grad(out, (x, y, s), dm)

    with e3j_amd.config.use(jit=False):
        slow = run()
    with e3j_amd.config.use(jit=True):
        packed = m._packed_coef("float32")
        dims = (m.source[0].dim, m.source[1].dim, m.target.dim, m.params.num_scalars)
        assert _Table.get(packed, np.float32).signature(dims, K, m.layout)[0] >= 0
        fast = run()
    for a, b in zip(slow, fast):
        assert float((a - b).detach().abs().max()) <= 2e-5 * float(a.detach().abs().max())


_TP_CASES = [(mode, layout, channels) for mode in ("MAP", "OUTER", "INNER")
             for layout, channels in (("TRAILING_CHANNELS", 16), ("TRAILING_CHANNELS", 32), ("TRAILING_CHANNELS", 64),
                                      ("TRAILING_CHANNELS", 128), ("LEADING_CHANNELS", 12), ("LEADING_CHANNELS", 128))
             # (channel sums in the leading layout need whole waves per row)
             if not (layout == "LEADING_CHANNELS" and channels == 12 and mode != "MAP")]


@pytest.mark.parametrize("mode,layout,channels", _TP_CASES)
def test_tensor_product_tables_run_on_generated_kernels(mode, layout, channels):
    from e3j_amd.coef import Coef
    from e3j_amd.tp_ops import TensorProductParams, _Table as TpTable
    from oracle import tp_oracle as T
    rng = np.random.default_rng(5)
    X, Y, Z, nnz, R = (5, 6, 11, 70, 91) if channels != 128 else (5, 20, 11, 120, 91)   # 20 y components at 128
    idx, val, _ = H.random_table(rng, nnz, X, Y, Z, 3)
    coef = Coef(val, idx, "float32", "uint8").pack()
    tr = layout == "TRAILING_CHANNELS"
    x = rng.normal(size=(R, X, channels) if tr else (R, channels, X)).astype(np.float32)
    y = (rng.normal(size=(R, Y)) if mode == "OUTER" else
         rng.normal(size=(R, Y, channels) if tr else (R, channels, Y))).astype(np.float32)
    kind = {"MAP": 0, "OUTER": 1, "INNER": 2}[mode]
    p = TensorProductParams(num_out=Z, mode=mode, layout=layout)
    with e3j_amd.config.use(jit=True):
        sig = TpTable.get(coef, np.float32).signature(X, Y, Z, channels, kind, e3j_amd.Layout.parse(layout))[0]
        assert sig >= 0, "the table must run on kernels compiled for it"
        xt, yt = dev(x).requires_grad_(True), dev(y).requires_grad_(True)
        z = e3j_amd.tensor_product(coef, xt, yt, p)
        dz = rng.normal(size=tuple(z.shape)).astype(np.float32)
        dx, dy = torch.autograd.grad(z, (xt, yt), dev(dz))
    f64 = lambda a: a.astype(np.float64)  # noqa: E731
    val_r = val.astype(np.float32).astype(np.float64)
    ref = T.tensor_product_unfused(idx, val_r, f64(x), f64(y), Z, mode, layout)
    mag = T.tensor_product_unfused(idx, np.abs(val_r), np.abs(f64(x)), np.abs(f64(y)), Z, mode, layout)
    H.assert_parity(z.detach().cpu().numpy(), ref, mag, "z")
    rdx, rdy = T.tensor_product_vjp(idx, val_r, f64(x), f64(y), f64(dz), mode, layout)
    mdx, mdy = T.tensor_product_vjp(idx, np.abs(val_r), np.abs(f64(x)), np.abs(f64(y)), np.abs(f64(dz)), mode, layout)
    H.assert_parity(dx.cpu().numpy(), rdx, mdx, "dx", ulps=32.0)
    H.assert_parity(dy.cpu().numpy(), rdy, mdy, "dy", ulps=32.0)


@pytest.mark.parametrize("dtype", ["float16", "float64"])
def test_tensor_product_generated_kernels_in_float16_and_float64(dtype):
    """A table that is not built in, compiled at run time, serves float16 and float64 operands too
    (trailing layout, 64 channels).  The float64 kernels exist when the table has at most 64
    distinct magnitudes: a real Clebsch-Gordan table (here 0e+1o (x) 0e+1o+2e, scaled) has few."""
    from e3j_amd import TensorProduct
    from e3j_amd.coef import Coef
    from e3j_amd.tp_ops import TensorProductParams, _Table as TpTable
    from oracle import tp_oracle as T
    rng = np.random.default_rng(8)
    np_dtype = np.dtype(dtype)
    tp = TensorProduct(("0e+1o", "0e+1o+2e"), None, layout="TRAILING_CHANNELS", mode="MAP")
    Z, X, Y = tp.shape
    idx = np.asarray(tp.indices, dtype=np.int64)
    val = (0.75 * np.asarray(tp.values, dtype=np.float64)).astype(np_dtype)
    coef = Coef(val, idx, dtype, "uint8").pack()
    K, R = 64, 53
    x = (0.5 * rng.normal(size=(R, X, K))).astype(np_dtype)
    y = (0.5 * rng.normal(size=(R, Y, K))).astype(np_dtype)
    p = TensorProductParams(num_out=Z, mode="MAP", layout="TRAILING_CHANNELS")
    with e3j_amd.config.use(jit=True):
        sig = TpTable.get(coef, np_dtype).signature(X, Y, Z, K, 0)[0]
        assert sig >= 0, "the table must run on kernels compiled for it"
        xt, yt = dev(x).requires_grad_(True), dev(y).requires_grad_(True)
        z = e3j_amd.tensor_product(coef, xt, yt, p)
        dz = (0.5 * rng.normal(size=tuple(z.shape))).astype(np_dtype)
        dx, dy = torch.autograd.grad(z, (xt, yt), dev(dz))
    f64 = lambda a: a.astype(np.float64)  # noqa: E731
    v = f64(val)
    lay = "TRAILING_CHANNELS"
    ref = T.tensor_product_unfused(idx, v, f64(x), f64(y), Z, "MAP", lay)
    mag = T.tensor_product_unfused(idx, np.abs(v), np.abs(f64(x)), np.abs(f64(y)), Z, "MAP", lay)
    rdx, rdy = T.tensor_product_vjp(idx, v, f64(x), f64(y), f64(dz), "MAP", lay)
    mdx, mdy = T.tensor_product_vjp(idx, np.abs(v), np.abs(f64(x)), np.abs(f64(y)), np.abs(f64(dz)), "MAP", lay)
    for got, r, m, name in ((z, ref, mag, "z"), (dx, rdx, mdx, "dx"), (dy, rdy, mdy, "dy")):
        err = np.abs(got.detach().double().cpu().numpy() - r)
        bound = 64 * 2.0 ** -52 * m + 1e-300 if dtype == "float64" else 8 * 2.0 ** -10 * m + 1e-3
        assert np.all(err <= bound), f"{name}: {err.max()} against magnitude {m.max()}"
