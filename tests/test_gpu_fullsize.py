"""Full-size benchmark workloads: comparison with the C checker where it finishes in
seconds, and size-independent properties at the 1M-edge configuration."""

import numpy as np
import pytest
import torch

import e3j_amd
from e3j_amd import workloads as W
from oracle import c_oracle
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _run(w, ordering=None):
    m = w.module
    coef = m._packed_coef("float32")
    ordering = ordering or m.graph_ordering
    out = e3j_amd.convolution(coef, w.x, w.y, w.s, w.sender, w.receiver, m.params, ordering,
                              layout=m.layout)
    grads = e3j_amd.convolution_bwd(coef, w.x, w.y, w.s, w.sender, w.receiver, w.dm, m.params, ordering,
                                    layout=m.layout)
    return out, grads


def _trailing(t, w):
    return (t.transpose(1, 2) if w.leading and t.dim() == 3 else t).cpu().numpy()


def _against_c_oracle(w, out, grads, tag):
    """Against the C checker's loops run in float64 (the exact value of every element) under the
    parity criterion of the small tests: 1e-5 relative / 1e-6 absolute, and for an element outside
    that band 16 float32 roundings of the sum of the absolute values of its terms (the same loops
    on the absolute values of the operands).  Prints the share of elements that needed the allowance."""
    idx, val, mix = w.table()
    a = w.numpy()
    Z = w.module.params.num_out
    args = (a["x"], a["y"], a["s"], a["sender"], a["receiver"])
    mag_args = tuple(np.abs(t) for t in args[:3]) + args[3:]
    f64 = np.float64
    ref = c_oracle.convolution(idx, val, mix, *args, Z, dtype=f64)
    mag = c_oracle.convolution(idx, np.abs(val), mix, *mag_args, Z, dtype=f64)
    shares = {"out": H.assert_parity(_trailing(out, w), ref, mag, f"{tag} out")}
    del ref, mag
    refs = c_oracle.convolution_vjp(idx, val, mix, *args, a["dm"], dtype=f64)
    mags = c_oracle.convolution_vjp(idx, np.abs(val), mix, *mag_args, np.abs(a["dm"]), dtype=f64)
    for g, r, m, name in zip(grads, refs, mags, ("dx", "dy", "ds")):
        shares[name] = H.assert_parity(_trailing(g, w), r, m, f"{tag} {name}")
    print(f"{tag}: share of elements outside 1e-5 relative / 1e-6 absolute (inside 16 roundings of their "
          "terms): " + ", ".join(f"{k} {v:.2e}" for k, v in shares.items()))


def test_config1_and_config2_full_size_match_checker():
    for w in (W.config1(device="cuda"), W.config2(device="cuda")):
        out, grads = _run(w)
        _against_c_oracle(w, out, grads, w.name)


def test_config2_full_size_in_float64_and_float16():
    """Configuration 2 at full size with float64 and float16 operands on the unrolled kernels of those
    dtypes, against the C checker's loops in float64: float64 within 64 float64 roundings of the
    terms' magnitudes, float16 (operands and table rounded to half, results summed in half by the
    atomics) within half-precision rounding of them."""
    w = W.config2(device="cuda")
    m = w.module
    idx, val, mix = w.table()
    Z = m.params.num_out
    for dtype, name, scale in ((torch.float64, "float64", 1.0), (torch.float16, "float16", 0.25)):
        coef = m._packed_coef(name)
        x, y, s, dm = ((t * scale).to(dtype) for t in (w.x, w.y, w.s, w.dm))
        out = e3j_amd.convolution(coef, x, y, s, w.sender, w.receiver, m.params, m.graph_ordering, layout=m.layout)
        grads = e3j_amd.convolution_bwd(coef, x, y, s, w.sender, w.receiver, dm, m.params, m.graph_ordering,
                                        layout=m.layout)
        torch.cuda.synchronize()
        assert out.dtype == dtype
        host = [t.double().cpu().numpy() for t in (x, y, s, dm)]
        snd, rcv = w.sender.cpu().numpy(), w.receiver.cpu().numpy()
        v = np.asarray(val).astype(np.float16 if dtype == torch.float16 else np.float64).astype(np.float64)
        args = (host[0], host[1], host[2], snd, rcv)
        mag_args = tuple(np.abs(t) for t in args[:3]) + args[3:]
        ref = c_oracle.convolution(idx, v, mix, *args, Z, dtype=np.float64)
        mag = c_oracle.convolution(idx, np.abs(v), mix, *mag_args, Z, dtype=np.float64)
        refs = c_oracle.convolution_vjp(idx, v, mix, *args, host[3], dtype=np.float64)
        mags = c_oracle.convolution_vjp(idx, np.abs(v), mix, *mag_args, np.abs(host[3]), dtype=np.float64)
        if dtype == torch.float64:
            bound = lambda m_, sums: 64 * 2.0 ** -52 * m_ + 1e-300   # noqa: E731
        else:   # (dx and the shared dy rows take one half rounding per addend)
            bound = lambda m_, sums: 6 * sums * 2.0 ** -10 * m_ + 1e-3   # noqa: E731
        for got, r, m_, what, sums in zip((out,) + tuple(grads), (ref,) + tuple(refs), (mag,) + tuple(mags),
                                          ("out", "dx", "dy", "ds"), (1.0, 4.0, 2.0, 1.0)):
            err = np.abs(got.double().cpu().numpy() - r)
            assert np.isfinite(err).all() and (err <= bound(m_, sums)).all(), (
                f"cfg2 {name} {what}: worst error {err.max():.3e}, {int((err > bound(m_, sums)).sum())} elements off")


def test_config2_leading_layout_full_size_matches_checker():
    """The configuration as the baseline names it: channels before the irreps axis."""
    w = W.config2(device="cuda").with_layout("LEADING_CHANNELS")
    out, grads = _run(w)
    _against_c_oracle(w, out, grads, "cfg2 leading")


def test_config4_unsorted_skewed_matches_checker():
    """Random edge order and hubs with ~120 incoming edges, through the device sort."""
    w = W.config4(device="cuda")
    assert w.module.graph_ordering.value == "NONE"
    assert not bool((w.receiver[1:] >= w.receiver[:-1]).all())
    out, grads = _run(w)
    _against_c_oracle(w, out, grads, "cfg4")


def test_config3_full_size_properties(config3_on_gpu):
    """32 000 atoms, ~0.96 M edges, 128 channels: properties that need no CPU reference."""
    w = config3_on_gpu
    assert 0.9e6 < w.num_edges < 1.05e6
    out, (dx, dy, ds) = _run(w)
    # Euler's identity of a trilinear form: <x,dx> = <y,dy> = <s,ds> = <out,dm>
    total = float((out.double() * w.dm.double()).sum())
    for a, g, name in ((w.x, dx, "x"), (w.y, dy, "y"), (w.s, ds, "s")):
        assert abs(float((a.double() * g.double()).sum()) - total) <= 2e-5 * abs(total), name
    # linearity in x and in s
    out2, _ = _run(W.Workload(**{**w.__dict__, "x": 2.0 * w.x}))
    torch.testing.assert_close(out2, 2.0 * out, rtol=1e-6, atol=1e-5)
    # the forward is bit-reproducible
    again, _ = _run(w)
    assert torch.equal(out, again)
    # the leading-channels layout gives the same numbers (forward: the same sums in the same order)
    wl = w.with_layout("LEADING_CHANNELS")
    out_l, (dx_l, dy_l, ds_l) = _run(wl)
    assert torch.equal(out_l.transpose(1, 2), out)
    torch.testing.assert_close(ds_l.transpose(1, 2), ds, rtol=1e-5, atol=1e-6)
    assert float((dx_l.transpose(1, 2) - dx).abs().max()) <= 2e-5 * float(dx.abs().max())
    assert float((dy_l - dy).abs().max()) <= 2e-5 * float(dy.abs().max())
    del wl, out_l, dx_l, dy_l, ds_l
    # a head of the workload agrees with the C checker
    head = w.head(64)
    idx, val, mix = w.table()
    a = head.numpy()
    ref = c_oracle.convolution(idx, val, mix, a["x"], a["y"], a["s"], a["sender"], a["receiver"],
                               w.module.params.num_out)
    got = out[:64].cpu().numpy()
    assert np.abs(got - ref[:64]).max() <= 2e-5 * np.abs(ref[:64]).max()


def _sub_problem(w, edge_ids):
    """The edges `edge_ids` of a workload as a problem of their own: the nodes they touch renumbered
    0.., host arrays in the trailing layout.  Returns (node ids, operands dict)."""
    snd, rcv = w.sender[edge_ids].long(), w.receiver[edge_ids].long()
    nodes, inv = torch.unique(torch.cat([snd, rcv]), return_inverse=True)
    t3 = (lambda t: t.transpose(1, 2)) if w.leading else (lambda t: t)
    ops = dict(x=t3(w.x[nodes]), y=w.y[edge_ids], s=t3(w.s[edge_ids]), dm=t3(w.dm[nodes]),
               sender=inv[:snd.numel()].int(), receiver=inv[snd.numel():].int())
    return nodes.cpu().numpy(), {k: v.contiguous().cpu().numpy() for k, v in ops.items()}


@pytest.fixture(scope="module")
def config3_on_gpu():
    return W.config3(device="cuda")


@pytest.mark.parametrize("layout,tile_rows", [("TRAILING_CHANNELS", -1), ("TRAILING_CHANNELS", 0),
                                              ("LEADING_CHANNELS", -1)])
def test_config3_full_size_elementwise_on_induced_subgraphs(config3_on_gpu, layout, tile_rows):
    """Elementwise at full size (32 000 atoms, 0.96 M edges, 128 channels): for the first 64, the
    last 64 and 64 scattered nodes R, the output rows of R and the dy / ds rows of every edge into R
    against the float64 checker on the sub-graph of those edges, and the dx rows of R against the
    checker on the sub-graph of every edge out of R (a dx row sums over all edges of its sender).
    Both layouts; the tiled backward and the one-wave-per-receiver backward."""
    from e3j_amd.options import config
    w = config3_on_gpu.with_layout(layout)
    n = w.num_nodes
    rng = np.random.default_rng(77)
    picked = np.unique(np.concatenate([np.arange(64), np.arange(n - 64, n), rng.choice(n, 64, replace=False)]))
    with config.use(tile_rows=tile_rows):
        out, (dx, dy, ds) = _run(w)
    torch.cuda.synchronize()
    idx, val, mix = w.table()
    Z = w.module.params.num_out
    t3 = (lambda t: t.transpose(1, 2)) if w.leading else (lambda t: t)
    f64 = np.float64
    member = torch.zeros(n, dtype=torch.bool, device="cuda")
    member[torch.as_tensor(picked, device="cuda")] = True
    tag = f"cfg3 {layout.split('_')[0].lower()} tile_rows={tile_rows}"
    shares = {}

    # edges into R: out rows of R, dy and ds of those edges
    into = torch.nonzero(member[w.receiver.long()]).flatten()
    assert 64 * 20 < into.numel() < 192 * 60
    nodes, a = _sub_problem(w, into)
    args = (a["x"], a["y"], a["s"], a["sender"], a["receiver"])
    mags = tuple(np.abs(t) for t in args[:3]) + args[3:]
    local = np.searchsorted(nodes, picked)
    ref = c_oracle.convolution(idx, val, mix, *args, Z, dtype=f64)[local]
    mag = c_oracle.convolution(idx, np.abs(val), mix, *mags, Z, dtype=f64)[local]
    got = t3(out[torch.as_tensor(picked, device="cuda")]).cpu().numpy()
    shares["out"] = H.assert_parity(got, ref, mag, f"{tag} out rows")
    _, rdy, rds = c_oracle.convolution_vjp(idx, val, mix, *args, a["dm"], dtype=f64)
    _, mdy, mds = c_oracle.convolution_vjp(idx, np.abs(val), mix, *mags, np.abs(a["dm"]), dtype=f64)
    shares["dy"] = H.assert_parity(dy[into].cpu().numpy(), rdy, mdy, f"{tag} dy of the edges into R")
    shares["ds"] = H.assert_parity(t3(ds[into]).cpu().numpy(), rds, mds, f"{tag} ds of the edges into R")

    # edges out of R: the whole dx rows of R
    out_of = torch.nonzero(member[w.sender.long()]).flatten()
    nodes, a = _sub_problem(w, out_of)
    args = (a["x"], a["y"], a["s"], a["sender"], a["receiver"])
    mags = tuple(np.abs(t) for t in args[:3]) + args[3:]
    local = np.searchsorted(nodes, picked)
    rdx = c_oracle.convolution_vjp(idx, val, mix, *args, a["dm"], dtype=f64)[0][local]
    mdx = c_oracle.convolution_vjp(idx, np.abs(val), mix, *mags, np.abs(a["dm"]), dtype=f64)[0][local]
    got = t3(dx[torch.as_tensor(picked, device="cuda")]).cpu().numpy()
    shares["dx"] = H.assert_parity(got, rdx, mdx, f"{tag} dx rows of R")
    print(f"{tag}: share of checked elements outside 1e-5 relative / 1e-6 absolute (inside 16 roundings of "
          "their terms): " + ", ".join(f"{k} {v:.2e}" for k, v in shares.items()))


def _dot(a, b, chunk=1 << 16):
    """<a, b> in float64 without a float64 copy of the operands."""
    return sum(float((a[i:i + chunk].double() * b[i:i + chunk].double()).sum()) for i in range(0, a.shape[0], chunk))


def test_radial_weights_beyond_two_to_32_elements():
    """51 200 atoms, ~1.5 M edges, 128 channels: `s` and `ds` hold more than 2^32 elements each
    (18 GB), so the rows of the last receivers sit behind offsets no 32-bit index reaches.  Their
    edges, passed again as a problem of their own (small offsets), must give the same bits."""
    import dataclasses
    w = W.config3(1.6, device="cuda")
    assert w.s.numel() > 2 ** 32
    out, (dx, dy, ds) = _run(w)
    total = _dot(out, w.dm)
    for a, g, name in ((w.x, dx, "x"), (w.y, dy, "y"), (w.s, ds, "s")):
        assert abs(_dot(a, g) - total) <= 2e-5 * abs(total), name
    first = w.num_nodes - 200
    e0 = int((w.receiver < first).sum())
    assert e0 * w.s.shape[1] * w.s.shape[2] > 2 ** 32
    tail = dataclasses.replace(w, s=w.s[e0:], y=w.y[e0:], sender=w.sender[e0:], receiver=w.receiver[e0:])
    out_t, (_, dy_t, ds_t) = _run(tail)
    assert torch.equal(out_t[first:], out[first:]) and not bool(out_t[:first].any())
    assert torch.equal(ds_t, ds[e0:])
    torch.testing.assert_close(dy_t, dy[e0:], rtol=1e-5, atol=1e-6)   # (summed over waves by float atomics)


@pytest.mark.parametrize("mode,layout", [("MAP", "TRAILING_CHANNELS"), ("OUTER", "TRAILING_CHANNELS"),
                                         ("INNER", "TRAILING_CHANNELS"), ("MAP", "LEADING_CHANNELS")])
def test_tensor_product_benchmark_size_properties(mode, layout):
    """The row-wise tensor product at the size `bench.py --op tensor_product` runs (262 144 rows,
    128 channels, l <= 3 table), through properties that do not depend on the size: the Euler
    identity of a bilinear form <dz, z> = <dx, x> = <dy, y>, linearity in x, bit-identical
    repetition, and a head of rows against the CPU checker."""
    from e3j_amd import TensorProduct
    from e3j_amd.tp_ops import TensorProductParams
    from oracle import tp_oracle as T
    R, K = 1 << 18, 128
    tr = layout == "TRAILING_CHANNELS"
    tp = TensorProduct(("0e+1o+2e+3o", "0e+1o+2e+3o"), "0e+1o+2e+3o", layout=layout, mode=mode)
    Z, X, Y = tp.shape
    coef = tp.packed_coef("float32")
    p = TensorProductParams(num_out=Z, mode=mode, layout=layout)
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn((R, X, K) if tr else (R, K, X), device="cuda", generator=g)
    y = torch.randn(((R, Y, K) if tr else (R, K, Y)) if mode != "OUTER" else (R, Y), device="cuda", generator=g)
    z = e3j_amd.tensor_product(coef, x, y, p)
    assert torch.equal(z, e3j_amd.tensor_product(coef, x, y, p))
    dz = torch.randn(tuple(z.shape), device="cuda", generator=g)
    dx, dy = e3j_amd.tensor_product_bwd(coef, x, y, dz, p)
    dot = lambda a, b: float((a.double() * b.double()).sum())  # noqa: E731
    ref = dot(dz, z)
    scale = float((dz.double().abs() * z.double().abs()).sum())
    assert abs(dot(dx, x) - ref) <= 1e-6 * scale and abs(dot(dy, y) - ref) <= 1e-6 * scale
    x2 = torch.randn(tuple(x.shape), device="cuda", generator=g)
    lin = e3j_amd.tensor_product(coef, x + 2.0 * x2, y, p) - (z + 2.0 * e3j_amd.tensor_product(coef, x2, y, p))
    assert float(lin.abs().max()) <= 2e-5 * float(z.abs().max())
    head = 64
    idx, val = np.asarray(tp.indices, dtype=np.int64), np.asarray(tp.values, dtype=np.float64)
    xs, ys = x[:head].cpu().numpy().astype(np.float64), y[:head].cpu().numpy().astype(np.float64)
    want = T.tensor_product_unfused(idx, val, xs, ys, Z, mode, layout)
    mag = T.tensor_product_unfused(idx, np.abs(val), np.abs(xs), np.abs(ys), Z, mode, layout)
    H.assert_parity(z[:head].cpu().numpy(), want, mag, f"head {mode} {layout}")


@pytest.mark.parametrize("layout", ["TRAILING_CHANNELS", "LEADING_CHANNELS"])
def test_sender_ordering_on_the_symmetric_config2_graph_matches_checker(layout):
    """SENDER ordering (`src/e3j/ops/convolution.py:166-176,413-425`) at the size of config 2: the
    radius graph is symmetric, y of a reversed edge is the parity image of y, and the radial
    weights are made symmetric; edges sorted by sender.  Forward and all three cotangents
    against the CPU checker, which knows nothing of orderings."""
    w = W.config2()
    n = w.num_nodes
    snd, rcv = w.sender.numpy().astype(np.int64), w.receiver.numpy().astype(np.int64)
    key, rev_key = snd * n + rcv, rcv * n + snd
    by_key = np.argsort(key)
    rev = by_key[np.searchsorted(key[by_key], rev_key)]
    assert np.array_equal(key[rev], rev_key), "every edge has its reverse"
    m = e3j_amd.Convolution((w.module.source[0], w.module.source[1]), "0e+1o+2e", graph_ordering="SENDER")
    parity = torch.as_tensor(np.asarray(m.y_parity, dtype=np.float32))
    torch.testing.assert_close(w.y[rev], w.y * parity[None, :], rtol=1e-5, atol=1e-5)
    s = 0.5 * (w.s + w.s[rev])                                    # s_ba = s_ab
    y = 0.5 * (w.y + w.y[rev] * parity[None, :])                  # y_ba = p y_ab to the last bit
    order = torch.as_tensor(np.argsort(snd, kind="stable"))
    base = W.Workload("cfg2 by sender", m, w.x, y[order], s[order], w.dm, w.sender[order], w.receiver[order],
                      w.positions, w.box)
    ws = base.with_layout(layout).to("cuda")
    m = ws.module
    assert m.graph_ordering.value == "SENDER" and m.layout.name == layout
    xs, ys, ss = (t.clone().requires_grad_(True) for t in (ws.x, ws.y, ws.s))
    out = m(xs, ys, ss, ws.sender, ws.receiver)
    grads = torch.autograd.grad(out, (xs, ys, ss), ws.dm)
    torch.cuda.synchronize()
    _against_c_oracle(ws, out.detach(), grads, f"cfg2 SENDER {layout}")
