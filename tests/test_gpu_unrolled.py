"""Parity of the compile-time-unrolled kernels against the CPU oracle on the benchmark signatures."""

import numpy as np
import pytest
import torch

import e3j_amd
from e3j_amd import _lib, workloads as W
from e3j_amd.ops import _Table
from tests import helpers as H

pytestmark = pytest.mark.gpu

CASES = {
    "cfg3_k32": lambda: W.config3(0.006, channels=32),
    "cfg3_k256": lambda: W.config3(0.003, channels=256),
    "cfg2_k32": lambda: W.config2(0.04, channels=32),
    "cfg2_k128": lambda: W.config2(0.03, channels=128),
    "cfg1": lambda: W.config1(0.2),
    "cfg2": lambda: W.config2(0.04),
    "cfg2_out3": lambda: W.config2(0.04, out_irreps="0e+1o+2e+3o"),
    "cfg3_k64": lambda: W.config3(0.006, channels=64),
    "cfg3": lambda: W.config3(0.006),
    # scalar node features (one x coordinate, four paths)
    "scalars_k64": lambda: W.make_workload("scalars", 200, "0e", 3, "0e+1o+2e+3o", 64, (51, 52, 53, 54)),
    "scalars_k256": lambda: W.make_workload("scalars", 120, "0e", 3, "0e+1o+2e+3o", 256, (55, 56, 57, 58)),
}


def _signature_of(w):
    packed = w.module._packed_coef("float32")
    d = 2 if w.leading else 1
    dims = (int(w.x.shape[d]), int(w.y.shape[1]), w.module.params.num_out, int(w.s.shape[d]))
    return _Table.get(packed, np.float32).signature(dims, w.channels, w.module.layout)


def _trailing(t, w):
    """Node/edge arrays of a workload as (rows, dim, channels) numpy arrays."""
    return (t.transpose(1, 2) if w.leading else t).cpu().numpy()


@pytest.mark.parametrize("layout", ["TRAILING_CHANNELS", "LEADING_CHANNELS"])
@pytest.mark.parametrize("name", list(CASES))
def test_unrolled_matches_oracle(name, layout):
    w = CASES[name]().with_layout(layout)
    sig, scale, flip = _signature_of(w)
    assert flip == 0
    assert sig >= 0, "benchmark signature must resolve to a built-in unrolled kernel"
    assert scale == 1.0
    d = w.to("cuda")
    m = w.module
    coef = m._packed_coef("float32")
    out = e3j_amd.convolution(coef, d.x, d.y, d.s, d.sender, d.receiver, m.params, m.graph_ordering,
                              layout=m.layout)
    dx, dy, ds = e3j_amd.convolution_bwd(coef, d.x, d.y, d.s, d.sender, d.receiver, d.dm, m.params,
                                         m.graph_ordering, layout=m.layout)
    torch.cuda.synchronize()
    idx, val, mix = w.table()
    a = w.numpy()
    ref, mag = H.forward_reference(idx, val, mix, a["x"], a["y"], a["s"], a["sender"], a["receiver"],
                                   m.params.num_out)
    H.assert_parity(_trailing(out, w), ref, mag, f"{name} out")
    (rx, ry, rs), (mx, my, ms) = H.backward_reference(idx, val, mix, a["x"], a["y"], a["s"],
                                                      a["sender"], a["receiver"], a["dm"])
    H.assert_parity(_trailing(dx, w), rx, mx, f"{name} dx")
    H.assert_parity(dy.cpu().numpy(), ry, my, f"{name} dy")
    H.assert_parity(_trailing(ds, w), rs, ms, f"{name} ds")


def test_scaled_table_uses_unrolled_kernel():
    """1/avg_num_neighbors folded into the coefficients still matches a built-in signature."""
    w = W.config2(0.04)
    m = e3j_amd.Convolution(("0e+1o+2e", "0e+1o+2e+3o"), "0e+1o+2e", graph_ordering="RECEIVER",
                            avg_num_neighbors=30.0)
    packed = m._packed_coef("float32")
    dims = (int(w.x.shape[1]), int(w.y.shape[1]), m.params.num_out, int(w.s.shape[1]))
    sig, scale, _ = _Table.get(packed, np.float32).signature(dims, w.channels, m.layout)
    assert sig >= 0 and abs(scale - 1.0 / 30.0) < 1e-8
    d = w.to("cuda")
    out = m(d.x, d.y, d.s, d.sender, d.receiver)
    base = w.module(d.x, d.y, d.s, d.sender, d.receiver)
    torch.testing.assert_close(out, base / 30.0, rtol=2e-6, atol=1e-6)


@pytest.mark.parametrize("layout", ["TRAILING_CHANNELS", "LEADING_CHANNELS"])
@pytest.mark.parametrize("name", ["cfg3", "cfg2"])
def test_every_launch_variant_gives_the_same_results(name, layout):
    """The launch shapes of a signature (channels per lane, parts, waves per block) differ in how
    the work is dealt to waves, not in what is computed: forward bit-identical, backward equal
    up to the order of the dx / dy atomic sums."""
    w = CASES[name]().with_layout(layout)
    d = w.to("cuda")
    m = w.module
    coef = m._packed_coef("float32")
    lib = _lib.load()

    def run():
        out = e3j_amd.convolution(coef, d.x, d.y, d.s, d.sender, d.receiver, m.params, m.graph_ordering,
                                  layout=m.layout)
        grads = e3j_amd.convolution_bwd(coef, d.x, d.y, d.s, d.sender, d.receiver, d.dm, m.params,
                                        m.graph_ordering, layout=m.layout)
        torch.cuda.synchronize()
        return out, grads

    try:
        lib.e3j_amd_set_launch_variant(0, 0)
        out0, grads0 = run()
        for variant in range(1, 8):  # numbers past the last variant fall back to the default
            lib.e3j_amd_set_launch_variant(variant, variant)
            out, grads = run()
            assert torch.equal(out, out0), f"forward variant {variant}"
            for g, g0, what in zip(grads, grads0, ("dx", "dy", "ds")):
                scale = float(g0.abs().max())
                assert float((g - g0).abs().max()) <= 2e-5 * scale, f"backward variant {variant} {what}"
    finally:
        lib.e3j_amd_set_launch_variant(0, 0)


def test_y_flip_mask_equals_negated_components():
    """`y_flip` through the C ABI: reading -y[:, k] for the masked components and returning
    -dy[:, k] is the same as handing the kernels the negated columns."""
    import ctypes
    from e3j_amd.graph import csr_row_ptr
    w = CASES["cfg2"]()
    d = w.to("cuda")
    m = w.module
    table = _Table.get(m._packed_coef("float32"), np.float32)
    sig, scale, _ = _signature_of(w)
    mask = 0b1111111000001110                               # the odd-parity components up to l = 3
    signs = torch.tensor([-1.0 if (mask >> k) & 1 else 1.0 for k in range(16)], device="cuda")
    ptr = csr_row_ptr(d.receiver, w.num_nodes)
    lib = _lib.load()
    stream = int(torch.cuda.current_stream().cuda_stream)

    def run(y, flip):
        p = _lib.ConvParams(num_nodes=w.num_nodes, num_edges=w.num_edges, num_coef=table.num_coef,
                            num_x=int(d.x.shape[1]), num_y=16, num_out=m.params.num_out,
                            num_scalars=int(d.s.shape[1]), channels=w.channels, layout=m.layout.value,
                            val_dtype=_lib.F32, coef_idx_bytes=table.idx_bytes, signature=sig,
                            coef_scale=scale, debug=0, y_flip=flip, row_order=None)
        out = torch.empty_like(d.dm)
        dx, dy, ds = torch.empty_like(d.x), torch.empty_like(y), torch.empty_like(d.s)
        coef = table.device(d.x.device)
        _lib.check(lib.e3j_amd_convolution_fwd(ctypes.byref(p), coef.data_ptr(), d.x.data_ptr(), y.data_ptr(),
                                               d.s.data_ptr(), d.sender.data_ptr(), ptr.data_ptr(), None,
                                               out.data_ptr(), stream))
        _lib.check(lib.e3j_amd_convolution_bwd_receiver(
            ctypes.byref(p), coef.data_ptr(), d.x.data_ptr(), y.data_ptr(), d.s.data_ptr(), d.dm.data_ptr(),
            d.sender.data_ptr(), ptr.data_ptr(), None, dx.data_ptr(), dy.data_ptr(), ds.data_ptr(), stream))
        torch.cuda.synchronize()
        return out, dx, dy, ds

    flipped = run(d.y, mask)
    negated = run((d.y * signs).contiguous(), 0)
    assert torch.equal(flipped[0], negated[0])
    assert torch.equal(flipped[3], negated[3])
    torch.testing.assert_close(flipped[1], negated[1], rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(flipped[2], negated[2] * signs, rtol=1e-5, atol=1e-5)
    # the table-driven kernels refuse the mask instead of ignoring it
    p = _lib.ConvParams(num_nodes=w.num_nodes, num_edges=w.num_edges, num_coef=table.num_coef,
                        num_x=int(d.x.shape[1]), num_y=16, num_out=m.params.num_out,
                        num_scalars=int(d.s.shape[1]), channels=w.channels, layout=m.layout.value,
                        val_dtype=_lib.F32, coef_idx_bytes=table.idx_bytes, signature=-1,
                        coef_scale=1.0, debug=0, y_flip=mask, row_order=None)
    out = torch.empty_like(d.dm)
    rc = lib.e3j_amd_convolution_fwd(ctypes.byref(p), table.device(d.x.device).data_ptr(), d.x.data_ptr(),
                                     d.y.data_ptr(), d.s.data_ptr(), d.sender.data_ptr(), ptr.data_ptr(), None,
                                     out.data_ptr(), stream)
    assert rc == _lib.INVALID_ARGUMENT and b"y_flip" in lib.e3j_amd_last_error()


@pytest.mark.parametrize("layout", ["TRAILING_CHANNELS", "LEADING_CHANNELS"])
@pytest.mark.parametrize("name", ["cfg1", "cfg2", "cfg3"])
def test_deterministic_backward_is_bit_reproducible_and_matches(name, layout):
    """`config(deterministic=True)`: the atomic-free backward of the unrolled kernels (dx rows per
    position summed in a fixed order).  Bit-identical over repeats like the reference's backward
    (`tests/test_ops/test_convolution_op.py:329-342`), same values as the oracle, and independent
    of the launch variant's wave count per edge only through float32 rounding."""
    w = CASES[name]().with_layout(layout)
    d = w.to("cuda")
    m = w.module
    coef = m._packed_coef("float32")
    # some padding edges inside the list and an unsorted variant below
    snd = d.sender.clone()
    snd[::17] = e3j_amd.DUMMY_INDEX
    lib = _lib.load()

    def run():
        g = e3j_amd.convolution_bwd(coef, d.x, d.y, d.s, snd, d.receiver, d.dm, m.params, m.graph_ordering,
                                    layout=m.layout)
        torch.cuda.synchronize()
        return g

    with e3j_amd.config.use(deterministic=True):
        base = run()
        for _ in range(50 if name == "cfg2" else 4):   # 50 repeats: the reference's count
            for a, b in zip(base, run()):
                assert torch.equal(a, b)
        if name == "cfg2":
            out = e3j_amd.convolution(coef, d.x, d.y, d.s, snd, d.receiver, m.params, m.graph_ordering,
                                      layout=m.layout)
            for _ in range(50):
                assert torch.equal(out, e3j_amd.convolution(coef, d.x, d.y, d.s, snd, d.receiver, m.params,
                                                            m.graph_ordering, layout=m.layout))
        try:  # another launch shape: other waves per edge, same sums up to rounding
            lib.e3j_amd_set_launch_variant(0, 2)
            other = run()
        finally:
            lib.e3j_amd_set_launch_variant(0, 0)
    atomic = run()
    for a, b, c, what in zip(base, atomic, other, ("dx", "dy", "ds")):
        scale = float(a.abs().max())
        assert float((a - b).abs().max()) <= 2e-5 * scale, what
        assert float((a - c).abs().max()) <= 2e-5 * scale, what
    idx, val, mix = w.table()
    a = w.numpy()
    a["sender"] = snd.cpu().numpy()
    (rx, ry, rs), (mx, my, ms) = H.backward_reference(idx, val, mix, a["x"], a["y"], a["s"], a["sender"],
                                                      a["receiver"], a["dm"])
    H.assert_parity(_trailing(base[0], w), rx, mx, f"{name} dx")
    H.assert_parity(base[1].cpu().numpy(), ry, my, f"{name} dy")
    H.assert_parity(_trailing(base[2], w), rs, ms, f"{name} ds")
    assert not base[1][::17].any() and not base[2][::17].any()     # padding edges: exact zeros


def test_deterministic_backward_on_unsorted_edges():
    """`GraphOrdering.NONE`: positions are sorted on the device first; the ordered backward then
    runs on the sorted positions and writes dy/ds through the permutation."""
    w = CASES["cfg2"]()
    d = w.to("cuda")
    m = w.module
    coef = m._packed_coef("float32")
    shuffle = torch.randperm(w.num_edges, generator=torch.Generator().manual_seed(3)).cuda()
    y, s, snd, rcv = d.y[shuffle].contiguous(), d.s[shuffle].contiguous(), d.sender[shuffle], d.receiver[shuffle]
    with e3j_amd.config.use(deterministic=True):
        got = e3j_amd.convolution_bwd(coef, d.x, y, s, snd, rcv, d.dm, m.params, "NONE")
        again = e3j_amd.convolution_bwd(coef, d.x, y, s, snd, rcv, d.dm, m.params, "NONE")
        want = e3j_amd.convolution_bwd(coef, d.x, d.y, d.s, d.sender, d.receiver, d.dm, m.params, "RECEIVER")
    for a, b in zip(got, again):
        assert torch.equal(a, b)
    assert torch.equal(got[0], want[0])                      # same positions after the stable sort
    assert torch.equal(got[1], want[1][shuffle]) and torch.equal(got[2], want[2][shuffle])


def test_kernel_entry_points_replay_from_a_captured_graph():
    """The forward and backward entry points only enqueue kernels on the stream they are given
    (zero fills included: no memset nodes), so a caller can record them into a HIP graph and
    replay it.  Each replay, with other work and new operand values in between, must equal the
    eager result of the same operands."""
    import ctypes
    from e3j_amd.graph import csr_row_ptr, locality_order
    w = CASES["cfg2"]()
    d = w.to("cuda")
    m = w.module
    table = _Table.get(m._packed_coef("float32"), np.float32)
    sig, scale, _ = _signature_of(w)
    ptr = csr_row_ptr(d.receiver, w.num_nodes)
    order = locality_order(d.sender, ptr, w.num_nodes, 2)
    lib = _lib.load()
    p = _lib.ConvParams(num_nodes=w.num_nodes, num_edges=w.num_edges, num_coef=table.num_coef,
                        num_x=int(d.x.shape[1]), num_y=16, num_out=m.params.num_out,
                        num_scalars=int(d.s.shape[1]), channels=w.channels, layout=m.layout.value,
                        val_dtype=_lib.F32, coef_idx_bytes=table.idx_bytes, signature=sig,
                        coef_scale=scale, debug=0, y_flip=0, row_order=order.data_ptr())
    coef = table.device(d.x.device)
    x, y, s, dm = d.x.clone(), d.y.clone(), d.s.clone(), d.dm.clone()
    out = torch.empty_like(dm)
    dx, dy, ds = torch.empty_like(x), torch.empty_like(y), torch.empty_like(s)

    def launch(stream):
        _lib.check(lib.e3j_amd_convolution_fwd(ctypes.byref(p), coef.data_ptr(), x.data_ptr(), y.data_ptr(),
                                               s.data_ptr(), d.sender.data_ptr(), ptr.data_ptr(), None,
                                               out.data_ptr(), stream))
        _lib.check(lib.e3j_amd_convolution_bwd_receiver(
            ctypes.byref(p), coef.data_ptr(), x.data_ptr(), y.data_ptr(), s.data_ptr(), dm.data_ptr(),
            d.sender.data_ptr(), ptr.data_ptr(), None, dx.data_ptr(), dy.data_ptr(), ds.data_ptr(), stream))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch(side.cuda_stream)                      # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        launch(side.cuda_stream)
    for trial in range(3):
        gen = torch.Generator(device="cuda").manual_seed(100 + trial)
        for t in (x, y, s, dm):
            t.copy_(torch.randn(t.shape, device="cuda", generator=gen))
        (x.sum() + s.sum()).item()                    # unrelated eager work and a synchronisation
        graph.replay()
        torch.cuda.synchronize()
        replayed = [t.clone() for t in (out, dx, dy, ds)]
        launch(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        assert torch.equal(replayed[0], out) and torch.equal(replayed[3], ds), trial
        for a, b in ((replayed[1], dx), (replayed[2], dy)):       # atomics: equal up to summation order
            assert float((a - b).abs().max()) <= 2e-5 * float(b.abs().max()), trial


@pytest.mark.parametrize("layout", ["TRAILING_CHANNELS", "LEADING_CHANNELS"])
def test_padding_edges_with_poisoned_features_never_reach_the_results(layout):
    """Padding edges (sender and/or receiver = INT32_MAX) may carry NaN/Inf features; nodes
    without live edges and the padding rows of dy/ds must come out as exact zeros and no NaN may
    leak into a neighbouring row (`tests/test_pallas_mosaic_gpu_convolution.py:1530-1563`,
    `tests/test_convolution_jax_transforms.py:229-306`), here on the unrolled kernels."""
    w = CASES["cfg2"]().with_layout(layout)
    d = w.to("cuda")
    m = w.module
    coef = m._packed_coef("float32")
    E, n = w.num_edges, w.num_nodes
    snd, rcv = d.sender.clone(), d.receiver.clone()
    y, s = d.y.clone(), d.s.clone()
    tail = E - 40                                  # the last receivers' edges become padding
    rcv[tail:] = e3j_amd.DUMMY_INDEX
    snd[tail + 20:] = e3j_amd.DUMMY_INDEX          # half of them with a padding sender as well
    inside = torch.arange(5, tail, 23, device="cuda")   # sender-only padding inside live rows
    snd[inside] = e3j_amd.DUMMY_INDEX
    poisoned = torch.cat([inside, torch.arange(tail, E, device="cuda")])
    y[poisoned] = float("nan")
    s[poisoned] = float("inf")
    out = e3j_amd.convolution(coef, d.x, y, s, snd, rcv, m.params, m.graph_ordering, layout=m.layout)
    dx, dy, ds = e3j_amd.convolution_bwd(coef, d.x, y, s, snd, rcv, d.dm, m.params, m.graph_ordering,
                                         layout=m.layout)
    with e3j_amd.config.use(deterministic=True):
        dx2, dy2, ds2 = e3j_amd.convolution_bwd(coef, d.x, y, s, snd, rcv, d.dm, m.params, m.graph_ordering,
                                                layout=m.layout)
    for t in (out, dx, dy, ds, dx2, dy2, ds2):
        assert torch.isfinite(t).all()
    for g in (dy, ds, dy2, ds2):
        assert not g[poisoned].any()
    # same as the graph without those edges
    keep = torch.ones(E, dtype=torch.bool, device="cuda")
    keep[poisoned] = False
    ref = e3j_amd.convolution(coef, d.x, d.y[keep].contiguous(), d.s[keep].contiguous(), d.sender[keep],
                              d.receiver[keep], m.params, m.graph_ordering, layout=m.layout)
    assert torch.equal(out, ref)
    last_rows = d.receiver[tail:].unique()
    emptied = [int(r) for r in last_rows if not bool((d.receiver[:tail] == r).any())]
    for r in emptied:
        assert not out[r].any()


def test_views_at_odd_element_offsets_are_served():
    """Operands that are only 4-byte aligned (contiguous views one element into an allocation)
    are outside what the unrolled kernels' 16-byte row pieces take: the operators serve them
    with the table-driven kernels, with the same results."""
    w = CASES["cfg2"]()
    d = w.to("cuda")
    m = w.module
    coef = m._packed_coef("float32")

    def shifted(t):
        flat = torch.empty(t.numel() + 1, dtype=t.dtype, device=t.device)
        view = flat[1:].view(t.shape)
        view.copy_(t)
        assert view.data_ptr() % 16 == 4 and view.is_contiguous()
        return view

    want = e3j_amd.convolution(coef, d.x, d.y, d.s, d.sender, d.receiver, m.params, m.graph_ordering)
    want_g = e3j_amd.convolution_bwd(coef, d.x, d.y, d.s, d.sender, d.receiver, d.dm, m.params, m.graph_ordering)
    got = e3j_amd.convolution(coef, shifted(d.x), d.y, shifted(d.s), d.sender, d.receiver, m.params, m.graph_ordering)
    got_g = e3j_amd.convolution_bwd(coef, shifted(d.x), d.y, shifted(d.s), d.sender, d.receiver, shifted(d.dm),
                                    m.params, m.graph_ordering)
    torch.testing.assert_close(got, want, rtol=2e-5, atol=2e-5)
    for a, b in zip(got_g, want_g):
        torch.testing.assert_close(a, b, rtol=2e-5, atol=2e-5 * float(b.abs().max()))
    # the entry points that have no table-driven form refuse such operands
    from e3j_amd.radial import radial_linear
    h = torch.randn(256, 32, device="cuda")
    wt = torch.randn(32, 64, device="cuda")
    torch.testing.assert_close(radial_linear(shifted(h), wt), h @ wt, rtol=1e-5, atol=1e-5)
    s_out = torch.empty(256 * 64 + 1, device="cuda")
    rc = _lib.load().e3j_amd_radial_linear_fwd(shifted(h).data_ptr(), wt.data_ptr(), s_out.data_ptr(), 256, 32, 64,
                                               int(torch.cuda.current_stream().cuda_stream))
    assert rc == _lib.INVALID_ARGUMENT and b"16-byte" in _lib.load().e3j_amd_last_error()


@pytest.mark.parametrize("name", ["cfg3", "cfg3_k64", "cfg2", "cfg2_k32", "cfg3_k256", "scalars_k64"])
def test_sender_grouped_backward_on_the_unrolled_kernels(name):
    """`e3j_amd_convolution_bwd_sender` with a signature: the reference's grouping (rows are senders,
    `lib/e3j_ops/ffi/e3j_ops.h:575-594`) on the unrolled kernels.  Against the oracle, with padding
    edges and through an edge permutation; dx (and dy up to 128 channels) the same bits in every run;
    a scaled table and a sign mask behave as on the receiver-grouped kernels."""
    import ctypes as C
    from oracle import conv_oracle as O
    w = CASES[name]()
    sig, scale, _ = _signature_of(w)
    assert sig >= 0
    a = w.numpy()
    n, e = w.num_nodes, w.num_edges
    rng = np.random.default_rng(17)
    snd, rcv = a["sender"].copy(), a["receiver"].copy()
    pad = rng.choice(e, size=max(e // 50, 2), replace=False)
    snd[pad[::2]] = np.iinfo(np.int32).max        # padding edges of both kinds
    rcv[pad[1::2]] = np.iinfo(np.int32).max
    perm, recv_t, sptr = O.transpose_graph(snd, rcv, n)   # positions grouped by sender
    m = w.module
    dims = (int(w.x.shape[1]), int(w.y.shape[1]), m.params.num_out, int(w.s.shape[1]))
    lib = _lib.load()
    dev = lambda t: torch.as_tensor(np.ascontiguousarray(t)).cuda()  # noqa: E731
    x, y, s, dm = (dev(a[k]) for k in ("x", "y", "s", "dm"))
    recv_d, sptr_d, perm_d = dev(recv_t.astype(np.int32)), dev(sptr.astype(np.int32)), dev(perm.astype(np.int32))
    idx, val, mix = w.table()
    (rx, ry, rs), (mx, my, ms) = H.backward_reference(idx, val, mix, a["x"], a["y"], a["s"], snd, rcv, a["dm"])

    def run(coef_scale=1.0, y_flip=0):
        p = _lib.ConvParams(num_nodes=n, num_edges=e, num_coef=len(val), num_x=dims[0], num_y=dims[1],
                            num_out=dims[2], num_scalars=dims[3], channels=w.channels, layout=_lib.LAYOUT_TRAILING,
                            val_dtype=_lib.F32, coef_idx_bytes=1, signature=sig, coef_scale=coef_scale * scale,
                            debug=0, y_flip=y_flip, row_order=None)
        dx, dy, ds = (torch.full_like(t, float("nan")) for t in (x, y, s))
        _lib.check(lib.e3j_amd_convolution_bwd_sender(
            C.byref(p), None, x.data_ptr(), y.data_ptr(), s.data_ptr(), dm.data_ptr(), recv_d.data_ptr(),
            sptr_d.data_ptr(), perm_d.data_ptr(), dx.data_ptr(), dy.data_ptr(), ds.data_ptr(),
            int(torch.cuda.current_stream().cuda_stream)))
        torch.cuda.synchronize()
        return dx, dy, ds

    dx, dy, ds = run()
    H.assert_parity(dx.cpu().numpy(), rx, mx, f"{name} dx")
    H.assert_parity(dy.cpu().numpy(), ry, my, f"{name} dy")
    H.assert_parity(ds.cpu().numpy(), rs, ms, f"{name} ds")
    dead = (snd >= n) | (rcv >= n)
    assert not dy.cpu().numpy()[dead].any() and not ds.cpu().numpy()[dead].any()      # exact zeros
    dx2, dy2, ds2 = run()
    assert torch.equal(dx, dx2) and torch.equal(ds, ds2)
    if w.channels <= 128:
        assert torch.equal(dy, dy2)
    # a uniformly scaled table
    dx3, dy3, ds3 = run(coef_scale=0.25)
    for g, g0 in ((dx3, dx), (dy3, dy), (ds3, ds)):
        assert float((g - 0.25 * g0).abs().max()) <= 2e-6 * float(g0.abs().max())
    # the sign mask on y: as if y[:, k] were negated, with dy[:, k] returned negated
    mask = 0b1010
    signs = torch.ones(dims[1], device="cuda")
    signs[1], signs[3] = -1.0, -1.0
    dx4, dy4, ds4 = run(y_flip=mask)
    y_keep = y.clone()
    y.mul_(signs)
    dx5, dy5, ds5 = run()
    y.copy_(y_keep)
    assert torch.equal(dx4, dx5) and torch.equal(ds4, ds5)
    if w.channels <= 128:
        assert torch.equal(dy4, dy5 * signs)
    else:   # four waves add into a dy row: equal up to the order of those additions
        assert float((dy4 - dy5 * signs).abs().max()) <= 1e-5 * float(dy5.abs().max())
