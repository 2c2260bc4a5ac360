"""The XLA-FFI handlers driven with hand-built call frames over GPU buffers."""

import ctypes as C

import numpy as np
import pytest
import torch

from e3j_amd import _lib
from e3j_amd.coef import Coef4D
from oracle import conv_oracle as O
from tests import helpers as H
from tests.xla_frame import F32, S32, U8, FakeXla

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _buf(xla, t, dtype):
    xla._keep.append(t)  # the frame only holds the address: keep the tensor alive
    return xla.buffer(dtype, t.data_ptr(), tuple(t.shape))


def _problem():
    rng = np.random.default_rng(12)
    N, E, X, Y, Z, S, K, nnz = 9, 50, 4, 5, 6, 3, 32, 40
    idx, val, mix = H.random_table(rng, nnz, X, Y, Z, S)
    snd, rcv = H.random_graph(rng, N, E)
    x, y, s, dm = H.random_operands(rng, N, E, X, Y, S, K, Z)
    return idx, val, mix, x, y, s, dm, snd, rcv, Z


def test_forward_and_both_backward_targets():
    idx, val, mix, x, y, s, dm, snd, rcv, Z = _problem()
    lib = _lib.load()
    xla = FakeXla(stream=torch.cuda.current_stream().cuda_stream)
    n = x.shape[0]
    packed = H.pack_table(idx, val, mix)
    coef = dev(packed)
    xd, yd, sd, dmd = dev(x), dev(y), dev(s), dev(dm)
    ptr = dev(O.receiver_ptr(rcv, n))
    ranges = dev(np.array([len(val)], dtype=np.int32))
    attrs = lambda: {"num_nodes": (S32, C.c_int32(n)), "debug": (S32, C.c_int32(1))}  # noqa: E731

    # "convolution": reference operand order, coef_ranges present and ignored
    out = torch.full((n, Z, x.shape[2]), float("nan"), device="cuda")
    frame = xla.frame([_buf(xla, coef, U8), _buf(xla, xd, F32), _buf(xla, yd, F32), _buf(xla, sd, F32),
                       _buf(xla, dev(snd), S32), _buf(xla, ptr, S32), _buf(xla, ranges, S32)],
                      [_buf(xla, out, F32)], attrs())
    keep = [frame]
    assert lib.e3j_amd_xla_convolution(C.addressof(frame)) is None, xla.errors
    torch.cuda.synchronize()
    ref, mag = H.forward_reference(idx, val, mix, x, y, s, snd, rcv, Z)
    H.assert_parity(out.cpu().numpy(), ref, mag, "xla out")

    refs, mags = H.backward_reference(idx, val, mix, x, y, s, snd, rcv, dm)

    def check(dx, dy, ds, tag):
        torch.cuda.synchronize()
        for g, r, m, name in zip((dx, dy, ds), refs, mags, ("dx", "dy", "ds")):
            H.assert_parity(g.cpu().numpy(), r, m, f"{tag} {name}")

    # "convolution_bwd": transposed CSR, permutation, and the reference's stack of three
    # transposed tables (src/e3j/ops/convolution.py:366-369,401-403)
    c = Coef4D.unpack(packed, np.float32)
    stacked = np.stack([c.transpose(a).pack() for a in ((1, 0, 2, 3), (2, 0, 1, 3), (3, 0, 2, 1))])
    perm, recv_t, sptr = O.transpose_graph(snd, rcv, n)
    dx, dy, ds = (torch.full_like(t, float("nan")) for t in (xd, yd, sd))
    operands = [_buf(xla, dev(stacked), U8), _buf(xla, xd, F32), _buf(xla, yd, F32), _buf(xla, sd, F32),
                _buf(xla, dmd, F32), _buf(xla, dev(recv_t.astype(np.int32)), S32), _buf(xla, dev(sptr), S32),
                _buf(xla, dev(perm), S32), _buf(xla, ranges, S32)]
    keep.append(operands)
    frame = xla.frame(operands, [_buf(xla, dx, F32), _buf(xla, dy, F32), _buf(xla, ds, F32)], attrs())
    assert lib.e3j_amd_xla_convolution_bwd(C.addressof(frame)) is None, xla.errors
    check(dx, dy, ds, "stacked tables")

    # same target with the forward table
    dx, dy, ds = (torch.full_like(t, float("nan")) for t in (xd, yd, sd))
    operands[0] = _buf(xla, coef, U8)
    frame = xla.frame(operands, [_buf(xla, dx, F32), _buf(xla, dy, F32), _buf(xla, ds, F32)], attrs())
    assert lib.e3j_amd_xla_convolution_bwd(C.addressof(frame)) is None, xla.errors
    check(dx, dy, ds, "forward table")

    # "convolution_bwd_receiver": forward CSR, empty permutation
    dx, dy, ds = (torch.full_like(t, float("nan")) for t in (xd, yd, sd))
    empty = torch.zeros(0, dtype=torch.int32, device="cuda")
    frame = xla.frame([_buf(xla, coef, U8), _buf(xla, xd, F32), _buf(xla, yd, F32), _buf(xla, sd, F32),
                       _buf(xla, dmd, F32), _buf(xla, dev(snd), S32), _buf(xla, ptr, S32),
                       xla.buffer(S32, 0, (0,))],
                      [_buf(xla, dx, F32), _buf(xla, dy, F32), _buf(xla, ds, F32)], attrs())
    assert lib.e3j_amd_xla_convolution_bwd_receiver(C.addressof(frame)) is None, xla.errors
    check(dx, dy, ds, "receiver grouping")

    # a runtime that hands out scratch: the plan of the table lives there for the length of a call
    xla.allocate = lambda nbytes: torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    dx, dy, ds = (torch.full_like(t, float("nan")) for t in (xd, yd, sd))
    frame = xla.frame([_buf(xla, coef, U8), _buf(xla, xd, F32), _buf(xla, yd, F32), _buf(xla, sd, F32),
                       _buf(xla, dmd, F32), _buf(xla, dev(snd), S32), _buf(xla, ptr, S32),
                       xla.buffer(S32, 0, (0,))],
                      [_buf(xla, dx, F32), _buf(xla, dy, F32), _buf(xla, ds, F32)], attrs())
    assert lib.e3j_amd_xla_convolution_bwd_receiver(C.addressof(frame)) is None, xla.errors
    check(dx, dy, ds, "receiver grouping, plan in the runtime's scratch")
    out2 = torch.full_like(out, float("nan"))
    frame = xla.frame([_buf(xla, coef, U8), _buf(xla, xd, F32), _buf(xla, yd, F32), _buf(xla, sd, F32),
                       _buf(xla, dev(snd), S32), _buf(xla, ptr, S32), _buf(xla, ranges, S32)],
                      [_buf(xla, out2, F32)], attrs())
    assert lib.e3j_amd_xla_convolution(C.addressof(frame)) is None, xla.errors
    torch.cuda.synchronize()
    H.assert_parity(out2.cpu().numpy(), ref, mag, "xla out, plan in the runtime's scratch")
    assert xla.allocations == 2 and not xla.scratch   # borrowed once per call and handed back
    del empty, keep


def test_ordered_backward_target_with_a_signature_and_scratch_result():
    """"convolution_bwd_ordered": the forward CSR, attributes `signature`/`coef_scale` from the
    host-side lookup, and the scratch of the atomic-free backward as a fourth result."""
    from e3j_amd import workloads as W
    from e3j_amd.ops import _Table
    w = W.config2(0.04)
    m = w.module
    packed = m._packed_coef("float32")
    dims = (int(w.x.shape[1]), int(w.y.shape[1]), m.params.num_out, int(w.s.shape[1]))
    sig, scale, _ = _Table.get(packed, np.float32).signature(dims, w.channels, m.layout)
    assert sig >= 0
    lib = _lib.load()
    xla = FakeXla(stream=torch.cuda.current_stream().cuda_stream)
    d = w.to("cuda")
    n = w.num_nodes
    ptr = dev(O.receiver_ptr(d.receiver.cpu().numpy(), n))
    p = _lib.ConvParams(num_nodes=n, num_edges=w.num_edges, num_coef=packed.shape[0], num_x=dims[0],
                        num_y=dims[1], num_out=dims[2], num_scalars=dims[3], channels=w.channels,
                        layout=m.layout.value, val_dtype=_lib.F32, coef_idx_bytes=1, signature=sig,
                        coef_scale=scale, debug=0, y_flip=0, row_order=None)
    nbytes = int(lib.e3j_amd_convolution_bwd_ordered_workspace_bytes(C.byref(p)))
    attrs = {"num_nodes": (S32, C.c_int32(n)), "debug": (S32, C.c_int32(0)),
             "signature": (S32, C.c_int32(sig)), "coef_scale": (F32, C.c_float(scale))}
    operands = [_buf(xla, dev(packed), U8), _buf(xla, d.x, F32), _buf(xla, d.y, F32), _buf(xla, d.s, F32),
                _buf(xla, d.dm, F32), _buf(xla, d.sender, S32), _buf(xla, ptr, S32), xla.buffer(S32, 0, (0,))]

    def run(workspace_bytes):
        dx, dy, ds = (torch.full_like(t, float("nan")) for t in (d.x, d.y, d.s))
        workspace = torch.empty(workspace_bytes, dtype=torch.uint8, device="cuda")
        frame = xla.frame(operands, [_buf(xla, dx, F32), _buf(xla, dy, F32), _buf(xla, ds, F32),
                                     _buf(xla, workspace, U8)], dict(attrs))
        err = lib.e3j_amd_xla_convolution_bwd_ordered(C.addressof(frame))
        torch.cuda.synchronize()
        return err, (dx, dy, ds)

    err, first = run(nbytes)
    assert err is None, xla.errors
    err, second = run(nbytes)
    assert err is None
    for a, b in zip(first, second):
        assert torch.equal(a, b)                               # bit-reproducible
    idx, val, mix = w.table()
    a = w.numpy()
    refs, mags = H.backward_reference(idx, val, mix, a["x"], a["y"], a["s"], a["sender"], a["receiver"], a["dm"])
    for g, r, mg, name in zip(first, refs, mags, ("dx", "dy", "ds")):
        H.assert_parity(g.cpu().numpy(), r, mg, f"ordered {name}")
    err, _ = run(nbytes // 2)                                  # a scratch result that is too small
    assert err is not None and "workspace" in xla.errors[-1][1]


@pytest.mark.parametrize("mode,layout", [(2, 1), (0, 1), (1, 0), (2, 0)])
def test_tensor_product_targets(mode, layout):
    """"tensor_product" and "tensor_product_bwd" with the reference's operand order and attributes
    (MAP / OUTER with a channel-free y / INNER; trailing and leading layouts)."""
    from e3j_amd.coef import Coef
    from oracle import tp_oracle as T
    rng = np.random.default_rng(31)
    R, X, Y, Z, K, nnz = 40, 6, 5, 9, 16, 70
    idx, val, _ = H.random_table(rng, nnz, X, Y, Z, 3)
    name = {0: "OUTER", 1: "INNER", 2: "MAP"}[mode]
    lay = "TRAILING_CHANNELS" if layout == 1 else "LEADING_CHANNELS"
    x = rng.normal(size=(R, X, K) if layout == 1 else (R, K, X)).astype(np.float32)
    y = (rng.normal(size=(R, Y)) if mode == 0 else
         rng.normal(size=(R, Y, K) if layout == 1 else (R, K, Y))).astype(np.float32)
    ref = T.tensor_product_unfused(idx, val, x.astype(np.float64), y.astype(np.float64), Z, name, lay)
    mag = T.tensor_product_unfused(idx, np.abs(val), np.abs(x).astype(np.float64), np.abs(y).astype(np.float64),
                                   Z, name, lay)
    lib = _lib.load()
    xla = FakeXla(stream=torch.cuda.current_stream().cuda_stream)
    c = Coef(val, idx, "float32", "int32")
    coef = dev(c.pack())
    xd, yd = dev(x), dev(y)
    z = torch.full(ref.shape, float("nan"), device="cuda")
    ranges = dev(np.zeros((0,), dtype=np.int32))
    attrs = {"num_out": (S32, C.c_int32(Z)), "mode": (S32, C.c_int32(mode)), "layout": (S32, C.c_int32(layout)),
             "debug": (S32, C.c_int32(1))}
    frame = xla.frame([_buf(xla, coef, S32), _buf(xla, xd, F32), _buf(xla, yd, F32), _buf(xla, ranges, S32)],
                      [_buf(xla, z, F32)], attrs)
    assert lib.e3j_amd_xla_tensor_product(C.addressof(frame)) is None, xla.errors
    torch.cuda.synchronize()
    H.assert_parity(z.cpu().numpy(), ref, mag, "xla tensor_product")

    dz = rng.normal(size=ref.shape).astype(np.float32)
    rdx, rdy = T.tensor_product_vjp(idx, val, x.astype(np.float64), y.astype(np.float64), dz.astype(np.float64), name, lay)
    mdx, mdy = T.tensor_product_vjp(idx, np.abs(val), np.abs(x).astype(np.float64), np.abs(y).astype(np.float64),
                                    np.abs(dz).astype(np.float64), name, lay)
    stacked = dev(np.stack([c.transpose((1, 0, 2)).pack(), c.transpose((2, 0, 1)).pack()]))
    dx, dy = torch.full_like(xd, float("nan")), torch.full_like(yd, float("nan"))
    attrs_b = {k: v for k, v in attrs.items() if k != "num_out"}
    frame_b = xla.frame([_buf(xla, stacked, S32), _buf(xla, xd, F32), _buf(xla, yd, F32), _buf(xla, dev(dz), F32),
                         _buf(xla, ranges, S32)], [_buf(xla, dx, F32), _buf(xla, dy, F32)], attrs_b)
    assert lib.e3j_amd_xla_tensor_product_bwd(C.addressof(frame_b)) is None, xla.errors
    torch.cuda.synchronize()
    H.assert_parity(dx.cpu().numpy(), rdx, mdx, "xla dx", ulps=32.0)
    H.assert_parity(dy.cpu().numpy(), rdy, mdy, "xla dy", ulps=32.0)

    # decoding errors come back as XLA errors, nothing is launched
    bad = xla.frame([_buf(xla, coef, S32), _buf(xla, xd, F32), _buf(xla, yd, F32)], [_buf(xla, z, F32)],
                    {k: v for k, v in attrs.items() if k != "num_out"})
    assert lib.e3j_amd_xla_tensor_product(C.addressof(bad)) is not None
    assert "num_out" in xla.errors[-1][1]
    wrong = torch.zeros(3, device="cuda")
    bad = xla.frame([_buf(xla, coef, S32), _buf(xla, xd, F32), _buf(xla, yd, F32)], [_buf(xla, wrong, F32)], attrs)
    assert lib.e3j_amd_xla_tensor_product(C.addressof(bad)) is not None
    assert "result shape" in xla.errors[-1][1]


def _time_ms(fn, reps=20):
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(reps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / reps


@pytest.mark.parametrize("size", ["config 2", "288k edges"])
def test_reference_frames_run_the_unrolled_kernels(size):
    """Exactly the operands and attributes the reference sends (`src/e3j/ops/convolution.py:229-242`:
    coef, x, y, s, sender, receiver_ptr, coef_ranges + num_nodes, debug; `:433-452`: the stack of
    three transposed tables, x, y, s, dm, sender_t, receiver_ptr_t, perm, coef_ranges + num_nodes,
    debug), with the table's rows in a permuted order as the reference's
    balancing leaves them: parity against the CPU checker, and the time of the unrolled kernels
    (within 1.3x of the direct C-ABI launches), not of the table-driven ones.  At the size of
    config 2 the backward frame runs the sender-grouped unrolled kernels on the operands as they are
    (nothing borrowed from the runtime); above a quarter of a million edges it rebuilds the receiver rows
    in scratch memory of the runtime and runs the receiver-grouped kernels."""
    from e3j_amd import workloads as W
    from e3j_amd.graph import csr_row_ptr
    from e3j_amd.ops import _Table
    from oracle import c_oracle
    w = W.config2() if size == "config 2" else W.config3(0.3)
    assert (w.num_edges < (1 << 18)) == (size == "config 2")
    m = w.module
    packed = m._packed_coef("float32")
    dims = (int(w.x.shape[1]), int(w.y.shape[1]), m.params.num_out, int(w.s.shape[1]))
    sig, scale, _ = _Table.get(packed, np.float32).signature(dims, w.channels, m.layout)
    assert sig >= 0
    lib = _lib.load()
    d = w.to("cuda")
    n, e = w.num_nodes, w.num_edges
    rng = np.random.default_rng(3)
    c = Coef4D.unpack(packed, np.float32)
    shuffled = Coef4D(c.val, c.idx, "float32", c.idx_dtype)
    order = rng.permutation(len(c.val))
    shuffled = Coef4D(c.val[order], c.idx[order], "float32", c.idx_dtype)
    stacked = np.stack([shuffled.transpose(a).pack() for a in ((1, 0, 2, 3), (2, 0, 1, 3), (3, 0, 2, 1))])
    snd, rcv = w.sender.numpy(), w.receiver.numpy()
    perm, recv_t, sptr = O.transpose_graph(snd, rcv, n)
    ptr = csr_row_ptr(d.receiver, n)
    ranges = dev(np.array([len(c.val)], dtype=np.int32))
    torch.cuda.synchronize()

    xla = FakeXla(stream=torch.cuda.current_stream().cuda_stream)
    xla.allocate = lambda nbytes: torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    attrs = lambda: {"num_nodes": (S32, C.c_int32(n)), "debug": (S32, C.c_int32(0))}  # noqa: E731
    out = torch.full_like(d.dm, float("nan"))
    fwd = xla.frame([_buf(xla, dev(shuffled.pack()), U8), _buf(xla, d.x, F32), _buf(xla, d.y, F32),
                     _buf(xla, d.s, F32), _buf(xla, d.sender, S32), _buf(xla, ptr, S32), _buf(xla, ranges, S32)],
                    [_buf(xla, out, F32)], attrs())
    dx, dy, ds = (torch.full_like(t, float("nan")) for t in (d.x, d.y, d.s))
    bwd = xla.frame([_buf(xla, dev(stacked), U8), _buf(xla, d.x, F32), _buf(xla, d.y, F32), _buf(xla, d.s, F32),
                     _buf(xla, d.dm, F32), _buf(xla, dev(recv_t.astype(np.int32)), S32), _buf(xla, dev(sptr), S32),
                     _buf(xla, dev(perm), S32), _buf(xla, ranges, S32)],
                    [_buf(xla, dx, F32), _buf(xla, dy, F32), _buf(xla, ds, F32)], attrs())
    torch.cuda.synchronize()
    assert lib.e3j_amd_xla_convolution(C.addressof(fwd)) is None, xla.errors
    assert lib.e3j_amd_xla_convolution_bwd(C.addressof(bwd)) is None, xla.errors
    torch.cuda.synchronize()
    # the rebuilt receiver rows: scratch borrowed once and handed back; the small graph borrows nothing
    assert xla.allocations == (0 if size == "config 2" else 1) and not xla.scratch

    idx, val, mix = w.table()
    a = w.numpy()
    args = (a["x"], a["y"], a["s"], a["sender"], a["receiver"])
    mag_args = tuple(np.abs(t) for t in args[:3]) + args[3:]
    ref = c_oracle.convolution(idx, val, mix, *args, dims[2])
    mag = c_oracle.convolution(idx, np.abs(val), mix, *mag_args, dims[2])
    H.assert_parity(out.cpu().numpy(), ref.astype(np.float64), 2.0 * mag.astype(np.float64), "reference frame out",
                    ulps=32.0)
    refs = c_oracle.convolution_vjp(idx, val, mix, *args, a["dm"])
    mags = c_oracle.convolution_vjp(idx, np.abs(val), mix, *mag_args, np.abs(a["dm"]))
    for g, r, mg, name in zip((dx, dy, ds), refs, mags, ("dx", "dy", "ds")):
        H.assert_parity(g.cpu().numpy(), r.astype(np.float64), 2.0 * mg.astype(np.float64), f"reference frame {name}",
                        ulps=32.0)

    # the direct launches of the same kernels through the C ABI
    p = _lib.ConvParams(num_nodes=n, num_edges=e, num_coef=packed.shape[0], num_x=dims[0], num_y=dims[1],
                        num_out=dims[2], num_scalars=dims[3], channels=w.channels, layout=m.layout.value,
                        val_dtype=_lib.F32, coef_idx_bytes=1, signature=sig, coef_scale=scale, debug=0, y_flip=0,
                        row_order=None)
    stream = int(torch.cuda.current_stream().cuda_stream)

    def direct_fwd():
        _lib.check(lib.e3j_amd_convolution_fwd(C.byref(p), None, d.x.data_ptr(), d.y.data_ptr(), d.s.data_ptr(),
                                               d.sender.data_ptr(), ptr.data_ptr(), None, out.data_ptr(), stream))

    def direct_bwd():
        _lib.check(lib.e3j_amd_convolution_bwd_receiver(
            C.byref(p), None, d.x.data_ptr(), d.y.data_ptr(), d.s.data_ptr(), d.dm.data_ptr(), d.sender.data_ptr(),
            ptr.data_ptr(), None, dx.data_ptr(), dy.data_ptr(), ds.data_ptr(), stream))

    t_direct = _time_ms(direct_fwd), _time_ms(direct_bwd)
    t_frames = (_time_ms(lambda: lib.e3j_amd_xla_convolution(C.addressof(fwd))),
                _time_ms(lambda: lib.e3j_amd_xla_convolution_bwd(C.addressof(bwd))))
    print(f"direct fwd/bwd {t_direct[0]:.3f}/{t_direct[1]:.3f} ms, reference frames {t_frames[0]:.3f}/{t_frames[1]:.3f} ms")
    assert t_frames[0] <= 1.3 * t_direct[0] + 0.02, (t_frames, t_direct)
    assert sum(t_frames) <= 1.3 * sum(t_direct) + 0.03, (t_frames, t_direct)

    # without scratch from the runtime the backward keeps the sender rows (their unrolled kernels), same results
    xla.allocate = None
    dx2, dy2, ds2 = (torch.full_like(t, float("nan")) for t in (d.x, d.y, d.s))
    bwd2 = xla.frame(bwd_operands(bwd), [_buf(xla, dx2, F32), _buf(xla, dy2, F32), _buf(xla, ds2, F32)], attrs())
    assert lib.e3j_amd_xla_convolution_bwd(C.addressof(bwd2)) is None, xla.errors
    torch.cuda.synchronize()
    for g, g0, name in zip((dx2, dy2, ds2), (dx, dy, ds), ("dx", "dy", "ds")):
        assert float((g - g0).abs().max()) <= 3e-5 * float(g0.abs().max()), name

    # a `signature` attribute that names kernels of another table size is refused
    bad = dict(attrs())
    bad["signature"] = (S32, C.c_int32(0))
    frame = xla.frame(bwd_operands(fwd), [_buf(xla, out, F32)], bad)
    if lib.e3j_amd_signature_name(0) and sig != 0:
        err = lib.e3j_amd_xla_convolution(C.addressof(frame))
        assert err is not None and ("entries" in xla.errors[-1][1] or "match" in xla.errors[-1][1])


def bwd_operands(frame):
    """The argument buffers of a frame, to build another frame over them."""
    from tests.xla_frame import Buffer
    n = frame.args.size
    return [C.cast(frame.args.args[i], C.POINTER(Buffer)).contents for i in range(n)]


def _reference_forward_frame(scale=0.05):
    from e3j_amd import workloads as W
    from e3j_amd.graph import csr_row_ptr
    w = W.config2(scale)
    d = w.to("cuda")
    n = w.num_nodes
    table = w.module._packed_coef("float32")
    packed = dev(table)
    ptr = csr_row_ptr(d.receiver, n)
    ranges = dev(np.array([1], dtype=np.int32))
    xla = FakeXla(stream=torch.cuda.current_stream().cuda_stream)
    out = torch.zeros_like(d.dm)
    frame = xla.frame([_buf(xla, packed, U8), _buf(xla, d.x, F32), _buf(xla, d.y, F32), _buf(xla, d.s, F32),
                       _buf(xla, d.sender, S32), _buf(xla, ptr, S32), _buf(xla, ranges, S32)],
                      [_buf(xla, out, F32)], {"num_nodes": (S32, C.c_int32(n)), "debug": (S32, C.c_int32(0))})
    keep = (w, d, ptr, ranges)
    return xla, frame, table, packed, out, keep


def _rescaled(table: np.ndarray, factor: float) -> np.ndarray:
    """The packed table (uint8 rows of {float32 val; 4 x uint8 index}) with every value times `factor`."""
    t = table.copy()
    vals = t[:, :4].copy().view(np.float32) * np.float32(factor)
    t[:, :4] = vals.view(np.uint8).reshape(-1, 4)
    return t


def test_reference_forward_frame_follows_a_table_rewritten_in_place():
    """The kernels of a frame without `signature` are found from the table's bytes at every call,
    never from its address: the same device buffer rewritten with a rescaled table (same shape, as
    the reference's signed and unsigned tables have) gives the rescaled result, also when the
    rewrite is still in flight on the caller's stream when the handler is called."""
    lib = _lib.load()
    xla, frame, table, packed, out, keep = _reference_forward_frame()
    torch.cuda.synchronize()
    assert lib.e3j_amd_xla_convolution(C.addressof(frame)) is None, xla.errors
    torch.cuda.synchronize()
    first = out.clone()
    assert float(first.abs().max()) > 0
    # rewritten on the caller's stream, handler called without waiting for it
    staged = torch.as_tensor(_rescaled(table, -2.5)).pin_memory()
    filler = torch.empty(1 << 26, device="cuda")
    for _ in range(4):
        filler.normal_()           # work ahead of the rewrite on the same stream
    packed.copy_(staged, non_blocking=True)
    assert lib.e3j_amd_xla_convolution(C.addressof(frame)) is None, xla.errors
    torch.cuda.synchronize()
    assert float((out + 2.5 * first).abs().max()) <= 2e-5 * float(first.abs().max()) * 2.5
    # and a table no signature matches (one value changed) runs the table-driven kernels: same contract
    odd = table.copy()
    v = odd[0, :4].copy().view(np.float32) * np.float32(1.5)
    odd[0, :4] = v.view(np.uint8)
    packed.copy_(torch.as_tensor(odd))
    assert lib.e3j_amd_xla_convolution(C.addressof(frame)) is None, xla.errors
    torch.cuda.synchronize()
    assert float((out - first).abs().max()) > 0


def test_reference_forward_frame_under_graph_capture_reads_the_table_at_every_replay():
    """Nothing can be read back while a stream is captured, and nothing is assumed about the table
    buffer: a frame without `signature` records the table-driven kernels, which read the table on
    the device.  Replays give the eager result; after the table buffer is rewritten in place with
    a rescaled table, the replays give the rescaled result.  A frame that names `signature`,
    `coef_scale` and `y_flip` records the unrolled kernels."""
    from e3j_amd.ops import _Table
    lib = _lib.load()
    xla, frame, table, packed, out, keep = _reference_forward_frame()
    xla.allocate = lambda nbytes: torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    w = keep[0]
    torch.cuda.synchronize()
    assert lib.e3j_amd_xla_convolution(C.addressof(frame)) is None, xla.errors
    torch.cuda.synchronize()
    eager = out.clone()
    tol = 2e-5 * float(eager.abs().max())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        xla.stream = torch.cuda.current_stream().cuda_stream
        assert lib.e3j_amd_xla_convolution(C.addressof(frame)) is None, xla.errors
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert float((out - eager).abs().max()) <= tol
    packed.copy_(torch.as_tensor(_rescaled(table, 3.0)))
    for _ in range(2):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert float((out - 3.0 * eager).abs().max()) <= 3.0 * tol
    packed.copy_(torch.as_tensor(table))

    # the path without a host wait: the frame names the kernels itself
    m = w.module
    dims = (int(w.x.shape[1]), int(w.y.shape[1]), m.params.num_out, int(w.s.shape[1]))
    sig, scale, flip = _Table.get(table, np.float32).signature(dims, w.channels, m.layout)
    assert sig >= 0
    named = xla.frame(bwd_operands(frame), [_buf(xla, out, F32)],
                      {"num_nodes": (S32, C.c_int32(w.num_nodes)), "debug": (S32, C.c_int32(0)),
                       "signature": (S32, C.c_int32(sig)), "coef_scale": (F32, C.c_float(scale)),
                       "y_flip": (S32, C.c_int32(flip))})
    graph2 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph2):
        xla.stream = torch.cuda.current_stream().cuda_stream
        assert lib.e3j_amd_xla_convolution(C.addressof(named)) is None, xla.errors
    for _ in range(2):
        out.zero_()
        graph2.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)   # the eager call resolved to the same unrolled kernels
