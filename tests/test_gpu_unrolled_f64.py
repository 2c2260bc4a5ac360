"""float64 operands on the compile-time-unrolled kernels (trailing layout): the kernels read one
coefficient per class of equal magnitude from the call, so a table with the structure of a
built-in signature is served to float64 accuracy whatever its values (here: Clebsch-Gordan values
divided by an average neighbour count and rounded to float32, as the modules store them, which
is not a multiple of the built-in table beyond float32 rounding).  Checked against the float64
oracle at float64 tolerances, against the table-driven kernels, through the C ABI and through
the operators."""

import ctypes

import numpy as np
import pytest
import torch

import e3j_amd
from e3j_amd import _lib, workloads as W
from e3j_amd.convolution import Convolution
from e3j_amd.ops import _Table
from oracle import conv_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu

EPS64 = 2.0 ** -52


def assert_parity64(got, ref, mag, what):
    """Within 64 float64 roundings of the sum of the absolute values of the terms."""
    got = np.asarray(got, dtype=np.float64)
    assert got.shape == ref.shape, f"{what}: shape {got.shape} != {ref.shape}"
    err = np.abs(got - ref)
    bound = 64 * EPS64 * mag + 1e-300
    assert (err <= bound).all(), (f"{what}: {int((err > bound).sum())} elements off; worst {err.max():.3e} "
                                  f"against a bound of {bound[np.unravel_index(err.argmax(), err.shape)]:.3e}")


CASES = {
    "cfg3_k64": lambda: W.config3(0.006, channels=64),
    "cfg3": lambda: W.config3(0.004),
    "cfg3_k256": lambda: W.config3(0.002, channels=256),
    "cfg2": lambda: W.config2(0.04),
    "cfg2_k128": lambda: W.config2(0.03, channels=128),
    "scalars_k64": lambda: W.make_workload("scalars", 200, "0e", 3, "0e+1o+2e+3o", 64, (51, 52, 53, 54)),
}


def _with_neighbour_count(w, avg):
    """The workload with `1 / avg` folded into its module's table (then rounded to float32, as the
    modules store it): no longer the built-in table times one factor beyond float32 rounding."""
    import dataclasses
    m = w.module
    out_filter = "+".join(dict.fromkeys(f"{ir.l}{'e' if ir.p == 1 else 'o'}" for _, ir in m.target))
    module = Convolution((m.source[0], m.source[1]), out_filter, graph_ordering=m.graph_ordering, layout=m.layout,
                         avg_num_neighbors=avg, normalization=m.normalization)
    ratio = np.asarray(module.coef.val, dtype=np.float64) * avg / np.asarray(m.coef.val, dtype=np.float64)
    distinct = len(set(np.abs(np.asarray(m.coef.val)).tolist()))
    assert np.ptp(ratio) < 1e-6 and (distinct == 1 or np.ptp(ratio) > 1e-9)
    return dataclasses.replace(w, module=module)


def _f64(w):
    """The workload's operands in float64 (values drawn in float32, widened, then perturbed so that
    they are not float32 numbers), host arrays and device tensors."""
    rng = np.random.default_rng(123)
    a = w.numpy()
    host = {}
    for f in ("x", "y", "s", "dm"):
        v = a[f].astype(np.float64)
        host[f] = v * (1.0 + 1e-9 * rng.standard_normal(v.shape))
    host["sender"], host["receiver"] = a["sender"], a["receiver"]
    dev = {f: torch.as_tensor(v).cuda() for f, v in host.items()}
    return host, dev


@pytest.mark.parametrize("name", list(CASES))
def test_float64_unrolled_kernels_match_the_float64_oracle(name):
    w = _with_neighbour_count(CASES[name](), 12.5)
    m = w.module
    coef = m._packed_coef("float64")
    dims = (int(w.x.shape[1]), int(w.y.shape[1]), m.params.num_out, int(w.s.shape[1]))
    sig, classes, flip = _Table.get(coef, np.float64).signature(dims, w.channels, m.layout)
    assert sig >= 0 and flip == 0, "the float64 table must resolve to the built-in signature"
    assert not isinstance(classes, float) and max(classes) > 0
    host, d = _f64(w)
    out = e3j_amd.convolution(coef, d["x"], d["y"], d["s"], d["sender"], d["receiver"], m.params, m.graph_ordering,
                              layout=m.layout)
    dx, dy, ds = e3j_amd.convolution_bwd(coef, d["x"], d["y"], d["s"], d["sender"], d["receiver"], d["dm"],
                                         m.params, m.graph_ordering, layout=m.layout)
    torch.cuda.synchronize()
    assert out.dtype == torch.float64
    idx, val, mix = w.table()
    val = np.asarray(val, dtype=np.float64)   # the float32 values of the module's table, as the packed table holds them
    args = (host["x"], host["y"], host["s"], host["sender"], host["receiver"])
    mags = tuple(np.abs(t) for t in args[:3]) + args[3:]
    ref = O.convolution_unfused(idx, val, mix, *args, m.params.num_out, dtype=np.float64)
    mag = O.convolution_unfused(idx, np.abs(val), mix, *mags, m.params.num_out, dtype=np.float64)
    assert_parity64(out.cpu().numpy(), ref, mag, f"{name} out")
    refs = O.convolution_vjp(idx, val, mix, *args, host["dm"], dtype=np.float64)
    mgs = O.convolution_vjp(idx, np.abs(val), mix, *mags, np.abs(host["dm"]), dtype=np.float64)
    for g, r, mg, what in zip((dx, dy, ds), refs, mgs, ("dx", "dy", "ds")):
        assert_parity64(g.cpu().numpy(), r, mg, f"{name} {what}")


def test_float64_through_the_c_abi_with_padding_permutation_and_sign_mask():
    """The C ABI with float64 operands and `coef_classes`: unsorted edges through `edge_perm`,
    padding edges (zero dy / ds rows), a receiver without edges, and a table whose y components of
    odd degree carry the opposite sign (`y_flip` from the look-up, as the SENDER ordering folds
    them).  Against the oracle on the table as given and against the table-driven kernels."""
    from tests.test_gpu_generic import _dev, _params
    lib = _lib.load()
    m = Convolution(("0e+1o+2e+3o", "0e+1o+2e+3o"), "0e+1o+2e+3o", graph_ordering="RECEIVER", avg_num_neighbors=7.3)
    c = m.coef
    parity = np.asarray(m.y_parity, dtype=np.float64)
    idx4 = np.asarray(c.idx, dtype=np.int64)
    val = np.asarray(c.val, dtype=np.float64) * parity[idx4[:, 2]]
    idx, mix = idx4[:, :3], m._mix.mix_indices
    rng = np.random.default_rng(17)
    N, E, X, Y, Z, S, K = 40, 900, 16, 16, 99, 23, 128
    snd = rng.integers(0, N, E)
    rcv = rng.integers(0, N - 1, E)          # the last receiver has no edges
    snd[rng.random(E) < 0.05] = N            # padding edges: sender out of range
    x, y, s, dm = (a.astype(np.float64) * (1 + 1e-9) for a in H.random_operands(rng, N, E, X, Y, S, K, Z))
    perm = np.argsort(rcv, kind="stable")
    packed = H.pack_table(idx, val, mix, val_dtype=np.float64)
    classes = (ctypes.c_double * _lib.F64_CLASSES)()
    flip = ctypes.c_uint32()
    sig = lib.e3j_amd_find_signature_f64(packed.ctypes.data, 1, len(val), X, Y,
                                         Z, S, K, 1, classes, ctypes.byref(flip))
    assert sig >= 0 and flip.value == sum(1 << k for k in range(Y) if parity[k] < 0)
    p = _params(N, E, len(val), X, Y, Z, S, K, 1, _lib.F64, 1)
    p.signature, p.y_flip = sig, flip.value
    p.coef_classes = ctypes.cast(classes, ctypes.c_void_p).value
    coef_d = _dev(packed.view(np.uint8).reshape(-1))
    xd, yd, sd, dmd = _dev(x), _dev(y), _dev(s), _dev(dm)
    other, perm_d, ptr = _dev(snd[perm].astype(np.int32)), _dev(perm.astype(np.int32)), _dev(O.receiver_ptr(rcv[perm], N))
    stream = torch.cuda.current_stream().cuda_stream

    def run(params):
        out = torch.full((N, Z, K), float("nan"), dtype=torch.float64, device="cuda")
        dx, dy, ds = (torch.full_like(t, float("nan")) for t in (xd, yd, sd))
        _lib.check(lib.e3j_amd_convolution_fwd(ctypes.byref(params), coef_d.data_ptr(), xd.data_ptr(), yd.data_ptr(),
                                               sd.data_ptr(), other.data_ptr(), ptr.data_ptr(), perm_d.data_ptr(),
                                               out.data_ptr(), stream))
        _lib.check(lib.e3j_amd_convolution_bwd_receiver(
            ctypes.byref(params), coef_d.data_ptr(), xd.data_ptr(), yd.data_ptr(), sd.data_ptr(), dmd.data_ptr(),
            other.data_ptr(), ptr.data_ptr(), perm_d.data_ptr(), dx.data_ptr(), dy.data_ptr(), ds.data_ptr(), stream))
        torch.cuda.synchronize()
        return [t.cpu().numpy() for t in (out, dx, dy, ds)]

    got = run(p)
    live = snd < N
    args = (x, y, s, snd, rcv)
    ref = O.convolution_unfused(idx, val, mix, *args, Z, dtype=np.float64)
    mag = O.convolution_unfused(idx, np.abs(val), mix, np.abs(x), np.abs(y), np.abs(s), args[3], rcv, Z, dtype=np.float64)
    assert_parity64(got[0], ref, mag, "out")
    assert not got[0][N - 1].any()                                   # the receiver without edges: a zero row
    refs = O.convolution_vjp(idx, val, mix, *args, dm, dtype=np.float64)
    mgs = O.convolution_vjp(idx, np.abs(val), mix, np.abs(x), np.abs(y), np.abs(s), args[3], rcv, np.abs(dm),
                            dtype=np.float64)
    for g, r, mg, what in zip(got[1:], refs, mgs, ("dx", "dy", "ds")):
        assert_parity64(g, r, mg, what)
    assert not got[2][~live].any() and not got[3][~live].any()       # padding edges: zero dy / ds rows
    # the table-driven kernels on the same operands
    q = _params(N, E, len(val), X, Y, Z, S, K, 1, _lib.F64, 1)
    for a, b, what in zip(got, run(q), ("out", "dx", "dy", "ds")):
        np.testing.assert_allclose(a, b, rtol=1e-11, atol=1e-12, err_msg=what)
    # float64 operands with a signature and no classes, and a grouping the float64 kernels do not serve
    p.coef_classes = None
    with pytest.raises(_lib.E3jAmdError, match="coef_classes"):
        run(p)
    p.coef_classes = ctypes.cast(classes, ctypes.c_void_p).value
    with pytest.raises(_lib.E3jAmdError, match="receiver-grouped"):
        _lib.check(lib.e3j_amd_convolution_bwd_sender(
            ctypes.byref(p), coef_d.data_ptr(), xd.data_ptr(), yd.data_ptr(), sd.data_ptr(), dmd.data_ptr(),
            other.data_ptr(), ptr.data_ptr(), perm_d.data_ptr(), xd.data_ptr(), yd.data_ptr(), sd.data_ptr(), stream))


def test_float64_module_gradients_and_the_deterministic_mode():
    """The module in float64 through autograd on the unrolled kernels against the dense form, and
    `config(deterministic=True)`, which takes the table-driven rows that own their dx instead of
    float64 atomics: the same bits in two runs, the same values to rounding."""
    from e3j_amd.options import config
    w = _with_neighbour_count(W.config2(0.03), 20.0)
    m = w.module
    host, d = _f64(w)
    x, y, s = (d[f].clone().requires_grad_(True) for f in ("x", "y", "s"))
    out = m(x, y, s, d["sender"], d["receiver"])
    gx, gy, gs = torch.autograd.grad(out, (x, y, s), d["dm"])
    idx, val, mix = w.table()
    val = np.asarray(val, dtype=np.float64)
    refs = O.convolution_vjp(idx, val, mix, host["x"], host["y"], host["s"], host["sender"], host["receiver"],
                             host["dm"], dtype=np.float64)
    for g, r, what in zip((gx, gy, gs), refs, ("dx", "dy", "ds")):
        np.testing.assert_allclose(g.cpu().numpy(), r, rtol=1e-11, atol=1e-12, err_msg=what)
    with config.use(deterministic=True):
        runs = []
        for _ in range(2):
            o = m(x, y, s, d["sender"], d["receiver"])
            runs.append(torch.autograd.grad(o, (x, y, s), d["dm"]))
    for a, b, g in zip(runs[0], runs[1], (gx, gy, gs)):
        assert torch.equal(a, b)
        torch.testing.assert_close(a, g, rtol=1e-11, atol=1e-12)


def test_run_time_compiled_kernels_serve_a_float64_table():
    """A random table of genuine float64 values (no float32 numbers) under `config(jit=True)`: the
    kernels compiled for its structure take its values as coefficient classes."""
    from e3j_amd import ConvolutionParams
    rng = np.random.default_rng(31)
    N, E, X, Y, Z, S, K, nnz = 40, 600, 5, 6, 7, 4, 64, 50
    idx, val, mix = H.random_table(rng, nnz, X, Y, Z, S)
    val = np.asarray(val, dtype=np.float64) * (1.0 + 1e-9 * rng.standard_normal(len(val)))
    assert not np.array_equal(val, val.astype(np.float32).astype(np.float64))
    snd, rcv = H.random_graph(rng, N, E)
    x, y, s, dm = (a.astype(np.float64) * (1 + 1e-9) for a in H.random_operands(rng, N, E, X, Y, S, K, Z))
    coef = H.pack_table(idx, val, mix, val_dtype=np.float64)
    params = ConvolutionParams(num_out=Z, num_scalars=S)
    dev = lambda a: torch.as_tensor(a).cuda()  # noqa: E731
    with e3j_amd.config.use(jit=True):
        sig = _Table.get(coef, np.float64).signature((X, Y, Z, S), K, e3j_amd.Layout.TRAILING_CHANNELS)[0]
        assert sig >= 0
        out = e3j_amd.convolution(coef, dev(x), dev(y), dev(s), dev(snd), dev(rcv), params, layout="TRAILING_CHANNELS")
        grads = e3j_amd.convolution_bwd(coef, dev(x), dev(y), dev(s), dev(snd), dev(rcv), dev(dm), params,
                                        layout="TRAILING_CHANNELS")
    torch.cuda.synchronize()
    ref = O.convolution_unfused(idx, val, mix, x, y, s, snd, rcv, Z, dtype=np.float64)
    mag = O.convolution_unfused(idx, np.abs(val), mix, np.abs(x), np.abs(y), np.abs(s), snd, rcv, Z, dtype=np.float64)
    assert_parity64(out.cpu().numpy(), ref, mag, "out")
    refs = O.convolution_vjp(idx, val, mix, x, y, s, snd, rcv, dm, dtype=np.float64)
    mgs = O.convolution_vjp(idx, np.abs(val), mix, np.abs(x), np.abs(y), np.abs(s), snd, rcv, np.abs(dm), dtype=np.float64)
    for g, r, mg, what in zip(grads, refs, mgs, ("dx", "dy", "ds")):
        assert_parity64(g.cpu().numpy(), r, mg, what)


def test_float64_frames_of_the_ffi_targets_run_the_float64_kernels():
    """`convolution` and `convolution_bwd_receiver` frames with float64 buffers and the reference's
    attributes only: the handler reads the table back, finds the signature's structure and passes the
    table's values as coefficient classes.  Same bits as the operators (the same kernels), and the
    time of the unrolled kernels, not of the table-driven ones."""
    import ctypes as C
    from e3j_amd.graph import csr_row_ptr
    from tests.xla_frame import F64, S32, U8, FakeXla
    lib = _lib.load()
    w = _with_neighbour_count(W.config2(0.2), 12.5)
    m = w.module
    coef = m._packed_coef("float64")
    host, d = _f64(w)
    n = w.num_nodes
    ptr = csr_row_ptr(d["receiver"], n)
    xla = FakeXla(stream=torch.cuda.current_stream().cuda_stream)
    xla.allocate = lambda nbytes: torch.empty(nbytes, dtype=torch.uint8, device="cuda")

    def buf(t, dtype):
        xla._keep.append(t)
        return xla.buffer(dtype, t.data_ptr(), tuple(t.shape))

    attrs = lambda: {"num_nodes": (S32, C.c_int32(n)), "debug": (S32, C.c_int32(0))}  # noqa: E731
    coef_d = torch.from_numpy(coef.copy()).cuda()
    none = torch.zeros(0, dtype=torch.int32, device="cuda")
    out = torch.full_like(d["dm"], float("nan"))
    fwd = xla.frame([buf(coef_d, U8), buf(d["x"], F64), buf(d["y"], F64), buf(d["s"], F64), buf(d["sender"], S32),
                     buf(ptr, S32)], [buf(out, F64)], attrs())
    dx, dy, ds = (torch.full_like(d[f], float("nan")) for f in ("x", "y", "s"))
    bwd = xla.frame([buf(coef_d, U8), buf(d["x"], F64), buf(d["y"], F64), buf(d["s"], F64), buf(d["dm"], F64),
                     buf(d["sender"], S32), buf(ptr, S32), buf(none, S32)],
                    [buf(dx, F64), buf(dy, F64), buf(ds, F64)], attrs())
    assert lib.e3j_amd_xla_convolution(C.addressof(fwd)) is None, xla.errors
    assert lib.e3j_amd_xla_convolution_bwd_receiver(C.addressof(bwd)) is None, xla.errors
    torch.cuda.synchronize()
    want = e3j_amd.convolution(coef, d["x"], d["y"], d["s"], d["sender"], d["receiver"], m.params, m.graph_ordering,
                               layout=m.layout)
    assert torch.equal(out, want)
    idx, val, mix = w.table()
    refs = O.convolution_vjp(idx, np.asarray(val, dtype=np.float64), mix, host["x"], host["y"], host["s"],
                             host["sender"], host["receiver"], host["dm"], dtype=np.float64)
    for g, r, what in zip((dx, dy, ds), refs, ("dx", "dy", "ds")):
        np.testing.assert_allclose(g.cpu().numpy(), r, rtol=1e-11, atol=1e-12, err_msg=what)

    # the reference's own backward frame: the three transposed tables stacked, the adjacency grouped by
    # sender.  The handler finds the signature through the dx-transposed table, rebuilds receiver rows in
    # scratch of the runtime and runs the float64 unrolled kernels on them.
    from e3j_amd.coef import Coef4D
    c = Coef4D.unpack(coef, np.float64)
    stacked = np.stack([c.transpose(a).pack() for a in ((1, 0, 2, 3), (2, 0, 1, 3), (3, 0, 2, 1))])
    perm_t, recv_t, sptr = O.transpose_graph(host["sender"], host["receiver"], n)
    xla.allocate = lambda nbytes: torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    before = xla.allocations
    dx2, dy2, ds2 = (torch.full_like(d[f], float("nan")) for f in ("x", "y", "s"))
    stacked_d = torch.from_numpy(stacked.copy()).cuda()
    ref_bwd = xla.frame([buf(stacked_d, U8), buf(d["x"], F64), buf(d["y"], F64), buf(d["s"], F64), buf(d["dm"], F64),
                         buf(torch.as_tensor(recv_t.astype(np.int32)).cuda(), S32), buf(torch.as_tensor(sptr).cuda(), S32),
                         buf(torch.as_tensor(perm_t.astype(np.int32)).cuda(), S32)],
                        [buf(dx2, F64), buf(dy2, F64), buf(ds2, F64)], attrs())
    assert lib.e3j_amd_xla_convolution_bwd(C.addressof(ref_bwd)) is None, xla.errors
    torch.cuda.synchronize()
    assert xla.allocations == before + 1, "the unrolled kernels run on receiver rows rebuilt in the runtime's scratch"
    for g, g0, what in zip((dx2, dy2, ds2), (dx, dy, ds), ("dx", "dy", "ds")):
        np.testing.assert_allclose(g.cpu().numpy(), g0.cpu().numpy(), rtol=1e-11, atol=1e-12, err_msg=what)

    def timed(fn, reps=5):
        fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / reps

    t_frame = timed(lambda: lib.e3j_amd_xla_convolution(C.addressof(fwd)))
    print(f"float64 forward frame {t_frame:.3f} ms at {w.num_edges} edges, K={w.channels}")
    assert t_frame < 0.5, "the table-driven float64 kernels take milliseconds at this size"


@pytest.mark.parametrize("dtype", ["float64", "float16"])
def test_float64_and_float16_entry_points_replay_from_a_captured_graph(dtype):
    """Forward and backward of the float64 / float16 unrolled kernels recorded into a HIP graph (their
    zero fills are kernels; the coefficient classes of a float64 call are copied into the launch when
    it is recorded) and replayed on new operand values with eager work in between."""
    from e3j_amd.graph import csr_row_ptr, locality_order
    f64 = dtype == "float64"
    w = _with_neighbour_count(W.config2(0.04), 12.5)
    m = w.module
    np_dtype, tdtype, code = (np.float64, torch.float64, _lib.F64) if f64 else (np.float16, torch.float16, _lib.F16)
    table = _Table.get(m._packed_coef(dtype), np_dtype)
    dims = (int(w.x.shape[1]), int(w.y.shape[1]), m.params.num_out, int(w.s.shape[1]))
    sig, scale, flip = table.signature(dims, w.channels, m.layout)
    assert sig >= 0
    d = w.to("cuda")
    ptr = csr_row_ptr(d.receiver, w.num_nodes)
    order = locality_order(d.sender, ptr, w.num_nodes, 2)
    lib = _lib.load()
    p = _lib.ConvParams(num_nodes=w.num_nodes, num_edges=w.num_edges, num_coef=table.num_coef, num_x=dims[0],
                        num_y=dims[1], num_out=dims[2], num_scalars=dims[3], channels=w.channels,
                        layout=m.layout.value, val_dtype=code, coef_idx_bytes=table.idx_bytes, signature=sig,
                        coef_scale=1.0 if f64 else scale, debug=0, y_flip=flip, row_order=order.data_ptr())
    if f64:
        p.coef_classes = ctypes.cast(scale, ctypes.c_void_p).value
    coef = table.device(d.x.device)
    x, y, s, dm = ((0.25 * t).to(tdtype) for t in (d.x, d.y, d.s, d.dm))
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
        launch(side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        launch(side.cuda_stream)
    if f64:
        p.coef_classes = None   # the recorded launches hold their own copy of the classes
    for trial in range(3):
        gen = torch.Generator(device="cuda").manual_seed(200 + trial)
        for t in (x, y, s, dm):
            t.copy_(0.25 * torch.randn(t.shape, device="cuda", generator=gen))
        (x.float().sum() + s.float().sum()).item()
        graph.replay()
        torch.cuda.synchronize()
        replayed = [t.clone() for t in (out, dx, dy, ds)]
        if f64:
            p.coef_classes = ctypes.cast(scale, ctypes.c_void_p).value
        launch(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        if f64:
            p.coef_classes = None
        assert torch.equal(replayed[0], out) and torch.equal(replayed[3], ds), trial
        tol = 1e-12 if f64 else 2e-2
        for a, b in ((replayed[1], dx), (replayed[2], dy)):       # atomics: equal up to summation order
            assert float((a.double() - b.double()).abs().max()) <= tol * float(b.double().abs().max()) + 1e-30, trial
