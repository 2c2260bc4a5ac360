"""float16 operands on the compile-time-unrolled kernels (trailing layout): values held as half,
the float kernels' arithmetic, dx by packed half atomics.  Checked against the float64 oracle on
the half-rounded operands and table within half-precision rounding of the terms, the bound the
reference's half-precision kernel is held to by the table-driven tests, and against the
table-driven kernels."""

import ctypes

import numpy as np
import pytest
import torch

import e3j_amd
from e3j_amd import _lib, workloads as W
from e3j_amd.ops import _Table
from oracle import conv_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu

EPS16 = 2.0 ** -10


def assert_parity16(got, ref, mag, what, sums=1.0):
    """Within 6 half-precision roundings of the sum of the absolute values of the terms (`sums`
    times that for results added up in half precision by atomics), plus 1e-3."""
    got = np.asarray(got.detach().float().cpu().numpy(), dtype=np.float64)
    assert got.shape == ref.shape, f"{what}: shape {got.shape} != {ref.shape}"
    assert np.isfinite(got).all(), f"{what}: non-finite values"
    err = np.abs(got - ref)
    bound = 6 * sums * EPS16 * mag + 1e-3
    assert (err <= bound).all(), (f"{what}: {int((err > bound).sum())} of {err.size} elements off; worst {err.max():.3e} "
                                  f"against {bound[np.unravel_index(err.argmax(), err.shape)]:.3e}")


CASES = {
    "cfg3_k64": lambda: W.config3(0.006, channels=64),
    "cfg3": lambda: W.config3(0.004),
    "cfg3_k256": lambda: W.config3(0.002, channels=256),
    "cfg2": lambda: W.config2(0.04),                      # y up to l = 3 on x up to l = 2
    "scalars_k64": lambda: W.make_workload("scalars", 200, "0e", 3, "0e+1o+2e+3o", 64, (51, 52, 53, 54)),
}


def _half(w, scale=0.25):
    """Operands of a workload rounded to half (scaled down so that sums of 30 messages stay well inside
    the half range), host arrays in float64 of the rounded values and device tensors in half."""
    a = w.numpy()
    host = {f: (a[f] * scale).astype(np.float16) for f in ("x", "y", "s", "dm")}
    dev = {f: torch.as_tensor(v).cuda() for f, v in host.items()}
    dev["sender"], dev["receiver"] = (torch.as_tensor(a[f]).cuda() for f in ("sender", "receiver"))
    f64 = {f: v.astype(np.float64) for f, v in host.items()}
    f64["sender"], f64["receiver"] = a["sender"], a["receiver"]
    return f64, dev


@pytest.mark.parametrize("name", list(CASES))
def test_float16_unrolled_kernels_match_the_oracle(name):
    w = CASES[name]()
    m = w.module
    coef = m._packed_coef("float16")
    dims = (int(w.x.shape[1]), int(w.y.shape[1]), m.params.num_out, int(w.s.shape[1]))
    sig, scale, flip = _Table.get(coef, np.float16).signature(dims, w.channels, m.layout)
    assert sig >= 0 and flip == 0, "the half-rounded table must resolve to the built-in signature"
    host, d = _half(w)
    out = e3j_amd.convolution(coef, d["x"], d["y"], d["s"], d["sender"], d["receiver"], m.params, m.graph_ordering,
                              layout=m.layout)
    dx, dy, ds = e3j_amd.convolution_bwd(coef, d["x"], d["y"], d["s"], d["sender"], d["receiver"], d["dm"],
                                         m.params, m.graph_ordering, layout=m.layout)
    torch.cuda.synchronize()
    assert out.dtype == torch.float16 and dx.dtype == torch.float16
    idx, val, mix = w.table()
    val = np.asarray(val).astype(np.float16).astype(np.float64)     # the table as the operand holds it
    args = (host["x"], host["y"], host["s"], host["sender"], host["receiver"])
    mags = tuple(np.abs(t) for t in args[:3]) + args[3:]
    ref = O.convolution_unfused(idx, val, mix, *args, m.params.num_out, dtype=np.float64)
    mag = O.convolution_unfused(idx, np.abs(val), mix, *mags, m.params.num_out, dtype=np.float64)
    assert_parity16(out, ref, mag, f"{name} out")
    refs = O.convolution_vjp(idx, val, mix, *args, host["dm"], dtype=np.float64)
    mgs = O.convolution_vjp(idx, np.abs(val), mix, *mags, np.abs(host["dm"]), dtype=np.float64)
    # dx and the shared dy rows are summed in half by the atomics, one rounding per edge or wave
    for g, r, mg, what, sums in zip((dx, dy, ds), refs, mgs, ("dx", "dy", "ds"), (4.0, 2.0, 1.0)):
        assert_parity16(g, r, mg, f"{name} {what}", sums)


def test_float16_through_the_c_abi_against_the_table_driven_kernels():
    """Unsorted edges through `edge_perm`, padding edges, a receiver without edges, and a table of
    9 y components (dy rows of an odd length: their shared sums go through compare-and-swap): the
    unrolled float16 kernels against the oracle and against the table-driven kernels of the same
    call with `signature = -1`."""
    from e3j_amd.convolution import Convolution
    from tests.test_gpu_generic import _dev, _params
    lib = _lib.load()
    m = Convolution(("0e+1o", "0e+1o+2e"), "0e+1o+2e", graph_ordering="RECEIVER", avg_num_neighbors=4.0)
    c = m.coef
    idx4 = np.asarray(c.idx, dtype=np.int64)
    val16 = np.asarray(c.val).astype(np.float16)
    idx, mix = idx4[:, :3], m._mix.mix_indices
    X, Y, Z, S, K, N, E = m.source[0].dim, m.source[1].dim, m.target.dim, m.params.num_scalars, 128, 40, 900
    assert Y == 9
    rng = np.random.default_rng(19)
    snd = rng.integers(0, N, E)
    rcv = rng.integers(0, N - 1, E)
    snd[rng.random(E) < 0.05] = N
    x, y, s, dm = ((0.5 * a).astype(np.float16) for a in H.random_operands(rng, N, E, X, Y, S, K, Z))
    perm = np.argsort(rcv, kind="stable")
    packed = H.pack_table(idx, val16, mix, val_dtype=np.float16)
    scale, flip = ctypes.c_float(), ctypes.c_uint32()
    sig = lib.e3j_amd_find_signature(packed.ctypes.data, 1, _lib.F16, len(val16), X, Y, Z, S, K, 1,
                                     ctypes.byref(scale), ctypes.byref(flip))
    assert sig >= 0 and abs(scale.value - 0.25) < 1e-3
    coef_d = _dev(packed.view(np.uint8).reshape(-1))
    xd, yd, sd, dmd = _dev(x), _dev(y), _dev(s), _dev(dm)
    other, perm_d, ptr = _dev(snd[perm].astype(np.int32)), _dev(perm.astype(np.int32)), _dev(O.receiver_ptr(rcv[perm], N))
    stream = torch.cuda.current_stream().cuda_stream

    def run(signature):
        p = _params(N, E, len(val16), X, Y, Z, S, K, 1, _lib.F16, 1)
        p.signature, p.coef_scale = signature, scale.value if signature >= 0 else 1.0
        out = torch.full((N, Z, K), float("nan"), dtype=torch.float16, device="cuda")
        dx, dy, ds = (torch.full_like(t, float("nan")) for t in (xd, yd, sd))
        _lib.check(lib.e3j_amd_convolution_fwd(ctypes.byref(p), coef_d.data_ptr(), xd.data_ptr(), yd.data_ptr(),
                                               sd.data_ptr(), other.data_ptr(), ptr.data_ptr(), perm_d.data_ptr(),
                                               out.data_ptr(), stream))
        if signature >= 0:
            _lib.check(lib.e3j_amd_convolution_bwd_receiver(
                ctypes.byref(p), coef_d.data_ptr(), xd.data_ptr(), yd.data_ptr(), sd.data_ptr(), dmd.data_ptr(),
                other.data_ptr(), ptr.data_ptr(), perm_d.data_ptr(), dx.data_ptr(), dy.data_ptr(), ds.data_ptr(), stream))
        torch.cuda.synchronize()
        return out, dx, dy, ds

    out, dx, dy, ds = run(sig)
    f64 = [a.astype(np.float64) for a in (x, y, s, dm)]
    v64 = val16.astype(np.float64)
    ref = O.convolution_unfused(idx, v64, mix, f64[0], f64[1], f64[2], snd, rcv, Z, dtype=np.float64)
    mag = O.convolution_unfused(idx, np.abs(v64), mix, *(np.abs(a) for a in f64[:3]), snd, rcv, Z, dtype=np.float64)
    assert_parity16(out, ref, mag, "out")
    assert not out[N - 1].any()
    refs = O.convolution_vjp(idx, v64, mix, f64[0], f64[1], f64[2], snd, rcv, f64[3], dtype=np.float64)
    mgs = O.convolution_vjp(idx, np.abs(v64), mix, *(np.abs(a) for a in f64[:3]), snd, rcv, np.abs(f64[3]), dtype=np.float64)
    for g, r, mg, what, sums in zip((dx, dy, ds), refs, mgs, ("dx", "dy", "ds"), (4.0, 2.0, 1.0)):
        assert_parity16(g, r, mg, what, sums)
    live = torch.as_tensor(snd < N).cuda()
    assert not dy[~live].any() and not ds[~live].any()
    # the table-driven kernels (half-precision arithmetic) on the same operands
    out_td = run(-1)[0]
    assert_parity16(out_td, ref, mag, "table-driven out")
    assert float((out.float() - out_td.float()).abs().max()) <= 12 * EPS16 * float(mag.max()) + 2e-3


def test_float16_module_through_autograd_and_the_deterministic_mode():
    """The module in half precision through autograd on the unrolled kernels; `config(deterministic=True)`
    keeps the table-driven rows that own their dx (no atomics): the same bits in two runs."""
    from e3j_amd.options import config
    w = W.config2(0.03)
    m = w.module
    host, d = _half(w)
    x, y, s = (d[f].clone().requires_grad_(True) for f in ("x", "y", "s"))
    out = m(x, y, s, d["sender"], d["receiver"])
    assert out.dtype == torch.float16
    gx, gy, gs = torch.autograd.grad(out, (x, y, s), d["dm"])
    idx, val, mix = w.table()
    val = np.asarray(val).astype(np.float16).astype(np.float64)
    args = (host["x"], host["y"], host["s"], host["sender"], host["receiver"])
    mags = tuple(np.abs(t) for t in args[:3]) + args[3:]
    refs = O.convolution_vjp(idx, val, mix, *args, host["dm"], dtype=np.float64)
    mgs = O.convolution_vjp(idx, np.abs(val), mix, *mags, np.abs(host["dm"]), dtype=np.float64)
    for g, r, mg, what, sums in zip((gx, gy, gs), refs, mgs, ("dx", "dy", "ds"), (4.0, 2.0, 1.0)):
        assert_parity16(g, r, mg, what, sums)
    with config.use(deterministic=True):
        runs = []
        for _ in range(2):
            o = m(x, y, s, d["sender"], d["receiver"])
            runs.append(torch.autograd.grad(o, (x, y, s), d["dm"]))
    for a, b, r, mg, what in zip(runs[0], runs[1], refs, mgs, ("dx", "dy", "ds")):
        assert torch.equal(a, b)
        assert_parity16(a, r, mg, f"deterministic {what}", 4.0)


def test_float16_frames_of_the_ffi_targets_run_the_float16_kernels():
    """`convolution` and `convolution_bwd_receiver` frames with float16 buffers and the reference's
    attributes only: the handler finds the half-valued table among the signatures and runs the
    float16 unrolled kernels, the operators' bits."""
    import ctypes as C
    from e3j_amd.graph import csr_row_ptr
    from tests.xla_frame import F16, S32, U8, FakeXla
    lib = _lib.load()
    w = W.config2(0.2)
    m = w.module
    coef = m._packed_coef("float16")
    host, d = _half(w)
    n = w.num_nodes
    ptr = csr_row_ptr(d["receiver"], n)
    xla = FakeXla(stream=torch.cuda.current_stream().cuda_stream)

    def buf(t, dtype):
        xla._keep.append(t)
        return xla.buffer(dtype, t.data_ptr(), tuple(t.shape))

    attrs = lambda: {"num_nodes": (S32, C.c_int32(n)), "debug": (S32, C.c_int32(0))}  # noqa: E731
    coef_d = torch.from_numpy(coef.copy()).cuda()
    none = torch.zeros(0, dtype=torch.int32, device="cuda")
    out = torch.full_like(d["dm"], float("nan"))
    fwd = xla.frame([buf(coef_d, U8), buf(d["x"], F16), buf(d["y"], F16), buf(d["s"], F16), buf(d["sender"], S32),
                     buf(ptr, S32)], [buf(out, F16)], attrs())
    dx, dy, ds = (torch.full_like(d[f], float("nan")) for f in ("x", "y", "s"))
    bwd = xla.frame([buf(coef_d, U8), buf(d["x"], F16), buf(d["y"], F16), buf(d["s"], F16), buf(d["dm"], F16),
                     buf(d["sender"], S32), buf(ptr, S32), buf(none, S32)],
                    [buf(dx, F16), buf(dy, F16), buf(ds, F16)], attrs())
    assert lib.e3j_amd_xla_convolution(C.addressof(fwd)) is None, xla.errors
    assert lib.e3j_amd_xla_convolution_bwd_receiver(C.addressof(bwd)) is None, xla.errors
    torch.cuda.synchronize()
    want = e3j_amd.convolution(coef, d["x"], d["y"], d["s"], d["sender"], d["receiver"], m.params, m.graph_ordering,
                               layout=m.layout)
    assert torch.equal(out, want)
    idx, val, mix = w.table()
    val = np.asarray(val).astype(np.float16).astype(np.float64)
    args = (host["x"], host["y"], host["s"], host["sender"], host["receiver"])
    mags = tuple(np.abs(t) for t in args[:3]) + args[3:]
    refs = O.convolution_vjp(idx, val, mix, *args, host["dm"], dtype=np.float64)
    mgs = O.convolution_vjp(idx, np.abs(val), mix, *mags, np.abs(host["dm"]), dtype=np.float64)
    for g, r, mg, what, sums in zip((dx, dy, ds), refs, mgs, ("dx", "dy", "ds"), (4.0, 2.0, 1.0)):
        assert_parity16(g, r, mg, what, sums)
    # the reference's own backward frame: the three transposed tables stacked, the adjacency grouped by
    # sender.  The handler finds the signature through the dx-transposed table, rebuilds receiver rows in
    # scratch of the runtime and runs the float16 unrolled kernels on them.
    from e3j_amd.coef import Coef4D
    c = Coef4D.unpack(coef, np.float16)
    stacked = np.stack([c.transpose(a).pack() for a in ((1, 0, 2, 3), (2, 0, 1, 3), (3, 0, 2, 1))])
    perm_t, recv_t, sptr = O.transpose_graph(host["sender"], host["receiver"], n)
    xla.allocate = lambda nbytes: torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    before = xla.allocations
    dx2, dy2, ds2 = (torch.full_like(d[f], float("nan")) for f in ("x", "y", "s"))
    stacked_d = torch.from_numpy(stacked.copy()).cuda()
    ref_bwd = xla.frame([buf(stacked_d, U8), buf(d["x"], F16), buf(d["y"], F16), buf(d["s"], F16), buf(d["dm"], F16),
                         buf(torch.as_tensor(recv_t.astype(np.int32)).cuda(), S32), buf(torch.as_tensor(sptr).cuda(), S32),
                         buf(torch.as_tensor(perm_t.astype(np.int32)).cuda(), S32)],
                        [buf(dx2, F16), buf(dy2, F16), buf(ds2, F16)], attrs())
    assert lib.e3j_amd_xla_convolution_bwd(C.addressof(ref_bwd)) is None, xla.errors
    torch.cuda.synchronize()
    assert xla.allocations == before + 1, "the unrolled kernels run on receiver rows rebuilt in the runtime's scratch"
    for g, r, mg, what, sums in zip((dx2, dy2, ds2), refs, mgs, ("dx", "dy", "ds"), (4.0, 2.0, 1.0)):
        assert_parity16(g, r, mg, "reference frame " + what, sums)
