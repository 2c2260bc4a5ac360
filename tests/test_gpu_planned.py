"""The two forms of the table-driven kernels through the C ABI (signature -1): over a plan of the
table that one workgroup builds on the device (float32 and float16 tables in which every output
coordinate uses one scalar, within the plan's size limits), and over LDS columns indexed by the table's
coordinates (everything else).  Which form a table gets is checked through
`e3j_amd_table_plan_status`; both forms are compared with the CPU oracle and with each other."""

import ctypes

import numpy as np
import pytest
import torch

from e3j_amd import _lib, workloads as W
from oracle import conv_oracle as O
from tests import helpers as H
from tests.test_gpu_generic import _dev, _params, check_all, run_abi

pytestmark = pytest.mark.gpu


@pytest.fixture
def plans_off():
    lib = _lib.load()
    lib.e3j_amd_set_table_plans(0)
    yield
    lib.e3j_amd_set_table_plans(1)


def _status(packed, X, Y, Z, S, K=8, cols_ji=0, val=_lib.F32):
    """(taken, cells, blocks, unused scalars) of the plan of a packed table."""
    coef_d = _dev(packed.view(np.uint8).reshape(-1))
    p = _params(4, 4, len(packed), X, Y, Z, S, K, 1, val, packed.dtype.itemsize)
    status = (ctypes.c_int32 * 4)()
    _lib.check(_lib.load().e3j_amd_table_plan_status(ctypes.byref(p), coef_d.data_ptr(), cols_ji, status,
                                                    torch.cuda.current_stream().cuda_stream))
    return tuple(int(v) for v in status)


def test_plan_of_the_l3_table():
    """cfg3's table: 353 entries on 311 (output, x) cells; the output coordinates sorted by the
    x coordinates of their paths leave 14 of the 28 blocks of 16 outputs x 4 x coordinates."""
    w = W.config3(0.002)
    idx, val, mix = w.table()
    packed = H.pack_table(idx, val, mix)
    i, j = np.asarray(idx)[:, 0], np.asarray(idx)[:, 1]
    cells = len(set(zip(i.tolist(), j.tolist())))
    taken, got_cells, blocks, unused = _status(packed, 16, 16, 99, 23)
    assert (taken, got_cells, unused) == (1, cells, 0) and cells == 311
    assert blocks == 14


def test_tables_the_plan_does_not_take():
    rng = np.random.default_rng(0)
    idx, val, mix = H.random_table(rng, 60, 5, 7, 6, 4)
    assert _status(H.pack_table(idx, val, mix), 5, 7, 6, 4)[0] == 1
    # an output coordinate with two scalars
    other_mix = (np.asarray(mix) + 1) % 4
    both = np.concatenate([H.pack_table(idx, val, mix, idx_dtype=np.uint8),
                           H.pack_table(idx[:5], val[:5], other_mix, idx_dtype=np.uint8)])
    assert _status(both, 5, 7, 6, 4)[0] == 0
    # sizes beyond the limits: x coordinates, y components, output coordinates, float64
    big = H.random_table(rng, 300, 17, 7, 6, 4)
    assert _status(H.pack_table(*big), 17, 7, 6, 4)[0] == 0
    big = H.random_table(rng, 300, 5, 65, 6, 4)
    assert _status(H.pack_table(*big), 5, 65, 6, 4)[0] == 0
    big = H.random_table(rng, 300, 5, 7, 129, 4)
    assert _status(H.pack_table(*big), 5, 7, 129, 4)[0] == 0
    assert _status(H.pack_table(idx, val, mix, val_dtype=np.float64), 5, 7, 6, 4, val=_lib.F64)[0] == 0
    # float16 tables are planned (values held as half, computed in float)
    assert _status(H.pack_table(idx, val.astype(np.float16), mix, val_dtype=np.float16), 5, 7, 6, 4,
                   val=_lib.F16)[0] == 1


def test_a_table_with_two_scalars_on_one_output_runs_the_column_kernels():
    """Not plannable; the result is still the sum of the two tables' results (the contraction is
    linear in the table)."""
    rng = np.random.default_rng(1)
    N, E, X, Y, Z, S, K = 9, 40, 5, 7, 6, 4, 24
    idx, val, mix = H.random_table(rng, 60, X, Y, Z, S)
    mix2 = (np.asarray(mix) + 1) % S
    sub = slice(0, 25)
    packed = np.concatenate([H.pack_table(idx, val, mix, idx_dtype=np.uint8),
                             H.pack_table(idx[sub], val[sub], mix2, idx_dtype=np.uint8)])
    snd, rcv = H.random_graph(rng, N, E)
    x, y, s, dm = H.random_operands(rng, N, E, X, Y, S, K, Z)
    lib = _lib.load()
    coef_d = _dev(packed.view(np.uint8).reshape(-1))
    xd, yd, sd, dmd = _dev(x), _dev(y), _dev(s), _dev(dm)
    other, ptr_d = _dev(snd.astype(np.int32)), _dev(O.receiver_ptr(rcv, N))
    p = _params(N, E, len(packed), X, Y, Z, S, K, 1, _lib.F32, packed.dtype.itemsize)
    out = torch.full((N, Z, K), float("nan"), device="cuda")
    dx, dy, ds = (torch.full_like(t, float("nan")) for t in (xd, yd, sd))
    stream = torch.cuda.current_stream().cuda_stream
    _lib.check(lib.e3j_amd_convolution_fwd(ctypes.byref(p), coef_d.data_ptr(), xd.data_ptr(), yd.data_ptr(),
                                           sd.data_ptr(), other.data_ptr(), ptr_d.data_ptr(), None,
                                           out.data_ptr(), stream))
    _lib.check(lib.e3j_amd_convolution_bwd_receiver(
        ctypes.byref(p), coef_d.data_ptr(), xd.data_ptr(), yd.data_ptr(), sd.data_ptr(), dmd.data_ptr(),
        other.data_ptr(), ptr_d.data_ptr(), None, dx.data_ptr(), dy.data_ptr(), ds.data_ptr(), stream))
    torch.cuda.synchronize()
    ref = mag = 0
    grads, mags = [0, 0, 0], [0, 0, 0]
    for ti, tv, tm in ((idx, val, mix), (idx[sub], val[sub], mix2)):
        r, m = H.forward_reference(ti, tv, tm, x, y, s, snd, rcv, Z)
        ref, mag = ref + r, mag + m
        g, gm = H.backward_reference(ti, tv, tm, x, y, s, snd, rcv, dm)
        grads = [a + b for a, b in zip(grads, g)]
        mags = [a + b for a, b in zip(mags, gm)]
    H.assert_parity(out.cpu().numpy(), ref, mag, "two scalars out")
    for got, r, m, name in zip((dx, dy, ds), grads, mags, ("dx", "dy", "ds")):
        H.assert_parity(got.cpu().numpy(), r, m, f"two scalars {name}")


# shapes: (X, Y, Z, S, nnz): one block, several blocks with a partial last one, the largest plan
SHAPES = [(3, 4, 5, 2, 30), (9, 16, 35, 11, 260), (16, 16, 99, 23, 353), (16, 64, 128, 64, 2048)]


@pytest.mark.parametrize("grouping", ["receiver", "sender"])
@pytest.mark.parametrize("channels", [1, 64, 70, 130])
@pytest.mark.parametrize("X, Y, Z, S, nnz", SHAPES)
def test_planned_kernels_match_oracle(X, Y, Z, S, nnz, channels, grouping):
    rng = np.random.default_rng(X * 1000 + channels)
    idx, val, mix = H.random_table(rng, nnz, X, Y, Z, S)
    assert _status(H.pack_table(idx, val, mix), X, Y, Z, S)[0] == 1
    N, E = 7, 30
    snd, rcv = H.random_graph(rng, N, E)
    x, y, s, dm = H.random_operands(rng, N, E, X, Y, S, channels, Z)
    res = run_abi(idx, val, mix, x, y, s, dm, snd, rcv, Z, grouping=grouping)
    check_all(idx, val, mix, x, y, s, dm, snd, rcv, Z, res, tag=f"{(X, Y, Z, S)} K={channels} {grouping}")


@pytest.mark.parametrize("seed", range(24))
def test_seeded_random_tables_and_graphs(seed):
    """Random sizes within the plan's limits, tables with holes (output coordinates and scalars no
    entry uses), graphs with empty rows, a hub, padding edges and unsorted edges behind a
    permutation, both layouts, both index widths, both groupings: the planned kernels against the
    CPU oracle."""
    rng = np.random.default_rng(7000 + seed)
    X, Y, Z = int(rng.integers(1, 17)), int(rng.integers(1, 65)), int(rng.integers(1, 129))
    S = int(rng.integers(1, min(Z, 64) + 1))
    nnz = int(rng.integers(max(X, Y, Z), min(2048, 6 * max(X, Y, Z)) + 1))
    K = int(rng.choice([1, 3, 32, 64, 65, 128, 200]))
    N, E = int(rng.integers(1, 30)), int(rng.integers(0, 400))
    idx, val, mix = H.random_table(rng, nnz, X, Y, Z, S)
    if rng.random() < 0.4 and len(val) > 4:
        keep = rng.random(len(val)) < 0.7
        keep[0] = True
        idx, val = idx[keep], val[keep]
    idx_dtype = np.int32 if rng.random() < 0.3 else None
    assert _status(H.pack_table(idx, val, mix, idx_dtype=idx_dtype), X, Y, Z, S)[0] == 1
    snd, rcv = H.random_graph(rng, N, E) if E else (np.zeros(0, np.int32), np.zeros(0, np.int32))
    grouping = "receiver" if rng.random() < 0.6 else "sender"
    if E and rng.random() < 0.5:                                   # a hub takes most of the edges
        rcv = rcv.copy()
        rcv[rng.random(E) < 0.6] = int(rng.integers(0, N))
        order = np.argsort(rcv, kind="stable")
        snd, rcv = snd[order], rcv[order]
    if E and grouping == "receiver" and rng.random() < 0.3:        # padding edges
        snd = snd.copy()
        snd[rng.random(E) < 0.2] = O.DUMMY_INDEX
    perm = None
    if E and grouping == "receiver" and rng.random() < 0.3:        # unsorted edges behind a permutation
        shuffle = rng.permutation(E)
        snd, rcv = snd[shuffle], rcv[shuffle]
        perm = np.argsort(rcv, kind="stable").astype(np.int32)
    x, y, s, dm = H.random_operands(rng, N, E, X, Y, S, K, Z)
    leading = bool(rng.random() < 0.3)
    args = [np.ascontiguousarray(a.swapaxes(1, 2)) if leading else a for a in (x, s, dm)]
    res = run_abi(idx, val, mix, args[0], y, args[1], args[2], snd, rcv, Z, leading=leading, grouping=grouping,
                  idx_dtype=idx_dtype, perm=perm)
    check_all(idx, val, mix, args[0], y, args[1], args[2], snd, rcv, Z, res, leading=leading,
              tag=f"seed {seed}: {(X, Y, Z, S)} nnz={len(val)} K={K} N={N} E={E} {grouping} leading={leading}")


def test_l3_table_with_padding_edges_and_permutation():
    """cfg3's table (7 blocks x 4 groups, 14 visited) on unsorted edges with padding among them."""
    w = W.config3(0.002)
    idx, val, mix = w.table()
    rng = np.random.default_rng(33)
    N, E, K = 12, 90, 128
    snd, rcv = H.random_graph(rng, N, E, sort_by=None)
    snd[rng.random(E) < 0.1] = O.DUMMY_INDEX
    x, y, s, dm = H.random_operands(rng, N, E, 16, 16, 23, K, 99)
    perm = np.argsort(rcv, kind="stable").astype(np.int32)
    out, dx, dy, ds = run_abi(idx, val, mix, x, y, s, dm, snd, rcv, 99, perm=perm)
    live = snd != O.DUMMY_INDEX
    assert not dy[~live].any() and not ds[~live].any()
    ref, mag = H.forward_reference(idx, val, mix, x, y[live], s[live], snd[live], rcv[live], 99)
    H.assert_parity(out, ref, mag, "out")
    refs, mags = H.backward_reference(idx, val, mix, x, y[live], s[live], snd[live], rcv[live], dm)
    H.assert_parity(dx, refs[0], mags[0], "dx")
    H.assert_parity(dy[live], refs[1], mags[1], "dy")
    H.assert_parity(ds[live], refs[2], mags[2], "ds")


def test_leading_layout_and_wide_indices():
    rng = np.random.default_rng(44)
    N, E, X, Y, Z, S, K, nnz = 9, 40, 9, 9, 20, 6, 40, 120
    idx, val, mix = H.random_table(rng, nnz, X, Y, Z, S)
    snd, rcv = H.random_graph(rng, N, E)
    x, y, s, dm = H.random_operands(rng, N, E, X, Y, S, K, Z)
    xl, sl, dml = (a.swapaxes(1, 2).copy() for a in (x, s, dm))
    res = run_abi(idx, val, mix, xl, y, sl, dml, snd, rcv, Z, leading=True, idx_dtype=np.int32)
    check_all(idx, val, mix, xl, y, sl, dml, snd, rcv, Z, res, leading=True, tag="leading int32")


def test_both_forms_agree_and_the_column_form_still_runs(plans_off):
    """With planning switched off the same calls run the LDS-column kernels: same results to rounding."""
    rng = np.random.default_rng(55)
    N, E, X, Y, Z, S, K, nnz = 9, 60, 9, 16, 35, 11, 96, 260
    idx, val, mix = H.random_table(rng, nnz, X, Y, Z, S)
    snd, rcv = H.random_graph(rng, N, E)
    x, y, s, dm = H.random_operands(rng, N, E, X, Y, S, K, Z)
    columns = run_abi(idx, val, mix, x, y, s, dm, snd, rcv, Z)
    check_all(idx, val, mix, x, y, s, dm, snd, rcv, Z, columns, tag="columns")
    _lib.load().e3j_amd_set_table_plans(1)
    planned = run_abi(idx, val, mix, x, y, s, dm, snd, rcv, Z)
    for a, b, name in zip(planned, columns, ("out", "dx", "dy", "ds")):
        np.testing.assert_allclose(a, b, rtol=2e-5, atol=2e-5, err_msg=name)


@pytest.mark.parametrize("grouping", ["receiver", "sender"])
def test_a_plan_built_once_serves_later_calls(grouping):
    """`table_plan_state`: with a plan built by the status call and declared ready, the calls launch
    the planned kernel alone, on the same plan contents as a call that builds it: the same bits (the
    sender-grouped backward has no atomics; for the receiver-grouped one dx is compared to rounding).
    Told not to plan, the calls run the column kernels; an unknown state and a ready state without a
    plan are refused before anything is launched."""
    rng = np.random.default_rng(91)
    N, E, X, Y, Z, S, K, nnz = 40, 700, 9, 16, 35, 11, 96, 260
    idx, val, mix = H.random_table(rng, nnz, X, Y, Z, S)
    snd, rcv = H.random_graph(rng, N, E)
    x, y, s, dm = H.random_operands(rng, N, E, X, Y, S, K, Z)
    built = run_abi(idx, val, mix, x, y, s, dm, snd, rcv, Z, grouping=grouping)
    ready = run_abi(idx, val, mix, x, y, s, dm, snd, rcv, Z, grouping=grouping, plan="ready")
    check_all(idx, val, mix, x, y, s, dm, snd, rcv, Z, ready, tag="ready plan")
    for a, b, name in zip(ready, built, ("out", "dx", "dy", "ds")):
        if name == "dx" and grouping == "receiver":
            np.testing.assert_allclose(a, b, rtol=2e-5, atol=2e-5, err_msg=name)
        else:
            assert np.array_equal(a, b), name
    columns = run_abi(idx, val, mix, x, y, s, dm, snd, rcv, Z, grouping=grouping, plan="none")
    check_all(idx, val, mix, x, y, s, dm, snd, rcv, Z, columns, tag="not planned")
    p = _params(N, E, nnz, X, Y, Z, S, K, 1, _lib.F32, 4)
    lib = _lib.load()
    some = _dev(np.zeros(4096, np.float32))
    for state, plan_ptr, message in ((7, None, "table_plan_state"), (_lib.PLAN_READY, None, "holds none")):
        p.table_plan_state, p.table_plan = state, plan_ptr
        with pytest.raises(_lib.E3jAmdError, match=message):
            _lib.check(lib.e3j_amd_convolution_fwd(ctypes.byref(p), some.data_ptr(), some.data_ptr(), some.data_ptr(),
                                                   some.data_ptr(), some.data_ptr(), some.data_ptr(), None,
                                                   some.data_ptr(), torch.cuda.current_stream().cuda_stream))


def test_the_operator_plans_a_table_once(monkeypatch):
    """The operators build the plan of a table on the first table-driven call and reuse it: later calls
    carry the ready state (one status call per table, sizes and device), and give the first call's bits."""
    from e3j_amd import ops
    from e3j_amd.ops import convolution
    w = W.config3(0.002)
    idx, val, mix = w.table()
    coef = H.pack_table(idx, np.asarray(val) * 1.25, mix)   # no unrolled kernel has these values
    rng = np.random.default_rng(5)
    N, E, K = 30, 400, 96
    snd, rcv = H.random_graph(rng, N, E)
    x, y, s, _ = H.random_operands(rng, N, E, 16, 16, 23, K, 99)
    calls, states = [], []
    lib = _lib.load()
    real_status, real_fwd = lib.e3j_amd_table_plan_status, lib.e3j_amd_convolution_fwd

    class Spy:
        def __getattr__(self, name):
            return getattr(lib, name)

        def e3j_amd_table_plan_status(self, *a):
            calls.append(1)
            return real_status(*a)

        def e3j_amd_convolution_fwd(self, p, *a):
            states.append(int(p._obj.table_plan_state))
            return real_fwd(p, *a)

    monkeypatch.setattr(ops._lib, "load", lambda: Spy())
    args = (_dev(x), _dev(y), _dev(s), _dev(snd.astype(np.int32)), _dev(rcv.astype(np.int32)), w.module.params)
    with pytest.warns(ops.TableDrivenKernelWarning):
        first = convolution(coef, *args)
    second = convolution(coef, *args)
    torch.cuda.synchronize()
    assert len(calls) == 1 and states == [_lib.PLAN_READY, _lib.PLAN_READY]
    assert torch.equal(first, second)
    ref, mag = H.forward_reference(idx, np.asarray(val) * 1.25, mix, x, y, s, snd, rcv, 99)
    H.assert_parity(first.cpu().numpy(), ref, mag, "operator on a cached plan")


@pytest.mark.parametrize("plans", [1, 0])
def test_float16_through_the_operator_in_both_forms(plans):
    """float16 operands with cfg3's table (7 blocks of outputs): the planned kernels hold the values
    as half and compute in float, the column kernels compute in half; both within half-precision
    rounding of the float64 checker on the rounded operands (forward, and the sender-grouped
    backward that float16 takes)."""
    from e3j_amd.ops import convolution
    w = W.config3(0.002)
    idx, val, mix = w.table()
    rng = np.random.default_rng(77)
    N, E, K = 12, 70, 128
    snd, rcv = H.random_graph(rng, N, E)
    x, y, s, dm = (a.astype(np.float16) for a in H.random_operands(rng, N, E, 16, 16, 23, K, 99))
    val16 = np.asarray(val).astype(np.float16)
    val16[0] *= np.float16(1.25)   # no longer the built-in table: the table-driven kernels serve it
    coef = H.pack_table(idx, val16, mix, val_dtype=np.float16)
    lib = _lib.load()
    lib.e3j_amd_set_table_plans(plans)
    try:
        xd, yd, sd = (_dev(a).requires_grad_(True) for a in (x, y, s))
        out = convolution(coef, xd, yd, sd, _dev(snd.astype(np.int32)), _dev(rcv.astype(np.int32)), w.module.params)
        grads = torch.autograd.grad(out, (xd, yd, sd), _dev(dm))
        torch.cuda.synchronize()
    finally:
        lib.e3j_amd_set_table_plans(1)
    assert out.dtype == torch.float16
    f64 = [a.astype(np.float64) for a in (x, y, s, dm)]
    ref, mag = H.forward_reference(idx, val16.astype(np.float64), mix, f64[0], f64[1], f64[2], snd, rcv, 99)
    refs, mags = H.backward_reference(idx, val16.astype(np.float64), mix, f64[0], f64[1], f64[2], snd, rcv, f64[3])
    eps = 2.0 ** -10
    for got, r, m, name in [(out, ref, mag, "out")] + list(zip(grads, refs, mags, ("dx", "dy", "ds"))):
        err = np.abs(got.detach().float().cpu().numpy().astype(np.float64) - r)
        assert np.all(err <= 6 * eps * m + 1e-3), f"{name} (plans={plans}): {err.max()} against magnitude {m.max()}"


def test_sender_grouped_backward_gives_the_same_bits_every_time():
    """The sender-grouped form owns dx and dy (no float atomics in global memory); the dy row of a
    wave is summed in LDS in a fixed order."""
    rng = np.random.default_rng(66)
    N, E, X, Y, Z, S, K, nnz = 64, 2000, 16, 16, 99, 23, 128, 353
    idx, val, mix = H.random_table(rng, nnz, X, Y, Z, S)
    snd, rcv = H.random_graph(rng, N, E)
    x, y, s, dm = H.random_operands(rng, N, E, X, Y, S, K, Z)
    base = run_abi(idx, val, mix, x, y, s, dm, snd, rcv, Z, grouping="sender")
    for _ in range(10):
        again = run_abi(idx, val, mix, x, y, s, dm, snd, rcv, Z, grouping="sender")
        for a, b in zip(base, again):
            assert np.array_equal(a, b)


def test_planned_kernels_at_120k_edges():
    """cfg3 at an eighth of its size (4 000 atoms, 120k edges, K = 128, l <= 3): the planned
    forward and backward against the column kernels' 9.1 ms and 24 ms on the same inputs."""
    import time

    w = W.config3(0.125).to("cuda")
    idx, val, mix = w.table()
    packed = H.pack_table(idx, val, mix)
    coef_d = _dev(packed.view(np.uint8).reshape(-1))
    lib = _lib.load()
    p = _params(w.num_nodes, w.num_edges, len(packed), 16, 16, 99, 23, 128, 1, _lib.F32, packed.dtype.itemsize,
                debug=0)
    from e3j_amd.graph import csr_row_ptr
    ptr = csr_row_ptr(w.receiver, w.num_nodes)
    out = torch.empty_like(w.dm)
    dx, dy, ds = torch.empty_like(w.x), torch.empty_like(w.y), torch.empty_like(w.s)
    stream = torch.cuda.current_stream().cuda_stream

    def fwd():
        _lib.check(lib.e3j_amd_convolution_fwd(ctypes.byref(p), coef_d.data_ptr(), w.x.data_ptr(), w.y.data_ptr(),
                                               w.s.data_ptr(), w.sender.data_ptr(), ptr.data_ptr(), None,
                                               out.data_ptr(), stream))

    def bwd():
        _lib.check(lib.e3j_amd_convolution_bwd_receiver(
            ctypes.byref(p), coef_d.data_ptr(), w.x.data_ptr(), w.y.data_ptr(), w.s.data_ptr(), w.dm.data_ptr(),
            w.sender.data_ptr(), ptr.data_ptr(), None, dx.data_ptr(), dy.data_ptr(), ds.data_ptr(), stream))

    times = {}
    for name, fn in (("fwd", fwd), ("bwd", bwd)):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        times[name] = (time.perf_counter() - t0) / 5 * 1e3
    print("planned kernels, ms:", times)
    assert times["fwd"] < 4.5 and times["bwd"] < 12.0, times
    # and they agree with the unrolled kernels of the same table on the same inputs
    from e3j_amd.ops import convolution
    ref = convolution(w.module._packed_coef("float32"), w.x, w.y, w.s, w.sender, w.receiver, w.module.params)
    torch.testing.assert_close(out, ref, rtol=2e-4, atol=2e-4)


def test_a_call_recorded_into_a_graph_allocates_nothing_and_replays():
    """On a stream that is being captured the table-driven call takes no plan memory from the pool:
    it records the LDS-column kernels, and the replays agree with eager calls (which plan the table)
    to rounding, with other work and new operand values in between."""
    w = W.config3(0.002)
    idx, val, mix = w.table()
    rng = np.random.default_rng(88)
    N, E, K = 40, 600, 64
    snd, rcv = H.random_graph(rng, N, E)
    packed = H.pack_table(idx, val, mix)
    coef_d = _dev(packed.view(np.uint8).reshape(-1))
    x, y, s, dm = (_dev(a) for a in H.random_operands(rng, N, E, 16, 16, 23, K, 99))
    other, ptr_d = _dev(snd.astype(np.int32)), _dev(O.receiver_ptr(rcv, N))
    p = _params(N, E, len(packed), 16, 16, 99, 23, K, 1, _lib.F32, packed.dtype.itemsize, debug=0)
    out = torch.empty((N, 99, K), device="cuda")
    dx, dy, ds = torch.empty_like(x), torch.empty_like(y), torch.empty_like(s)
    lib = _lib.load()

    def launch(stream):
        _lib.check(lib.e3j_amd_convolution_fwd(ctypes.byref(p), coef_d.data_ptr(), x.data_ptr(), y.data_ptr(),
                                               s.data_ptr(), other.data_ptr(), ptr_d.data_ptr(), None,
                                               out.data_ptr(), stream))
        _lib.check(lib.e3j_amd_convolution_bwd_receiver(
            ctypes.byref(p), coef_d.data_ptr(), x.data_ptr(), y.data_ptr(), s.data_ptr(), dm.data_ptr(),
            other.data_ptr(), ptr_d.data_ptr(), None, dx.data_ptr(), dy.data_ptr(), ds.data_ptr(), stream))

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
        gen = torch.Generator(device="cuda").manual_seed(200 + trial)
        for t in (x, y, s, dm):
            t.copy_(torch.randn(t.shape, device="cuda", generator=gen))
        (x.sum() + s.sum()).item()                    # unrelated eager work and a synchronisation
        graph.replay()
        torch.cuda.synchronize()
        replayed = [t.clone() for t in (out, dx, dy, ds)]
        launch(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        for a, b, name in zip(replayed, (out, dx, dy, ds), ("out", "dx", "dy", "ds")):
            assert float((a - b).abs().max()) <= 5e-5 * float(b.abs().max()), (trial, name)


def test_plan_memory_of_the_caller_serves_eager_calls_and_graph_capture():
    """With `table_plan` memory from the caller the call takes nothing from the stream's pool and a
    captured call records the planned kernels: the forward of every replay has the bits of an eager
    planned call (the LDS-column kernels round differently), the backward agrees to the order of its
    dx atomics; the size comes from `e3j_amd_table_plan_bytes`, which answers 0 for what the plan
    does not take."""
    w = W.config3(0.002)
    idx, val, mix = w.table()
    rng = np.random.default_rng(91)
    N, E, K = 40, 600, 64
    snd, rcv = H.random_graph(rng, N, E)
    packed = H.pack_table(idx, val, mix)
    coef_d = _dev(packed.view(np.uint8).reshape(-1))
    x, y, s, dm = (_dev(a) for a in H.random_operands(rng, N, E, 16, 16, 23, K, 99))
    other, ptr_d = _dev(snd.astype(np.int32)), _dev(O.receiver_ptr(rcv, N))
    lib = _lib.load()
    p = _params(N, E, len(packed), 16, 16, 99, 23, K, 1, _lib.F32, packed.dtype.itemsize, debug=0)
    nbytes = int(lib.e3j_amd_table_plan_bytes(ctypes.byref(p)))
    assert 0 < nbytes < (1 << 20) and nbytes % 4 == 0
    wide = _params(N, E, len(packed), 16, 16, 99, 23, K, 1, _lib.F64, packed.dtype.itemsize, debug=0)
    assert int(lib.e3j_amd_table_plan_bytes(ctypes.byref(wide))) == 0          # float64: LDS columns
    big = _params(N, E, len(packed), 17, 16, 99, 23, K, 1, _lib.F32, packed.dtype.itemsize, debug=0)
    assert int(lib.e3j_amd_table_plan_bytes(ctypes.byref(big))) == 0           # 17 x coordinates
    plan = torch.full((nbytes // 4,), -1, dtype=torch.int32, device="cuda")
    out = torch.empty((N, 99, K), device="cuda")
    dx, dy, ds = torch.empty_like(x), torch.empty_like(y), torch.empty_like(s)

    def launch(params, stream):
        _lib.check(lib.e3j_amd_convolution_fwd(ctypes.byref(params), coef_d.data_ptr(), x.data_ptr(), y.data_ptr(),
                                               s.data_ptr(), other.data_ptr(), ptr_d.data_ptr(), None,
                                               out.data_ptr(), stream))
        _lib.check(lib.e3j_amd_convolution_bwd_receiver(
            ctypes.byref(params), coef_d.data_ptr(), x.data_ptr(), y.data_ptr(), s.data_ptr(), dm.data_ptr(),
            other.data_ptr(), ptr_d.data_ptr(), None, dx.data_ptr(), dy.data_ptr(), ds.data_ptr(), stream))

    def results():
        torch.cuda.synchronize()
        return [t.clone() for t in (out, dx, dy, ds)]

    current = torch.cuda.current_stream().cuda_stream
    launch(p, current)
    pooled = results()                               # plan memory from the stream's pool
    lib.e3j_amd_set_table_plans(0)
    try:
        launch(p, current)
        columns = results()
    finally:
        lib.e3j_amd_set_table_plans(1)
    assert not torch.equal(pooled[0], columns[0]), "the two forms round differently on this problem"
    p.table_plan = plan.data_ptr()
    launch(p, current)
    own = results()
    assert int(plan[0].item()) == 1                  # the plan was written to the caller's memory
    assert torch.equal(own[0], pooled[0]) and torch.equal(own[3], pooled[3])
    p.table_plan = plan.data_ptr() + 2
    with pytest.raises(_lib.E3jAmdError, match="aligned"):
        launch(p, current)
    p.table_plan = plan.data_ptr()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        launch(p, side.cuda_stream)
    for trial in range(3):
        gen = torch.Generator(device="cuda").manual_seed(300 + trial)
        for t in (x, y, s, dm):
            t.copy_(torch.randn(t.shape, device="cuda", generator=gen))
        (x.sum() + s.sum()).item()                   # unrelated eager work and a synchronisation
        graph.replay()
        replayed = results()
        launch(p, torch.cuda.current_stream().cuda_stream)
        eager = results()
        assert torch.equal(replayed[0], eager[0]), trial         # forward: the planned kernels' bits
        assert torch.equal(replayed[3], eager[3]), trial         # ds belongs to the edge alone
        for a, b, name in zip(replayed[1:3], eager[1:3], ("dx", "dy")):
            assert float((a - b).abs().max()) <= 5e-5 * float(b.abs().max()), (trial, name)
