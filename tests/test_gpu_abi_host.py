"""The C ABI from a host program in plain C (no Python or torch in the process that calls it):
`tests/abi_host/conv_host.c` reads a problem from a file, runs the graph preparation, the forward
and the receiver-grouped backward through `include/e3j_amd.h` and writes the results, which are
compared with the CPU checker."""

import os
import subprocess

import numpy as np
import pytest

import e3j_amd
from e3j_amd import workloads as W
from tests import abi_host
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _run_host(tmp_path, coef, x, y, s, dm, sender, receiver, dims, layout):
    binary = abi_host.binary()
    N, E, K, X, Y, Z, S = dims
    problem, result = tmp_path / "problem.bin", tmp_path / "result.bin"
    with open(problem, "wb") as f:
        np.asarray([N, E, K, X, Y, Z, S, coef.shape[0], coef.dtype.itemsize, layout], dtype=np.int32).tofile(f)
        for a in (coef, x, y, s, dm, sender, receiver):
            np.ascontiguousarray(a).tofile(f)
    done = subprocess.run([binary, str(problem), str(result)], capture_output=True, text=True, timeout=100)
    assert done.returncode == 0, done.stderr
    flat = np.fromfile(result, dtype=np.float32)
    sizes = [N * Z * K, N * X * K, E * Y, E * S * K]
    assert flat.size == sum(sizes)
    out, dx, dy, ds = np.split(flat, np.cumsum(sizes)[:-1])
    return done.stdout, out, dx, dy.reshape(E, Y), ds


@pytest.mark.parametrize("layout", ["TRAILING_CHANNELS", "LEADING_CHANNELS"])
def test_compiled_table_from_a_c_host(tmp_path, layout):
    """l <= 3 table at 64 channels: the lookup finds the compiled kernels."""
    w = W.config3(0.006, channels=64).with_layout(layout)
    a = w.numpy()   # node and edge arrays as (rows, dim, channels)
    m = w.module
    lead = w.leading
    put = (lambda t: np.ascontiguousarray(t.transpose(0, 2, 1))) if lead else (lambda t: t)
    N, X, K = a["x"].shape
    E, Y = a["y"].shape
    S, Z = a["s"].shape[1], a["dm"].shape[1]
    text, out, dx, dy, ds = _run_host(tmp_path, m._packed_coef("float32"), put(a["x"]), a["y"], put(a["s"]),
                                      put(a["dm"]), a["sender"], a["receiver"], (N, E, K, X, Y, Z, S),
                                      m.layout.value)
    assert "signature -1" not in text and "K=64" in text, text
    back = (lambda t, d: t.reshape(-1, K, d).transpose(0, 2, 1)) if lead else (lambda t, d: t.reshape(-1, d, K))
    idx, val, mix = w.table()
    ref, mag = H.forward_reference(idx, val, mix, a["x"], a["y"], a["s"], a["sender"], a["receiver"], Z)
    H.assert_parity(back(out, Z), ref, mag, "out")
    refs, mags = H.backward_reference(idx, val, mix, a["x"], a["y"], a["s"], a["sender"], a["receiver"], a["dm"])
    for got, r, g, name in zip((back(dx, X), dy, back(ds, S)), refs, mags, ("dx", "dy", "ds")):
        H.assert_parity(got, r, g, name)


def test_unknown_table_from_a_c_host(tmp_path):
    """A random table: no compiled kernel, the table-driven kernels serve it."""
    rng = np.random.default_rng(11)
    N, E, X, Y, Z, S, K = 30, 400, 5, 6, 9, 4, 48
    idx, val, mix = H.random_table(rng, 70, X, Y, Z, S)
    snd, rcv = H.random_graph(rng, N, E)
    x, y, s, dm = H.random_operands(rng, N, E, X, Y, S, K, Z)
    text, out, dx, dy, ds = _run_host(tmp_path, H.pack_table(idx, val, mix), x, y, s, dm, snd, rcv,
                                      (N, E, K, X, Y, Z, S), e3j_amd.Layout.TRAILING_CHANNELS.value)
    assert "signature -1" in text
    ref, mag = H.forward_reference(idx, val, mix, x, y, s, snd, rcv, Z)
    H.assert_parity(out.reshape(N, Z, K), ref, mag, "out")
    refs, mags = H.backward_reference(idx, val, mix, x, y, s, snd, rcv, dm)
    for got, r, g, name in zip((dx.reshape(N, X, K), dy, ds.reshape(E, S, K)), refs, mags, ("dx", "dy", "ds")):
        H.assert_parity(got, r, g, name)
