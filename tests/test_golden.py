"""The committed golden fixtures (`tests/golden/*.npz`, written by `tests/golden/make_fixtures.py`):
the CPU checkers must reproduce them (guards the oracle, the table construction and the
fixtures against drift), and the HIP kernels must match them to the parity criterion.
Only `strip` holds values the reference itself holds (its closed-form known-answer case,
`lib/e3j_ops/tests/test_convolution.cpp:128-183`); `l3_k64`, `padding` and `unsorted_skewed` were
written by this repository's own oracle and are regression pins, as the test names say."""

import os

import numpy as np
import pytest

from oracle import c_oracle
from oracle import conv_oracle as O
from tests import helpers as H

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
CASES = ["strip", "l3_k64", "padding", "unsorted_skewed"]


def load(name):
    with np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False) as f:
        return {k: f[k] for k in f.files}


def magnitudes(g):
    if "mag_out" in g:
        return {k: g["mag_" + k] for k in ("out", "dx", "dy", "ds")}
    a = {k: np.abs(g[k]) for k in ("val", "x", "y", "s", "dm")}
    out = O.convolution_unfused(g["idx"], a["val"], g["mix"], a["x"], a["y"], a["s"], g["sender"],
                                g["receiver"], int(g["num_out"]), dtype=np.float64)
    dx, dy, ds = O.convolution_vjp(g["idx"], a["val"], g["mix"], a["x"], a["y"], a["s"], g["sender"],
                                   g["receiver"], a["dm"], dtype=np.float64)
    return dict(out=out, dx=dx, dy=dy, ds=ds)


@pytest.mark.parametrize("name", CASES)
def test_numpy_oracle_reproduces_its_own_regression_fixture(name):
    g = load(name)
    tol = dict(rtol=1e-6, atol=1e-6) if g["out"].dtype == np.float32 else dict(rtol=1e-12, atol=1e-12)
    out = O.convolution_unfused(g["idx"], g["val"], g["mix"], g["x"], g["y"], g["s"], g["sender"],
                                g["receiver"], int(g["num_out"]), dtype=np.float64)
    np.testing.assert_allclose(out, g["out"], **tol)
    grads = O.convolution_vjp(g["idx"], g["val"], g["mix"], g["x"], g["y"], g["s"], g["sender"],
                              g["receiver"], g["dm"], dtype=np.float64)
    for got, key in zip(grads, ("dx", "dy", "ds")):
        np.testing.assert_allclose(got, g[key], err_msg=key, **tol)


@pytest.mark.parametrize("name", ["strip", "l3_k64", "padding"])
def test_c_checker_matches_regression_fixture(name):
    """The float32 C restatement of the reference's CPU loops (receiver-sorted cases)."""
    g = load(name)
    mag = magnitudes(g)
    out = c_oracle.convolution(g["idx"], g["val"], g["mix"], g["x"], g["y"], g["s"], g["sender"],
                               g["receiver"], int(g["num_out"]))
    H.assert_parity(out, g["out"].astype(np.float64), mag["out"], f"{name} out")
    grads = c_oracle.convolution_vjp(g["idx"], g["val"], g["mix"], g["x"], g["y"], g["s"], g["sender"],
                                     g["receiver"], g["dm"])
    for got, key in zip(grads, ("dx", "dy", "ds")):
        H.assert_parity(got, g[key].astype(np.float64), mag[key], f"{name} {key}")


def test_strip_fixture_is_the_reference_held_closed_form():
    """out[r, 2t+a, c] = (a+1) * 12 * sum over the row's edges of s[e, t]
    (`lib/e3j_ops/tests/test_convolution.cpp:122-207`), exact in float32."""
    g = load("strip")
    ptr = O.receiver_ptr(g["receiver"], int(g["num_nodes"]))
    want = np.zeros_like(g["out"])
    for r in range(int(g["num_nodes"])):
        for t in range(int(g["num_scalars"])):
            total = g["s"][ptr[r]:ptr[r + 1], t, :].astype(np.float64).sum(axis=0)
            for a in range(2):
                want[r, 2 * t + a] = (a + 1) * 12.0 * total
    np.testing.assert_array_equal(g["out"], want)


@pytest.mark.gpu
@pytest.mark.parametrize("layout", ["TRAILING_CHANNELS", "LEADING_CHANNELS"])
@pytest.mark.parametrize("name", CASES)
def test_hip_kernels_match_regression_fixture(name, layout):
    import torch
    import e3j_amd
    g = load(name)
    mag = magnitudes(g)
    leading = layout == "LEADING_CHANNELS"
    params = e3j_amd.ConvolutionParams(num_out=int(g["num_out"]), num_scalars=int(g["num_scalars"]))
    coef = H.pack_table(g["idx"], g["val"], g["mix"])

    def dev(a):
        t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
        return t.transpose(1, 2).contiguous() if leading and t.dim() == 3 else t

    def host(t):
        return (t.transpose(1, 2) if leading and t.dim() == 3 else t).cpu().numpy()

    x, y, s, dm = dev(g["x"]), dev(g["y"]), dev(g["s"]), dev(g["dm"])
    snd, rcv = dev(g["sender"]), dev(g["receiver"])
    ordering = str(g["ordering"])
    out = e3j_amd.convolution(coef, x, y, s, snd, rcv, params, ordering, layout=layout)
    dx, dy, ds = e3j_amd.convolution_bwd(coef, x, y, s, snd, rcv, dm, params, ordering, layout=layout)
    H.assert_parity(host(out), g["out"].astype(np.float64), mag["out"], f"{name} out")
    for got, key in zip((dx, dy, ds), ("dx", "dy", "ds")):
        H.assert_parity(host(got), g[key].astype(np.float64), mag[key], f"{name} {key}")
    if name == "strip" and not leading:
        assert np.array_equal(host(out), g["out"].astype(np.float32))  # bit-exact, small integers
    if name == "padding":
        assert not host(out)[4].any() and not host(ds)[33:].any() and not host(dy)[33:].any()
