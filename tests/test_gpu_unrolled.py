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
    "cfg1": lambda: W.config1(0.2),
    "cfg2": lambda: W.config2(0.04),
    "cfg2_out3": lambda: W.config2(0.04, out_irreps="0e+1o+2e+3o"),
    "cfg3_k64": lambda: W.config3(0.006, channels=64),
    "cfg3": lambda: W.config3(0.006),
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
    sig, scale = _signature_of(w)
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
    sig, scale = _Table.get(packed, np.float32).signature(dims, w.channels, m.layout)
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
