"""The access-pattern probe of `bench.py --access-floor` touches the memory it claims to touch."""

import ctypes
import os

import pytest
import torch

from e3j_amd import build as lib_build

pytestmark = pytest.mark.gpu


def _probe():
    assert os.path.exists(lib_build.PROBE_LIB_PATH), "run `python -m e3j_amd.build` first"
    fn = ctypes.CDLL(lib_build.PROBE_LIB_PATH).e3j_amd_probe_access_pattern
    fn.restype = ctypes.c_int
    fn.argtypes = ([ctypes.c_uint] + [ctypes.c_int] * 4 + [ctypes.c_void_p] * 9 + [ctypes.c_int]
                   + [ctypes.c_void_p] * 2)
    return fn


def _operands(n=50, degree=7, seed=0):
    g = torch.Generator().manual_seed(seed)
    e = n * degree
    dev = "cuda:0"
    t = dict(
        x=torch.randn(n, 16, 128, generator=g), s=torch.randn(e, 23, 128, generator=g),
        dm=torch.randn(n, 99, 128, generator=g),
        sender=torch.randint(0, n, (e,), generator=g, dtype=torch.int32),
        row_ptr=torch.arange(0, e + 1, degree, dtype=torch.int32),
        order=torch.randperm(n, generator=g).to(torch.int32),
    )
    return n, e, {k: v.to(dev) for k, v in t.items()}


def _call(fn, mask, n, t, ds=None, dx=None, out=None):
    sink = torch.zeros(1, device="cuda:0")
    ptr = lambda a: a.data_ptr() if a is not None else None  # noqa: E731
    rc = fn(mask, 16, 23, 99, 128, ptr(t["x"]), ptr(t["s"]), ptr(t["dm"]), ptr(t["sender"]), ptr(t["row_ptr"]),
            ptr(t["order"]), ptr(ds), ptr(dx), ptr(out), n, sink.data_ptr(),
            int(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return rc


def test_streams_and_atomics_of_the_backward_pattern():
    fn = _probe()
    n, e, t = _operands()
    ds = torch.full_like(t["s"], float("nan"))
    dx = torch.zeros_like(t["x"])
    assert _call(fn, 1 | 2 | 4 | 8 | 32, n, t, ds=ds, dx=dx) == 0
    # ds row l of an edge = s row l + x[sender] row l mod 16; dx[sender] row j += x row j + s row j
    xs = t["x"][t["sender"].long()]
    want_ds = t["s"] + xs[:, torch.arange(23) % 16, :]
    assert torch.equal(ds, want_ds)
    want_dx = torch.zeros_like(dx).index_add_(0, t["sender"].long(), xs + t["s"][:, :16, :])
    assert torch.allclose(dx, want_dx, rtol=1e-5, atol=1e-5)


def test_output_rows_of_the_forward_pattern():
    fn = _probe()
    n, e, t = _operands(seed=1)
    out = torch.full_like(t["dm"], float("nan"))
    assert _call(fn, 1 | 2 | 16, n, t, out=out) == 0
    xs = t["x"][t["sender"].long()]
    per_edge = t["s"].sum(1) + xs.sum(1)                       # (E, 128)
    acc = per_edge.view(n, -1, 128).sum(1)                     # rows are 7 consecutive edges
    want = acc[:, None, :] + torch.arange(99, device=acc.device, dtype=acc.dtype)[None, :, None]
    assert torch.allclose(out, want, rtol=1e-4, atol=1e-3)


def test_unknown_mask_and_shape_are_refused():
    fn = _probe()
    n, e, t = _operands()
    assert _call(fn, 2, n, t) == -1
    sink = torch.zeros(1, device="cuda:0")
    assert fn(1, 9, 23, 99, 128, None, None, None, None, None, None, None, None, None, n, sink.data_ptr(), None) == -1
