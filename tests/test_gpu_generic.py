"""Parity of the table-driven HIP kernels against the CPU oracle, through the C ABI."""

import ctypes

import numpy as np
import pytest
import torch

from e3j_amd import _lib
from oracle import conv_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _params(n, e, nnz, X, Y, Z, S, K, layout, val, idx_bytes, debug=1):
    return _lib.ConvParams(num_nodes=n, num_edges=e, num_coef=nnz, num_x=X, num_y=Y, num_out=Z,
                           num_scalars=S, channels=K, layout=layout, val_dtype=val,
                           coef_idx_bytes=idx_bytes, signature=-1, coef_scale=1.0, debug=debug)


def run_abi(idx, val, mix, x, y, s, dm, snd, rcv, Z, *, leading=False, dtype=np.float32,
            idx_dtype=None, grouping="receiver", perm=None):
    """Forward and backward through the C ABI on receiver-sorted (or permuted) edges."""
    lib = _lib.load()
    n, e = x.shape[0], y.shape[0]
    X, S = (x.shape[2], s.shape[2]) if leading else (x.shape[1], s.shape[1])
    K = x.shape[1] if leading else x.shape[2]
    packed = H.pack_table(idx, val, mix, val_dtype=dtype, idx_dtype=idx_dtype)
    coef_d = _dev(packed.view(np.uint8).reshape(-1))
    xd, yd, sd, dmd = _dev(x), _dev(y), _dev(s), _dev(dm)
    if perm is None:
        ptr = O.receiver_ptr(rcv, n)
        other, perm_d = _dev(snd.astype(np.int32)), None
    else:
        ptr = O.receiver_ptr(rcv[perm], n)
        other, perm_d = _dev(snd[perm].astype(np.int32)), _dev(perm.astype(np.int32))
    ptr_d = _dev(ptr)
    p = _params(n, e, len(val), X, y.shape[1], Z, S, K, 0 if leading else 1,
                _lib.F32 if dtype == np.float32 else _lib.F64, packed.dtype.itemsize)
    out = torch.full((n,) + ((K, Z) if leading else (Z, K)), float("nan"),
                     dtype=xd.dtype, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    _lib.check(lib.e3j_amd_convolution_fwd(ctypes.byref(p), coef_d.data_ptr(), xd.data_ptr(),
                                           yd.data_ptr(), sd.data_ptr(), other.data_ptr(),
                                           ptr_d.data_ptr(),
                                           perm_d.data_ptr() if perm_d is not None else None,
                                           out.data_ptr(), stream))
    dx = torch.full_like(xd, float("nan"))
    dy = torch.full_like(yd, float("nan"))
    ds = torch.full_like(sd, float("nan"))
    if grouping == "receiver":
        _lib.check(lib.e3j_amd_convolution_bwd_receiver(
            ctypes.byref(p), coef_d.data_ptr(), xd.data_ptr(), yd.data_ptr(), sd.data_ptr(),
            dmd.data_ptr(), other.data_ptr(), ptr_d.data_ptr(),
            perm_d.data_ptr() if perm_d is not None else None,
            dx.data_ptr(), dy.data_ptr(), ds.data_ptr(), stream))
    else:
        perm_t, recv_t, sptr = O.transpose_graph(snd, rcv, n)
        recv_t_d, sptr_d, perm_t_d = _dev(recv_t.astype(np.int32)), _dev(sptr), _dev(perm_t)
        _lib.check(lib.e3j_amd_convolution_bwd_sender(
            ctypes.byref(p), coef_d.data_ptr(), xd.data_ptr(), yd.data_ptr(), sd.data_ptr(),
            dmd.data_ptr(), recv_t_d.data_ptr(), sptr_d.data_ptr(), perm_t_d.data_ptr(),
            dx.data_ptr(), dy.data_ptr(), ds.data_ptr(), stream))
    torch.cuda.synchronize()
    return out.cpu().numpy(), dx.cpu().numpy(), dy.cpu().numpy(), ds.cpu().numpy()


def check_all(idx, val, mix, x, y, s, dm, snd, rcv, Z, results, leading=False, tag=""):
    out, dx, dy, ds = results
    ref, mag = H.forward_reference(idx, val, mix, x, y, s, snd, rcv, Z, leading=leading)
    H.assert_parity(out, ref, mag, f"{tag} out")
    (rx, ry, rs), (mx, my, ms) = H.backward_reference(idx, val, mix, x, y, s, snd, rcv, dm, leading=leading)
    H.assert_parity(dx, rx, mx, f"{tag} dx")
    H.assert_parity(dy, ry, my, f"{tag} dy")
    H.assert_parity(ds, rs, ms, f"{tag} ds")


@pytest.mark.parametrize("scale_s", [False, True])
@pytest.mark.parametrize("channels", [32, 64, 96, 128])
@pytest.mark.parametrize("idx_dtype", [np.int32, np.uint8])
def test_strip_case_bit_exact(channels, scale_s, idx_dtype):
    """Known-answer case of the reference's C++ test, required bit-exact
    (lib/e3j_ops/tests/test_convolution.cpp:288-290,316-384)."""
    c = O.strip_case(3, channels, scale_s)
    dm = np.ones((4, c["num_out"], channels), dtype=np.float32)
    out, *_ = run_abi(c["idx"], c["val"], c["mix_idx"], c["x"], c["y"], c["s"], dm, c["sender"],
                      c["receiver"], c["num_out"], idx_dtype=idx_dtype)
    assert np.array_equal(out, c["expect"])


# channel counts of the reference's op tests (tests/test_ops/test_convolution_op.py:209-282)
@pytest.mark.parametrize("channels", [1, 2, 4, 8, 16, 32, 128, 256])
@pytest.mark.parametrize("grouping", ["receiver", "sender"])
def test_random_table_fwd_bwd(channels, grouping):
    rng = np.random.default_rng(100 + channels)
    N, E, X, Y, Z, S, nnz = 8, 24, 9, 16, 9, 3, 200
    idx, val, mix = H.random_table(rng, nnz, X, Y, Z, S)
    snd, rcv = H.random_graph(rng, N, E)
    x, y, s, dm = H.random_operands(rng, N, E, X, Y, S, channels, Z)
    res = run_abi(idx, val, mix, x, y, s, dm, snd, rcv, Z, grouping=grouping)
    check_all(idx, val, mix, x, y, s, dm, snd, rcv, Z, res, tag=f"K={channels} {grouping}")
