"""ctypes binding of `conv_oracle.c` (trailing-channels layout; float32, or the same loops in float64).

TEST INFRASTRUCTURE ONLY: used by `tests/`, `__graft_entry__.smoke()` and the
`cpu_baseline` leg of `bench.py`; never by the `e3j_amd` package.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libconv_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile `conv_oracle.c` with the Makefile next to it."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        for name in ("conv_oracle_fwd", "conv_oracle_bwd", "conv_oracle_fwd_f64", "conv_oracle_bwd_f64"):
            getattr(_lib, name).restype = None
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _prep(idx, val, mix_idx, senders, receivers, dtype=np.float32):
    idx = np.asarray(idx)
    ci = np.ascontiguousarray(idx[:, 0], dtype=np.int32)
    cj = np.ascontiguousarray(idx[:, 1], dtype=np.int32)
    ck = np.ascontiguousarray(idx[:, 2], dtype=np.int32)
    cv = np.ascontiguousarray(val, dtype=dtype)
    mix = np.ascontiguousarray(mix_idx, dtype=np.int32)
    snd = np.ascontiguousarray(senders, dtype=np.int32)
    rcv = np.ascontiguousarray(receivers, dtype=np.int32)
    return ci, cj, ck, cv, mix, snd, rcv


def _dtype(dtype):
    dtype = np.dtype(dtype)
    if dtype not in (np.dtype(np.float32), np.dtype(np.float64)):
        raise TypeError("the C checker is built for float32 and float64")
    return dtype


def convolution(idx, val, mix_idx, x, y, s, senders, receivers, num_out: int, dtype=np.float32) -> np.ndarray:
    """`dtype=np.float64`: the same loops with every value (table included) in double."""
    lib = _load()
    dtype = _dtype(dtype)
    ci, cj, ck, cv, mix, snd, rcv = _prep(idx, val, mix_idx, senders, receivers, dtype)
    x = np.ascontiguousarray(x, dtype=dtype)
    y = np.ascontiguousarray(y, dtype=dtype)
    s = np.ascontiguousarray(s, dtype=dtype)
    n, X, K = x.shape
    E, Y = y.shape
    S = s.shape[1]
    out = np.empty((n, num_out, K), dtype=dtype)
    fn = lib.conv_oracle_fwd if dtype == np.float32 else lib.conv_oracle_fwd_f64
    fn(_p(ci), _p(cj), _p(ck), _p(cv), ctypes.c_int32(len(cv)), _p(mix),
       _p(x), _p(y), _p(s), _p(snd), _p(rcv),
       ctypes.c_int32(n), ctypes.c_int64(E),
       ctypes.c_int32(X), ctypes.c_int32(Y), ctypes.c_int32(S),
       ctypes.c_int32(num_out), ctypes.c_int32(K), _p(out))
    return out


def convolution_vjp(idx, val, mix_idx, x, y, s, senders, receivers, dm, dtype=np.float32):
    lib = _load()
    dtype = _dtype(dtype)
    ci, cj, ck, cv, mix, snd, rcv = _prep(idx, val, mix_idx, senders, receivers, dtype)
    x = np.ascontiguousarray(x, dtype=dtype)
    y = np.ascontiguousarray(y, dtype=dtype)
    s = np.ascontiguousarray(s, dtype=dtype)
    dm = np.ascontiguousarray(dm, dtype=dtype)
    n, X, K = x.shape
    E, Y = y.shape
    S = s.shape[1]
    Z = dm.shape[1]
    dx, dy, ds = np.empty_like(x), np.empty_like(y), np.empty_like(s)
    fn = lib.conv_oracle_bwd if dtype == np.float32 else lib.conv_oracle_bwd_f64
    fn(_p(ci), _p(cj), _p(ck), _p(cv), ctypes.c_int32(len(cv)), _p(mix),
       _p(x), _p(y), _p(s), _p(dm), _p(snd), _p(rcv),
       ctypes.c_int32(n), ctypes.c_int64(E),
       ctypes.c_int32(X), ctypes.c_int32(Y), ctypes.c_int32(S),
       ctypes.c_int32(Z), ctypes.c_int32(K), _p(dx), _p(dy), _p(ds))
    return dx, dy, ds
