"""ctypes binding of `conv_oracle.c` (float32, trailing-channels layout).

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
        _lib.conv_oracle_fwd.restype = None
        _lib.conv_oracle_bwd.restype = None
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _prep(idx, val, mix_idx, senders, receivers):
    idx = np.asarray(idx)
    ci = np.ascontiguousarray(idx[:, 0], dtype=np.int32)
    cj = np.ascontiguousarray(idx[:, 1], dtype=np.int32)
    ck = np.ascontiguousarray(idx[:, 2], dtype=np.int32)
    cv = np.ascontiguousarray(val, dtype=np.float32)
    mix = np.ascontiguousarray(mix_idx, dtype=np.int32)
    snd = np.ascontiguousarray(senders, dtype=np.int32)
    rcv = np.ascontiguousarray(receivers, dtype=np.int32)
    return ci, cj, ck, cv, mix, snd, rcv


def convolution(idx, val, mix_idx, x, y, s, senders, receivers, num_out: int) -> np.ndarray:
    lib = _load()
    ci, cj, ck, cv, mix, snd, rcv = _prep(idx, val, mix_idx, senders, receivers)
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.ascontiguousarray(y, dtype=np.float32)
    s = np.ascontiguousarray(s, dtype=np.float32)
    n, X, K = x.shape
    E, Y = y.shape
    S = s.shape[1]
    out = np.empty((n, num_out, K), dtype=np.float32)
    lib.conv_oracle_fwd(_p(ci), _p(cj), _p(ck), _p(cv), ctypes.c_int32(len(cv)), _p(mix),
                        _p(x), _p(y), _p(s), _p(snd), _p(rcv),
                        ctypes.c_int32(n), ctypes.c_int64(E),
                        ctypes.c_int32(X), ctypes.c_int32(Y), ctypes.c_int32(S),
                        ctypes.c_int32(num_out), ctypes.c_int32(K), _p(out))
    return out


def convolution_vjp(idx, val, mix_idx, x, y, s, senders, receivers, dm):
    lib = _load()
    ci, cj, ck, cv, mix, snd, rcv = _prep(idx, val, mix_idx, senders, receivers)
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.ascontiguousarray(y, dtype=np.float32)
    s = np.ascontiguousarray(s, dtype=np.float32)
    dm = np.ascontiguousarray(dm, dtype=np.float32)
    n, X, K = x.shape
    E, Y = y.shape
    S = s.shape[1]
    Z = dm.shape[1]
    dx, dy, ds = np.empty_like(x), np.empty_like(y), np.empty_like(s)
    lib.conv_oracle_bwd(_p(ci), _p(cj), _p(ck), _p(cv), ctypes.c_int32(len(cv)), _p(mix),
                        _p(x), _p(y), _p(s), _p(dm), _p(snd), _p(rcv),
                        ctypes.c_int32(n), ctypes.c_int64(E),
                        ctypes.c_int32(X), ctypes.c_int32(Y), ctypes.c_int32(S),
                        ctypes.c_int32(Z), ctypes.c_int32(K), _p(dx), _p(dy), _p(ds))
    return dx, dy, ds
