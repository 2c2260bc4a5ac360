"""Unrolled kernels for coefficient tables the library was not built for, compiled at run time.

The generator that writes the built-in signatures (`e3j_amd/codegen/gen_conv.py`) takes any
forward table; here its output for one table and channel count is compiled with hipcc into a
small shared library, cached on disk under a hash of the table, and handed to the kernel
library's registry (`e3j_amd_register_signature`).  From then on the table is served like a
built-in one, in both memory layouts.  This is the counterpart of the trace-time unrolling of
the reference's Pallas kernels (`src/e3j/pallas_ops/convolution/mosaic_gpu/fwd.py:162-177`,
`src/e3j/pallas_ops/utils/coef.py:102-126`); switched on with `config(jit=True)` or
`E3J_AMD_JIT=1`, because the first call with a new table waits for the compiler.
"""

from __future__ import annotations

import ctypes
import hashlib
import os
import subprocess
import tempfile
import threading
import warnings

import numpy as np

from . import _lib
from . import build as _build
from .codegen import gen_conv, gen_tp

#: where compiled signature libraries are kept (in-tree by default, so that they travel with it)
CACHE_DIR = os.environ.get("E3J_AMD_JIT_CACHE", os.path.join(_build.HERE, "lib", "jit"))

_lock = threading.Lock()
_loaded = {}   # key -> (ctypes.CDLL kept alive, [signature ids])
_failed = set()


# the parameter structs the compiled kernels read
_PUBLIC_HEADER = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "e3j_amd.h")


def _key(val: np.ndarray, idx4: np.ndarray, dims, channels: int) -> str:
    h = hashlib.sha256()
    h.update(np.ascontiguousarray(val, dtype=np.float32).tobytes())
    h.update(np.ascontiguousarray(idx4, dtype=np.int64).tobytes())
    h.update(repr((tuple(int(d) for d in dims), int(channels))).encode())
    for path in (gen_conv.__file__, os.path.join(_build.CSRC, "unrolled.h"),
                 os.path.join(_build.CSRC, "unrolled_f64.h"), os.path.join(_build.CSRC, "unrolled_f16.h"),
                 os.path.join(_build.CSRC, "common.h"), _PUBLIC_HEADER):
        with open(path, "rb") as fh:      # kernels of another version of the templates are stale
            h.update(fh.read())
    return h.hexdigest()[:20]


def _compile(source: str, out_path: str) -> None:
    os.makedirs(os.path.dirname(out_path), exist_ok=True)
    with tempfile.TemporaryDirectory(dir=os.path.dirname(out_path)) as tmp:
        src = os.path.join(tmp, "signature.hip")
        lib = os.path.join(tmp, "signature.so")
        with open(src, "w") as fh:
            fh.write(source)
        # undefined symbols (error reporting, fills, tuning) bind to the loaded kernel library
        cmd = [_build.HIPCC, *_build.COMMON_FLAGS, "-shared", "-I", _build.CSRC, src, "-o", lib]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed for a run-time signature:\n{' '.join(cmd)}\n{proc.stderr[-4000:]}")
        with open(os.path.join(tmp, "signature.hip.txt"), "w") as fh:
            fh.write(source)
        os.replace(src, out_path[:-3] + ".hip")
        os.replace(lib, out_path)


def signature_library(val, idx4, dims, channels: int, build: bool = True) -> str | None:
    """Path of the compiled library of a table (compiled now if missing and `build`), or None
    when the kernel templates cannot take the table."""
    num_x, num_y, num_out, num_scalars = (int(d) for d in dims)
    try:
        table = gen_conv.Table(val, idx4, num_x, num_y, num_out, num_scalars)
    except ValueError:
        return None            # an output coordinate scaled by several scalars
    if not gen_conv.supports(table, channels) or np.asarray(idx4).max(initial=0) > 255:
        return None
    key = _key(val, idx4, dims, channels)
    path = os.path.join(CACHE_DIR, key, "signature.so")
    if not os.path.exists(path):
        if not build:
            return None
        trailing, leading = gen_conv.plugin_launch(channels)
        name = f"jit_{key}"
        desc = (f"{name}: run-time table (x {num_x}, y {num_y}, out {num_out}, paths {num_scalars}), "
                f"K={channels}, trailing, nnz={len(table.val)}")
        source = gen_conv.emit_table_source(table, name, desc, channels,
                                            symbols=(f"kTrailing_{key}", f"kLeading_{key}"),
                                            include='"unrolled.h"', launch=trailing, lead=leading, plugin=True)
        _compile(source, path)
    return path


def register(val, idx4, dims, channels: int) -> list[int]:
    """Compile (or find in the cache) and register the kernels of a table; ids of the new
    signatures, empty when the table cannot be served."""
    key = _key(val, idx4, dims, channels)
    with _lock:
        if key in _loaded:
            return _loaded[key][1]
        if key in _failed:
            return []
        try:
            path = signature_library(val, idx4, dims, channels)
        except (RuntimeError, OSError) as err:   # no compiler, or the templates reject the shape
            warnings.warn(f"e3j_amd: no run-time kernels for this table ({err}); "
                          "the table-driven kernels serve it", RuntimeWarning)
            path = None
        if path is None:
            _failed.add(key)
            return []
        main = _lib.load()
        # local scope: every signature library resolves its own objects, and the kernel
        # library's (loaded with global scope) for everything it leaves undefined
        plugin = ctypes.CDLL(path, mode=ctypes.RTLD_LOCAL)
        plugin.e3j_amd_plugin_signature.restype = ctypes.c_void_p
        plugin.e3j_amd_plugin_signature.argtypes = [ctypes.c_int]
        ids = []
        for which in (0, 1):
            entry = plugin.e3j_amd_plugin_signature(which)
            if entry:
                sig = main.e3j_amd_register_signature(entry)
                if sig >= 0:
                    ids.append(int(sig))
        _loaded[key] = (plugin, ids)
        return ids


# ---------------------------------------------------------------------------
# row-wise tensor product
# ---------------------------------------------------------------------------
def _tp_key(val: np.ndarray, idx: np.ndarray, shape, channels: int) -> str:
    h = hashlib.sha256()
    h.update(b"tensor_product")
    h.update(np.ascontiguousarray(val, dtype=np.float32).tobytes())
    h.update(np.ascontiguousarray(idx, dtype=np.int64).tobytes())
    h.update(repr((tuple(int(d) for d in shape), int(channels))).encode())
    for path in (gen_tp.__file__, os.path.join(_build.CSRC, "tp_unrolled.h"),
                 os.path.join(_build.CSRC, "unrolled.h"), os.path.join(_build.CSRC, "common.h"),
                 _PUBLIC_HEADER):
        with open(path, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:20]


def tp_signature_library(val, idx, shape, channels: int, build: bool = True) -> str | None:
    """Path of the compiled tensor-product library of a table `(val; i, j, k)` with dense shape
    `(num_out, num_x, num_y)`: trailing-layout kernels for `channels` (a multiple of 64), or the
    leading-layout kernels (any channel count) for `channels` 0.  None when the kernel templates
    cannot take the table."""
    num_out, num_x, num_y = (int(d) for d in shape)
    idx = np.asarray(idx)
    if not gen_tp.supports(num_x, num_y, num_out, channels or 64) or idx.max(initial=0) > 255 or not len(val):
        return None
    key = _tp_key(val, idx, shape, channels)
    path = os.path.join(CACHE_DIR, key, "signature.so")
    if not os.path.exists(path):
        if not build:
            return None
        name = f"jit_{key}"
        where = f"K={channels}, trailing" if channels else "leading"
        desc = f"{name}: run-time table (x {num_x}, y {num_y}, out {num_out}), {where}, nnz={len(val)}"
        symbols = tuple(f"kTp_{key}_{t}" for t in range(3))
        source = gen_tp.emit_source(name, desc, np.asarray(val, dtype=np.float32), idx, (num_out, num_x, num_y),
                                    channels, symbols, include='"tp_unrolled.h"', plugin=True)
        _compile(source, path)
    return path


def register_tp(val, idx, shape, channels: int) -> list[int]:
    """Compile (or find in the cache) and register the tensor-product kernels of a table (MAP,
    channel-free y, INNER); `channels` 0 = the leading layout.  Ids of the new signatures, empty
    when the table cannot be served."""
    key = _tp_key(val, idx, shape, channels)
    with _lock:
        if key in _loaded:
            return _loaded[key][1]
        if key in _failed:
            return []
        try:
            path = tp_signature_library(val, idx, shape, channels)
        except (RuntimeError, OSError) as err:
            warnings.warn(f"e3j_amd: no run-time kernels for this table ({err}); "
                          "the table-driven kernels serve it", RuntimeWarning)
            path = None
        if path is None:
            _failed.add(key)
            return []
        main = _lib.load()
        plugin = ctypes.CDLL(path, mode=ctypes.RTLD_LOCAL)
        plugin.e3j_amd_tp_plugin_signature.restype = ctypes.c_void_p
        plugin.e3j_amd_tp_plugin_signature.argtypes = [ctypes.c_int]
        ids = []
        for which in range(3):
            entry = plugin.e3j_amd_tp_plugin_signature(which)
            if entry:
                sig = main.e3j_amd_tp_register_signature(entry)
                if sig >= 0:
                    ids.append(int(sig))
        _loaded[key] = (plugin, ids)
        return ids
