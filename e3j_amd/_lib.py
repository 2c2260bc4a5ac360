"""ctypes binding of `libe3j_amd.so` (declarations of `include/e3j_amd.h`).

There is no fallback: if the library has not been built, loading raises and
every operator of this package fails.  Takes the place of the reference's
`e3j_ops` pybind11 module and its registration (`lib/e3j_ops/ffi/e3j_ops.cpp:79-100`,
`src/e3j/ops/__init__.py:22-23`).
"""

from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
#: E3J_AMD_LIBRARY overrides the in-tree build (e.g. to compare two builds of the kernels).
LIB_PATH = os.environ.get("E3J_AMD_LIBRARY") or os.path.join(_HERE, "lib", "libe3j_amd.so")

OK, INVALID_ARGUMENT, UNIMPLEMENTED, INTERNAL = 0, 1, 2, 3
LAYOUT_LEADING, LAYOUT_TRAILING = 0, 1
F32, F64, F16 = 0, 1, 2
PLAN_BUILD, PLAN_READY, PLAN_NONE = 0, 1, 2
F64_CLASSES = 64


class ConvParams(ctypes.Structure):
    """`e3j_amd_conv_params`."""

    _fields_ = [
        ("num_nodes", ctypes.c_int32),
        ("num_edges", ctypes.c_int64),
        ("num_coef", ctypes.c_int32),
        ("num_x", ctypes.c_int32),
        ("num_y", ctypes.c_int32),
        ("num_out", ctypes.c_int32),
        ("num_scalars", ctypes.c_int32),
        ("channels", ctypes.c_int32),
        ("layout", ctypes.c_int32),
        ("val_dtype", ctypes.c_int32),
        ("coef_idx_bytes", ctypes.c_int32),
        ("signature", ctypes.c_int32),
        ("coef_scale", ctypes.c_float),
        ("debug", ctypes.c_int32),
        ("y_flip", ctypes.c_uint32),
        ("row_order", ctypes.c_void_p),
        ("row_cap", ctypes.c_int32),
        ("row_piece", ctypes.c_int32),
        ("max_segments", ctypes.c_int32),
        ("segments", ctypes.c_void_p),
        ("partials", ctypes.c_void_p),
        ("table_plan", ctypes.c_void_p),
        ("table_plan_state", ctypes.c_int32),
        ("coef_classes", ctypes.c_void_p),
    ]


MODE_OUTER, MODE_INNER, MODE_MAP = 0, 1, 2


class TileSchedule(ctypes.Structure):
    """`e3j_amd_tile_schedule`."""

    _fields_ = [
        ("tile_rows", ctypes.c_int32),
        ("num_work", ctypes.c_int32),
        ("work", ctypes.c_void_p),
        ("sender", ctypes.c_void_p),
        ("edge", ctypes.c_void_p),
        ("local", ctypes.c_void_p),
    ]


class TpParams(ctypes.Structure):
    """`e3j_amd_tp_params`."""

    _fields_ = [
        ("num_rows", ctypes.c_int64),
        ("num_coef", ctypes.c_int32),
        ("num_x", ctypes.c_int32),
        ("num_y", ctypes.c_int32),
        ("num_out", ctypes.c_int32),
        ("channels_x", ctypes.c_int32),
        ("channels_y", ctypes.c_int32),
        ("mode", ctypes.c_int32),
        ("layout", ctypes.c_int32),
        ("val_dtype", ctypes.c_int32),
        ("coef_idx_bytes", ctypes.c_int32),
        ("coef_sorted", ctypes.c_int32),
        ("debug", ctypes.c_int32),
        ("signature", ctypes.c_int32),
        ("coef_scale", ctypes.c_float),
        ("coef_classes", ctypes.c_void_p),
    ]


class EdgeFeaturesParams(ctypes.Structure):
    """`e3j_amd_edge_features_params`."""

    _fields_ = [
        ("num_edges", ctypes.c_int64),
        ("num_nodes", ctypes.c_int32),
        ("l_max", ctypes.c_int32),
        ("normalization", ctypes.c_int32),
        ("num_basis", ctypes.c_int32),
        ("hidden", ctypes.c_int32),
        ("layers", ctypes.c_int32),
        ("cutoff", ctypes.c_float),
        ("val_dtype", ctypes.c_int32),
    ]


class E3jAmdError(RuntimeError):
    """Failure reported by the kernel library; `.code` is the status code."""

    def __init__(self, code: int, message: str):
        super().__init__(message)
        self.code = code


_P = ctypes.c_void_p
_PARAMS = ctypes.POINTER(ConvParams)
_TP_PARAMS = ctypes.POINTER(TpParams)

#: name -> (restype, argtypes): every symbol `include/e3j_amd.h` declares.
SYMBOLS = {
    "e3j_amd_last_error": (ctypes.c_char_p, []),
    "e3j_amd_version": (ctypes.c_char_p, []),
    "e3j_amd_convolution_fwd": (ctypes.c_int, [_PARAMS] + [_P] * 9),
    "e3j_amd_convolution_bwd_sender": (ctypes.c_int, [_PARAMS] + [_P] * 12),
    "e3j_amd_convolution_bwd_receiver": (ctypes.c_int, [_PARAMS] + [_P] * 12),
    "e3j_amd_convolution_bwd_ordered_workspace_bytes": (ctypes.c_size_t, [_PARAMS]),
    "e3j_amd_convolution_bwd_ordered": (ctypes.c_int, [_PARAMS] + [_P] * 13),
    "e3j_amd_row_segments_max": (ctypes.c_int64, [ctypes.c_int64, ctypes.c_int32]),
    "e3j_amd_row_segments_build": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32,
                                                  ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p]),
    "e3j_amd_pair_rows_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int32, ctypes.c_int64]),
    "e3j_amd_pair_rows": (ctypes.c_int, [_P, _P, ctypes.c_int32, ctypes.c_int64, _P, _P, _P, _P]),
    "e3j_amd_tile_rows": (ctypes.c_int32, [ctypes.c_int32]),
    "e3j_amd_tile_rows_default": (ctypes.c_int32, [ctypes.c_int32]),
    "e3j_amd_tile_schedule_num_work": (ctypes.c_int64, [ctypes.c_int32, ctypes.c_int64, ctypes.c_int32, ctypes.c_int32]),
    "e3j_amd_tile_schedule_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int32, ctypes.c_int64, ctypes.c_int32]),
    "e3j_amd_tile_schedule_build": (ctypes.c_int, [_P] * 4 + [ctypes.c_int32, ctypes.c_int64, ctypes.c_int32,
                                                              ctypes.c_int32] + [_P] * 6),
    "e3j_amd_convolution_bwd_tiled": (ctypes.c_int, [_PARAMS] + [_P] * 7 + [ctypes.POINTER(TileSchedule)] + [_P] * 4),
    "e3j_amd_find_signature": (ctypes.c_int, [_P] + [ctypes.c_int32] * 9 + [ctypes.POINTER(ctypes.c_float),
                                                                             ctypes.POINTER(ctypes.c_uint32)]),
    "e3j_amd_find_signature_f64": (ctypes.c_int, [_P] + [ctypes.c_int32] * 8 + [ctypes.POINTER(ctypes.c_double),
                                                                                 ctypes.POINTER(ctypes.c_uint32)]),
    "e3j_amd_num_signatures": (ctypes.c_int, []),
    "e3j_amd_signature_name": (ctypes.c_char_p, [ctypes.c_int]),
    "e3j_amd_csr_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int32, ctypes.c_int64]),
    "e3j_amd_csr_row_ptr": (ctypes.c_int, [_P, ctypes.c_int64, ctypes.c_int32, _P, _P, _P]),
    "e3j_amd_csr_row_ptr_static_max_nodes": (ctypes.c_int32, []),
    "e3j_amd_csr_row_ptr_static": (ctypes.c_int, [_P, ctypes.c_int64, ctypes.c_int32, _P, _P]),
    "e3j_amd_sort_edges": (ctypes.c_int, [_P, _P, ctypes.c_int64, ctypes.c_int32, _P, _P, _P, _P, _P]),
    "e3j_amd_order_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int32]),
    "e3j_amd_register_signature": (ctypes.c_int, [_P]),
    "e3j_amd_set_table_plans": (None, [ctypes.c_int32]),
    "e3j_amd_row_partials_bytes": (ctypes.c_size_t, [ctypes.c_int64, ctypes.c_int32, ctypes.c_int32]),
    "e3j_amd_table_plan_bytes": (ctypes.c_size_t, [ctypes.POINTER(ConvParams)]),
    "e3j_amd_table_plan_status": (ctypes.c_int, [ctypes.POINTER(ConvParams), ctypes.c_void_p, ctypes.c_int32,
                                                 ctypes.POINTER(ctypes.c_int32), ctypes.c_void_p]),
    "e3j_amd_harmonics": (ctypes.c_int, [_P, ctypes.c_int64] + [ctypes.c_int32] * 4 + [_P, _P]),
    "e3j_amd_harmonics_bwd": (ctypes.c_int, [_P, _P, ctypes.c_int64] + [ctypes.c_int32] * 4 + [_P, _P]),
    "e3j_amd_edge_features_fwd": (ctypes.c_int, [ctypes.POINTER(EdgeFeaturesParams)] + [_P] * 9),
    "e3j_amd_edge_features_bwd": (ctypes.c_int, [ctypes.POINTER(EdgeFeaturesParams)] + [_P] * 10),
    "e3j_amd_channel_mix": (ctypes.c_int, [_P, _P, _P, ctypes.c_int64, ctypes.c_int32, ctypes.c_int32,
                                           ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int32),
                                           ctypes.c_int32, _P]),
    "e3j_amd_rows_regroup": (ctypes.c_int, [_P, _P, ctypes.c_int64, ctypes.c_int32, ctypes.c_int32, _P, _P,
                                            ctypes.c_int32, ctypes.c_int32, _P]),
    "e3j_amd_radial_linear_fwd": (ctypes.c_int, [_P, _P, _P, ctypes.c_int64, ctypes.c_int32, ctypes.c_int32, _P]),
    "e3j_amd_radial_linear_bwd_input": (ctypes.c_int, [_P, _P, _P, ctypes.c_int64, ctypes.c_int32, ctypes.c_int32, _P]),
    "e3j_amd_radial_linear_bwd_weight_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int64, ctypes.c_int32, ctypes.c_int32]),
    "e3j_amd_radial_linear_bwd_weight": (ctypes.c_int, [_P, _P, _P, _P, ctypes.c_int64, ctypes.c_int32, ctypes.c_int32, _P]),
    "e3j_amd_wrap_index": (ctypes.c_int, [_P, ctypes.c_int64, ctypes.c_int32, _P, _P]),
    "e3j_amd_locality_order": (ctypes.c_int, [_P, _P, ctypes.c_int32, ctypes.c_int32, _P, _P, _P]),
    "e3j_amd_tensor_product_fwd": (ctypes.c_int, [_TP_PARAMS] + [_P] * 5),
    "e3j_amd_tensor_product_bwd": (ctypes.c_int, [_TP_PARAMS] + [_P] * 7),
    "e3j_amd_tp_find_signature": (ctypes.c_int, [_P] + [ctypes.c_int32] * 9 + [ctypes.POINTER(ctypes.c_float)]),
    "e3j_amd_tp_find_signature_f64": (ctypes.c_int, [_P] + [ctypes.c_int32] * 8 + [ctypes.POINTER(ctypes.c_double)]),
    "e3j_amd_tp_num_signatures": (ctypes.c_int, []),
    "e3j_amd_tp_register_signature": (ctypes.c_int, [_P]),
    "e3j_amd_tp_signature_name": (ctypes.c_char_p, [ctypes.c_int]),
    "e3j_amd_xla_convolution": (_P, [_P]),
    "e3j_amd_xla_convolution_bwd": (_P, [_P]),
    "e3j_amd_xla_convolution_bwd_receiver": (_P, [_P]),
    "e3j_amd_xla_convolution_bwd_ordered": (_P, [_P]),
    "e3j_amd_xla_tensor_product": (_P, [_P]),
    "e3j_amd_xla_tensor_product_bwd": (_P, [_P]),
}

#: exported for the in-tree tests only, declared in `csrc/tuning_api.h`, not in the public header
INTERNAL_SYMBOLS = {
    "e3j_amd_set_launch_variant": (None, [ctypes.c_int32, ctypes.c_int32]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Load the library once; raise if it is missing or lacks a declared symbol."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m e3j_amd.build` "
            "(hipcc, gfx950). e3j_amd has no fallback implementation.")
    # global symbols: signature libraries compiled at run time resolve against this one
    lib = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    for name, (restype, argtypes) in {**SYMBOLS, **INTERNAL_SYMBOLS}.items():
        fn = getattr(lib, name)  # AttributeError if the export is missing
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(code: int) -> None:
    if code != OK:
        raise E3jAmdError(code, load().e3j_amd_last_error().decode())
