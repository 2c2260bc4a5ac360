"""The C-ABI library: exports, argument validation and XLA-FFI frame decoding (no kernel launch)."""

import ctypes as C
import os
import re

import numpy as np
import pytest

from e3j_amd import Convolution, _lib
from tests.xla_frame import ERR_INVALID_ARGUMENT, ERR_UNIMPLEMENTED, F32, F64, S32, U8, FakeXla

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _params(**kw):
    base = dict(num_nodes=4, num_edges=6, num_coef=3, num_x=2, num_y=3, num_out=2, num_scalars=1,
                channels=8, layout=1, val_dtype=0, coef_idx_bytes=1, signature=-1, coef_scale=1.0, debug=0)
    base.update(kw)
    return _lib.ConvParams(**base)


def test_every_declared_symbol_is_exported():
    header = open(os.path.join(ROOT, "include", "e3j_amd.h")).read()
    declared = set(re.findall(r"\b(e3j_amd_[a-z0-9_]+)\s*\(", header))
    assert declared == set(_lib.SYMBOLS), "binding table and header disagree"
    lib = _lib.load()
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.e3j_amd_version().startswith(b"e3j_amd")


def test_params_struct_matches_header():
    header = open(os.path.join(ROOT, "include", "e3j_amd.h")).read()
    body = re.search(r"typedef struct e3j_amd_conv_params \{(.*?)\} e3j_amd_conv_params;", header, re.S).group(1)
    fields = re.findall(r"^\s*(const int32_t \*|const double \*|float \*|int32_t \*|uint32_t|int32_t|int64_t|float)\s*(\w+);",
                        body, re.M)
    assert [name for _, name in fields] == [name for name, _ in _lib.ConvParams._fields_]
    ctype = {"int32_t": C.c_int32, "uint32_t": C.c_uint32, "int64_t": C.c_int64, "float": C.c_float, "const int32_t *": C.c_void_p,
             "float *": C.c_void_p, "int32_t *": C.c_void_p, "const double *": C.c_void_p}
    assert [ctype[t] for t, _ in fields] == [t for _, t in _lib.ConvParams._fields_]


def test_tensor_product_params_struct_matches_header():
    header = open(os.path.join(ROOT, "include", "e3j_amd.h")).read()
    body = re.search(r"typedef struct e3j_amd_tp_params \{(.*?)\} e3j_amd_tp_params;", header, re.S).group(1)
    fields = re.findall(r"^\s*(const double \*|int32_t|int64_t|float)\s*(\w+);", body, re.M)
    assert [name for _, name in fields] == [name for name, _ in _lib.TpParams._fields_]
    ctype = {"int32_t": C.c_int32, "int64_t": C.c_int64, "float": C.c_float, "const double *": C.c_void_p}
    assert [ctype[t] for t, _ in fields] == [t for _, t in _lib.TpParams._fields_]
    modes = re.search(r"E3J_AMD_MODE_OUTER = (\d), E3J_AMD_MODE_INNER = (\d), E3J_AMD_MODE_MAP = (\d)", header)
    assert tuple(map(int, modes.groups())) == (_lib.MODE_OUTER, _lib.MODE_INNER, _lib.MODE_MAP)


def test_header_is_plain_c_and_ctypes_mirrors_its_layout(tmp_path):
    """The header compiles as strict C99 (what a cgo / JNI / FFI binding would include), and the
    compiler's sizes and field offsets of the parameter structs are those of the ctypes mirrors."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no C compiler")
    fields = {"e3j_amd_conv_params": _lib.ConvParams, "e3j_amd_tp_params": _lib.TpParams,
              "e3j_amd_tile_schedule": _lib.TileSchedule}
    lines = ['#include <stdio.h>', '#include <stddef.h>', f'#include "{os.path.join(ROOT, "include", "e3j_amd.h")}"',
             'int main(void) {']
    for struct, mirror in fields.items():
        lines.append(f'    printf("{struct} %zu\\n", sizeof({struct}));')
        for name, _ in mirror._fields_:
            lines.append(f'    printf("{struct}.{name} %zu\\n", offsetof({struct}, {name}));')
    lines += ['    return 0;', '}']
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", str(src), "-o", str(exe)], check=True)
    got = dict(line.split() for line in subprocess.run([str(exe)], check=True, capture_output=True,
                                                       text=True).stdout.splitlines())
    for struct, mirror in fields.items():
        assert int(got[struct]) == C.sizeof(mirror)
        for name, _ in mirror._fields_:
            assert int(got[f"{struct}.{name}"]) == getattr(mirror, name).offset, (struct, name)


def test_tensor_product_argument_errors_need_no_launch():
    lib = _lib.load()
    assert lib.e3j_amd_tensor_product_fwd(None, None, None, None, None, None) == _lib.INVALID_ARGUMENT
    assert "null params" in lib.e3j_amd_last_error().decode()
    p = _lib.TpParams(num_rows=0, num_coef=0, num_x=1, num_y=1, num_out=1, channels_x=1, channels_y=1,
                      mode=_lib.MODE_OUTER, layout=_lib.LAYOUT_LEADING, val_dtype=_lib.F32, coef_idx_bytes=1,
                      signature=-1, coef_scale=1.0)
    assert lib.e3j_amd_tensor_product_fwd(C.byref(p), None, None, None, None, None) == _lib.OK   # no rows: a no-op
    p.num_rows = 3
    assert lib.e3j_amd_tensor_product_fwd(C.byref(p), None, None, None, None, None) == _lib.INVALID_ARGUMENT
    assert "null operand" in lib.e3j_amd_last_error().decode()
    p.mode = 9
    assert lib.e3j_amd_tensor_product_bwd(C.byref(p), *[None] * 7) == _lib.INVALID_ARGUMENT
    assert "unknown mode" in lib.e3j_amd_last_error().decode()
    p.mode, p.signature = _lib.MODE_OUTER, 10_000
    assert lib.e3j_amd_tensor_product_fwd(C.byref(p), None, None, None, None, None) == _lib.INVALID_ARGUMENT
    assert "unknown signature" in lib.e3j_amd_last_error().decode()
    p.signature = 0      # a built-in kernel: trailing layout, 64 channels, MAP
    assert lib.e3j_amd_tensor_product_fwd(C.byref(p), None, None, None, None, None) == _lib.INVALID_ARGUMENT
    assert "do not match signature" in lib.e3j_amd_last_error().decode()


def test_tensor_product_signature_lookup():
    from e3j_amd import TensorProduct
    lib = _lib.load()
    assert lib.e3j_amd_tp_num_signatures() >= 27
    tp = TensorProduct(("0e+1o+2e+3o", "0e+1o+2e+3o"), "0e+1o+2e+3o")
    packed = tp.packed_coef("float32")
    Z, X, Y = tp.shape
    scale = C.c_float(0)

    def find(buf, channels, uniform, layout=_lib.LAYOUT_TRAILING):
        return lib.e3j_amd_tp_find_signature(buf.ctypes.data, buf.dtype.itemsize, _lib.F32, buf.shape[0],
                                             X, Y, Z, channels, uniform, layout, C.byref(scale))
    a, b = find(packed, 128, 0), find(packed, 128, 1)
    assert a >= 0 and b >= 0 and a != b and scale.value == 1.0
    assert b"K=128" in lib.e3j_amd_tp_signature_name(a) and b"MAP" in lib.e3j_amd_tp_signature_name(a)
    assert b"without channel axis" in lib.e3j_amd_tp_signature_name(b)
    assert find(packed, 128, 2) >= 0 and b"INNER" in lib.e3j_amd_tp_signature_name(find(packed, 128, 2))
    assert find(packed, 64, 0) >= 0 and find(packed, 96, 0) == -1 and find(packed, 16, 0) == -1
    assert b"K=32" in lib.e3j_amd_tp_signature_name(find(packed, 32, 2))   # two rows side by side in a wave
    # leading layout: one kernel for every multiple of 4 channels (MAP); whole waves per row (uniform y)
    lead = find(packed, 100, 0, _lib.LAYOUT_LEADING)
    assert lead >= 0 and lead == find(packed, 4, 0, _lib.LAYOUT_LEADING) and lead not in (a, b)
    assert b"leading" in lib.e3j_amd_tp_signature_name(lead)
    assert find(packed, 6, 0, _lib.LAYOUT_LEADING) == -1
    assert find(packed, 128, 1, _lib.LAYOUT_LEADING) >= 0 and find(packed, 100, 1, _lib.LAYOUT_LEADING) == -1
    from e3j_amd.coef import Coef
    c = Coef.unpack(packed, np.float32)
    assert find(Coef(3.0 * c.val, c.idx, "float32", "int32").pack(), 128, 0) == a and abs(scale.value - 3.0) < 1e-6
    bent = c.val.copy()
    bent[5] *= 1.001
    assert find(Coef(bent, c.idx, "float32", "int32").pack(), 128, 0) == -1
    assert find(Coef(-c.val, c.idx, "float32", "int32").pack(), 128, 0) == -1
    other = TensorProduct(("0e+1o+2e+3o", "0e+1o+2e+3o"), "0e+1o+2e+3o", normalization="SQRT_DIM_OUT")
    assert find(other.packed_coef("float32"), 128, 0) == -1     # one factor per path is not one factor


@pytest.mark.parametrize("kw, code, needle", [
    (dict(layout=7), _lib.INVALID_ARGUMENT, "unknown layout"),
    (dict(channels=0), _lib.INVALID_ARGUMENT, "must be >= 1"),
    (dict(val_dtype=5), _lib.INVALID_ARGUMENT, "unsupported (IDX, VAL) dtype pair"),
    (dict(coef_idx_bytes=2), _lib.INVALID_ARGUMENT, "unsupported (IDX, VAL) dtype pair"),
    (dict(num_edges=-1), _lib.INVALID_ARGUMENT, "negative size"),
    (dict(signature=10_000), _lib.INVALID_ARGUMENT, "unknown signature"),
    (dict(), _lib.INVALID_ARGUMENT, "null operand"),
])
def test_forward_argument_errors(kw, code, needle):
    lib = _lib.load()
    p = _params(**kw)
    rc = lib.e3j_amd_convolution_fwd(C.byref(p), None, None, None, None, None, None, None, None, None)
    assert rc == code
    message = lib.e3j_amd_last_error().decode()
    assert needle in message and message.startswith("E3J_AMD_ERROR[")
    with pytest.raises(_lib.E3jAmdError, match=re.escape(needle)):
        _lib.check(rc)


def test_null_params_and_backward_errors():
    lib = _lib.load()
    assert lib.e3j_amd_convolution_fwd(None, *([None] * 9)) == _lib.INVALID_ARGUMENT
    p = _params()
    for fn in (lib.e3j_amd_convolution_bwd_sender, lib.e3j_amd_convolution_bwd_receiver):
        assert fn(C.byref(p), *([None] * 12)) == _lib.INVALID_ARGUMENT
        assert "null operand" in lib.e3j_amd_last_error().decode()
    # mismatching shapes for a built-in signature
    p = _params(signature=0)
    assert lib.e3j_amd_convolution_fwd(C.byref(p), *([None] * 9)) == _lib.INVALID_ARGUMENT
    assert "do not match signature" in lib.e3j_amd_last_error().decode()


def test_empty_problem_is_a_no_op():
    lib = _lib.load()
    p = _params(num_nodes=0, num_edges=0)
    assert lib.e3j_amd_convolution_fwd(C.byref(p), *([None] * 9)) == _lib.OK
    assert lib.e3j_amd_convolution_bwd_receiver(C.byref(p), *([None] * 12)) == _lib.OK


def test_graph_entry_point_errors():
    lib = _lib.load()
    assert lib.e3j_amd_csr_row_ptr(None, -1, 4, None, None, None) == _lib.INVALID_ARGUMENT
    assert lib.e3j_amd_sort_edges(None, None, 4, 4, None, None, None, None, None) == _lib.INVALID_ARGUMENT
    assert lib.e3j_amd_csr_workspace_bytes(1000, 100000) > 0
    # the row order, the tile schedule and the pieces of long rows
    assert lib.e3j_amd_pair_rows(None, None, 4, 8, None, None, None, None) == _lib.INVALID_ARGUMENT
    assert "null operand" in lib.e3j_amd_last_error().decode()
    assert lib.e3j_amd_pair_rows(None, None, -1, 8, None, None, None, None) == _lib.INVALID_ARGUMENT
    assert lib.e3j_amd_pair_rows(None, None, 0, 0, None, None, None, None) == _lib.OK
    assert lib.e3j_amd_pair_rows_workspace_bytes(1000, 30000) > 4 * 30000
    assert lib.e3j_amd_row_segments_max(1000, 64) == 15 and lib.e3j_amd_row_segments_max(1000, 0) == 0
    assert lib.e3j_amd_row_segments_build(None, 4, 64, 64, 10, None, None) == _lib.INVALID_ARGUMENT
    assert lib.e3j_amd_row_segments_build(None, 4, 32, 64, 10, None, None) == _lib.INVALID_ARGUMENT   # piece > cap
    assert lib.e3j_amd_tile_rows(-1) == 0 and lib.e3j_amd_tile_rows_default(10_000) == 0
    p = _params(row_cap=-1)
    assert lib.e3j_amd_convolution_fwd(C.byref(p), *([C.c_void_p(64)] * 6), None, C.c_void_p(64), None) \
        == _lib.INVALID_ARGUMENT
    assert "row_cap" in lib.e3j_amd_last_error().decode()


def test_find_signature_matches_benchmark_tables():
    lib = _lib.load()
    assert lib.e3j_amd_num_signatures() >= 10
    module = Convolution(("0e+1o+2e+3o", "0e+1o+2e+3o"), "0e+1o+2e+3o", graph_ordering="RECEIVER")
    packed = module._packed_coef("float32")
    scale, flip = C.c_float(0), C.c_uint32(0)

    def find(buf, channels, idx_bytes=1, layout=1, signs=False):
        return lib.e3j_amd_find_signature(buf.ctypes.data, idx_bytes, _lib.F32, buf.shape[0], 16, 16, 99, 23,
                                          channels, layout, C.byref(scale), C.byref(flip) if signs else None)
    sig = find(packed, 128)
    assert sig >= 0 and scale.value == 1.0
    assert b"K=128" in lib.e3j_amd_signature_name(sig)
    assert find(packed, 64) >= 0 and find(packed, 64) != sig
    assert find(packed, 256) >= 0 and find(packed, 32) >= 0
    assert find(packed, 96) == -1                        # no kernel built for 96 channels
    lead = find(packed, 128, layout=0)                   # the leading layout has kernels of its own
    assert lead >= 0 and lead != sig and b"leading" in lib.e3j_amd_signature_name(lead)
    # int32 indices describe the same table
    from e3j_amd.coef import Coef4D
    c = module.coef
    wide = Coef4D(c.val, c.idx, "float32", "int32").pack()
    assert find(wide, 128, idx_bytes=4) == sig
    # a uniform positive factor is recognised and returned
    scaled = Convolution(("0e+1o+2e+3o", "0e+1o+2e+3o"), "0e+1o+2e+3o", graph_ordering="RECEIVER",
                         avg_num_neighbors=12.5)._packed_coef("float32")
    assert find(scaled, 128) == sig and abs(scale.value - 0.08) < 1e-7
    # one changed value or index breaks the match
    broken = packed.copy()
    broken[5, 4] ^= 1
    assert find(broken, 128) == -1
    v = packed.copy().view(np.uint8)
    c2 = Coef4D(c.val.copy(), c.idx, "float32", "uint8")
    c2.val[7] *= 1.001
    assert find(c2.pack(), 128) == -1
    # the parity signs of y folded into the values (SENDER ordering) come back as a bit mask
    parity = module.y_parity
    signed = Coef4D(c.val * parity[c.idx[:, 2].astype(np.int64)], c.idx, "float32", "uint8").pack()
    assert find(signed, 128) == -1                       # not asked for: no match
    assert find(signed, 128, signs=True) == sig and scale.value == 1.0
    assert flip.value == sum(1 << k for k in range(16) if parity[k] < 0) == 0b1111111000001110
    assert find(packed, 128, signs=True) == sig and flip.value == 0
    # signs that differ within one y component are no parity pattern
    c3 = Coef4D(c.val.copy(), c.idx, "float32", "uint8")
    first_k1 = int(np.flatnonzero(c.idx[:, 2] == 1)[0])
    c3.val[first_k1] *= -1.0
    assert find(c3.pack(), 128, signs=True) == -1


# --- XLA-FFI handlers -----------------------------------------------------------------
def test_xla_metadata_query():
    lib = _lib.load()
    for handler in (lib.e3j_amd_xla_convolution, lib.e3j_amd_xla_convolution_bwd,
                    lib.e3j_amd_xla_convolution_bwd_receiver, lib.e3j_amd_xla_convolution_bwd_ordered,
                    lib.e3j_amd_xla_tensor_product, lib.e3j_amd_xla_tensor_product_bwd):
        xla = FakeXla()
        frame, md = xla.metadata_frame()
        assert handler(C.addressof(frame)) is None
        assert (md.api_version.major_version, md.api_version.minor_version) == (0, 2)
        assert md.traits == 0 and md.state_type_id == 0
        assert not xla.errors


def test_xla_tensor_product_decoding_errors():
    """Operand and attribute checks of the tensor-product handlers (host addresses, no launch)."""
    lib = _lib.load()
    xla = FakeXla()
    host = np.zeros(4096, dtype=np.float32)
    coef = xla.buffer(S32, host.ctypes.data, (5, 4))
    x = xla.buffer(F32, host.ctypes.data, (3, 4, 8))
    y = xla.buffer(F32, host.ctypes.data, (3, 2, 8))
    z = xla.buffer(F32, host.ctypes.data, (3, 6, 8))
    i32 = lambda v: (S32, C.c_int32(v))  # noqa: E731
    full = {"num_out": i32(6), "mode": i32(2), "layout": i32(1), "debug": i32(0)}

    def run(args, rets, attrs, handler=lib.e3j_amd_xla_tensor_product):
        frame = xla.frame(args, rets, attrs)
        assert handler(C.addressof(frame)) is not None
        return xla.errors[-1]

    assert "3 or 4 operands" in run([coef, x], [z], full)[1]
    assert "mode and layout" in run([coef, x, y], [z], {"num_out": i32(6)})[1]
    assert "as many rows" in run([coef, x, xla.buffer(F32, host.ctypes.data, (4, 2, 8))], [z], full)[1]
    code, msg = run([xla.buffer(F64, host.ctypes.data, (5, 4)), x, y], [z], full)
    assert code == ERR_INVALID_ARGUMENT and "dtype pair" in msg
    assert "share one dtype" in run([coef, x, xla.buffer(F64, host.ctypes.data, (3, 2, 8))], [z], full)[1]
    assert "result shape" in run([coef, x, y], [xla.buffer(F32, host.ctypes.data, (3, 5, 8))], full)[1]
    assert "same number" in run([coef, x, xla.buffer(F32, host.ctypes.data, (3, 2, 4))],
                                [z], full)[1]                       # MAP with 8 and 4 channels
    back = {k: v for k, v in full.items() if k != "num_out"}
    stacked = xla.buffer(S32, host.ctypes.data, (2, 5, 4))
    dz_bad = xla.buffer(F32, host.ctypes.data, (3, 6, 4))
    assert "cotangent shape" in run([stacked, x, y, dz_bad], [x, y], back, lib.e3j_amd_xla_tensor_product_bwd)[1]
    assert "2 results" in run([stacked, x, y, z], [x], back, lib.e3j_amd_xla_tensor_product_bwd)[1]
    outer = dict(back, mode=i32(0))
    dz_outer = xla.buffer(F32, host.ctypes.data, (3, 6, 8, 8))
    code, msg = run([stacked, x, y, dz_outer], [x, y], outer, lib.e3j_amd_xla_tensor_product_bwd)
    assert code == ERR_UNIMPLEMENTED and "one channel" in msg


def _conv_frame(xla, *, x_dtype=F32, coef_dtype=U8, y_dims=(6, 3), n_attr=4, drop=None, channels=8):
    bufs = dict(coef=xla.buffer(coef_dtype, 0x1000, (3, 8)), x=xla.buffer(x_dtype, 0x2000, (4, 2, channels)),
                y=xla.buffer(F32, 0x3000, y_dims), s=xla.buffer(F32, 0x4000, (6, 1, channels)),
                sender=xla.buffer(S32, 0x5000, (6,)), ptr=xla.buffer(S32, 0x6000, (5,)),
                ranges=xla.buffer(S32, 0x7000, (1,)))
    out = xla.buffer(F32, 0x8000, (4, 2, channels))
    attrs = {"num_nodes": (S32, C.c_int32(n_attr)), "debug": (S32, C.c_int32(0))}
    if drop:
        attrs.pop(drop)
    return xla.frame(list(bufs.values()), [out], attrs)


@pytest.mark.parametrize("kw, code, needle", [
    (dict(x_dtype=16), ERR_INVALID_ARGUMENT, "unsupported (IDX, VAL) dtype pair"),    # BF16
    (dict(coef_dtype=F32), ERR_INVALID_ARGUMENT, "unsupported (IDX, VAL) dtype pair"),
    (dict(y_dims=(6, 3, 2)), ERR_UNIMPLEMENTED, "RHS y should have only one channel"),
    (dict(n_attr=5), ERR_INVALID_ARGUMENT, "num_nodes rows"),
    (dict(drop="num_nodes"), ERR_INVALID_ARGUMENT, "num_nodes (i32) is required"),
])
def test_xla_forward_decoding_errors(kw, code, needle):
    lib = _lib.load()
    xla = FakeXla()
    frame = _conv_frame(xla, **kw)
    err = lib.e3j_amd_xla_convolution(C.addressof(frame))
    assert err is not None and len(xla.errors) == 1
    assert xla.errors[0][0] == code and needle in xla.errors[0][1]


def test_xla_wrong_operand_count_and_stage():
    lib = _lib.load()
    xla = FakeXla()
    frame = xla.frame([xla.buffer(U8, 0x1000, (3, 8))], [], {"num_nodes": (S32, C.c_int32(4))})
    assert lib.e3j_amd_xla_convolution(C.addressof(frame)) is not None
    assert "expected 6 to 8 operands" in xla.errors[-1][1]
    assert lib.e3j_amd_xla_convolution_bwd(C.addressof(frame)) is not None
    assert "expected 8 or 9 operands" in xla.errors[-1][1]
    # stages other than EXECUTE are accepted and ignored
    frame = xla.frame([], [], {}, stage=1)
    assert lib.e3j_amd_xla_convolution(C.addressof(frame)) is None


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "absent.so"))
    with pytest.raises(ImportError, match="no fallback"):
        _lib.load()


def test_edge_features_and_regroup_validate_before_launching():
    lib = _lib.load()
    p = _lib.EdgeFeaturesParams(num_edges=4, num_nodes=3, l_max=7, normalization=1, num_basis=8, hidden=4, layers=1,
                                cutoff=5.0, val_dtype=0)
    assert lib.e3j_amd_edge_features_fwd(C.byref(p), *[None] * 9) == _lib.UNIMPLEMENTED      # degree 7
    p.l_max, p.num_basis = 3, 17
    assert lib.e3j_amd_edge_features_fwd(C.byref(p), *[None] * 9) == _lib.UNIMPLEMENTED      # 17 basis functions
    p.num_basis, p.cutoff = 8, 0.0
    assert lib.e3j_amd_edge_features_bwd(C.byref(p), *[None] * 10) == _lib.INVALID_ARGUMENT
    p.cutoff, p.normalization = 5.0, 9
    assert lib.e3j_amd_edge_features_fwd(C.byref(p), *[None] * 9) == _lib.INVALID_ARGUMENT
    p.normalization = 1
    assert lib.e3j_amd_edge_features_fwd(C.byref(p), *[None] * 9) == _lib.INVALID_ARGUMENT   # null y
    assert lib.e3j_amd_edge_features_fwd(None, *[None] * 9) == _lib.INVALID_ARGUMENT
    assert lib.e3j_amd_rows_regroup(None, None, 3, 4, 8, None, None, 0, 0, None) == _lib.INVALID_ARGUMENT
    assert lib.e3j_amd_rows_regroup(None, None, 0, 4, 8, None, None, 0, 0, None) == _lib.OK
    assert lib.e3j_amd_rows_regroup(None, None, -1, 4, 8, None, None, 0, 0, None) == _lib.INVALID_ARGUMENT


def test_float64_look_up_refuses_tables_of_another_structure():
    """One magnitude per class: a table in which two entries of one class differ, or with a sign
    that is not a sign of a whole y component, is not the built-in structure."""
    from e3j_amd.convolution import Convolution
    from tests import helpers as H
    lib = _lib.load()
    m = Convolution(("0e+1o+2e", "0e+1o+2e+3o"), "0e+1o+2e", graph_ordering="RECEIVER", avg_num_neighbors=3.0)
    c = m.coef
    idx4 = np.asarray(c.idx, dtype=np.int64)
    val = np.asarray(c.val, dtype=np.float64)
    dims = (m.source[0].dim, m.source[1].dim, m.target.dim, m.params.num_scalars)

    def find(values):
        packed = H.pack_table(idx4[:, :3], values, m._mix.mix_indices, val_dtype=np.float64)
        classes = (C.c_double * _lib.F64_CLASSES)()
        flip = C.c_uint32()
        return lib.e3j_amd_find_signature_f64(packed.ctypes.data, 1, len(values), *dims, 64, 1, classes,
                                              C.byref(flip)), list(classes), flip.value

    sig, classes, flip = find(val)
    assert sig >= 0 and flip == 0
    assert sorted(set(np.round(np.abs(val), 15))) == sorted(set(np.round([v for v in classes if v > 0], 15)))
    mags = np.abs(val)
    twin = np.flatnonzero(mags == mags[0])
    assert len(twin) > 1
    one_off = val.copy()
    one_off[twin[1]] *= 1.0 + 1e-9
    assert find(one_off)[0] == -1
    one_sign = val.copy()
    k0 = idx4[0, 2]
    members = np.flatnonzero(idx4[:, 2] == k0)
    assert len(members) > 1
    one_sign[members[0]] *= -1.0
    assert find(one_sign)[0] == -1
    whole_component = val.copy()
    whole_component[members] *= -1.0
    assert find(whole_component)[2] == 1 << int(k0)


@pytest.mark.parametrize("avg", [None, 4.0, 12.5, 30.0, 7.3])
def test_half_valued_tables_resolve_to_their_signature(avg):
    """A table of half values (the built-in table times a factor, every entry rounded to half on its
    own) is found among the signatures that have float16 kernels, with the factor."""
    lib = _lib.load()
    m = Convolution(("0e+1o+2e+3o", "0e+1o+2e+3o"), "0e+1o+2e+3o", graph_ordering="RECEIVER", avg_num_neighbors=avg)
    packed = m._packed_coef("float16")
    scale, flip = C.c_float(), C.c_uint32()
    for channels, found in ((64, True), (128, True), (32, False)):
        sig = lib.e3j_amd_find_signature(packed.ctypes.data, 1, _lib.F16, packed.shape[0], 16, 16, 99, 23, channels, 1,
                                         C.byref(scale), C.byref(flip))
        assert (sig >= 0) == found
        if found:
            assert abs(scale.value * (avg or 1.0) - 1.0) < 2e-3 and flip.value == 0
    # the same values with one entry off by a percent are another table
    from e3j_amd.coef import Coef4D
    c = Coef4D.unpack(packed, np.float16)
    val = np.asarray(c.val).copy()
    val[3] *= np.float16(1.01)
    other = Coef4D(val, c.idx, val_dtype=np.float16, idx_dtype=c.idx_dtype).pack()
    assert lib.e3j_amd_find_signature(other.ctypes.data, 1, _lib.F16, other.shape[0], 16, 16, 99, 23, 128, 1,
                                      C.byref(scale), C.byref(flip)) == -1
