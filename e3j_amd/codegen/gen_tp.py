"""Generator of the compile-time-unrolled row-wise tensor product kernels.

For every built-in Clebsch-Gordan table and channel count it writes one HIP source with a
`Sig` type holding the straight-line arithmetic of the table (`fwd`: every output coordinate as
a sum of `c * x[j] * y[k]`, stored once; `bwd`: per output coordinate one load of the cotangent
and two fused multiply-adds per coefficient) and the registry entries of the three channel modes
the kernel templates of `csrc/tp_unrolled.h` serve (MAP, OUTER with a channel-free `y`, INNER).
The tables are those `e3j_amd.TensorProduct` builds with its default normalisation
(`src/e3j/core/tensor_product.py:202-274`); a uniform factor between a caller's table and the
built-in one is passed to the kernels at run time.
"""

from __future__ import annotations

import os
from collections import OrderedDict

import numpy as np

from ..tensor_product import TensorProduct
from .gen_conv import F64_MAX_CLASSES, _f32_bits, _lit

#: (name, x irreps, y irreps, output filter or None for the full product, channel counts)
TP_TABLES = [
    ("tp_l2_l2_full", "0e+1o+2e", "0e+1o+2e", None, (32, 64, 128)),
    ("tp_l2_l3_to_l3", "0e+1o+2e", "0e+1o+2e+3o", "0e+1o+2e+3o", (64, 128)),
    ("tp_l3_l3_to_l3", "0e+1o+2e+3o", "0e+1o+2e+3o", "0e+1o+2e+3o", (32, 64, 128)),
]


def supports(num_x: int, num_y: int, num_out: int, channels: int) -> bool:
    """Whether the kernel templates can take a table of these sizes."""
    return num_y <= 64 and num_x <= 64 and num_out <= 255 and (
        (channels % 64 == 0 and channels >= 64) or channels in (16, 32))


def _rows(val, idx, num_out):
    rows = OrderedDict((i, []) for i in range(num_out))
    for v, (i, j, k) in zip(val, idx):
        if v != 0:
            rows[int(i)].append((float(np.float32(v)), int(j), int(k)))
    return rows


def coefficient_classes(val):
    """Classes of equal magnitude in the order of their first entry (`class of each entry`, number
    of classes): the float64 kernels read one value per class from a kernel argument."""
    classes = OrderedDict()
    for v in np.asarray(val, dtype=np.float32):
        if v != 0:
            classes.setdefault(_f32_bits(abs(float(v))), len(classes))
    return [classes[_f32_bits(abs(float(v)))] if v != 0 else 255 for v in np.asarray(val, dtype=np.float32)], len(classes)


def _emit_arith(val, idx, shape, f64: bool) -> list[str]:
    """`fwd` and `bwd` of a table: coefficients as float literals with float operands, or (float64)
    read from the coefficient classes `cf` under the sign of the entry."""
    Z = int(shape[0])
    T = "double" if f64 else "float"
    fma = "fma" if f64 else "fmaf"
    zero = "0.0" if f64 else "0.f"
    class_of, _ = coefficient_classes(val)
    rows = OrderedDict((i, []) for i in range(Z))
    for n, (v, (i, j, k)) in enumerate(zip(val, idx)):
        if v != 0:
            c = float(np.float32(v))
            text = (("-" if c < 0 else "") + f"cf.v[{class_of[n]}]") if f64 else _lit(c)
            rows[int(i)].append((text, int(j), int(k)))
    tail = ", const F64Coefs &cf" if f64 else ", TpNoCoefs = {}"
    out = ["    template <typename Store>",
           f"    __device__ static __forceinline__ void fwd(const {T} *x, const {T} *y, const Store &st{tail}) {{"]
    for i, terms in rows.items():
        if not terms:
            out.append(f"        st.template put<{i}>({zero});")
            continue
        out.append("        {")
        for n, (c, j, k) in enumerate(terms):
            if n == 0:
                out.append(f"            {T} m = {c} * (x[{j}] * y[{k}]);")
            else:
                out.append(f"            m = {fma}({c}, x[{j}] * y[{k}], m);")
        out.append(f"            st.template put<{i}>(m);")
        out.append("        }")
    out += ["    }", "",
            "    // dx and dy are accumulated into: the caller clears them",
            "    template <typename Load>",
            f"    __device__ static __forceinline__ void bwd(const {T} *x, const {T} *y, const Load &ld,",
            f"                                                {T} *dx, {T} *dy{tail}) {{"]
    for i, terms in rows.items():
        if not terms:
            continue
        out.append("        {")
        out.append(f"            const {T} g = ld.template get<{i}>();")
        scaled = OrderedDict()
        for c, j, k in terms:
            if c not in scaled:
                scaled[c] = f"t{len(scaled)}"
                out.append(f"            const {T} {scaled[c]} = {c} * g;")
            t = scaled[c]
            out.append(f"            dx[{j}] = {fma}({t}, y[{k}], dx[{j}]);")
            out.append(f"            dy[{k}] = {fma}({t}, x[{j}], dy[{k}]);")
        out.append("        }")
    out += ["    }"]
    return out


def emit_sig(struct_name: str, val, idx, shape, f64: bool = False) -> list[str]:
    Z, X, Y = (int(d) for d in shape)
    out = [f"struct {struct_name} {{",
           f"    static constexpr int X = {X}, Y = {Y}, Z = {Z};",
           ""]
    out += _emit_arith(val, idx, shape, False)
    if f64:
        out += ["", "    // float64: one coefficient per class of equal magnitude, from the kernel's argument"]
        out += _emit_arith(val, idx, shape, True)
    out += ["};", ""]
    return out


def emit_source(name: str, desc: str, val, idx, shape, channels: int, symbols, include='"../tp_unrolled.h"',
                plugin: bool = False) -> str:
    """HIP source of the kernels and the three registry entries (MAP, channel-free y, INNER) of one table:
    at one channel count in the trailing layout, or (`channels` 0) for the leading layout, whose
    kernels take the channel count at run time."""
    Z, X, Y = (int(d) for d in shape)
    leading = channels == 0
    sig = f"TpSig_{name}"
    vals = ", ".join(_lit(v) for v in val)
    idxs = ", ".join(str(int(a)) for row in idx for a in row)
    out = ["// GENERATED by e3j_amd/codegen/gen_tp.py -- do not edit.",
           f"// {desc}",
           f"#include {include}",
           "",
           "namespace e3j_amd {",
           "namespace {",
           ""]
    # float16 and float64 kernels: trailing layout, whole waves of channels
    wide = not leading and channels % 64 == 0
    class_of, num_classes = coefficient_classes(val)
    wide64 = wide and num_classes <= F64_MAX_CLASSES   # (a table of more magnitudes than the argument holds: no float64 kernels)
    out += emit_sig(sig, val, idx, shape, f64=wide64)
    out += ["}  // namespace", "",
            "// host pass only: the registry entries hold host function pointers",
            "#if !defined(__HIP_DEVICE_COMPILE__)",
            f"static const float kVal[] = {{{vals}}};",
            f"static const uint8_t kIdx[] = {{{idxs}}};",
            f"static const uint8_t kClass[] = {{{', '.join(str(c) for c in class_of)}}};"]
    layout = "E3J_AMD_LAYOUT_LEADING" if leading else "E3J_AMD_LAYOUT_TRAILING"
    for kind, symbol in zip((0, 1, 2), symbols):
        uniform = kind
        mode = ("MAP", "y without channel axis", "INNER")[kind]
        args = f"{sig}, {kind}" if leading else f"{sig}, {channels}, {kind}"
        suffix = "_leading" if leading else ""
        out += [f"extern const TpSignature {symbol} = {{",
                f'    "{desc}, {mode}",',
                f"    {X}, {Y}, {Z}, {len(val)}, {channels}, {uniform}, {layout}, kVal, kIdx,",
                f"    &launch_tp_unrolled_fwd{suffix}<{args}>,",
                f"    &launch_tp_unrolled_bwd{suffix}<{args}>,",
                f"    {num_classes}, kClass,"]
        out += [f"    &launch_tp_unrolled_fwd_f16<{args}>, &launch_tp_unrolled_bwd_f16<{args}>," if wide
                else "    nullptr, nullptr,",
                f"    &launch_tp_unrolled_fwd_f64<{args}>, &launch_tp_unrolled_bwd_f64<{args}>," if wide64
                else "    nullptr, nullptr,"]
        out += ["};"]
    if plugin:  # accessor a run-time compiled library is loaded through
        out += ["", f"static const TpSignature *const kPlugin[] = {{{', '.join('&' + sym for sym in symbols)}}};",
                'extern "C" const void *e3j_amd_tp_plugin_signature(int which) {',
                f"    return (which >= 0 && which < {len(symbols)}) ? kPlugin[which] : nullptr;",
                "}"]
    out += ["#else", "// device pass: the kernels must be instantiated"]
    fwd_args = "    const float *, const float *, float *, int64_t, {}float);"
    bwd_args = "    const float *, const float *, const float *, float *, float *, int64_t, {}float);"

    def typed(kind: str, V: str) -> str:
        """Argument list of a trailing-layout kernel for values held as `V`."""
        A, cf = ("double", "F64Coefs") if V == "double" else ("float", "TpNoCoefs")
        if kind == "fwd":
            return f"    const {V} *, const {V} *, {V} *, int64_t, {A}, {cf});"
        return f"    const {V} *, const {V} *, const {V} *, {V} *, {V} *, int64_t, {A}, {cf});"
    if leading:
        for uniform in ("false", "true"):
            out.append(f"template __global__ void tp_unrolled_fwd_leading_kernel<{sig}, 4, {uniform}>(")
            out.append(fwd_args.format("int, "))
        out.append(f"template __global__ void tp_unrolled_fwd_inner_leading_kernel<{sig}, 4>(")
        out.append(fwd_args.format("int, "))
        for inner in ("false", "true"):
            out.append(f"template __global__ void tp_unrolled_bwd_map_leading_kernel<{sig}, 4, {inner}>(")
            out.append(bwd_args.format("int, "))
        out.append(f"template __global__ void tp_unrolled_bwd_uniform_leading_kernel<{sig}, 4>(")
        out.append(bwd_args.format("int, "))
        out.append(f"template __global__ void tp_unrolled_bwd_uniform_leading_lds_kernel<{sig}, 2>(")
        out.append(bwd_args.format("int, "))
    else:
        narrow = channels < 64   # 16 or 32 channels: several rows side by side in a wave
        for V in ("float",) + (("half_t",) if wide else ()) + (("double",) if wide64 else ()):
            for uniform in ("false", "true"):
                out.append(f"template __global__ void tp_unrolled_fwd_kernel<{sig}, {channels}, 4, {uniform}, {V}>(")
                out.append(typed("fwd", V))
            if narrow:
                out.append(f"template __global__ void tp_unrolled_fwd_inner_narrow_kernel<{sig}, {channels}, 4>(")
                out.append(fwd_args.format(""))
            else:
                out.append(f"template __global__ void tp_unrolled_fwd_inner_kernel<{sig}, {channels}, {V}>(")
                out.append(typed("fwd", V))
            out.append(f"template __global__ void tp_unrolled_bwd_inner_kernel<{sig}, {channels}, 4, {V}>(")
            out.append(typed("bwd", V))
            out.append(f"template __global__ void tp_unrolled_bwd_map_kernel<{sig}, {channels}, 4, {V}>(")
            out.append(typed("bwd", V))
            if narrow:
                out.append(f"template __global__ void tp_unrolled_bwd_uniform_narrow_kernel<{sig}, {channels}, 4>(")
                out.append(bwd_args.format(""))
            else:
                out.append(f"template __global__ void tp_unrolled_bwd_uniform_kernel<{sig}, {channels}, {V}>(")
                out.append(typed("bwd", V))
    out += ["#endif", "", "}  // namespace e3j_amd", ""]
    return "\n".join(out)


def builtin_signatures():
    """(file stem, description, val, idx, shape, channels) of every compiled table; channels 0
    is the leading layout (any channel count)."""
    for name, xi, yi, filt, ks in TP_TABLES:
        tp = TensorProduct((xi, yi), filt)
        val = np.asarray(tp.values, dtype=np.float32)
        idx = np.asarray(tp.indices, dtype=np.int64)
        head = f"{name}: x {tp.source[0]} (x) y {tp.source[1]} -> {tp.target}"
        for k in ks:
            yield f"{name}_k{k}", f"{head}, K={k}, trailing, nnz={len(val)}", val, idx, tp.shape, k
        yield f"{name}_leading", f"{head}, leading, nnz={len(val)}", val, idx, tp.shape, 0


def write_all(out_dir: str) -> list[str]:
    os.makedirs(out_dir, exist_ok=True)
    written, symbols = [], []
    for n, (stem, desc, val, idx, shape, k) in enumerate(builtin_signatures()):
        if not supports(shape[1], shape[2], shape[0], k or 64):
            raise ValueError(f"{stem}: sizes outside the kernel templates")
        pair = tuple(f"kTpSignature_{3 * n + t}" for t in range(3))
        symbols += pair
        path = os.path.join(out_dir, f"{stem}.hip")
        _write_if_changed(path, emit_source(stem, desc, val, idx, shape, k, pair))
        written.append(path)
    reg = ["// GENERATED by e3j_amd/codegen/gen_tp.py -- do not edit.",
           '#include "../tp_unrolled.h"', "", "namespace e3j_amd {", ""]
    reg += [f"extern const TpSignature {s};" for s in symbols]
    reg += ["", "static const TpSignature *const kAll[] = {"]
    reg += [f"    &{s}," for s in symbols]
    reg += ["};", "",
            f"int num_builtin_tp_signatures() {{ return {len(symbols)}; }}",
            "const TpSignature &builtin_tp_signature(int id) { return *kAll[id]; }", "",
            "}  // namespace e3j_amd", ""]
    path = os.path.join(out_dir, "tp_registry.hip")
    _write_if_changed(path, "\n".join(reg))
    written.append(path)
    return written


def _write_if_changed(path: str, text: str) -> None:
    if os.path.exists(path) and open(path).read() == text:
        return
    with open(path, "w") as f:
        f.write(text)
