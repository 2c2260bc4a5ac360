"""Generator of the compile-time-unrolled convolution kernels.

For one irreps signature (x irreps, y irreps, output filter, channel count) it
turns the stacked Clebsch-Gordan table into straight-line HIP: every non-zero
coefficient becomes a fused multiply-add with a literal constant, and nothing
of the table is read at run time.  This is the gfx950 counterpart of the
trace-time unrolling of the reference's Pallas kernels
(`src/e3j/pallas_ops/convolution/mosaic_gpu/fwd.py:162-177`,
`src/e3j/pallas_ops/utils/coef.py:102-126`); the reference's CUDA kernel walks
the table at run time instead (`lib/e3j_ops/cuda/convolution/fwd.cuh:88-153`).

Per edge and lane (a lane owns CPL channels; `y` is the same for all lanes):

    p_m      = |c_m| * y[k_m]                      one product per distinct (|c|, k)
    w_ij     = sum of +-p_m                         the edge's (output, x) weights
    forward  : msg_i = sum_j w_ij x_j ;  acc_i += s_l(i) msg_i
    backward : g_i = dm_i s_l(i) ;  dx_j += w_ij g_i
               a_k = sum_ij c_ijk (dm_i x_j) per path ;  ds_l = sum_k y_k a_k ;
               dy_k += sum_channels(s_l a_k)

`python -m e3j_amd.codegen.gen_conv` rewrites `e3j_amd/csrc/generated/`.
"""

from __future__ import annotations

import os
import struct
from collections import OrderedDict

import numpy as np

from ..scalar_mixing import ScalarMixing
from ..tensor_product import TensorProduct

#: Tables compiled into the library: (name, x irreps, y irreps, output filter), the irreps
#: combinations of the benchmark configurations (SQRT_DIM_OUT normalisation, the default of
#: `Convolution`), each for the power-of-two channel counts the reference's fused kernel is
#: used with (`tests/test_convolution.py:245-246`: multiples of 32).
BUILTIN_TABLES = [
    ("l1_l2_to_l2", "0e+1o", "0e+1o+2e", "0e+1o+2e", (32, 64, 128)),
    ("l2_l3_to_l2", "0e+1o+2e", "0e+1o+2e+3o", "0e+1o+2e", (32, 64, 128)),
    ("l2_l3_to_l3", "0e+1o+2e", "0e+1o+2e+3o", "0e+1o+2e+3o", (64, 128)),
    ("l3_l3_to_l3", "0e+1o+2e+3o", "0e+1o+2e+3o", "0e+1o+2e+3o", (32, 64, 128, 256)),
    # scalar node features times the harmonics: the first layer of a model whose input is invariant
    ("l0_l3_to_l3", "0e", "0e+1o+2e+3o", "0e+1o+2e+3o", (64, 128, 256)),
]
#: (name, x irreps, y irreps, output filter, channels) of every compiled signature
BUILTIN_SIGNATURES = [(f"{name}_k{k}", xi, yi, oi, k) for name, xi, yi, oi, ks in BUILTIN_TABLES for k in ks]

#: launch shapes per channel count: (channels per lane, waves per block, parts[, resident
#: waves per SIMD the register allocation must allow]) variants for fwd and bwd.  `parts` splits the paths of the signature over that many waves.  Variant 0
#: is the default; the others are selected with the environment variables
#: E3J_AMD_FWD_VARIANT / E3J_AMD_BWD_VARIANT (read once) for tuning runs.
LAUNCH = {
    32: dict(fwd=[(1, 4, 1)], bwd=[(1, 4, 2), (1, 4, 1)]),
    64: dict(fwd=[(1, 4, 1), (1, 4, 2)], bwd=[(1, 4, 2), (1, 4, 1), (1, 4, 3), (1, 4, 4)],
             bwd_tile=[(1, 8, 3, 1, 4), (1, 8, 4), (1, 16, 4)]),   # (tiles of 4: the same kernel time as 8, a cheaper schedule)
    128: dict(fwd=[(1, 4, 1), (1, 4, 2), (2, 4, 2), (2, 4, 4)],
              bwd=[(2, 4, 3), (1, 4, 1), (1, 4, 3), (1, 4, 4), (2, 4, 4), (1, 4, 2)],
              bwd_tile=[(2, 4, 3, 3, 2), (2, 8, 3, 1, 8), (2, 12, 3, 3, 8), (2, 4, 3, 2, 4), (1, 8, 4, 1, 8)]),
    256: dict(fwd=[(1, 4, 1), (1, 4, 2)], bwd=[(2, 4, 3), (1, 4, 2), (1, 4, 3)],
              bwd_tile=[(2, 8, 3), (1, 8, 4)]),
}
#: parts of the float64 kernels: (forward, backward).  A double takes the registers of two channels
#: of a float kernel, so these are the splits the two-channel float kernels use.
F64_SPLIT = (3, 4)
#: float16 kernels (values held as half, computed in float): (channels per lane, parts forward,
#: parts backward) by whether the channel count is a multiple of 128; the splits of the float
#: kernels with as many channels per lane
F16_SHAPE = {True: (2, 2, 3), False: (1, 1, 3)}
#: the float64 kernels take one coefficient per class of equal magnitude as a kernel argument
F64_MAX_CLASSES = 64
#: `bwd_tile`: variants of the backward over tiles of receivers (trailing layout, at least 64
#: channels): a block of `waves per block` waves shares the dm rows of a tile in LDS.  A fifth
#: number is the receivers per tile the variant is tuned for (8 if absent): few enough that the
#: LDS of a CU holds the tiles of as many blocks as its wave slots take.


#: leading-channels layout: (waves per block, parts) variants.  The forward pass is never
#: split; a backward block is the parts of one (receiver, channel slice), so its wave count
#: is the part count (the first number is ignored there).
LAUNCH_LEADING = {
    32: dict(fwd=[(4, 1)], bwd=[(2, 2), (1, 1)]),
    64: dict(fwd=[(4, 1)], bwd=[(3, 3), (1, 1), (2, 2), (4, 4)]),
    128: dict(fwd=[(4, 1)], bwd=[(3, 3), (1, 1), (2, 2), (4, 4)]),
    256: dict(fwd=[(4, 1)], bwd=[(3, 3), (2, 2)]),
}


def _f32_bits(v: float) -> int:
    return struct.unpack("<I", struct.pack("<f", float(v)))[0]


def _lit(v: float) -> str:
    """Exact float32 literal."""
    f = np.float32(v)
    text = repr(float(f))
    if "e" not in text and "." not in text and "inf" not in text and "nan" not in text:
        text += ".0"
    return text + "f"


class Table:
    """A forward table `(val; i, j, k, l)` organised for emission.

    Output coordinates are grouped by their scalar index `l`: one group is one
    Clebsch-Gordan path (one output irrep copy), whose rows share an x block, a y
    block and one normalisation, so the products `|c| * y[k]` of a group are few
    and die with the group.
    """

    def __init__(self, val, idx4, num_x, num_y, num_out, num_scalars):
        self.val = np.asarray(val, dtype=np.float32)
        self.idx = np.asarray(idx4, dtype=np.int64)
        self.X, self.Y, self.Z, self.S = int(num_x), int(num_y), int(num_out), int(num_scalars)
        # paths[l] = OrderedDict i -> OrderedDict j -> [(c, k)]
        self.paths = OrderedDict()
        row_scalar = {}
        for v, (i, j, k, l) in zip(self.val, self.idx):
            if v == 0:
                continue
            if row_scalar.setdefault(int(i), int(l)) != int(l):
                raise ValueError("an output coordinate must map to one scalar")
            rows = self.paths.setdefault(int(l), OrderedDict())
            rows.setdefault(int(i), OrderedDict()).setdefault(int(j), []).append((float(v), int(k)))
        # Classes of equal magnitude, in the order of their first entry: the float64 kernels read
        # one value per class from a kernel argument instead of carrying the values as literals,
        # so that they serve every table of this structure to float64 accuracy.
        self.classes = OrderedDict()
        for v in self.val:
            if v != 0:
                self.classes.setdefault(_f32_bits(abs(float(v))), len(self.classes))
        self.class_of = [self.classes[_f32_bits(abs(float(v)))] if v != 0 else 255 for v in self.val]

    def lit(self, c: float, f64: bool) -> str:
        """Coefficient `c` in generated code: a float literal, or (float64 kernels) the value of
        its class in the kernel's coefficient argument `cf`, under the sign of `c`."""
        if not f64:
            return _lit(c)
        return ("-" if c < 0 else "") + f"cf[{self.classes[_f32_bits(abs(float(c)))]}]"

    def path_products(self, rows, f64: bool = False):
        """Distinct `(|c|, k)` of one path -> local product id, and their definitions."""
        ids = OrderedDict()
        for cols in rows.values():
            for terms in cols.values():
                for c, k in terms:
                    ids.setdefault((_f32_bits(abs(c)), k), len(ids))
        defs = []
        for (bits, k), m in ids.items():
            c = struct.unpack("<f", struct.pack("<I", bits))[0]
            defs.append(f"            const {'double' if f64 else 'float'} p{m} = {self.lit(c, f64)} * y[{k}];")
        return ids, defs

    @staticmethod
    def weight_expr(terms, ids):
        """C expression of w_ij and whether it is a bare (possibly negated) product."""
        parts = [(c < 0, ids[(_f32_bits(abs(c)), k)]) for c, k in terms]
        if len(parts) == 1:
            neg, m = parts[0]
            return ("-" if neg else "") + f"p{m}", True
        expr = ""
        for n, (neg, m) in enumerate(parts):
            if n == 0:
                expr = ("-" if neg else "") + f"p{m}"
            else:
                expr += (" - " if neg else " + ") + f"p{m}"
        return expr, False

    def op_counts(self):
        """(products, weight adds, (i, j) pairs, coefficients, rows) - VALU work per edge and lane."""
        prods = sum(len(self.path_products(rows)[0]) for rows in self.paths.values())
        pairs = sum(len(cols) for rows in self.paths.values() for cols in rows.values())
        nnz = sum(len(t) for rows in self.paths.values() for cols in rows.values() for t in cols.values())
        nrows = sum(len(rows) for rows in self.paths.values())
        return prods, nnz - pairs, pairs, nnz, nrows


class Part:
    """A subset of the paths of a table with its local row numbering."""

    def __init__(self, t: Table, paths: list[int], extra_zero_rows=(), extra_zero_paths=()):
        self.t = t
        self.paths = OrderedDict((l, t.paths[l]) for l in paths)
        self.zero_paths = list(extra_zero_paths)      # paths without coefficients: ds = 0
        z_rows = sorted({i for rows in self.paths.values() for i in rows} | set(extra_zero_rows))
        x_rows = sorted({j for rows in self.paths.values() for cols in rows.values() for j in cols})
        self.kZ, self.kX, self.kS = z_rows, x_rows, list(self.paths)
        self.zi = {i: n for n, i in enumerate(self.kZ)}
        self.xj = {j: n for n, j in enumerate(self.kX)}
        self.sl = {l: n for n, l in enumerate(self.kS)}

    def cost(self) -> int:
        return sum(len(terms) for rows in self.paths.values() for cols in rows.values()
                   for terms in cols.values())


def split_parts(t: Table, count: int) -> list[Part]:
    """Split the paths into at most `count` parts that read disjoint sets of x rows.

    Paths are first grouped by the x rows they read (one group per x irrep block), so a
    part's x gathers and dx scatters are never repeated by another part; the groups are
    then packed into parts of similar work, largest first.
    """
    def path_cost(l):
        return sum(len(terms) for cols in t.paths[l].values() for terms in cols.values())

    groups = []  # [set of x rows, [paths]]
    for l, rows in t.paths.items():
        xs = {j for cols in rows.values() for j in cols}
        merged = [xs, [l]]
        rest = []
        for g in groups:
            if g[0] & merged[0]:
                merged = [g[0] | merged[0], g[1] + merged[1]]
            else:
                rest.append(g)
        groups = rest + [merged]
    groups.sort(key=lambda g: -sum(path_cost(l) for l in g[1]))
    count = max(1, min(count, len(groups)))
    bins = [[] for _ in range(count)]
    load = [0] * count
    for _, paths in groups:
        b = load.index(min(load))
        bins[b] += paths
        load[b] += sum(path_cost(l) for l in paths)
    covered_rows = {i for rows in t.paths.values() for i in rows}
    gap_rows = [i for i in range(t.Z) if i not in covered_rows]
    gap_paths = [l for l in range(t.S) if l not in t.paths]
    return [Part(t, sorted(b), gap_rows if n == 0 else (), gap_paths if n == 0 else ())
            for n, b in enumerate(bins)]


def _arr(name: str, values) -> str:
    body = ", ".join(str(v) for v in values) if values else "0"
    return f"    static constexpr int {name}[{max(len(values), 1)}] = {{{body}}};"


def _mask(indices) -> str:
    """Bit set of small indices; indices past 63 (no leading-layout kernels then) are dropped."""
    return hex(sum(1 << i for i in indices if i < 64))


def emit_edge_fwd(p: Part, f64: bool = False) -> list[str]:
    """`f64`: the float64 form (`edge_fwd_f64`): one double per lane, coefficients from `cf`."""
    V, R = ("Vec<1, double>", "double") if f64 else ("Vec<C>", "float")
    if f64:
        lines = ["    __device__ static __forceinline__ void edge_fwd_f64(const Vec<1, double> *x, const double *y,",
                 "                                                         const Vec<1, double> *s, Vec<1, double> *acc,",
                 "                                                         const double *cf) {"]
    else:
        lines = ["    template <int C>",
                 "    __device__ static __forceinline__ void edge_fwd(const Vec<C> *x, const float *y,",
                 "                                                     const Vec<C> *s, Vec<C> *acc) {"]
    for l, rows in p.paths.items():
        ids, defs = p.t.path_products(rows, f64)
        lines.append(f"        {{  // path {l}: rows {min(rows)}..{max(rows)}")
        lines += defs
        for i, cols in rows.items():
            lines.append("            {")
            first = True
            for j, terms in cols.items():
                expr, bare = Table.weight_expr(terms, ids)
                if not bare:
                    lines.append(f"                const {R} w{j} = {expr};")
                    expr = f"w{j}"
                if first:
                    lines.append(f"                {V} m = vmul(x[{p.xj[j]}], {expr});")
                    first = False
                else:
                    lines.append(f"                m = vfma(x[{p.xj[j]}], {expr}, m);")
            lines.append(f"                acc[{p.zi[i]}] = vfmav(s[{p.sl[l]}], m, acc[{p.zi[i]}]);")
            lines.append("            }")
        lines.append("        }")
    lines.append("    }")
    return lines


def emit_edge_bwd(p: Part, f64: bool = False) -> list[str]:
    """Backward of one edge for the paths of a part.

    Per path l (rows i, x columns j, y components k):
        a_k   = sum_{ij} c_ijk (dm_i x_j)          channel-wise, independent of s and y
        ds_l  = sum_k y_k a_k
        dy_k += sum_channels s_l a_k
        dx_j += w_ij (dm_i s_l),  w_ij = sum_k c_ijk y_k
    One product dm_i x_j per (i, j) pair serves both ds and dy.
    """
    t = p.t
    V, R = ("Vec<1, double>", "double") if f64 else ("Vec<C>", "float")
    if f64:
        lines = ["    // the float64 form of edge_bwd: one double per lane, coefficients from `cf`",
                 "    template <bool kAcc = false, bool kPin = false, typename Dm, typename DsSink>",
                 "    __device__ static __forceinline__ void edge_bwd_f64(const Vec<1, double> *x, const double *y,",
                 "                                                         const Vec<1, double> *s, const Dm &dm,",
                 "                                                         Vec<1, double> *dx, double *dy, const DsSink &ds,",
                 "                                                         const double *cf) {"]
    else:
        lines = ["    // dx (this part's x rows) and dy (all Y) are written here; ds rows go to `ds` path by path.",
                 "    // `dm`: anything indexable by the part's local output row (registers or LDS).",
                 "    // kAcc: dx holds running sums the edge's contributions are added to (else it is overwritten).",
                 "    // kPin: each row's dx sums are computed where the row is (see `pin`); for dm rows read from LDS.",
                 "    template <int C, bool kAcc = false, bool kPin = false, typename Dm, typename DsSink>",
                 "    __device__ static __forceinline__ void edge_bwd(const Vec<C> *x, const float *y,",
                 "                                                     const Vec<C> *s, const Dm &dm,",
                 "                                                     Vec<C> *dx, float *dy, const DsSink &ds) {"]
    dx_init, dy_init = set(), set()
    for l, rows in p.paths.items():
        ids, defs = t.path_products(rows, f64)
        ks = sorted({k for cols in rows.values() for terms in cols.values() for _, k in terms})
        lines.append(f"        {{  // path {l}: rows {min(rows)}..{max(rows)}, y components {ks[0]}..{ks[-1]}")
        lines += defs
        a_init = set()
        for k in ks:
            lines.append(f"            {V} a{k};")
        for i, cols in rows.items():
            zi = p.zi[i]
            lines.append("            {")
            lines.append(f"                const {V} dmi = dm[{zi}];")
            lines.append(f"                const {V} g = vmulv(dmi, s[{p.sl[l]}]);")
            for j, terms in cols.items():
                xj = p.xj[j]
                expr, bare = Table.weight_expr(terms, ids)
                if not bare:
                    lines.append(f"                const {R} w{j} = {expr};")
                    expr = f"w{j}"
                if j in dx_init:
                    lines.append(f"                dx[{xj}] = vfma(g, {expr}, dx[{xj}]);")
                else:
                    lines.append(f"                dx[{xj}] = kAcc ? vfma(g, {expr}, dx[{xj}]) : vmul(g, {expr});")
                    dx_init.add(j)
                lines.append(f"                {{ const {V} pr = vmulv(dmi, x[{xj}]);")
                for c, k in terms:
                    if k in a_init:
                        lines.append(f"                  a{k} = vfma(pr, {t.lit(c, f64)}, a{k});")
                    else:
                        lines.append(f"                  a{k} = vmul(pr, {t.lit(c, f64)});")
                        a_init.add(k)
                lines.append("                }")
            lines.append("            }")
            lines.append("            if (kPin) { " + " ".join(f"pin(dx[{p.xj[j]}]);" for j in cols) + " }")
        first = True
        for k in ks:
            if first:
                lines.append(f"            {V} dsl = vmul(a{k}, y[{k}]);")
                first = False
            else:
                lines.append(f"            dsl = vfma(a{k}, y[{k}], dsl);")
            if k in dy_init:
                lines.append(f"            dy[{k}] = vdot(s[{p.sl[l]}], a{k}, dy[{k}]);")
            else:
                lines.append(f"            dy[{k}] = vdot(s[{p.sl[l]}], a{k});")
                dy_init.add(k)
        lines.append(f"            ds.template put<{l}>(dsl);")
        lines.append("        }")
    for l in p.zero_paths:  # paths no coefficient touches get exact zeros
        lines.append(f"        ds.template put<{l}>({'vzero<1, double>()' if f64 else 'vzero<C>()'});")
    for k in range(t.Y):
        if k not in dy_init:
            lines.append(f"        dy[{k}] = {'0.0' if f64 else '0.f'};")
    lines.append("    }")
    return lines


def emit_part(struct_name: str, p: Part, f64: bool = False) -> list[str]:
    """`f64`: also the float64 forms of the arithmetic (for the parts the float64 kernels use)."""
    t = p.t
    out = [f"struct {struct_name} {{",
           f"    static constexpr int X = {t.X}, Y = {t.Y}, S = {t.S}, Z = {t.Z};",
           f"    static constexpr int NX = {len(p.kX)}, NS = {len(p.kS)}, NZ = {len(p.kZ)};",
           _arr("kX", p.kX), _arr("kS", p.kS), _arr("kZ", p.kZ),
           "    // x coordinates whose dx, and paths whose ds, this part writes (bit per index)",
           f"    static constexpr unsigned long long kDxMask = {_mask(p.kX)}ull, "
           f"kDsMask = {_mask(list(p.kS) + list(p.zero_paths))}ull;", ""]
    out += emit_edge_fwd(p)
    out.append("")
    out += emit_edge_bwd(p)
    if f64:
        out.append("")
        out += emit_edge_fwd(p, f64=True)
        out.append("")
        out += emit_edge_bwd(p, f64=True)
    out += ["};", ""]
    return out


def build_table(x_irreps, y_irreps, out_filter):
    tp = TensorProduct((x_irreps, y_irreps), out_filter, normalization="SQRT_DIM_OUT")
    mix = ScalarMixing(tp.target)
    idx = tp.indices.astype(np.int64)
    idx4 = np.concatenate([idx, mix.mix_indices[idx[:, 0]][:, None]], axis=1)
    return Table(tp.values, idx4, tp.source[0].dim, tp.source[1].dim, tp.target.dim, mix.num_irreps), tp


def emit_signature(sig_id: int, name: str, x_irreps: str, y_irreps: str, out_filter: str,
                   channels: int) -> str:
    t, tp = build_table(x_irreps, y_irreps, out_filter)
    desc = (f"{name}: x {tp.source[0]} | y {tp.source[1]} -> {tp.target}, "
            f"K={channels}, trailing, nnz={len(t.val)}")
    return emit_table_source(t, name, desc, channels, symbols=(f"kSignature_{2 * sig_id}",
                                                                 f"kSignature_{2 * sig_id + 1}"))


def plugin_launch(channels: int):
    """Launch shapes of a signature compiled at run time: the default variant of each pass."""
    if channels % 128 == 0:
        trailing = dict(fwd=[(1, 4, 1)], bwd=[(2, 4, 3)], bwd_tile=[LAUNCH[128]["bwd_tile"][0]])
    elif channels % 64 == 0:
        trailing = dict(fwd=[(1, 4, 1)], bwd=[(1, 4, 2)], bwd_tile=[LAUNCH[64]["bwd_tile"][0]])
    else:
        trailing = dict(fwd=[(1, 4, 1)], bwd=[(1, 4, 2)])
    width = min(channels, 64)
    leading = None
    if channels % width == 0 and width >= 4 and (width & (width - 1)) == 0:  # power-of-two wave width
        parts = 3 if channels >= 64 else 2
        leading = dict(fwd=[(4, 1)], bwd=[(parts, parts)])
    return trailing, leading


def supports(t: "Table", channels: int) -> bool:
    """Whether the kernel templates can take this table (register-resident dy sums, bit masks)."""
    return t.Y <= 64 and t.X <= 64 and t.S <= 64 and t.Z <= 255 and channels >= 1


def emit_table_source(t: "Table", name: str, desc: str, channels: int, symbols, include='"../unrolled.h"',
                      launch=None, lead="builtin", plugin: bool = False) -> str:
    """HIP source of the kernels and registry entries of one table at one channel count.

    `symbols`: names of the trailing- and leading-layout `Signature` objects.  `plugin` adds
    the C accessor a run-time compiled library is loaded through.
    """
    launch = LAUNCH[channels] if launch is None else launch
    vals = ", ".join(_lit(v) for v in t.val)
    idxs = ", ".join(str(int(a)) for row in t.idx for a in row)
    out = [
        "// GENERATED by e3j_amd/codegen/gen_conv.py -- do not edit.",
        f"// {desc}",
        f"#include {include}",
        "#include " + include.replace("unrolled.h", "unrolled_f64.h"),
        "#include " + include.replace("unrolled.h", "unrolled_f16.h"),
        "",
        "namespace e3j_amd {",
        "namespace {",
        "",
    ]
    if lead == "builtin":
        lead = LAUNCH_LEADING[channels] if (t.X <= 64 and t.S <= 64) else None
    tile = launch.get("bwd_tile", [])
    # float64 kernels: trailing layout, whole waves of channels, few enough coefficient classes
    f64 = channels % 64 == 0 and 0 < len(t.classes) <= F64_MAX_CLASSES
    f16 = channels % 64 == 0   # float16 kernels: trailing layout, whole waves of channels
    splits = sorted({v[2] for v in launch["fwd"] + launch["bwd"] + tile} |
                    ({v[1] for v in lead["fwd"] + lead["bwd"]} if lead else set()) |
                    (set(F64_SPLIT) if f64 else set()) | (set(F16_SHAPE[channels % 128 == 0][1:]) if f16 else set()))
    part_names = {}
    for zs in splits:
        names = []
        for n, part in enumerate(split_parts(t, zs)):
            sname = f"Sig_{name}_z{zs}p{n}"
            out += emit_part(sname, part, f64=f64 and zs in F64_SPLIT)
            names.append(sname)
        part_names[zs] = ", ".join(names)
    fwd_args = ["    const float *, const float *, const float *, const int32_t *, const int32_t *,",
                "    const int32_t *, const int32_t *, float *, int, float, unsigned);"]
    bwd_args = ["    const float *, const float *, const float *, const float *, const int32_t *,",
                "    const int32_t *, const int32_t *, const int32_t *, float *, float *, float *, int, float,",
                "    unsigned);"]
    out += ["}  // namespace", "", "// both passes: the device pass needs the kernels instantiated"]
    fwd_args_trailing = [fwd_args[0], fwd_args[1].replace("unsigned);", "unsigned, int, int, const int32_t *, int);")]
    for v in launch["fwd"]:
        cpl, wpb, zs, minw = (*v, 1)[:4]
        out += [f"template __global__ void unrolled_fwd_kernel<{channels}, {cpl}, {wpb}, {minw}, "
                f"{part_names[zs]}>("] + fwd_args_trailing
    for v in launch["bwd"]:
        cpl, wpb, zs, minw = (*v, 1)[:4]
        for ordered in ("false", "true"):
            out += [f"template __global__ void unrolled_bwd_kernel<{channels}, {cpl}, {wpb}, {minw}, {ordered}, "
                    f"{part_names[zs]}>("] + bwd_args
    tile_args = ["    const float *, const float *, const float *, const float *, const int32_t *,",
                 "    const int32_t *, const int32_t *, const int32_t *, const int32_t *, float *, float *, float *,",
                 "    int, int, int, float, unsigned);"]
    for v in tile:
        cpl, wpb, zs, minw = (*v, 1)[:4]
        out += [f"template __global__ void unrolled_bwd_tile_kernel<{channels}, {cpl}, {wpb}, {minw}, "
                f"{part_names[zs]}>("] + tile_args
    # sender-grouped backward: the finest split of the paths (parts run one after another in a wave)
    sender_split = max(v[2] for v in launch["bwd"] + tile)
    sender_minw = 2
    out += [f"template __global__ void unrolled_bwd_sender_kernel<{channels}, 4, {sender_minw}, "
            f"{part_names[sender_split]}>("] + bwd_args
    if f16:
        as_f16 = lambda lines: [ln.replace("float *", "half_t *") for ln in lines]  # noqa: E731
        h_cpl, h_fwd, h_bwd = F16_SHAPE[channels % 128 == 0]
        out += [f"template __global__ void unrolled_fwd_f16_kernel<{channels}, {h_cpl}, 4, {part_names[h_fwd]}>("] + as_f16(fwd_args)
        out += [f"template __global__ void unrolled_bwd_f16_kernel<{channels}, {h_cpl}, 4, {part_names[h_bwd]}>("] + as_f16(bwd_args)
    if f64:
        as_f64 = lambda lines: [ln.replace("float", "double").replace("unsigned);", "unsigned, F64Coefs);")  # noqa: E731
                                for ln in lines]
        out += [f"template __global__ void unrolled_fwd_f64_kernel<{channels}, 4, {part_names[F64_SPLIT[0]]}>("] + as_f64(fwd_args)
        out += [f"template __global__ void unrolled_bwd_f64_kernel<{channels}, 4, {part_names[F64_SPLIT[1]]}>("] + as_f64(bwd_args)
    if lead:
        for wpb, zs in lead["fwd"]:
            out += [f"template __global__ void unrolled_fwd_leading_kernel<{channels}, {wpb}, {part_names[zs]}>("] + fwd_args
        for wpb, zs in lead["bwd"]:
            for ordered in ("false", "true"):
                out += [f"template __global__ void unrolled_bwd_leading_kernel<{channels}, {ordered}, "
                        f"{part_names[zs]}>("] + bwd_args

    fwd_sig = ["(const e3j_amd_conv_params &p, const float *x, const float *y, const float *s,",
               "                   const int32_t *sender, const int32_t *row_ptr, const int32_t *perm,",
               "                   float *out, hipStream_t stream) {"]
    bwd_sig = ["(const e3j_amd_conv_params &p, const float *x, const float *y, const float *s,",
               "                   const float *dm, const int32_t *sender, const int32_t *row_ptr,",
               "                   const int32_t *perm, float *dx, float *dy, float *ds, hipStream_t stream,",
               "                   OrderedBwd *ordered) {"]

    def switch(variants, call):
        body = ["    switch (VARIANT) {"]
        for n, v in reversed(list(enumerate(variants))):
            label = f"case {n}:" if n else "default:"
            body.append(f"        {label} return {call(v)}")
        return body + ["    }", "}", ""]

    out += ["", "// host pass only: the registry entries hold host function pointers",
            "#if !defined(__HIP_DEVICE_COMPILE__)",
            f"static const float kVal[] = {{{vals}}};",
            f"static const uint8_t kIdx[] = {{{idxs}}};",
            ""]
    if f16:
        out += ["static int run_fwd_f16(const e3j_amd_conv_params &p, const half_t *x, const half_t *y, const half_t *s,",
                "                       const int32_t *sender, const int32_t *row_ptr, const int32_t *perm, half_t *out,",
                "                       hipStream_t stream) {",
                f"    return launch_unrolled_fwd_f16<{channels}, {h_cpl}, 4, {part_names[h_fwd]}>(",
                "        p, x, y, s, sender, row_ptr, perm, out, stream);",
                "}",
                "static int run_bwd_f16(const e3j_amd_conv_params &p, const half_t *x, const half_t *y, const half_t *s,",
                "                       const half_t *dm, const int32_t *sender, const int32_t *row_ptr,",
                "                       const int32_t *perm, half_t *dx, half_t *dy, half_t *ds, hipStream_t stream) {",
                f"    return launch_unrolled_bwd_f16<{channels}, {h_cpl}, 4, {t.Y}, {t.X}, {part_names[h_bwd]}>(",
                "        p, x, y, s, dm, sender, row_ptr, perm, dx, dy, ds, stream);",
                "}", ""]
    if f64:
        out += ["// class of equal magnitude of every entry (the float64 kernels read one coefficient per class)",
                f"static const uint8_t kClass[] = {{{', '.join(str(c) for c in t.class_of)}}};",
                "static int run_fwd_f64(const e3j_amd_conv_params &p, const double *x, const double *y, const double *s,",
                "                       const int32_t *sender, const int32_t *row_ptr, const int32_t *perm, double *out,",
                "                       hipStream_t stream) {",
                f"    return launch_unrolled_fwd_f64<{channels}, 4, {part_names[F64_SPLIT[0]]}>(",
                "        p, x, y, s, sender, row_ptr, perm, out, stream);",
                "}",
                "static int run_bwd_f64(const e3j_amd_conv_params &p, const double *x, const double *y, const double *s,",
                "                       const double *dm, const int32_t *sender, const int32_t *row_ptr,",
                "                       const int32_t *perm, double *dx, double *dy, double *ds, hipStream_t stream) {",
                f"    return launch_unrolled_bwd_f64<{channels}, 4, {t.Y}, {t.X}, {part_names[F64_SPLIT[1]]}>(",
                "        p, x, y, s, dm, sender, row_ptr, perm, dx, dy, ds, stream);",
                "}", ""]
    out += ["static int run_fwd" + fwd_sig[0]] + fwd_sig[1:]
    out += [ln.replace("VARIANT", "tuning().fwd_variant.load(std::memory_order_relaxed)") for ln in switch(
        launch["fwd"], lambda v: f"launch_unrolled_fwd<{channels}, {v[0]}, {v[1]}, {(*v, 1)[3]}, {part_names[v[2]]}>("
                                 "p, x, y, s, sender, row_ptr, perm, out, stream);")]
    out += ["static int run_bwd" + bwd_sig[0]] + bwd_sig[1:]
    out += [ln.replace("VARIANT", "tuning().bwd_variant.load(std::memory_order_relaxed)") for ln in switch(
        launch["bwd"], lambda v: f"launch_unrolled_bwd<{channels}, {v[0]}, {v[1]}, {(*v, 1)[3]}, {t.Y}, {t.X}, "
                                 f"{part_names[v[2]]}>(p, x, y, s, dm, sender, row_ptr, perm, dx, dy, ds, stream, ordered);")]
    if tile:
        out += ["static int run_bwd_tiled(const e3j_amd_conv_params &p, const float *x, const float *y,",
                "                         const float *s, const float *dm, const e3j_amd_tile_schedule &schedule,",
                "                         float *dx, float *dy, float *ds, hipStream_t stream) {"]
        out += [ln.replace("VARIANT", "tuning().bwd_variant.load(std::memory_order_relaxed)") for ln in switch(
            tile, lambda v: f"launch_unrolled_bwd_tile<{channels}, {v[0]}, {v[1]}, {(*v, 1)[3]}, {t.Y}, {t.X}, "
                            f"{part_names[v[2]]}>(p, x, y, s, dm, schedule, dx, dy, ds, stream);")]
        out += ["static int run_tile_row_bytes() {"]
        out += [ln.replace("VARIANT", "tuning().bwd_variant.load(std::memory_order_relaxed)") for ln in switch(
            tile, lambda v: f"tile_row_bytes<{v[0]}, {part_names[v[2]]}>();")]
        out += ["static int run_tile_rows_default() {"]
        out += [ln.replace("VARIANT", "tuning().bwd_variant.load(std::memory_order_relaxed)") for ln in switch(
            tile, lambda v: f"{v[4] if len(v) > 4 else 8};")]
    out += ["static int run_bwd_sender(const e3j_amd_conv_params &p, const float *x, const float *y, const float *s,",
            "                          const float *dm, const int32_t *receiver_t, const int32_t *row_ptr,",
            "                          const int32_t *perm, float *dx, float *dy, float *ds, hipStream_t stream) {",
            f"    return launch_unrolled_bwd_sender<{channels}, 4, {sender_minw}, {t.Y}, {part_names[sender_split]}>(",
            "        p, x, y, s, dm, receiver_t, row_ptr, perm, dx, dy, ds, stream);",
            "}", ""]
    tiled = "&run_bwd_tiled, &run_tile_row_bytes, &run_tile_rows_default" if tile else "nullptr, nullptr, nullptr"
    out += [f"extern const Signature {symbols[0]} = {{",
            f'    "{desc}",',
            f"    {t.X}, {t.Y}, {t.Z}, {t.S}, {len(t.val)}, {channels}, E3J_AMD_LAYOUT_TRAILING, kVal, kIdx,",
            f"    &run_fwd, &run_bwd, {tiled}, &run_bwd_sender,",
            f"    {len(t.classes)}, kClass, &run_fwd_f64, &run_bwd_f64," if f64 else "    0, nullptr, nullptr, nullptr,",
            "    &run_fwd_f16, &run_bwd_f16," if f16 else "    nullptr, nullptr,",
            "};", ""]
    if lead:
        out += ["static int run_fwd_leading" + fwd_sig[0]] + fwd_sig[1:]
        out += [ln.replace("VARIANT", "tuning().fwd_variant.load(std::memory_order_relaxed)") for ln in switch(
            lead["fwd"], lambda v: f"launch_unrolled_fwd_leading<{channels}, {v[0]}, {part_names[v[1]]}>("
                                   "p, x, y, s, sender, row_ptr, perm, out, stream);")]
        out += ["static int run_bwd_leading" + bwd_sig[0]] + bwd_sig[1:]
        out += [ln.replace("VARIANT", "tuning().bwd_variant.load(std::memory_order_relaxed)") for ln in switch(
            lead["bwd"], lambda v: f"launch_unrolled_bwd_leading<{channels}, {t.Y}, {t.X}, "
                                   f"{part_names[v[1]]}>(p, x, y, s, dm, sender, row_ptr, perm, dx, dy, ds, stream, ordered);")]
        out += [f"extern const Signature {symbols[1]} = {{",
                f'    "{desc.replace("trailing", "leading")}",',
                f"    {t.X}, {t.Y}, {t.Z}, {t.S}, {len(t.val)}, {channels}, E3J_AMD_LAYOUT_LEADING, kVal, kIdx,",
                "    &run_fwd_leading, &run_bwd_leading, nullptr, nullptr,",
                "};"]
    else:  # no leading-layout kernels: an entry that never matches keeps the numbering regular
        out += [f"extern const Signature {symbols[1]} = {{",
                f'    "{desc.replace("trailing", "leading (not built)")}",',
                "    -1, -1, -1, -1, -1, -1, E3J_AMD_LAYOUT_LEADING, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr,",
                "};"]
    if plugin:
        out += ["",
                "// entry point of a run-time compiled signature library: 0 trailing, 1 leading layout",
                'extern "C" const void *e3j_amd_plugin_signature(int which) {',
                f"    return which == 0 ? &{symbols[0]} : which == 1 ? &{symbols[1]} : nullptr;",
                "}"]
    out += ["#endif",
            "",
            "}  // namespace e3j_amd",
            ""]
    return "\n".join(out)


def emit_registry(count: int) -> str:
    out = ["// GENERATED by e3j_amd/codegen/gen_conv.py -- do not edit.",
           '#include "../common.h"', "", "namespace e3j_amd {", ""]
    for n in range(count):
        out.append(f"extern const Signature kSignature_{n};")
    out += ["", f"int num_builtin_signatures() {{ return {count}; }}", "",
            "const Signature &builtin_signature(int id) {",
            "    static const Signature *const table[] = {" +
            ", ".join(f"&kSignature_{n}" for n in range(count)) + (", " if count else "") + "nullptr};",
            "    return *table[id];", "}", "", "}  // namespace e3j_amd", ""]
    return "\n".join(out)


def _write_if_changed(path: str, text: str) -> None:
    if os.path.exists(path):
        with open(path) as fh:
            if fh.read() == text:
                return
    with open(path, "w") as fh:
        fh.write(text)


def write_all(out_dir: str, signatures=None) -> list[str]:
    signatures = BUILTIN_SIGNATURES if signatures is None else signatures
    os.makedirs(out_dir, exist_ok=True)
    wanted = {"registry.hip"}
    paths = []
    for n, (name, xi, yi, oi, k) in enumerate(signatures):
        fname = f"sig_{name}.hip"
        wanted.add(fname)
        _write_if_changed(os.path.join(out_dir, fname), emit_signature(n, name, xi, yi, oi, k))
        paths.append(os.path.join(out_dir, fname))
    _write_if_changed(os.path.join(out_dir, "registry.hip"), emit_registry(2 * len(signatures)))
    for stale in os.listdir(out_dir):
        if stale.startswith("sig_") and stale.endswith(".hip") and stale not in wanted:
            os.remove(os.path.join(out_dir, stale))
    return paths


if __name__ == "__main__":
    here = os.path.dirname(os.path.abspath(__file__))
    for p in write_all(os.path.join(os.path.dirname(here), "csrc", "generated")):
        print(p)
