"""Option enums and the small configuration object of the fused convolution path.

Mirrors the option names of the reference (`src/e3j/utils/options.py:76-180`,
`src/e3j/utils/config.py:42-216`) for the one path this package implements.
There is deliberately no unfused/CPU evaluation strategy here: the only
evaluation strategy is the HIP kernel library, and it fails loudly when the
library is missing.
"""

from __future__ import annotations

import contextlib
import dataclasses
import os
from enum import Enum


class _ParsedEnum(Enum):
    """Enum with a forgiving `parse` accepting members, names and values."""

    @classmethod
    def parse(cls, value):
        if isinstance(value, cls):
            return value
        if isinstance(value, str):
            key = value.strip().upper()
            if key in cls.__members__:
                return cls.__members__[key]
        for member in cls:
            if member.value == value:
                return member
        raise ValueError(f"{value!r} is not a valid {cls.__name__}; "
                         f"expected one of {list(cls.__members__)}")


class Layout(_ParsedEnum):
    """Memory layout of equivariant arrays (`src/e3j/utils/options.py:122-151`).

    LEADING_CHANNELS: `(rows, channels, dim)`; TRAILING_CHANNELS: `(rows, dim, channels)`.
    The integer values are the ones the reference hands to its FFI.
    """

    LEADING_CHANNELS = 0
    TRAILING_CHANNELS = 1


class GraphOrdering(_ParsedEnum):
    """Edge ordering contract (`src/e3j/utils/options.py:95-112`).

    RECEIVER / SENDER: edges sorted by that endpoint. NONE: no ordering is
    promised; the kernel library then sorts on the device before reducing.
    """

    RECEIVER = "RECEIVER"
    SENDER = "SENDER"
    NONE = "NONE"


class MixingMode(_ParsedEnum):
    """How a bilinear product mixes the channel axes (`src/e3j/utils/options.py:154-168`).

    OUTER: `u, v -> (u, v)` (also broadcasts an operand without channel axis); INNER:
    `v, v -> 1`; MAP: `v, v -> v`.  The integer values are the ones the reference hands to
    its FFI.
    """

    OUTER = 0
    INNER = 1
    MAP = 2


class TensorProductNormalization(_ParsedEnum):
    """Scaling of the stacked Clebsch-Gordan blocks (`src/e3j/utils/options.py:171-180`)."""

    NONE = "NONE"
    SQRT_DIM_OUT = "SQRT_DIM_OUT"


class Convolution(_ParsedEnum):
    """Evaluation strategy of `e3j_amd.Convolution` (`src/e3j/utils/options.py:76-92`).

    FUSED_HIP is the only strategy: hand-written gfx950 kernels behind the C ABI.
    """

    FUSED_HIP = "FUSED_HIP"


@dataclasses.dataclass(frozen=True)
class Config:
    """Frozen settings snapshot (`src/e3j/utils/config.py:42-105`)."""

    layout: Layout = Layout.TRAILING_CHANNELS
    convolution: Convolution = Convolution.FUSED_HIP
    #: 0 = asynchronous launches; >0 = synchronise the stream after each launch
    #: so that device-side failures surface at the faulting call.
    debug_level: int = 0
    #: atomic-free backward for `dx` (bit-reproducible, slower).
    deterministic: bool = False
    #: sweeps of label propagation behind the locality-aware row order of the kernels
    #: (0 = rows are processed in index order).
    locality_rounds: int = 2
    #: keep the adjacencies prepared for the index tensors seen last and reuse them when the same
    #: tensors (identity and in-place version) come again.  Off by default: a buffer rewritten behind
    #: torch's back (raw pointer, DLPack, `.data`) would get a stale adjacency; `prepare_graph`
    #: handles are the explicit way to reuse one.
    graph_cache: bool = False
    #: receivers per tile of the backward that sums dx per (tile, sender) on chip before the float
    #: atomics and shares long rows between workgroups (trailing layout, unrolled kernels, at least
    #: 64 channels; capped by what the LDS holds).  -1: the size the kernel of the signature is
    #: tuned for; 0: one wave per receiver and one set of atomics per edge (no schedule to build).
    tile_rows: int = -1
    #: put rows that share most of their senders side by side in the row order, so that the tiles
    #: of the default backward (two receivers at K = 128) sum more dx contributions on chip: 19 %
    #: fewer atomic requests and a 2-3 % faster backward at 1M edges, for 0.28 ms more graph
    #: preparation.  "prepared" (default): only for the handles of `prepare_graph`, whose adjacency
    #: serves many calls; True: also for the adjacency an operator call prepares for itself; False: never
    pair_rows: object = "prepared"
    #: positions of a row one wave of the forward pass sums; longer rows are shared between waves
    #: (their sums then come from float atomics).  -1: twice the mean row length, at least 64;
    #: 0: never share a row.
    row_cap: int = -1
    #: add the pieces of a shared row to its output row in a fixed order (a scratch row per piece,
    #: up to 256 MB per prepared graph; the forward then gives the same bits in every run, as the
    #: reference's does); off: the pieces are added with float atomics (no scratch, and about 0.1 ms
    #: less for a hub of 50 000 edges)
    fixed_order_rows: bool = True
    #: compile unrolled kernels at run time for coefficient tables the library was not built
    #: for (needs hipcc; about half a minute per new table, cached on disk); off: such tables
    #: run the table-driven kernels.
    jit: bool = False


class _ConfigHolder:
    """Mutable process-wide holder with `use(**kw)` scoping (`src/e3j/utils/config.py:107-216`)."""

    def __init__(self):
        self._current = Config(
            debug_level=int(os.environ.get("E3J_AMD_DEBUG", "0")),
            deterministic=os.environ.get("E3J_AMD_DETERMINISTIC", "0") not in ("0", ""),
            locality_rounds=int(os.environ.get("E3J_AMD_LOCALITY_ROUNDS", "2")),
            tile_rows=int(os.environ.get("E3J_AMD_TILE_ROWS", "-1")),
            row_cap=int(os.environ.get("E3J_AMD_ROW_CAP", "-1")),
            fixed_order_rows=os.environ.get("E3J_AMD_FIXED_ORDER_ROWS", "1") not in ("0", ""),
            pair_rows={"0": False, "": False, "1": True}.get(os.environ.get("E3J_AMD_PAIR_ROWS", "prepared"),
                                                             "prepared"),
            graph_cache=os.environ.get("E3J_AMD_GRAPH_CACHE", "0") not in ("0", ""),
            jit=os.environ.get("E3J_AMD_JIT", "0") not in ("0", ""),
        )

    def __call__(self, **updates) -> Config:
        if updates:
            self._current = self._coerce(updates)
        return self._current

    def _coerce(self, updates) -> Config:
        fields = {f.name for f in dataclasses.fields(Config)}
        unknown = set(updates) - fields
        if unknown:
            raise TypeError(f"unknown config field(s): {sorted(unknown)}")
        if "layout" in updates:
            updates["layout"] = Layout.parse(updates["layout"])
        if "convolution" in updates:
            updates["convolution"] = Convolution.parse(updates["convolution"])
        return dataclasses.replace(self._current, **updates)

    @contextlib.contextmanager
    def use(self, **updates):
        previous = self._current
        self._current = self._coerce(updates)
        try:
            yield self._current
        finally:
            self._current = previous

    def snapshot(self, config: Config | None = None) -> Config:
        """Modules freeze the settings they were built under."""
        return self._current if config is None else config


config = _ConfigHolder()
