"""The fused convolution operators: `convolution` and `convolution_bwd`.

Same signatures, argument meaning and errors as the reference's primitives
(`src/e3j/ops/convolution.py:106-116,334-345`), with tensors in GPU memory
and the HIP library of this package behind them instead of the CUDA `e3j_ops`
binding.  `convolution` is differentiable in `(x, y, s)` to any reverse-mode
order: its backward is `convolution_bwd`, whose own backward is expressed with
three `convolution` and three `convolution_bwd` calls
(`src/e3j/ops/convolution.py:535-562`).

Extensions over the reference's operator: a `layout` keyword (the reference's
fused kernel is trailing-channels only), any channel count (no power-of-two
rule), and `GraphOrdering.NONE` (edges are sorted on the device first).
"""

from __future__ import annotations

import ctypes
import dataclasses
import warnings
import weakref

import numpy as np
import torch

from . import _lib
from .coef import Coef4D
from .graph import (RowSegments, TileSchedule, csr_row_ptr, fold_endpoints, locality_order,
                    pair_rows, row_cap_for, row_piece_for, sort_edges, wrap_global_index, ROW_PIECE)
from .options import GraphOrdering, Layout, config


@dataclasses.dataclass
class ConvolutionParams:
    """Static sizes of the operator (`src/e3j/ops/convolution.py:81-84`)."""

    num_out: int
    num_scalars: int


#: name used by code written against the reference
CUDAConvolutionParams = ConvolutionParams


class ConvolutionBatchingWarning(UserWarning):
    """Emitted when the convolution is batched over graph adjacencies."""


class TableDrivenKernelWarning(UserWarning):
    """Emitted once per coefficient table that runs the table-driven kernels (no built-in
    unrolled kernel and run-time compilation switched off): they are an order of magnitude
    slower than the unrolled ones."""


_VAL_DTYPES = {torch.float32: (_lib.F32, np.float32), torch.float64: (_lib.F64, np.float64),
               torch.float16: (_lib.F16, np.float16)}


class _Table:
    """A packed coefficient table with its device copies and kernel selection."""

    _cache: dict = {}

    def __init__(self, packed: np.ndarray, val_np_dtype):
        self.packed = np.ascontiguousarray(packed)
        self.idx_bytes = self.packed.dtype.itemsize
        self.val_np_dtype = np.dtype(val_np_dtype)
        self.num_coef = int(self.packed.shape[0])
        self._device = {}
        self._signature = {}
        self._signed = {}
        self._plans = {}   # (device, value dtype, sizes) -> (plan of the table-driven kernels, taken)

    #: tables by the identity of the packed array (a module hands over the same array on every
    #: call): the bytes of a table are hashed once, not per call
    _by_identity: dict = {}

    @classmethod
    def get(cls, coef, val_np_dtype) -> "_Table":
        if isinstance(coef, torch.Tensor):
            raise TypeError("`coef` must be concrete: it is read on the host.")
        val_key = np.dtype(val_np_dtype).str
        seen = cls._by_identity.get((id(coef), val_key))
        if seen is not None and seen[0]() is coef:
            return seen[1]
        packed = np.asarray(coef)
        if packed.dtype not in (np.dtype(np.uint8), np.dtype(np.int32)):
            raise TypeError(f"unsupported coefficient index dtype {packed.dtype}")
        key = (packed.dtype.str, packed.shape, packed.tobytes(), val_key)
        table = cls._cache.get(key)
        if table is None:
            if len(cls._cache) > 256:
                cls._cache.clear()
            table = cls._cache[key] = cls(packed, val_np_dtype)
        if isinstance(coef, np.ndarray) and not coef.flags.writeable:
            # only arrays that cannot change under the cache (modules freeze their packed tables)
            ident = (id(coef), val_key)
            if len(cls._by_identity) > 256:
                cls._by_identity.clear()
            cls._by_identity[ident] = (weakref.ref(coef, lambda _, k=ident: cls._by_identity.pop(k, None)), table)
        return table

    def signed(self, y_parity) -> "_Table":
        """The table with the parity signs of y folded in (SENDER ordering), built once per parity."""
        key = np.asarray(y_parity, dtype=np.float64).tobytes()
        hit = self._signed.get(key)
        if hit is None:
            c = self.unpack()
            signs = np.asarray(y_parity, dtype=c.val.dtype)[c.idx[:, 2].astype(np.int64)]
            hit = self._signed[key] = _Table.get(Coef4D(c.val * signs, c.idx, c.val_dtype, c.idx_dtype).pack(),
                                                 self.val_np_dtype)
        return hit

    def unpack(self) -> Coef4D:
        return Coef4D.unpack(self.packed, self.val_np_dtype)

    def device(self, device: torch.device) -> torch.Tensor:
        t = self._device.get(device)
        if t is None:
            t = torch.from_numpy(self.packed.view(np.uint8).reshape(-1).copy()).to(device)
            self._device[device] = t
        return t

    def signature(self, dims, channels: int, layout: Layout):
        """`(id, scale, y_flip)` of a built-in unrolled kernel, `(-1, 1.0, 0)` if none matches.

        `y_flip`: bit mask of the y components whose coefficients carry the opposite sign of
        the built-in table (the parity signs of the SENDER ordering).  For a float64 table `scale`
        is not a number but the array of coefficient classes the float64 kernels read
        (`e3j_amd_conv_params.coef_classes`, kept alive by this table).
        """
        jit = config().jit
        key = (dims, channels, layout, jit)
        hit = self._signature.get(key)
        if hit is None:
            scale, flip = ctypes.c_float(1.0), ctypes.c_uint32(0)
            val_code = {np.dtype(np.float32): _lib.F32, np.dtype(np.float64): _lib.F64,
                        np.dtype(np.float16): _lib.F16}[self.val_np_dtype]

            classes = (ctypes.c_double * _lib.F64_CLASSES)()

            def find():
                if self.val_np_dtype == np.float64:
                    return int(_lib.load().e3j_amd_find_signature_f64(
                        self.packed.ctypes.data, self.idx_bytes, self.num_coef, dims[0], dims[1], dims[2],
                        dims[3], channels, layout.value, classes, ctypes.byref(flip)))
                return int(_lib.load().e3j_amd_find_signature(
                    self.packed.ctypes.data, self.idx_bytes, val_code, self.num_coef, dims[0], dims[1],
                    dims[2], dims[3], channels, layout.value, ctypes.byref(scale), ctypes.byref(flip)))

            sig = find()
            if sig < 0 and jit and self.num_coef > 0:
                # not built in: generate and compile the kernels of this table, then look again
                from . import jit as _jit
                c = self.unpack()
                if _jit.register(c.val, c.idx.astype(np.int64), dims, channels):
                    sig = find()
            if sig < 0 and not jit and self.val_np_dtype == np.float32:
                warnings.warn(
                    f"no unrolled kernel is built for this coefficient table (x {dims[0]}, y {dims[1]}, "
                    f"out {dims[2]}, paths {dims[3]}, {channels} channels, {layout.name.lower()}): the "
                    "table-driven kernels serve it, an order of magnitude slower; config(jit=True) "
                    "(or E3J_AMD_JIT=1) compiles unrolled kernels for it with hipcc on first use",
                    TableDrivenKernelWarning, stacklevel=3)
            hit = self._signature[key] = (sig, classes if self.val_np_dtype == np.float64 else float(scale.value),
                                          int(flip.value))
        return hit


@dataclasses.dataclass
class _Meta:
    """Everything static about one call."""

    table: _Table
    signed_table: _Table | None  # forward table under SENDER ordering
    params: ConvolutionParams
    ordering: GraphOrdering
    layout: Layout
    y_parity: np.ndarray | None
    num_nodes: int
    squeeze_channels: bool       # x was (N, X): channel axis added internally
    y_shape: tuple


def _stream(device) -> int:
    return int(torch.cuda.current_stream(device).cuda_stream)


def _shape(meta: _Meta, x: torch.Tensor, y: torch.Tensor, s: torch.Tensor):
    """`((num_x, num_y, num_out, num_scalars), channels)` of a call."""
    if meta.layout == Layout.TRAILING_CHANNELS:
        num_x, channels, num_s = x.shape[1], x.shape[2], s.shape[1]
    else:
        channels, num_x, num_s = x.shape[1], x.shape[2], s.shape[2]
    return (int(num_x), int(y.shape[1]), int(meta.params.num_out), int(num_s)), int(channels)


def _fill_params(meta: _Meta, x: torch.Tensor, y: torch.Tensor, s: torch.Tensor, table: _Table,
                 use_signature: bool = True, row_order: torch.Tensor | None = None):
    layout = meta.layout
    val_code = _VAL_DTYPES[x.dtype][0]
    dims, channels = _shape(meta, x, y, s)
    sig, scale, flip = table.signature(dims, channels, layout) if use_signature else (-1, 1.0, 0)
    cfg = config()
    p = _lib.ConvParams(
        num_nodes=int(x.shape[0]), num_edges=int(y.shape[0]), num_coef=table.num_coef,
        num_x=dims[0], num_y=dims[1], num_out=dims[2], num_scalars=dims[3], channels=int(channels),
        layout=layout.value, val_dtype=val_code, coef_idx_bytes=table.idx_bytes,
        signature=sig, coef_scale=scale if isinstance(scale, float) else 1.0, debug=int(cfg.debug_level),
        y_flip=flip, row_order=row_order.data_ptr() if row_order is not None else None)
    if sig >= 0 and not isinstance(scale, float):   # float64: the classes of the table (host memory of the table)
        p.coef_classes = ctypes.cast(scale, ctypes.c_void_p).value
    return p, table


def _table_plan(p, table, device) -> torch.Tensor | None:
    """The plan of a table-driven call.  Outside a graph capture it is built once per (table, sizes,
    device) by the status call, which also says whether the planned kernels take the table: later
    calls launch that kernel alone (`PLAN_READY`) or skip planning (`PLAN_NONE`).  While the stream is
    captured (the status call synchronises) a table not seen before gets memory for a plan built
    inside the call, which the caller keeps until the call is enqueued: the library then allocates
    nothing."""
    if p.signature >= 0:
        return None
    lib = _lib.load()
    nbytes = int(lib.e3j_amd_table_plan_bytes(ctypes.byref(p)))
    if nbytes == 0:
        p.table_plan_state = _lib.PLAN_NONE
        return None
    key = (device, int(p.val_dtype), p.num_x, p.num_y, p.num_out, p.num_scalars)
    hit = table._plans.get(key)
    if hit is None:
        plan = torch.empty((nbytes + 3) // 4, dtype=torch.int32, device=device)
        p.table_plan = plan.data_ptr()
        if torch.cuda.is_current_stream_capturing():
            return plan
        status = (ctypes.c_int32 * 4)()
        _lib.check(lib.e3j_amd_table_plan_status(ctypes.byref(p), table.device(device).data_ptr(), 0, status,
                                                 _stream(device)))
        hit = table._plans[key] = (plan, bool(status[0]))
    plan, taken = hit
    p.table_plan = plan.data_ptr() if taken else None
    p.table_plan_state = _lib.PLAN_READY if taken else _lib.PLAN_NONE
    return plan


def _check_operands(x, y, s, sender, receiver):
    for name, t in (("x", x), ("y", y), ("s", s), ("sender", sender), ("receiver", receiver)):
        if not isinstance(t, torch.Tensor):
            raise TypeError(f"`{name}` must be a torch.Tensor")
        if t.device.type != "cuda":
            raise RuntimeError(f"`{name}` must live in GPU memory; e3j_amd has no CPU implementation")
    if x.dtype not in _VAL_DTYPES:
        raise TypeError(f"Fused ops support value dtypes ('float16', 'float32', 'float64'), got {x.dtype}. "
                        "Cast the operands.")
    if y.dtype != x.dtype or s.dtype != x.dtype:
        raise TypeError("x, y and s must share one dtype")


def _row_order(other: torch.Tensor, row_ptr: torch.Tensor, n: int, pair: bool | None = None):
    """Locality-aware processing order of the rows of a CSR, or None when switched off.
    `pair`: also put rows with common senders side by side (None: only if `config().pair_rows` is
    True; the handles of `prepare_graph` ask for it by default)."""
    rounds = config().locality_rounds
    if rounds <= 0 or n < 2 or other.numel() == 0:
        return None
    order = locality_order(other, row_ptr, n, rounds)
    if pair is None:
        pair = config().pair_rows is True
    if pair:
        order = pair_rows(other, row_ptr, n, order)
    return order


#: Opt-in (`config(graph_cache=True)`): adjacencies prepared for the index tensors seen last, keyed by
#: the identity and the in-place version counter of both tensors, dropped when either tensor dies.
#: The version counter only sees writes that go through torch: a buffer rewritten through its raw
#: pointer, a DLPack / numpy view or `.data` keeps its version and would get the adjacency of its
#: old contents.  Callers that reuse an adjacency should hold a `prepare_graph` handle instead.
_GRAPH_CACHE: dict = {}
_GRAPH_CACHE_SIZE = 8


def clear_graph_cache() -> None:
    """Forget the cached adjacencies (only filled under `config(graph_cache=True)`)."""
    _GRAPH_CACHE.clear()


class PreparedGraph:
    """A prepared adjacency: CSR (`other`, `row_ptr`), optional permutation of the edge rows,
    row order and, built on first use, the schedules of the tiled backward.

    Returned by `prepare_graph`; valid for as long as the contents of the index tensors it was
    built from do not change.  It remembers the stream it was prepared on and makes any other
    stream that uses it wait for the preparation.  The scratch rows of the forward's long-row sums
    belong to the handle: calls that share a handle must not overlap on different streams.
    """

    def __init__(self, other, row_ptr, perm, order, num_nodes: int, ordering=None):
        self.other, self.row_ptr, self.perm, self.order = other, row_ptr, perm, order
        self.num_nodes = int(num_nodes)
        self.ordering = ordering
        self._schedules = {}
        self._segments = {}
        self._mark()

    def _mark(self):
        self.stream = torch.cuda.current_stream(self.row_ptr.device)
        self.event = torch.cuda.Event()
        self.event.record(self.stream)

    def ready(self):
        """Order the current stream after the kernels that prepared this adjacency."""
        current = torch.cuda.current_stream(self.row_ptr.device)
        if current != self.stream:
            current.wait_event(self.event)

    @property
    def num_edges(self) -> int:
        return int(self.other.numel())

    def __iter__(self):
        return iter((self.other, self.row_ptr, self.perm, self.order))

    def __getitem__(self, i):
        return (self.other, self.row_ptr, self.perm, self.order)[i]

    def schedule(self, tile_rows: int) -> TileSchedule:
        hit = self._schedules.get(tile_rows)
        if hit is None:
            self.ready()
            hit = self._schedules[tile_rows] = TileSchedule(self.other, self.row_ptr, self.perm, self.order,
                                                            self.num_nodes, tile_rows)
            self._mark()
        return hit


    def segments(self, row_cap: int, row_piece: int = ROW_PIECE) -> RowSegments:
        """The pieces of the rows longer than `row_cap` (second call of the forward pass), of
        `row_piece` positions each."""
        key = (int(row_cap), int(row_piece))
        hit = self._segments.get(key)
        if hit is None:
            self.ready()
            hit = self._segments[key] = RowSegments(self.row_ptr, self.num_nodes, self.num_edges, *key)
            self._mark()
        return hit


_Graph = PreparedGraph


def prepare_graph(sender: torch.Tensor, receiver: torch.Tensor, num_nodes: int,
                  graph_ordering=GraphOrdering.RECEIVER, pair_rows: bool | None = None) -> PreparedGraph:
    """Prepare the adjacency of `(sender, receiver)` once, for every call that passes it as `graph=`.

    `pair_rows`: put rows with common senders side by side (fewer dx atomics in every backward that
    uses the handle, 0.3 ms more preparation at 1M edges); None: as `config().pair_rows` says, which
    by default pairs for these handles.  A caller that rebuilds the handle for every step passes False.

    The counterpart of the reference's per-call `GraphCSR` (`src/e3j/ops/convolution.py:227,426-431`)
    for callers whose graph outlives one call: the layers of a model, the steps between two
    neighbour-list rebuilds.  Build a new handle whenever the contents of the index tensors change.
    """
    ordering = GraphOrdering.parse(graph_ordering)
    if pair_rows is None:
        pair_rows = config().pair_rows in (True, "prepared")
    return _prepare_graph(ordering, int(num_nodes), sender, receiver, pair=bool(pair_rows))


def _check_graph(graph: PreparedGraph, meta: "_Meta", num_edges: int) -> None:
    if graph.num_nodes != meta.num_nodes or graph.num_edges != num_edges:
        raise ValueError(f"`graph` was prepared for {graph.num_nodes} nodes and {graph.num_edges} edges; the "
                         f"operands have {meta.num_nodes} and {num_edges}")
    if graph.ordering is not None and graph.ordering != meta.ordering:
        raise ValueError(f"`graph` was prepared for {graph.ordering.name} ordering, the call asks for "
                         f"{meta.ordering.name}")


def _forward_graph(meta: _Meta, sender: torch.Tensor, receiver: torch.Tensor, build: bool = True):
    """Adjacency used by the forward kernel.  Without the opt-in cache it is prepared on every call
    (`build` off: None, the caller prepares what it needs)."""
    if not config().graph_cache:
        return _prepare_graph(meta.ordering, meta.num_nodes, sender, receiver) if build else None
    key = (id(sender), id(receiver), sender._version, receiver._version, meta.num_nodes,
           meta.ordering, config().locality_rounds)
    hit = _GRAPH_CACHE.get(key)
    if hit is not None and hit[0]() is sender and hit[1]() is receiver:
        return hit[2]
    if not build:
        return None
    graph = _prepare_graph(meta.ordering, meta.num_nodes, sender, receiver)
    if len(_GRAPH_CACHE) >= _GRAPH_CACHE_SIZE:
        _GRAPH_CACHE.pop(next(iter(_GRAPH_CACHE)))

    def evict(_, key=key):
        _GRAPH_CACHE.pop(key, None)

    _GRAPH_CACHE[key] = (weakref.ref(sender, evict), weakref.ref(receiver, evict), graph)
    return graph


def _prepare_graph(ordering: GraphOrdering, n: int, sender: torch.Tensor, receiver: torch.Tensor,
                   pair: bool | None = None) -> PreparedGraph:
    sender_l, receiver_l = wrap_global_index(sender, n), wrap_global_index(receiver, n)
    if ordering == GraphOrdering.RECEIVER:
        other, row_ptr, perm = sender_l.contiguous(), csr_row_ptr(receiver_l, n), None
    elif ordering == GraphOrdering.SENDER:
        # aggregate over reversed edges; y parities are folded into the coefficients
        other, row_ptr, perm = receiver_l.contiguous(), csr_row_ptr(sender_l, n), None
    else:
        perm, other, row_ptr = sort_edges(receiver_l, sender_l, n)
    return PreparedGraph(other, row_ptr, perm, _row_order(other, row_ptr, n, pair), n, ordering)


def _raw_forward(meta: _Meta, x, y, s, sender, receiver, graph=None) -> torch.Tensor:
    x, y, s = x.contiguous(), y.contiguous(), s.contiguous()
    if graph is None:
        graph = _forward_graph(meta, sender, receiver)
    graph.ready()
    other, row_ptr, perm, order = graph
    # SENDER ordering: the table carries the parity signs of y (unrolled kernels take them as
    # a sign mask on the unsigned built-in table instead)
    p, table = _fill_params(meta, x, y, s, meta.signed_table or meta.table, row_order=order)
    if meta.layout == Layout.TRAILING_CHANNELS:
        out = torch.empty((x.shape[0], meta.params.num_out, x.shape[2]), dtype=x.dtype, device=x.device)
    else:
        out = torch.empty((x.shape[0], x.shape[1], meta.params.num_out), dtype=x.dtype, device=x.device)
    # Rows much longer than the mean are shared between waves: the first call cuts every row at
    # `cap` positions, a second call sums the remaining pieces, each into a scratch row, and adds
    # them to their output rows in a fixed order (unrolled kernels of the trailing layout): the
    # result is the same bits in every run, as for a row that one wave sums
    cap = 0
    fixed_order = bool(config().fixed_order_rows)
    if (p.signature >= 0 and meta.layout == Layout.TRAILING_CHANNELS and x.dtype == torch.float32
            and (fixed_order or not config().deterministic)
            and isinstance(graph, PreparedGraph) and y.shape[0] > 0
            and all(t.data_ptr() % 16 == 0 for t in (x, s, out))):
        want = int(config().row_cap)
        cap = row_cap_for(x.shape[0], y.shape[0]) if want < 0 else want
    lib = _lib.load()
    with torch.cuda.device(x.device):
        plan = _table_plan(p, table, x.device)  # noqa: F841 (kept alive until the call is enqueued)
        args = (table.device(x.device).data_ptr(), x.data_ptr(), y.data_ptr(), s.data_ptr(),
                other.data_ptr(), row_ptr.data_ptr(), perm.data_ptr() if perm is not None else None,
                out.data_ptr(), _stream(x.device))
        pieces = None
        if cap > 0:
            row_floats = int(out.shape[1]) * int(out.shape[2])
            pieces = graph.segments(cap, row_piece_for(int(y.shape[0]), row_floats) if fixed_order else ROW_PIECE)
            p.row_cap, p.row_piece = pieces.row_cap, pieces.row_piece
        _lib.check(lib.e3j_amd_convolution_fwd(ctypes.byref(p), *args))
        if pieces is not None and pieces.count > 0:
            p.segments, p.max_segments = pieces.buffer.data_ptr(), pieces.count
            if fixed_order:
                p.partials = pieces.partials(int(out.shape[1]), int(out.shape[2])).data_ptr()
            _lib.check(lib.e3j_amd_convolution_fwd(ctypes.byref(p), *args))
    return out


def _raw_backward(meta: _Meta, x, y, s, dm, sender, receiver, graph=None):
    """`graph`: the forward's `(other, row_ptr, perm, row_order)` when it can be reused."""
    x, y, s, dm = x.contiguous(), y.contiguous(), s.contiguous(), dm.contiguous()
    n = meta.num_nodes
    dx, dy, ds = torch.empty_like(x), torch.empty_like(y), torch.empty_like(s)
    lib = _lib.load()
    table = meta.table
    has_kernel = table.signature(*_shape(meta, x, y, s), meta.layout)[0] >= 0
    # float16 without an unrolled kernel: the table-driven kernels have no half-precision form of dx by
    # atomics, rows must own their dx
    deterministic = config().deterministic or (x.dtype == torch.float16 and not has_kernel)
    if x.dtype != torch.float32 and deterministic:
        has_kernel = False   # the float64 / float16 unrolled backward adds dx with atomics; rows that own dx: table-driven
    # SENDER ordering: the cotangents belong to the edges as given (dy[e], ds[e] come from
    # dm[receiver(e)]), not to the reversed edges the forward walks
    # (`src/e3j/ops/convolution.py:413-431`).  With an unrolled kernel for the table the edges
    # are sorted by receiver on the device and the receiver-grouped backward runs on them
    # (results land on the edges' own rows through the permutation); otherwise the
    # table-driven kernel keeps the sender rows, gathers dm and owns dx.
    # deterministic, with an unrolled kernel: in the trailing layout up to 128 channels the
    # sender-grouped unrolled backward (rows own their dx, an edge's dy comes from at most two waves:
    # the same bits in every run, no workspace); otherwise the atomic-free backward on receiver rows
    # (per-position dx rows in a workspace, summed in a fixed order); tables without a kernel fall
    # back to the table-driven kernel on sender rows
    channels = _shape(meta, x, y, s)[1]
    sender_kernel = (deterministic and has_kernel and meta.layout == Layout.TRAILING_CHANNELS and channels <= 128
                     and x.dtype == torch.float32
                     and all(t.data_ptr() % 16 == 0 for t in (x, y, s, dm, dx, dy, ds)))
    sender_rows = meta.ordering == GraphOrdering.SENDER and (not has_kernel or sender_kernel)
    resort = meta.ordering in (GraphOrdering.NONE, GraphOrdering.SENDER) and not sender_rows
    ordered = deterministic and has_kernel and not sender_kernel
    forward_rows = meta.ordering != GraphOrdering.SENDER   # the forward's rows are receivers
    reuse = graph is not None and (
        (forward_rows and (not deterministic or ordered)) or sender_rows)
    prepared = None  # the receiver-grouped adjacency as an object that keeps tile schedules
    if graph is not None:
        graph.ready()
    if reuse:
        other, row_ptr, perm, order = graph
        group_receiver = not sender_rows
        if isinstance(graph, _Graph) and group_receiver:
            prepared = graph
    else:
        sender_l, receiver_l = wrap_global_index(sender, n), wrap_global_index(receiver, n)
        if sender_rows:
            # already grouped by sender: rows own their dx, no permutation
            group_receiver, other, row_ptr, perm = False, receiver_l.contiguous(), csr_row_ptr(sender_l, n), None
        elif deterministic and not ordered:
            if meta.ordering == GraphOrdering.NONE:
                # by receiver first (stable), then by sender (stable): the order in which a sender's
                # contributions are summed then does not depend on the order the edges came in
                by_rcv, snd_sorted, _ = sort_edges(receiver_l, sender_l, n)
                perm2, other, row_ptr = sort_edges(snd_sorted, receiver_l[by_rcv.long()].contiguous(), n)
                perm = by_rcv[perm2.long()].contiguous()
            else:
                perm, other, row_ptr = sort_edges(sender_l, receiver_l, n)
            group_receiver = False
        elif resort:
            perm, other, row_ptr = sort_edges(receiver_l, sender_l, n)
            group_receiver = True
        else:
            group_receiver, other, row_ptr, perm = True, sender_l.contiguous(), csr_row_ptr(receiver_l, n), None
        order = (graph[3] if graph is not None and forward_rows else _row_order(other, row_ptr, n))
    p, table = _fill_params(meta, x, y, s, table, use_signature=group_receiver or sender_kernel, row_order=order)
    args = (ctypes.byref(p), table.device(x.device).data_ptr(), x.data_ptr(), y.data_ptr(),
            s.data_ptr(), dm.data_ptr(), other.data_ptr(), row_ptr.data_ptr(),
            perm.data_ptr() if perm is not None else None,
            dx.data_ptr(), dy.data_ptr(), ds.data_ptr())
    # tiles of receivers whose dm rows fit the LDS of a workgroup: dx summed per (tile, sender)
    tile_rows = 0
    aligned = all(t.data_ptr() % 16 == 0 for t in (x, y, s, dm, dx, dy, ds))  # what the unrolled kernels take
    if (group_receiver and not ordered and y.shape[0] > 0 and p.layout == _lib.LAYOUT_TRAILING and aligned
            and x.dtype == torch.float32):
        tile_rows = _tile_rows(p.signature)
    with torch.cuda.device(x.device):
        plan = _table_plan(p, table, x.device)  # noqa: F841 (kept alive until the call is enqueued)
        if tile_rows >= 1:
            if prepared is None:
                prepared = PreparedGraph(other, row_ptr, perm, order, n)
            schedule = prepared.schedule(tile_rows)
            _lib.check(lib.e3j_amd_convolution_bwd_tiled(
                ctypes.byref(p), x.data_ptr(), y.data_ptr(), s.data_ptr(), dm.data_ptr(), other.data_ptr(),
                row_ptr.data_ptr(), perm.data_ptr() if perm is not None else None,
                ctypes.byref(schedule.struct), dx.data_ptr(), dy.data_ptr(), ds.data_ptr(), _stream(x.device)))
        elif ordered:
            nbytes = int(lib.e3j_amd_convolution_bwd_ordered_workspace_bytes(ctypes.byref(p)))
            workspace = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
            _lib.check(lib.e3j_amd_convolution_bwd_ordered(*args, workspace.data_ptr(), _stream(x.device)))
        else:
            fn = lib.e3j_amd_convolution_bwd_receiver if group_receiver else lib.e3j_amd_convolution_bwd_sender
            _lib.check(fn(*args, _stream(x.device)))
    return dx, dy, ds


def _tile_rows(signature: int) -> int:
    """Receivers per tile of the tiled backward for a compiled signature under the current
    configuration; 0: the one-wave-per-receiver backward runs."""
    want = int(config().tile_rows)
    if signature < 0 or want == 0:
        return 0
    lib = _lib.load()
    if want < 0:
        return int(lib.e3j_amd_tile_rows_default(signature))
    return min(want, int(lib.e3j_amd_tile_rows(signature)))


def _sum(*terms):
    terms = [t for t in terms if t is not None]
    if not terms:
        return None
    total = terms[0]
    for t in terms[1:]:
        total = total + t
    return total


def _lead(t: torch.Tensor, dim, batch: int) -> torch.Tensor:
    """Batch axis first; an operand that is not batched is broadcast over the batch."""
    if dim is None:
        return t.unsqueeze(0).expand((batch,) + tuple(t.shape))
    return t.movedim(dim, 0)


def _fold_rows(t: torch.Tensor) -> torch.Tensor:
    return t.reshape((t.shape[0] * t.shape[1],) + tuple(t.shape[2:]))


def _unfold_rows(t: torch.Tensor, batch: int) -> torch.Tensor:
    return t.reshape((batch, t.shape[0] // batch) + tuple(t.shape[1:]))


def _fold_graphs(meta: _Meta, sender, receiver, dims, batch: int):
    """Endpoints of `batch` graphs as one disjoint graph (`src/e3j/ops/convolution.py:54-78,271-308`);
    returns the folded endpoints and the meta of the folded problem."""
    if dims[0] is not None or dims[1] is not None:
        warnings.warn("Convolution is being batched over graph adjacency. Batch graphs into a "
                      "single, disconnected graph upstream or silence this warning by filtering "
                      "`ConvolutionBatchingWarning`.", ConvolutionBatchingWarning, stacklevel=3)
    snd = _lead(sender, dims[0], batch).to(torch.int64)
    rcv = _lead(receiver, dims[1], batch).to(torch.int64)
    if meta.ordering == GraphOrdering.SENDER:
        snd_f, rcv_f = fold_endpoints(snd, rcv, batch, meta.num_nodes)
    else:
        rcv_f, snd_f = fold_endpoints(rcv, snd, batch, meta.num_nodes)
    return snd_f, rcv_f, dataclasses.replace(meta, num_nodes=batch * meta.num_nodes)


class _Convolution(torch.autograd.Function):
    """Differentiable in (x, y, s) to any reverse-mode order; composes with `torch.func`
    transforms (the batching rule folds the graphs of a batch into one disjoint graph)."""

    @staticmethod
    def forward(x, y, s, sender, receiver, meta, graph):
        if graph is None:
            graph = _forward_graph(meta, sender, receiver)
        return _raw_forward(meta, x, y, s, sender, receiver, graph)

    @staticmethod
    def setup_context(ctx, inputs, output):
        x, y, s, sender, receiver, meta, graph = inputs
        ctx.meta, ctx.graph = meta, graph
        # the index tensors themselves (not copies): the adjacency prepared for them by the
        # forward pass is found again by their identity
        ctx.index = (sender, receiver)
        ctx.save_for_backward(x, y, s)

    @staticmethod
    def backward(ctx, dm):
        x, y, s = ctx.saved_tensors
        sender, receiver = ctx.index
        dx, dy, ds = _ConvolutionBwd.apply(x, y, s, dm, sender, receiver, ctx.meta, ctx.graph)
        return dx, dy, ds, None, None, None, None

    @staticmethod
    def vmap(info, in_dims, x, y, s, sender, receiver, meta, graph):
        batch = info.batch_size
        snd, rcv, folded = _fold_graphs(meta, sender, receiver, in_dims[3:5], batch)
        out = _Convolution.apply(_fold_rows(_lead(x, in_dims[0], batch)), _fold_rows(_lead(y, in_dims[1], batch)),
                                 _fold_rows(_lead(s, in_dims[2], batch)), snd, rcv, folded, None)
        return _unfold_rows(out, batch), 0


class _ConvolutionBwd(torch.autograd.Function):
    @staticmethod
    def forward(x, y, s, dm, sender, receiver, meta, graph):
        if graph is None:  # the adjacency the forward pass prepared for these index tensors
            graph = _forward_graph(meta, sender, receiver, build=False)
        return _raw_backward(meta, x, y, s, dm, sender, receiver, graph)

    @staticmethod
    def setup_context(ctx, inputs, output):
        x, y, s, dm, sender, receiver, meta, graph = inputs
        ctx.meta, ctx.graph = meta, graph
        ctx.index = (sender, receiver)
        ctx.save_for_backward(x, y, s, dm)

    @staticmethod
    def backward(ctx, ddx, ddy, dds):
        # (Dx, Dy, Ds, Ddm) from (Ddx, Ddy, Dds): the trilinear form's second variation
        # (`src/e3j/ops/convolution.py:535-562`).
        x, y, s, dm = ctx.saved_tensors
        sender, receiver = ctx.index
        meta = ctx.meta

        graph = ctx.graph

        def conv(a, b, c):
            return _Convolution.apply(a, b, c, sender, receiver, meta, graph)

        def conv_bwd(a, b, c):
            return _ConvolutionBwd.apply(a, b, c, dm, sender, receiver, meta, graph)

        d_dm, d_x, d_y, d_s = [], [], [], []
        if ddx is not None:
            d_dm.append(conv(ddx, y, s))
            _, gy, gs = conv_bwd(ddx, y, s)
            d_y.append(gy)
            d_s.append(gs)
        if ddy is not None:
            d_dm.append(conv(x, ddy, s))
            gx, _, gs = conv_bwd(x, ddy, s)
            d_x.append(gx)
            d_s.append(gs)
        if dds is not None:
            d_dm.append(conv(x, y, dds))
            gx, gy, _ = conv_bwd(x, y, dds)
            d_x.append(gx)
            d_y.append(gy)
        return _sum(*d_x), _sum(*d_y), _sum(*d_s), _sum(*d_dm), None, None, None, None

    @staticmethod
    def vmap(info, in_dims, x, y, s, dm, sender, receiver, meta, graph):
        batch = info.batch_size
        snd, rcv, folded = _fold_graphs(meta, sender, receiver, in_dims[4:6], batch)
        dx, dy, ds = _ConvolutionBwd.apply(
            _fold_rows(_lead(x, in_dims[0], batch)), _fold_rows(_lead(y, in_dims[1], batch)),
            _fold_rows(_lead(s, in_dims[2], batch)), _fold_rows(_lead(dm, in_dims[3], batch)), snd, rcv, folded, None)
        return (_unfold_rows(dx, batch), _unfold_rows(dy, batch), _unfold_rows(ds, batch)), (0, 0, 0)


def _make_meta(coef, x, y, s, params, graph_ordering, y_parity, layout) -> _Meta:
    ordering = GraphOrdering.parse(graph_ordering)
    layout = Layout.parse(layout)
    val_np = _VAL_DTYPES[x.dtype][1]
    table = _Table.get(coef, val_np)
    signed = None
    if ordering == GraphOrdering.SENDER:
        if y_parity is None:
            raise ValueError("SENDER graph ordering requires `y_parity`.")
        signed = table.signed(y_parity)
    return _Meta(table=table, signed_table=signed, params=params, ordering=ordering, layout=layout,
                 y_parity=None if y_parity is None else np.asarray(y_parity),
                 num_nodes=int(x.shape[0]), squeeze_channels=False, y_shape=tuple(y.shape))


def _under_transform() -> bool:
    return torch._C._functorch.peek_interpreter_stack() is not None


def _canonical(x, y, s, layout: Layout):
    """Add the channel axis of a 2-D `x`/`s`, drop a unit channel axis of `y`."""
    squeeze = x.ndim == 2
    if y.ndim == x.ndim and y.shape[-1] != 1 and not squeeze:
        raise NotImplementedError("RHS y should have only one channel.")
    if squeeze:
        axis = -1 if layout == Layout.TRAILING_CHANNELS else 1
        x = x.unsqueeze(axis)
        if s.ndim == 2:
            s = s.unsqueeze(axis)
        if y.ndim == 3:
            y = y.reshape(y.shape[0], -1)
    elif y.ndim == 3:
        y = y[..., 0]
    if x.ndim != 3 or s.ndim != 3 or y.ndim != 2:
        raise ValueError(f"unexpected operand ranks: x {tuple(x.shape)}, y {tuple(y.shape)}, "
                         f"s {tuple(s.shape)}")
    return x, y, s, squeeze


def convolution(coef, x, y, s, sender, receiver, params: ConvolutionParams,
                graph_ordering=GraphOrdering.RECEIVER, y_parity=None, *,
                layout=Layout.TRAILING_CHANNELS, graph: PreparedGraph | None = None) -> torch.Tensor:
    """`out[r] = sum_{e: recv(e)=r} (x[send(e)] (x) y[e]) . s[e]` with the fused HIP kernels.

    Args:
        coef: packed `Coef4D` table (host numpy array, opaque index dtype).
        x: node features `(num_nodes, num_x, channels)` [leading layout: `(num_nodes, channels, num_x)`].
        y: edge embeddings `(num_edges, num_y)`, single channel.
        s: radial scalars `(num_edges, num_scalars, channels)` [leading: `(num_edges, channels, num_scalars)`].
        sender, receiver: `(num_edges,)` integer endpoints; `DUMMY_INDEX` marks padding.
            Sorted by receiver (RECEIVER) or sender (SENDER), or in any order (NONE).
        params: `ConvolutionParams(num_out, num_scalars)`.
        y_parity: per-`y`-component parity, required under SENDER ordering.
        graph: optional handle from `prepare_graph(sender, receiver, num_nodes, graph_ordering)`; the
            adjacency is then not prepared again (forward and backward).
    """
    _check_operands(x, y, s, sender, receiver)
    layout = Layout.parse(layout)
    x3, y2, s3, squeeze = _canonical(x, y, s, layout)
    meta = _make_meta(coef, x3, y2, s3, params, graph_ordering, y_parity, layout)
    if graph is not None:
        _check_graph(graph, meta, int(y2.shape[0]))
    elif not _under_transform():
        # prepared here, so that the backward pass finds it in its context; under a torch.func
        # transform the operator prepares it itself, on the plain tensors the transform hands it
        # (the batching rule first folds batched index tensors into one graph)
        graph = _forward_graph(meta, sender, receiver)
    out = _Convolution.apply(x3, y2, s3, sender, receiver, meta, graph)
    if squeeze:
        out = out.squeeze(-1 if layout == Layout.TRAILING_CHANNELS else 1)
    return out


def convolution_bwd(coef, x, y, s, sender, receiver, dm, params: ConvolutionParams,
                    graph_ordering=GraphOrdering.RECEIVER, y_parity=None, *,
                    layout=Layout.TRAILING_CHANNELS, graph: PreparedGraph | None = None):
    """Cotangents `(dx, dy, ds)` of `convolution` for the output cotangent `dm`."""
    _check_operands(x, y, s, sender, receiver)
    layout = Layout.parse(layout)
    y_in_shape = tuple(y.shape)
    x3, y2, s3, squeeze = _canonical(x, y, s, layout)
    dm3 = dm.unsqueeze(-1 if layout == Layout.TRAILING_CHANNELS else 1) if squeeze else dm
    meta = _make_meta(coef, x3, y2, s3, params, graph_ordering, y_parity, layout)
    if graph is not None:
        _check_graph(graph, meta, int(y2.shape[0]))
    dx, dy, ds = _ConvolutionBwd.apply(x3, y2, s3, dm3, sender, receiver, meta, graph)
    if squeeze:
        axis = -1 if layout == Layout.TRAILING_CHANNELS else 1
        dx = dx.squeeze(axis)
        if s.ndim == 2:
            ds = ds.squeeze(axis)
    return dx, dy.reshape(y_in_shape), ds


def convolution_batched(coef, x, y, s, sender, receiver, params: ConvolutionParams,
                        graph_ordering=GraphOrdering.RECEIVER, y_parity=None, *,
                        layout=Layout.TRAILING_CHANNELS) -> torch.Tensor:
    """Batch of graphs on a leading axis, folded into one disjoint graph.

    The counterpart of the reference's batching rule (`src/e3j/ops/convolution.py:271-308`):
    `x (B, N, ...)`, `y (B, E, Y)`, `s (B, E, ...)`; `sender`/`receiver` either `(E,)`
    (one graph shared by the batch) or `(B, E)` (one graph per batch entry, which
    emits `ConvolutionBatchingWarning`).
    """
    ordering = GraphOrdering.parse(graph_ordering)
    batch, num_nodes, num_edges = x.shape[0], x.shape[1], y.shape[1]
    if sender.ndim != receiver.ndim:
        raise ValueError("Graph adjacency inconsistently batched.")
    if sender.ndim == 2:
        warnings.warn("Convolution is being batched over graph adjacency. Batch graphs into a "
                      "single, disconnected graph upstream or silence this warning by filtering "
                      "`ConvolutionBatchingWarning`.", ConvolutionBatchingWarning, stacklevel=2)
    else:
        sender = sender.unsqueeze(0).expand(batch, -1)
        receiver = receiver.unsqueeze(0).expand(batch, -1)
    sender, receiver = sender.to(torch.int64), receiver.to(torch.int64)
    if ordering == GraphOrdering.SENDER:
        sender_f, receiver_f = fold_endpoints(sender, receiver, batch, num_nodes)
    else:
        receiver_f, sender_f = fold_endpoints(receiver, sender, batch, num_nodes)
    out = convolution(coef, x.reshape((batch * num_nodes,) + tuple(x.shape[2:])),
                      y.reshape((batch * num_edges,) + tuple(y.shape[2:])),
                      s.reshape((batch * num_edges,) + tuple(s.shape[2:])),
                      sender_f, receiver_f, params, ordering, y_parity, layout=layout)
    return out.reshape((batch, num_nodes) + tuple(out.shape[1:]))


convolution.Params = ConvolutionParams
