"""CSR adjacency of a directed graph, built on the device.

Mirrors `GraphCSR` of the reference (`src/e3j/data/graph.py:21-91`): edges are
grouped by receiver so a kernel can reduce a receiver's messages without
atomics; `DUMMY_INDEX` (INT32_MAX) marks padding endpoints, which drop out of
the adjacency.  The derived buffers (`receiver_ptr`, the permutations of `sort`
and `transpose`) are int32 and are computed by the HIP kernels of
`csrc/graph.hip`; the index arithmetic of `mask_edges` and of the folding
helpers is plain tensor arithmetic.
"""

from __future__ import annotations


import numpy as np
import torch

from . import _lib

DUMMY_INDEX = int(np.iinfo(np.int32).max)
INDEX_DTYPE = torch.int32


def is_dummy_index(index: torch.Tensor) -> torch.Tensor:
    return index == DUMMY_INDEX


def is_dummy_edge(sender: torch.Tensor, receiver: torch.Tensor) -> torch.Tensor:
    return is_dummy_index(sender) | is_dummy_index(receiver)


def _require_device(*tensors: torch.Tensor) -> torch.device:
    device = tensors[0].device
    for t in tensors:
        if t.device.type != "cuda":
            raise RuntimeError("e3j_amd graph kernels need tensors in GPU memory; got a "
                               f"{t.device.type} tensor (there is no CPU implementation)")
        if t.device != device:
            raise RuntimeError("adjacency tensors must live on one device")
    return device


def _stream_ptr(device: torch.device) -> int:
    return int(torch.cuda.current_stream(device).cuda_stream)


def _as_index(t: torch.Tensor) -> torch.Tensor:
    return t.to(INDEX_DTYPE).contiguous()


def _workspace(num_nodes: int, num_edges: int, device) -> torch.Tensor:
    nbytes = _lib.load().e3j_amd_csr_workspace_bytes(num_nodes, num_edges)
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


def csr_row_ptr(key: torch.Tensor, num_nodes: int) -> torch.Tensor:
    """`[0] + cumsum(bincount(key, length=num_nodes))` as int32; out-of-range keys dropped."""
    device = _require_device(key)
    key = _as_index(key)
    row_ptr = torch.empty(num_nodes + 1, dtype=INDEX_DTYPE, device=device)
    ws = _workspace(num_nodes, key.numel(), device)
    with torch.cuda.device(device):
        _lib.check(_lib.load().e3j_amd_csr_row_ptr(
            key.data_ptr(), key.numel(), num_nodes, row_ptr.data_ptr(), ws.data_ptr(),
            _stream_ptr(device)))
    return row_ptr


def sort_edges(key: torch.Tensor, other: torch.Tensor, num_nodes: int):
    """Stable sort of edge positions by `key`: `(perm, other[perm], row_ptr)`, all int32."""
    device = _require_device(key, other)
    key, other = _as_index(key), _as_index(other)
    num_edges = key.numel()
    perm = torch.empty(num_edges, dtype=INDEX_DTYPE, device=device)
    other_sorted = torch.empty(num_edges, dtype=INDEX_DTYPE, device=device)
    row_ptr = torch.empty(num_nodes + 1, dtype=INDEX_DTYPE, device=device)
    ws = _workspace(num_nodes, num_edges, device)
    with torch.cuda.device(device):
        _lib.check(_lib.load().e3j_amd_sort_edges(
            key.data_ptr(), other.data_ptr(), num_edges, num_nodes, perm.data_ptr(),
            other_sorted.data_ptr(), row_ptr.data_ptr(), ws.data_ptr(), _stream_ptr(device)))
    return perm, other_sorted, row_ptr


def locality_order(other: torch.Tensor, row_ptr: torch.Tensor, num_nodes: int,
                   rounds: int = 2) -> torch.Tensor:
    """Processing order of the nodes in which graph neighbours are close together (int32 permutation).

    `(other, row_ptr)`: a CSR adjacency (e.g. senders per receiver-sorted position and
    `receiver_ptr`).  Kernels that walk rows in this order gather sender rows that the rows
    running beside them gather too, so those rows are served from cache.  Results do not
    depend on the order.
    """
    device = _require_device(other, row_ptr)
    other, row_ptr = _as_index(other), _as_index(row_ptr)
    order = torch.empty(num_nodes, dtype=INDEX_DTYPE, device=device)
    lib = _lib.load()
    ws = torch.empty(max(int(lib.e3j_amd_order_workspace_bytes(num_nodes)), 256), dtype=torch.uint8,
                     device=device)
    with torch.cuda.device(device):
        _lib.check(lib.e3j_amd_locality_order(other.data_ptr(), row_ptr.data_ptr(), num_nodes,
                                              int(rounds), order.data_ptr(), ws.data_ptr(),
                                              _stream_ptr(device)))
    return order


def pair_rows(other: torch.Tensor, row_ptr: torch.Tensor, num_nodes: int,
              order: torch.Tensor | None = None) -> torch.Tensor:
    """`order` (or the index order) rearranged so that rows sharing most of their senders sit side
    by side on positions 2q, 2q + 1: the tiles of the backward over two receivers per tile
    (`e3j_amd_pair_rows`).  Results do not depend on it."""
    device = _require_device(other, row_ptr)
    other, row_ptr = _as_index(other), _as_index(row_ptr)
    lib = _lib.load()
    num_edges = int(other.numel())
    out = torch.empty(num_nodes, dtype=INDEX_DTYPE, device=device)
    ws = torch.empty(max(int(lib.e3j_amd_pair_rows_workspace_bytes(num_nodes, num_edges)), 256),
                     dtype=torch.uint8, device=device)
    with torch.cuda.device(device):
        _lib.check(lib.e3j_amd_pair_rows(other.data_ptr(), row_ptr.data_ptr(), num_nodes, num_edges,
                                         order.data_ptr() if order is not None else None, out.data_ptr(),
                                         ws.data_ptr(), _stream_ptr(device)))
    return out


#: edge positions per work item of the tiled backward: longer tile lists (hub rows) are cut
#: into pieces of this many positions, each taken by a workgroup of its own
MAX_WORK_EDGES = 256


#: smallest row length above which the forward pass shares a row between waves, and the
#: positions per wave of a shared row
MIN_ROW_CAP = 64
ROW_PIECE = 64


def row_cap_for(num_nodes: int, num_edges: int) -> int:
    """Row length above which the forward pass shares a row between waves: twice the mean
    degree (at least 64), which no row of a radius graph of even density reaches."""
    mean = num_edges / max(num_nodes, 1)
    return max(MIN_ROW_CAP, int(2 * mean))


#: bytes of scratch the fixed-order sums of long rows may take (a row of the output per piece):
#: larger graphs get longer pieces instead of more of them
PARTIALS_BUDGET = 256 << 20


def row_piece_for(num_edges: int, row_floats: int, row_piece: int = ROW_PIECE) -> int:
    """Positions per piece such that a scratch row for every possible piece (`num_edges //
    piece` of them, `row_floats` floats each) stays within `PARTIALS_BUDGET`."""
    need = -(-int(num_edges) * int(row_floats) * 4 // PARTIALS_BUDGET)
    return max(int(row_piece), need)


class RowSegments:
    """The pieces of long rows for the second call of the forward pass
    (`e3j_amd_row_segments_build`).  `count`: pieces to launch, the bound `num_edges // row_piece`
    (the list's own count, which the kernel reads on the device, is never read back: the
    surplus workgroups of the second call leave at once, which costs less than a wait).
    `partials(num_out, channels)`: the scratch of the fixed-order sums (`e3j_amd_conv_params.partials`)."""

    def __init__(self, row_ptr: torch.Tensor, num_nodes: int, num_edges: int, row_cap: int,
                 row_piece: int = ROW_PIECE):
        device = _require_device(row_ptr)
        lib = _lib.load()
        self.row_cap = max(int(row_cap), int(row_piece)) if row_piece > ROW_PIECE else int(row_cap)
        self.row_piece = min(int(row_piece), self.row_cap)
        self._partials = {}
        self.max_segments = int(lib.e3j_amd_row_segments_max(int(num_edges), self.row_piece))
        self.buffer = torch.empty(4 + 3 * self.max_segments, dtype=INDEX_DTYPE, device=device)
        with torch.cuda.device(device):
            _lib.check(lib.e3j_amd_row_segments_build(
                row_ptr.data_ptr(), int(num_nodes), self.row_cap, self.row_piece, self.max_segments,
                self.buffer.data_ptr(), _stream_ptr(device)))
        self.count = self.max_segments

    def partials(self, num_out: int, channels: int) -> torch.Tensor:
        key = (int(num_out), int(channels))
        hit = self._partials.get(key)
        if hit is None:
            nbytes = int(_lib.load().e3j_amd_row_partials_bytes(self.max_segments, *key))
            hit = self._partials[key] = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=self.buffer.device)
        return hit


class TileSchedule:
    """Schedule of the backward over tiles of receivers (`e3j_amd_tile_schedule`).

    The edge positions of every tile of `tile_rows` receivers (consecutive in `row_order`),
    sorted by sender, and the work descriptors that hand them to the workgroups.  Built on
    the device; holds the buffers the C struct points to.
    """

    def __init__(self, other: torch.Tensor, row_ptr: torch.Tensor, perm, row_order, num_nodes: int,
                 tile_rows: int, max_work_edges: int = MAX_WORK_EDGES):
        device = _require_device(other, row_ptr)
        lib = _lib.load()
        num_edges = int(other.numel())
        self.tile_rows = int(tile_rows)
        self.num_work = int(lib.e3j_amd_tile_schedule_num_work(num_nodes, num_edges, tile_rows, max_work_edges))
        self.work = torch.empty((max(self.num_work, 1), 4), dtype=INDEX_DTYPE, device=device)
        self.sender = torch.empty(num_edges, dtype=INDEX_DTYPE, device=device)
        self.edge = torch.empty(num_edges, dtype=INDEX_DTYPE, device=device)
        self.local = torch.empty(num_edges, dtype=INDEX_DTYPE, device=device)
        nbytes = int(lib.e3j_amd_tile_schedule_workspace_bytes(num_nodes, num_edges, tile_rows))
        ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=device)
        with torch.cuda.device(device):
            _lib.check(lib.e3j_amd_tile_schedule_build(
                other.data_ptr(), row_ptr.data_ptr(), perm.data_ptr() if perm is not None else None,
                row_order.data_ptr() if row_order is not None else None, num_nodes, num_edges,
                self.tile_rows, int(max_work_edges), self.work.data_ptr(), self.sender.data_ptr(),
                self.edge.data_ptr(), self.local.data_ptr(), ws.data_ptr(), _stream_ptr(device)))
        self.struct = _lib.TileSchedule(
            tile_rows=self.tile_rows, num_work=self.num_work, work=self.work.data_ptr(),
            sender=self.sender.data_ptr(), edge=self.edge.data_ptr(), local=self.local.data_ptr())


class GraphCSR:
    """Edges grouped by receiver (`src/e3j/data/graph.py:38-73`)."""

    def __init__(self, num_nodes: int, sender: torch.Tensor, receiver: torch.Tensor,
                 receiver_ptr: torch.Tensor | None = None):
        self.num_nodes = int(num_nodes)
        self.sender = sender
        self.receiver = receiver
        self._receiver_ptr = receiver_ptr

    @property
    def receiver_ptr(self) -> torch.Tensor:
        if self._receiver_ptr is None:
            self._receiver_ptr = csr_row_ptr(self.receiver, self.num_nodes)
        return self._receiver_ptr

    @property
    def num_neighbors(self) -> torch.Tensor:
        return self.receiver_ptr[1:] - self.receiver_ptr[:-1]

    @classmethod
    def sort(cls, num_nodes: int, sender: torch.Tensor, receiver: torch.Tensor):
        """`(sigma, graph', sigma_inv)` sorting edges by receiver (stable)."""
        perm, sender_sorted, ptr = sort_edges(receiver, sender, num_nodes)
        graph = cls(num_nodes, sender_sorted, _as_index(receiver)[perm.long()], receiver_ptr=ptr)
        inverse = torch.empty_like(perm)
        inverse[perm.long()] = torch.arange(perm.numel(), dtype=INDEX_DTYPE, device=perm.device)
        return perm, graph, inverse

    def transpose(self):
        """`(sigma, graph_t, sigma_inv)` sorting edges by sender instead."""
        return GraphCSR.sort(self.num_nodes, self.receiver, self.sender)

    @staticmethod
    def mask_edges(sender: torch.Tensor, receiver: torch.Tensor, node_mask: torch.Tensor):
        """Mark edges touching a padding node (at or past `count_nonzero(node_mask)`) as dummies."""
        num_real = torch.count_nonzero(node_mask)
        keep = (sender < num_real) & (receiver < num_real)
        dummy = torch.full_like(sender, DUMMY_INDEX)
        return torch.where(keep, sender, dummy), torch.where(keep, receiver, dummy)


def wrap_global_index(index: torch.Tensor, num_nodes: int) -> torch.Tensor:
    """Reduce modulo `num_nodes`, keeping the sentinel (`src/e3j/ops/convolution.py:39-51`)."""
    if index.device.type != "cuda" or index.dtype != INDEX_DTYPE or num_nodes <= 0:
        # host-side planning and wide index types: plain tensor arithmetic
        local = torch.where(is_dummy_index(index), index, index % max(num_nodes, 1))
        return local.to(INDEX_DTYPE)
    index = index.contiguous()
    out = torch.empty_like(index)
    with torch.cuda.device(index.device):
        _lib.check(_lib.load().e3j_amd_wrap_index(index.data_ptr(), index.numel(), num_nodes,
                                                  out.data_ptr(), _stream_ptr(index.device)))
    return out


def fold_endpoints(group: torch.Tensor, guard: torch.Tensor, axis_size: int, num_nodes: int):
    """Fold `axis_size` graphs into one disjoint graph (`src/e3j/ops/convolution.py:54-78`).

    `group`, `guard`: `(axis_size, E)`.  Padding grouping endpoints move to their
    graph's last node so the folded key stays non-decreasing; guard endpoints keep
    the sentinel so kernels skip the edge.
    """
    offsets = (torch.arange(axis_size, dtype=group.dtype, device=group.device) * num_nodes)[:, None]
    last = offsets + (num_nodes - 1)
    group = torch.where(is_dummy_index(group), last.expand_as(group), group + offsets)
    guard = torch.where(is_dummy_index(guard), guard, guard + offsets)
    return group.reshape(-1), guard.reshape(-1)
