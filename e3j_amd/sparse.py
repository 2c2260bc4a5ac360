"""Sparse COO arrays of compile-time constant coefficients (host side, numpy).

Follows `src/e3j/utils/sparse.py:29-126`: coalescing sorts coordinates
lexicographically, sums duplicates and drops exact zeros; coordinates are
narrowed to `uint8` when every dimension fits, else `int32`; values are
stored as float32 (the canonical value dtype of the reference without x64).
"""

from __future__ import annotations

import dataclasses
import math

import numpy as np


def narrow_index_dtype(shape) -> np.dtype:
    """`uint8` when all dims are <= 255, else `int32` (`src/e3j/utils/sparse.py:29-46`)."""
    return np.dtype(np.uint8) if max(shape) <= np.iinfo(np.uint8).max else np.dtype(np.int32)


@dataclasses.dataclass(frozen=True, eq=False)
class SparseCOO:
    data: np.ndarray      # (nnz,)
    indices: np.ndarray   # (nnz, ndim)
    shape: tuple

    @property
    def nnz(self) -> int:
        return int(self.indices.shape[0])

    def todense(self) -> np.ndarray:
        dense = np.zeros(self.shape, dtype=self.data.dtype)
        np.add.at(dense, tuple(self.indices.astype(np.int64).T), self.data)
        return dense


def sparse_coo(values, indices, shape, coalesce: bool = True, dtype=np.float32) -> SparseCOO:
    """Build a `SparseCOO`; coalesced by default: entries in lexicographic order of their
    coordinates, repeated coordinates merged by summation, entries that sum to exactly zero
    removed (behaviour of `src/e3j/utils/sparse.py:76-126`)."""
    shape = tuple(int(n) for n in shape)
    coords = np.asarray(indices, dtype=np.int64)
    vals = np.asarray(values).astype(dtype)
    rank = len(shape)
    if coords.ndim != 2 or coords.shape[1] != rank:
        raise ValueError(f"indices must be (nnz, {rank}) for a rank-{rank} array of shape {shape}; got {coords.shape}")
    if len(vals) != len(coords):
        raise ValueError(f"{len(vals)} values do not pair with {len(coords)} coordinate rows")
    limits = np.asarray(shape, dtype=np.int64).reshape(1, rank)
    if coords.size and not ((coords >= 0) & (coords < limits)).all():
        raise ValueError(f"Out of bounds indices for shape {shape}.")
    if coalesce and len(coords):
        # The distinct coordinates in lexicographic order and, per entry, which of them it falls
        # on.  Duplicates are added in the value dtype, one after another in the order the
        # entries were given (`np.add.at` is unbuffered), and an entry is dropped when that sum is
        # exactly zero in the value dtype: the arithmetic of `src/e3j/utils/sparse.py:116-124`.
        if math.prod(shape) <= np.iinfo(np.int64).max:
            # row-major linear positions: ascending positions = lexicographic coordinates
            strides = np.concatenate([np.cumprod(limits[0, :0:-1])[::-1], [1]]).astype(np.int64)
            distinct, slot = np.unique(coords @ strides, return_inverse=True)
            distinct = np.stack(np.unravel_index(distinct, shape), axis=1).astype(np.int64)
        else:  # the linear position would overflow: compare coordinate rows
            distinct, slot = np.unique(coords, axis=0, return_inverse=True)
        merged = np.zeros(len(distinct), dtype=vals.dtype)
        np.add.at(merged, slot.reshape(-1), vals)
        alive = merged != 0
        coords, vals = distinct[alive], merged[alive]
    return SparseCOO(vals, coords.astype(narrow_index_dtype(shape)), shape)
