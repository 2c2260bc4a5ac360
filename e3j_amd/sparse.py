"""Sparse COO arrays of compile-time constant coefficients (host side, numpy).

Follows `src/e3j/utils/sparse.py:29-126`: coalescing sorts coordinates
lexicographically, sums duplicates and drops exact zeros; coordinates are
narrowed to `uint8` when every dimension fits, else `int32`; values are
stored as float32 (the canonical value dtype of the reference without x64).
"""

from __future__ import annotations

import dataclasses

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
    """Build a `SparseCOO`, coalesced by default (`src/e3j/utils/sparse.py:76-126`)."""
    shape = tuple(int(n) for n in shape)
    values = np.asarray(values).astype(dtype)
    indices = np.asarray(indices, dtype=np.int64)
    if indices.ndim != 2 or indices.shape[1] != len(shape):
        raise ValueError(f"Expected indices of shape (nnz, {len(shape)}) for shape {shape}, "
                         f"got {indices.shape}.")
    if indices.shape[0] != values.shape[0]:
        raise ValueError(f"Got {values.shape[0]} values for {indices.shape[0]} indices.")
    if indices.size and ((indices < 0).any() or (indices >= np.asarray(shape)).any()):
        raise ValueError(f"Out of bounds indices for shape {shape}.")
    if coalesce and indices.shape[0]:
        keys = np.ravel_multi_index(tuple(indices.T), shape)
        order = np.argsort(keys, kind="stable")
        keys = keys[order]
        first = np.ones(keys.shape[0], dtype=bool)
        np.not_equal(keys[1:], keys[:-1], out=first[1:])
        summed = np.zeros(int(first.sum()), dtype=values.dtype)
        np.add.at(summed, np.cumsum(first) - 1, values[order])
        indices = indices[order[first]]
        keep = summed != 0
        indices, values = indices[keep], summed[keep]
    return SparseCOO(values, indices.astype(narrow_index_dtype(shape)), shape)
