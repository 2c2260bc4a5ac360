"""Packed wire format of the sparse coefficient operand.

A table entry is the C struct `{val; i; j; k[; l]}` padded to the next power
of two of `sizeof(val) + rank*sizeof(idx)`, `val` at offset 0 and the indices
from `ceil(sizeof(val)/sizeof(idx))*sizeof(idx)`; the table travels as an
opaque `(nnz, itemsize/sizeof(idx))` array of the index dtype.  Byte layout
and API follow `src/e3j/ops/coef.py:68-235` and the struct it mirrors,
`lib/e3j_ops/cuda/convolution.cuh:31-44` (sizes 8/16/32 bytes).
"""

from __future__ import annotations

import numpy as np

SUPPORTED_VAL_DTYPES = ("float16", "float32", "float64")
SUPPORTED_IDX_DTYPES = ("int32", "uint8")


def next_pow2(n: int) -> int:
    return 1 if n <= 1 else 1 << (int(n) - 1).bit_length()


def resolve_val_dtype(input_dtype) -> str:
    """Value dtype the kernels run in; raises `TypeError` outside f16/f32/f64."""
    name = np.dtype(input_dtype).name
    if name not in SUPPORTED_VAL_DTYPES:
        raise TypeError(f"Fused ops support value dtypes {SUPPORTED_VAL_DTYPES}, "
                        f"got {name!r}. Cast the operands.")
    return name


class Coef:
    """`(val, idx)` COO pair with its packed representation; rank 3: `(i, j, k)`."""

    rank = 3
    index_names = ("i", "j", "k")

    def __init__(self, val, idx, val_dtype="float32", idx_dtype="int32"):
        self.val = np.asarray(val)
        self.idx = np.asarray(idx)
        self.val_dtype = np.dtype(val_dtype).name
        self.idx_dtype = np.dtype(idx_dtype).name
        if self.val_dtype not in SUPPORTED_VAL_DTYPES:
            raise ValueError(f"unsupported value dtype {self.val_dtype}")
        if self.idx_dtype not in SUPPORTED_IDX_DTYPES:
            raise ValueError(f"unsupported index dtype {self.idx_dtype}")
        if self.idx.shape[:-1] != self.val.shape or self.idx.shape[-1] != self.rank:
            raise ValueError(f"idx must have shape val.shape + ({self.rank},), "
                             f"got {self.idx.shape} for {self.val.shape}")

    @classmethod
    def _numpy_dtype(cls, val_t, idx_t) -> np.dtype:
        """The entry as a numpy record: the value first, the indices behind it at the first
        multiple of the index size, the record padded to a power of two (the `alignas` of
        `lib/e3j_ops/cuda/convolution.cuh:31-44`)."""
        val_t, idx_t = np.dtype(val_t), np.dtype(idx_t)
        step = idx_t.itemsize
        first_index = -(-val_t.itemsize // step) * step
        offsets = {"val": 0}
        for n, name in enumerate(cls.index_names):
            offsets[name] = first_index + n * step
        names = ["val", *cls.index_names]
        return np.dtype({
            "names": names,
            "formats": [val_t] + [idx_t] * cls.rank,
            "offsets": [offsets[n] for n in names],
            "itemsize": next_pow2(val_t.itemsize + cls.rank * step),
        })

    @property
    def dtype(self) -> np.dtype:
        return self._numpy_dtype(self.val_dtype, self.idx_dtype)

    def __iter__(self):
        return zip(self.val, self.idx)

    def __len__(self):
        return int(self.val.shape[0])

    def pack_numpy(self) -> np.ndarray:
        out = np.zeros(self.val.shape[0], dtype=self.dtype)  # zeroed padding bytes
        out["val"] = self.val.astype(self.val_dtype)
        for col, name in enumerate(self.index_names):
            out[name] = self.idx[:, col].astype(self.idx_dtype)
        return out

    def pack(self) -> np.ndarray:
        packed = self.pack_numpy()
        idx_t = np.dtype(self.idx_dtype)
        numel, rem = divmod(self.dtype.itemsize, idx_t.itemsize)
        if rem:
            raise TypeError(f"Cannot pack dtype pair: size of {idx_t} does not divide "
                            f"the struct size {self.dtype.itemsize}.")
        return packed.view(idx_t).reshape(-1, numel)

    def transpose(self, argnums):
        """The table with its index columns reordered to `argnums` and its entries grouped by the
        new leading column, earlier entries first within a group (behaviour of
        `src/e3j/ops/coef.py:174-184`)."""
        columns = self.idx[:, list(argnums)]
        order = np.argsort(columns[:, 0], kind="stable")
        return type(self)(self.val[order], columns[order], self.val_dtype, self.idx_dtype)

    @classmethod
    def unpack(cls, data, val_dtype):
        """Inverse of `pack` / `pack_numpy`: read the records back through the record dtype."""
        data = np.ascontiguousarray(data)
        idx_t = data.dtype if data.dtype.fields is None else data.dtype["i"]
        record = cls._numpy_dtype(val_dtype, idx_t)
        table = data.view(np.uint8).reshape(-1).view(record) if data.size else np.zeros(0, dtype=record)
        idx = np.stack([table[name] for name in cls.index_names], axis=1) if len(table) else \
            np.zeros((0, cls.rank), dtype=idx_t)
        return cls(np.array(table["val"]), idx, np.dtype(val_dtype), idx_t)


class Coef4D(Coef):
    """Rank 4: `(i, j, k, l)` = (output, x, y, scalar) coordinates."""

    rank = 4
    index_names = ("i", "j", "k", "l")
