"""The stacked Clebsch-Gordan coefficient table and its row-wise evaluation.

Host side: selection rules, block stacking and the canonical sort of output blocks
(`src/e3j/core/tensor_product.py:169-274`, `src/e3j/core/permutation.py:55-74`), which
the fused convolution consumes.  Calling a `TensorProduct` evaluates the bilinear map
row by row with the fused HIP kernels of `e3j_amd.tp_ops`
(`src/e3j/core/tensor_product.py:322-343,404-420`).
"""

from __future__ import annotations


import numpy as np

from .clebsch_gordan import clebsch_gordan
from .options import Layout, MixingMode, TensorProductNormalization, config as _config
from .sparse import SparseCOO, sparse_coo
from .spaces import O3Space


def block_sort_permutation(space: O3Space):
    """Coordinate permutation sorting the blocks of `space` by (degree, parity).

    Returns `(sigma, sigma_inv, target)`: `sorted[i] = unsorted[sigma[i]]`, and
    `target` is the sorted space with equal irreps merged
    (`src/e3j/core/permutation.py:55-74`).
    """
    space = O3Space(space)
    sorted_space, order = space.sort(return_inverse=True)
    slices = space.slices()
    sigma = np.concatenate(
        [np.arange(slices[b].start, slices[b].stop) for b in order]
    ) if len(order) else np.zeros((0,), dtype=np.int64)
    return sigma, np.argsort(sigma), sorted_space.regroup()


class TensorProduct:
    r"""Coefficients of the bilinear map `z_i = \sum_{jk} c_{ijk} x_j y_k`."""

    def __init__(self, source, target=None, coef: SparseCOO | None = None, sort: bool = True,
                 config=None, layout=Layout.LEADING_CHANNELS, mode=MixingMode.OUTER,
                 normalization=TensorProductNormalization.NONE):
        if len(source) != 2:
            raise TypeError("TensorProduct expects a binary tuple as source argument.")
        self.source = tuple(O3Space(s) for s in source)
        self.config = _config.snapshot(config)
        self.layout = Layout.parse(layout)
        self.mode = MixingMode.parse(mode)
        self.normalization = TensorProductNormalization.parse(normalization)
        infer = coef is None
        if target is None:
            self.target = self.infer_target(self.source)
        elif infer:
            self.target = self.infer_target(self.source, O3Space(target))
        else:
            self.target = O3Space(target)
        self._coef = coef
        if sort and infer:
            other = self.sort()
            self.target, self._coef = other.target, other.coef

    # --- coefficient access ----------------------------------------------
    @property
    def coef(self) -> SparseCOO:
        if self._coef is None:
            self._coef = self.clebsch_gordan(self.target, *self.source, self.normalization)
        return self._coef

    @coef.setter
    def coef(self, value: SparseCOO):
        self._coef = value

    @property
    def values(self) -> np.ndarray:
        return self.coef.data

    @property
    def indices(self) -> np.ndarray:
        return self.coef.indices

    @property
    def shape(self):
        return self.coef.shape

    # --- construction ----------------------------------------------------
    @staticmethod
    def infer_target(source, target=None, sort: bool = False) -> O3Space:
        return O3Space.otimes(source[0], source[1], target, sort)

    def sort(self) -> "TensorProduct":
        """Permute output coordinates so blocks are ordered by (degree, parity)."""
        _, sigma_inv, target = block_sort_permutation(self.target)
        idx = self.indices.astype(np.int64)
        idx = np.concatenate((sigma_inv[idx[:, 0]][:, None], idx[:, 1:]), axis=-1)
        return TensorProduct(self.source, target, coef=sparse_coo(self.values, idx, self.shape),
                             sort=False, config=self.config, layout=self.layout, mode=self.mode,
                             normalization=self.normalization)

    # --- evaluation ------------------------------------------------------
    def packed_coef(self, val_dtype="float32") -> np.ndarray:
        """The table in the operator's wire format (`src/e3j/core/tensor_product.py:340-343`)."""
        from .coef import Coef
        idx = self.indices
        return Coef(self.values, idx, val_dtype=val_dtype, idx_dtype=idx.dtype).pack()

    def __call__(self, x, y):
        """Evaluate the bilinear map on GPU tensors with the fused HIP kernels (the
        counterpart of the reference's `FUSED_CUDA` branch,
        `src/e3j/core/tensor_product.py:322-343`); there is no other evaluation strategy."""
        import torch
        from .coef import resolve_val_dtype
        from .tp_ops import TensorProductParams, tensor_product
        dtype = torch.result_type(x, y)
        val_dtype = resolve_val_dtype(str(dtype).replace("torch.", ""))
        params = TensorProductParams(num_out=self.target.dim, mode=self.mode, layout=self.layout)
        return tensor_product(self.packed_coef(val_dtype), x.to(dtype), y.to(dtype), params)

    @staticmethod
    def clebsch_gordan(target, source_1, source_2,
                       normalization=TensorProductNormalization.NONE) -> SparseCOO:
        """Stack one Clebsch-Gordan block per path, in x-major / y / l_out order.

        `target` only filters which `(l, p)` are kept; the output coordinates are
        laid out path after path (`src/e3j/core/tensor_product.py:202-274`).
        """
        target, in1, in2 = O3Space(target), O3Space(source_1), O3Space(source_2)
        normalization = TensorProductNormalization.parse(normalization)
        wanted = {(ir.l, ir.p) for _, ir in target}
        scaled = normalization == TensorProductNormalization.SQRT_DIM_OUT
        shape = (target.dim, in1.dim, in2.dim)
        rows, vals = [], []
        out_at = 0   # first output coordinate of the next path
        for (mul_x, ir_x), at_x in zip(in1, in1.slices()):
            for (mul_y, ir_y), at_y in zip(in2, in2.slices()):
                for _, ir_o in ir_x * ir_y:
                    if (ir_o.l, ir_o.p) not in wanted:
                        continue
                    block = clebsch_gordan(ir_o.l, ir_x.l, ir_y.l)
                    if scaled:
                        block = block * np.sqrt(2 * ir_o.l + 1)
                    i, j, k = np.nonzero(block)
                    # every pair of copies (a of x, b of y) gets its own copy a * mul_y + b of
                    # the output irrep, all with the same block
                    for a in range(mul_x):
                        for b in range(mul_y):
                            copy = a * mul_y + b
                            rows.append(np.stack([out_at + copy * ir_o.dim + i,
                                                  at_x.start + a * ir_x.dim + j,
                                                  at_y.start + b * ir_y.dim + k], axis=1))
                            vals.append(block[i, j, k])
                    out_at += mul_x * mul_y * ir_o.dim
        if not rows:
            return sparse_coo(np.zeros((0,)), np.zeros((0, 3), dtype=np.int64), shape)
        return sparse_coo(np.concatenate(vals), np.concatenate(rows, axis=0), shape)
