"""`Convolution`: the equivariant message-passing block, backed by the HIP kernels.

Same constructor and call signature as the reference's class
(`src/e3j/core/convolution.py:85-95,342-350`):

    m_b = 1/N * sum_a (x_a (x) y_ab) . s_ab

with the sum over the senders `a` of receiver `b`.  It builds the stacked
Clebsch-Gordan table and the scalar-mixing index map on the host, folds
`1/avg_num_neighbors` into the coefficients (`:135-140`), packs them as
`Coef4D(val, [i, j, k, mix_idx[i]])` (`:159-170`) and calls the fused operator.
"""

from __future__ import annotations

import numpy as np
import torch

from .coef import Coef4D, resolve_val_dtype
from .graph import GraphCSR
from .ops import ConvolutionParams, convolution
from .options import Convolution as ConvolutionImpl
from .options import GraphOrdering, Layout, TensorProductNormalization, config as _config
from .scalar_mixing import ScalarMixing
from .sparse import sparse_coo
from .spaces import O3Space
from .tensor_product import TensorProduct

_NP_OF_TORCH = {torch.float32: np.float32, torch.float64: np.float64, torch.float16: np.float16}


class Convolution:
    """Equivariant message-passing convolution (no parameters of its own)."""

    def __init__(self, source, target=None, *, graph_ordering, layout=Layout.TRAILING_CHANNELS,
                 avg_num_neighbors: float | None = None,
                 normalization=TensorProductNormalization.SQRT_DIM_OUT, config=None):
        self.config = _config.snapshot(config)
        otimes = TensorProduct((source[0], source[1]), target, normalization=normalization,
                               layout=layout, config=self.config)
        if avg_num_neighbors is not None:
            otimes.coef = sparse_coo(otimes.values / avg_num_neighbors, otimes.indices,
                                     otimes.coef.shape)
        mix = ScalarMixing(otimes.target, layout=layout)
        self.source = (*otimes.source, O3Space([(mix.num_irreps, (0, 1))]))
        self.target = otimes.target
        self.avg_num_neighbors = avg_num_neighbors
        self.layout = Layout.parse(layout)
        self.normalization = otimes.normalization
        self.graph_ordering = GraphOrdering.parse(graph_ordering)
        self._otimes = otimes
        self._mix = mix
        self._coef = None
        self._packed = {}

    @property
    def coef(self) -> Coef4D:
        """Packed-ready `Coef4D` of the forward pass."""
        if self._coef is None:
            idx = self._otimes.indices.T
            mix_idx = self._mix.mix_indices.astype(idx.dtype)
            self._coef = Coef4D(self._otimes.values,
                                np.stack([idx[0], idx[1], idx[2], mix_idx[idx[0]]], axis=-1),
                                val_dtype=np.float32, idx_dtype=idx.dtype)
        return self._coef

    @property
    def params(self) -> ConvolutionParams:
        return ConvolutionParams(num_out=self.target.dim, num_scalars=self._mix.num_irreps)

    @property
    def y_parity(self) -> np.ndarray:
        """Parity of every `y` coordinate, used to sign coefficients under SENDER ordering."""
        return np.concatenate([np.full(m * ir.dim, float(ir.p), dtype=np.float32)
                               for m, ir in self._otimes.source[1]])

    def _packed_coef(self, val_dtype: str) -> np.ndarray:
        packed = self._packed.get(val_dtype)
        if packed is None:
            c = self.coef
            packed = self._packed[val_dtype] = Coef4D(c.val, c.idx, val_dtype=val_dtype,
                                                      idx_dtype=c.idx_dtype).pack()
            packed.setflags(write=False)   # frozen: the operators may key their caches on its identity
        return packed

    def _fused_eval(self, node_features, edge_features, edge_scalars, senders, receivers, graph=None):
        dtype = torch.promote_types(torch.promote_types(node_features.dtype, edge_features.dtype),
                                    edge_scalars.dtype)
        val_dtype = resolve_val_dtype(_NP_OF_TORCH.get(dtype, "int64"))
        node_features = node_features.to(dtype)
        edge_features = edge_features.to(dtype)
        edge_scalars = edge_scalars.to(dtype)
        y_parity = self.y_parity if self.graph_ordering == GraphOrdering.SENDER else None
        return convolution(self._packed_coef(val_dtype), node_features, edge_features, edge_scalars,
                           senders, receivers, self.params, self.graph_ordering, y_parity,
                           layout=self.layout, graph=graph)

    def __call__(self, node_features, edge_features, edge_scalars, senders, receivers,
                 node_mask=None, graph=None):
        """Sum of messages on receiver nodes.

        node_features `(num_nodes, num_x, channels)`, edge_features `(num_edges, num_y)`,
        edge_scalars `(num_edges, num_scalars, channels)` (leading layout: channels before
        the irreps axis); `node_mask` marks real nodes, padding nodes lie at the tail.
        `graph`: optional `prepare_graph` handle of `(senders, receivers)` in this module's
        ordering (not together with `node_mask`, which changes the edges).
        """
        if node_mask is not None and graph is not None:
            raise ValueError("`graph` was prepared for the unmasked edges; pass either `node_mask` or `graph`")
        if node_mask is not None:
            senders, receivers = GraphCSR.mask_edges(senders, receivers, node_mask)
        if self.config.convolution == ConvolutionImpl.FUSED_HIP:
            return self._fused_eval(node_features, edge_features, edge_scalars, senders, receivers, graph)
        raise RuntimeError("Unknown convolution implementation.")
