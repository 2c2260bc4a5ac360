"""MI355X-native fused equivariant message-passing convolution.

Public names follow the reference package for this path: `Convolution`,
`convolution`, `convolution_bwd`, `TensorProduct`, `tensor_product`, `tensor_product_bwd`,
`Harmonics`, `GraphCSR`, `Coef4D`, `O3Space`, `config`; `edge_features` (positions to harmonics and
hidden radial layers in one launch), `radial_linear` (the radial network's last layer) and `ChannelMix`
(the per-degree mixing after a convolution) have no counterpart there.
Importing the package does not load the kernel library; the first operator call does,
and fails if `e3j_amd/lib/libe3j_amd.so` has not been built.
"""

from .channel_mix import ChannelMix
from .coef import Coef, Coef4D, resolve_val_dtype
from .convolution import Convolution
from .edge_features import edge_features
from .graph import DUMMY_INDEX, GraphCSR
from .harmonics import Harmonics
from .ops import (ConvolutionBatchingWarning, ConvolutionParams, CUDAConvolutionParams, TableDrivenKernelWarning,
                  PreparedGraph, clear_graph_cache, convolution, convolution_batched, convolution_bwd,
                  prepare_graph)
from .options import Config, GraphOrdering, Layout, MixingMode, TensorProductNormalization, config
from .radial import radial_linear
from .scalar_mixing import ScalarMixing
from .spaces import O3Irrep, O3Space
from .tensor_product import TensorProduct
from .tp_ops import (CUDATensorProductParams, TensorProductParams, tensor_product, tensor_product_batched,
                     tensor_product_bwd)

Space = O3Space

__all__ = [
    "Coef", "Coef4D", "Config", "Convolution", "ConvolutionBatchingWarning", "ConvolutionParams",
    "TableDrivenKernelWarning",
    "CUDAConvolutionParams", "DUMMY_INDEX", "GraphCSR", "GraphOrdering", "Harmonics", "Layout", "O3Irrep",
    "O3Space", "ScalarMixing", "Space", "TensorProduct", "TensorProductNormalization", "config",
    "convolution", "convolution_batched", "convolution_bwd", "radial_linear", "resolve_val_dtype",
    "edge_features", "ChannelMix",
    "PreparedGraph", "prepare_graph", "clear_graph_cache",
    "CUDATensorProductParams", "MixingMode", "TensorProductParams", "tensor_product", "tensor_product_batched", "tensor_product_bwd",
]
