"""Edge featurisation from atom positions in one kernel launch, forward and backward.

`edge_features(positions, sender, receiver, shift, w1, ...)` returns, for every edge, the harmonics
`y` of the direction of `positions[sender] - positions[receiver] + shift` and the hidden layer
`h = silu(basis @ w1[layer])` of the radial network of each convolution layer, where `basis` are
Bessel functions of the edge length under a polynomial cutoff envelope (`csrc/harmonics.hip`).
With `radial_linear` (the network's last layer) this is the whole producer chain of the convolution's
operands `y` and `s`; its backward adds the gradient of every edge vector to the two atoms of the edge
in one launch as well.  The reference leaves these steps to its callers as separate XLA operations
(`Harmonics`: `src/e3j/core/harmonics.py:45-101`; `edge_scalars` of
`src/e3j/core/convolution.py:342-350` arrive ready-made).
"""

from __future__ import annotations

import ctypes

import torch

from . import _lib
from .harmonics import _NORMALIZATIONS

_DTYPES = {torch.float32: _lib.F32, torch.float64: _lib.F64}


def _params(positions, sender, w1, l_max, normalization, cutoff):
    layers, num_basis, hidden = (int(d) for d in w1.shape)
    return _lib.EdgeFeaturesParams(
        num_edges=int(sender.shape[0]), num_nodes=int(positions.shape[0]), l_max=int(l_max),
        normalization=_NORMALIZATIONS[normalization], num_basis=num_basis, hidden=hidden, layers=layers,
        cutoff=float(cutoff), val_dtype=_DTYPES[positions.dtype])


class _EdgeFeatures(torch.autograd.Function):
    @staticmethod
    def forward(positions, shift, w1, sender, receiver, l_max, normalization, cutoff):
        p = _params(positions, sender, w1, l_max, normalization, cutoff)
        edges = int(sender.shape[0])
        y = torch.empty((edges, (l_max + 1) ** 2), dtype=positions.dtype, device=positions.device)
        h = torch.empty((p.layers, edges, p.hidden), dtype=positions.dtype, device=positions.device)
        with torch.cuda.device(positions.device):
            _lib.check(_lib.load().e3j_amd_edge_features_fwd(
                ctypes.byref(p), positions.data_ptr(), sender.data_ptr(), receiver.data_ptr(),
                shift.data_ptr() if shift is not None else None, w1.data_ptr(), y.data_ptr(), None, h.data_ptr(),
                int(torch.cuda.current_stream(positions.device).cuda_stream)))
        return y, h

    @staticmethod
    def setup_context(ctx, inputs, output):
        positions, shift, w1, sender, receiver, l_max, normalization, cutoff = inputs
        ctx.args = (l_max, normalization, cutoff)
        ctx.has_shift = shift is not None
        ctx.save_for_backward(positions, w1, sender, receiver, *((shift,) if shift is not None else ()))

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, dy, dh):
        positions, w1, sender, receiver, *rest = ctx.saved_tensors
        shift = rest[0] if ctx.has_shift else None
        if ctx.needs_input_grad[1] or ctx.needs_input_grad[2]:
            raise NotImplementedError("edge_features is differentiable with respect to the positions only")
        p = _params(positions, sender, w1, *ctx.args)
        dpos = torch.empty_like(positions)
        dy = dy.contiguous() if dy is not None else None
        dh = dh.contiguous() if dh is not None else None
        with torch.cuda.device(positions.device):
            _lib.check(_lib.load().e3j_amd_edge_features_bwd(
                ctypes.byref(p), positions.data_ptr(), sender.data_ptr(), receiver.data_ptr(),
                shift.data_ptr() if shift is not None else None, w1.data_ptr(),
                dy.data_ptr() if dy is not None else None, None, dh.data_ptr() if dh is not None else None,
                dpos.data_ptr(), int(torch.cuda.current_stream(positions.device).cuda_stream)))
        return dpos, None, None, None, None, None, None, None


def supported(positions: torch.Tensor, w1: torch.Tensor, l_max: int) -> bool:
    """Whether `edge_features` has a kernel for these operands."""
    return (positions.is_cuda and positions.dtype in _DTYPES and w1.dim() == 3 and 0 <= l_max <= 6
            and 1 <= int(w1.shape[1]) <= 16)


def edge_features(positions: torch.Tensor, sender: torch.Tensor, receiver: torch.Tensor,
                  shift: torch.Tensor | None, w1: torch.Tensor, l_max: int, cutoff: float,
                  normalization: str = "component"):
    """`(y, h)`: harmonics `(E, (l_max + 1)^2)` of the unit edge vectors and hidden layers
    `(layers, E, hidden)` of the radial networks, `w1 (layers, num_basis, hidden)`.

    `positions (N, 3)` float32 or float64 in GPU memory, `sender` / `receiver (E,)` int32, `shift (E, 3)`
    or None.  Differentiable once, with respect to `positions`.
    """
    if not supported(positions, w1, l_max):
        raise ValueError("edge_features: GPU positions in float32 or float64, w1 (layers, num_basis <= 16, hidden), "
                         "l_max <= 6")
    if sender.dtype != torch.int32 or receiver.dtype != torch.int32:
        sender, receiver = sender.to(torch.int32), receiver.to(torch.int32)
    positions = positions.contiguous()
    w1 = w1.to(dtype=positions.dtype).contiguous()
    shift = shift.to(dtype=positions.dtype).contiguous() if shift is not None else None
    return _EdgeFeatures.apply(positions, shift, w1, sender.contiguous(), receiver.contiguous(), int(l_max),
                               normalization, float(cutoff))
