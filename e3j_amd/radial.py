"""Last layer of the radial network: `s = h @ w` on the matrix cores.

The per-edge, per-path weights `s (E, paths * channels)` are the operand the convolution reads
most; the layer that writes them is a product with a small inner size (the hidden width of the
radial network), bound by the stream it writes.  `radial_linear` runs it as one HIP kernel
(`csrc/radial_linear.hip`); the products of its backward, `ds @ w.T` and `h.T @ ds`, read the
stream along the contracted index and are left to the library.
"""

from __future__ import annotations

import torch

from . import _lib

INNER_SIZES = (8, 16, 32, 64, 128)


def supported(h: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether `radial_linear` has a kernel for these operands."""
    return (h.is_cuda and w.is_cuda and h.dtype == torch.float32 and w.dtype == torch.float32 and h.dim() == 2
            and w.dim() == 2 and h.shape[1] == w.shape[0] and int(w.shape[0]) in INNER_SIZES
            and int(w.shape[1]) % 32 == 0)


class _RadialLinear(torch.autograd.Function):
    @staticmethod
    def forward(h, w):
        h, w = h.contiguous(), w.contiguous()
        s = torch.empty((h.shape[0], w.shape[1]), dtype=h.dtype, device=h.device)
        with torch.cuda.device(h.device):
            _lib.check(_lib.load().e3j_amd_radial_linear_fwd(
                h.data_ptr(), w.data_ptr(), s.data_ptr(), int(h.shape[0]), int(w.shape[0]), int(w.shape[1]),
                torch.cuda.current_stream(h.device).cuda_stream))
        return s

    @staticmethod
    def setup_context(ctx, inputs, output):
        ctx.save_for_backward(*inputs)

    @staticmethod
    def backward(ctx, ds):
        h, w = ctx.saved_tensors
        dh = ds @ w.t() if ctx.needs_input_grad[0] else None
        dw = h.t() @ ds if ctx.needs_input_grad[1] else None
        return dh, dw


def radial_linear(h: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """`h (E, inner) @ w (inner, n)`, float32 tensors in GPU memory; inner in `INNER_SIZES`, n a
    multiple of 32.  Differentiable in both operands."""
    if not supported(h, w):
        raise ValueError("radial_linear: float32 GPU matrices (E, inner) and (inner, n) with inner in "
                         f"{INNER_SIZES} and n a multiple of 32; got {tuple(h.shape)} {h.dtype} on {h.device} and "
                         f"{tuple(w.shape)} {w.dtype} on {w.device}")
    return _RadialLinear.apply(h, w)
