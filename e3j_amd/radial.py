"""Last layer of the radial network: `s = h @ w` on the matrix cores.

The per-edge, per-path weights `s (E, paths * channels)` are the operand the convolution reads
most; the layer that writes them is a product with a small inner size (the hidden width of the
radial network), bound by the stream it writes.  `radial_linear` runs it as one HIP kernel
(`csrc/radial_linear.hip`), and so does `dw = h.T @ ds` of its backward (the contraction runs over
the edges: both operands arrive coalesced) and, from inner size 64 on, `dh = ds @ w.T` (the stream
transposed through LDS); below that the library product already reads `ds` near the rate of the memory.
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


def _aligned(t: torch.Tensor) -> torch.Tensor:
    """Contiguous and 16-byte aligned (a contiguous view at an odd element offset is copied)."""
    t = t.contiguous()
    return t if t.data_ptr() % 16 == 0 else t.clone()


class _RadialLinear(torch.autograd.Function):
    @staticmethod
    def forward(h, w):
        h, w = _aligned(h), _aligned(w)
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
        dh = _input_gradient(ds, w) if ctx.needs_input_grad[0] else None
        dw = _weight_gradient(h, ds) if ctx.needs_input_grad[1] else None
        return dh, dw


def _input_gradient(ds: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """`ds @ w.T`: from inner size 64 on the kernel that transposes `ds` through LDS; below, and when
    autograd records the backward, the library product (which reads `ds` near the rate of the memory)."""
    if (int(w.shape[0]) < 64 or ds.dtype != torch.float32
            or torch.is_grad_enabled() and (ds.requires_grad or w.requires_grad)):
        return ds @ w.t()
    ds, wt = _aligned(ds), w.t().contiguous()
    dh = torch.empty((ds.shape[0], w.shape[0]), dtype=ds.dtype, device=ds.device)
    with torch.cuda.device(ds.device):
        _lib.check(_lib.load().e3j_amd_radial_linear_bwd_input(
            ds.data_ptr(), wt.data_ptr(), dh.data_ptr(), int(ds.shape[0]), int(w.shape[0]), int(w.shape[1]),
            torch.cuda.current_stream(ds.device).cuda_stream))
    return dh


def _weight_gradient(h: torch.Tensor, ds: torch.Tensor) -> torch.Tensor:
    """`h.T @ ds` on the matrix cores (the library product when autograd records the backward,
    e.g. for a second derivative, or for tensors the kernel does not take)."""
    if torch.is_grad_enabled() and (h.requires_grad or ds.requires_grad) or ds.dtype != torch.float32:
        return h.t() @ ds
    lib = _lib.load()
    h, ds = _aligned(h), _aligned(ds)
    edges, inner, n = int(h.shape[0]), int(h.shape[1]), int(ds.shape[1])
    dw = torch.empty((inner, n), dtype=h.dtype, device=h.device)
    ws = torch.empty(max(int(lib.e3j_amd_radial_linear_bwd_weight_workspace_bytes(edges, inner, n)), 4),
                     dtype=torch.uint8, device=h.device)
    with torch.cuda.device(h.device):
        _lib.check(lib.e3j_amd_radial_linear_bwd_weight(
            h.data_ptr(), ds.data_ptr(), dw.data_ptr(), ws.data_ptr(), edges, inner, n,
            torch.cuda.current_stream(h.device).cuda_stream))
    return dw


def radial_linear(h: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """`h (E, inner) @ w (inner, n)`, float32 tensors in GPU memory; inner in `INNER_SIZES`, n a
    multiple of 32.  Differentiable in both operands."""
    if not supported(h, w):
        raise ValueError("radial_linear: float32 GPU matrices (E, inner) and (inner, n) with inner in "
                         f"{INNER_SIZES} and n a multiple of 32; got {tuple(h.shape)} {h.dtype} on {h.device} and "
                         f"{tuple(w.shape)} {w.dtype} on {w.device}")
    return _RadialLinear.apply(h, w)
