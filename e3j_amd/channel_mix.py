"""Per-degree channel mixing after a convolution: `x'[n, m, c] = sum_{u, k} out[n, (l, u, m), k] W_l[u, k, c]`.

The convolution writes, for every output degree `l`, `mul` copies of `2l + 1` rows; the linear layer
that follows mixes copies and channels per degree (`src/e3j/core/linear.py:125-243` in the reference:
slices, a product per block, a join).  Here float32 rows of 64 or 128 channels are mixed by one
launch of a matrix-core kernel each way (`e3j_amd_channel_mix`, `csrc/channel_mix.hip`); other
dtypes and channel counts take one kernel launch that regroups all rows into the operands
`A_l[(n, m), (u, k)]` of one library matrix product per degree, and a second that puts the results
into `(N, X, K)`; the backward pass runs the same moves in the other direction, so that every
cotangent row is written once.
"""

from __future__ import annotations

import numpy as np
import torch

from . import _lib

_DTYPES = {torch.float32: _lib.F32, torch.float64: _lib.F64}


def _regroup(src, dst, num_nodes, rows, channels, base, stride, to_plain):
    with torch.cuda.device(src.device):
        _lib.check(_lib.load().e3j_amd_rows_regroup(
            src.data_ptr(), dst.data_ptr(), int(num_nodes), int(rows), int(channels), base.data_ptr(),
            stride.data_ptr(), int(to_plain), _DTYPES[src.dtype],
            int(torch.cuda.current_stream(src.device).cuda_stream)))


class _Mix(torch.autograd.Function):
    @staticmethod
    def forward(out, mixer, weights):
        return mixer._forward(out.contiguous(), weights)

    @staticmethod
    def setup_context(ctx, inputs, output):
        out, mixer, weights = inputs
        ctx.mixer, ctx.weights, ctx.num_nodes = mixer, weights, int(out.shape[0])

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, dx):
        return ctx.mixer._backward(dx.contiguous(), ctx.weights, ctx.num_nodes), None, None


class ChannelMix:
    """`blocks`: `(mul, dim)` of every output degree in row order; `weights[l] (mul, K, K)` numpy arrays.
    Call with `out (N, Z, K)` in GPU memory (float32 or float64): returns `(N, X, K)`, `X = sum dim`.
    Differentiable once, with respect to `out` (the weights are constants of the layer)."""

    def __init__(self, blocks, channels: int, weights):
        self.blocks = [(int(m), int(d)) for m, d in blocks]
        self.channels = int(channels)
        self.rows_in = sum(m * d for m, d in self.blocks)
        self.rows_out = sum(d for _, d in self.blocks)
        self._weights = [np.ascontiguousarray(w).reshape(m * self.channels, self.channels)
                         for w, (m, _) in zip(weights, self.blocks)]
        self._device = {}

    def _tables(self, num_nodes: int, device):
        """Row tables of the two regroupings for `num_nodes` nodes, and the weights, on `device`."""
        key = (int(num_nodes), device)
        hit = self._device.get(key)
        if hit is not None:
            return hit
        K, n = self.channels, int(num_nodes)
        a_base, a_stride, c_base, c_stride, spans = [], [], [], [], []
        a_off = c_off = 0
        for mul, dim in self.blocks:
            for u in range(mul):
                for m in range(dim):
                    a_base.append(a_off + m * mul * K + u * K)
                    a_stride.append(dim * mul * K)
            for m in range(dim):
                c_base.append(c_off + m * K)
                c_stride.append(dim * K)
            spans.append((a_off, n * dim, mul * K, c_off))
            a_off += n * dim * mul * K
            c_off += n * dim * K
        as_dev = lambda v: torch.as_tensor(np.asarray(v, dtype=np.int64), device=device)  # noqa: E731
        hit = self._device[key] = (as_dev(a_base), as_dev(a_stride), as_dev(c_base), as_dev(c_stride), spans)
        return hit

    def _weight(self, l: int, like: torch.Tensor) -> torch.Tensor:
        key = ("w", l, like.dtype, like.device)
        hit = self._device.get(key)
        if hit is None:
            hit = self._device[key] = torch.as_tensor(self._weights[l], dtype=like.dtype, device=like.device)
        return hit

    def _fused(self, src: torch.Tensor, transpose: bool):
        """The mixing (or its transpose) in one launch of the library's matrix-core kernel, or None
        where that kernel does not apply (it takes float32 at 64 or 128 channels, up to 8 degrees)."""
        import ctypes
        K = self.channels
        if src.dtype != torch.float32 or K not in (64, 128) or len(self.blocks) > 8 or src.data_ptr() % 16:
            return None
        key = ("fused", transpose, src.device)
        w = self._device.get(key)
        if w is None:
            parts = [wl.reshape(m, K, K) for wl, (m, _) in zip(self._weights, self.blocks)]
            if transpose:
                parts = [p.transpose(0, 2, 1) for p in parts]
            flat = np.concatenate([np.ascontiguousarray(p, dtype=np.float32).reshape(-1) for p in parts])
            w = self._device[key] = torch.as_tensor(flat, device=src.device)
        n = int(src.shape[0])
        dst = torch.empty((n, self.rows_in if transpose else self.rows_out, K), dtype=src.dtype, device=src.device)
        mul = (ctypes.c_int32 * len(self.blocks))(*[m for m, _ in self.blocks])
        dim = (ctypes.c_int32 * len(self.blocks))(*[d for _, d in self.blocks])
        with torch.cuda.device(src.device):
            _lib.check(_lib.load().e3j_amd_channel_mix(
                src.data_ptr(), dst.data_ptr(), w.data_ptr(), n, K, len(self.blocks), mul, dim, int(transpose),
                int(torch.cuda.current_stream(src.device).cuda_stream)))
        return dst

    def _forward(self, out: torch.Tensor, weights) -> torch.Tensor:
        fused = self._fused(out, transpose=False)
        if fused is not None:
            return fused
        n, K = int(out.shape[0]), self.channels
        a_base, a_stride, c_base, c_stride, spans = self._tables(n, out.device)
        grouped = torch.empty(n * self.rows_in * K, dtype=out.dtype, device=out.device)
        _regroup(out, grouped, n, self.rows_in, K, a_base, a_stride, to_plain=False)
        mixed = torch.empty(n * self.rows_out * K, dtype=out.dtype, device=out.device)
        for l, (a_off, rows, inner, c_off) in enumerate(spans):
            torch.mm(grouped[a_off:a_off + rows * inner].view(rows, inner), self._weight(l, out),
                     out=mixed[c_off:c_off + rows * K].view(rows, K))
        x = torch.empty((n, self.rows_out, K), dtype=out.dtype, device=out.device)
        _regroup(mixed, x, n, self.rows_out, K, c_base, c_stride, to_plain=True)
        return x

    def _backward(self, dx: torch.Tensor, weights, n: int) -> torch.Tensor:
        fused = self._fused(dx, transpose=True)
        if fused is not None:
            return fused
        K = self.channels
        a_base, a_stride, c_base, c_stride, spans = self._tables(n, dx.device)
        dmixed = torch.empty(n * self.rows_out * K, dtype=dx.dtype, device=dx.device)
        _regroup(dx, dmixed, n, self.rows_out, K, c_base, c_stride, to_plain=False)
        dgrouped = torch.empty(n * self.rows_in * K, dtype=dx.dtype, device=dx.device)
        for l, (a_off, rows, inner, c_off) in enumerate(spans):
            torch.mm(dmixed[c_off:c_off + rows * K].view(rows, K), self._weight(l, dx).t(),
                     out=dgrouped[a_off:a_off + rows * inner].view(rows, inner))
        dout = torch.empty((n, self.rows_in, K), dtype=dx.dtype, device=dx.device)
        _regroup(dgrouped, dout, n, self.rows_in, K, a_base, a_stride, to_plain=True)
        return dout

    def __call__(self, out: torch.Tensor) -> torch.Tensor:
        if not (out.is_cuda and out.dtype in _DTYPES and out.dim() == 3 and int(out.shape[1]) == self.rows_in
                and int(out.shape[2]) == self.channels):
            raise ValueError(f"ChannelMix: expected a GPU tensor (N, {self.rows_in}, {self.channels}) in float32 or "
                             f"float64, got {tuple(out.shape)} {out.dtype} on {out.device}")
        return _Mix.apply(out, self, None)
