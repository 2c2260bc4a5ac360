"""The fused row-wise tensor product operators: `tensor_product` and `tensor_product_bwd`.

Same signatures, argument meaning and errors as the reference's primitives
(`src/e3j/ops/tensor_product.py:50-145,276-326`), with tensors in GPU memory and the
HIP library of this package behind them.  `tensor_product` is differentiable in
`(x, y)` to any reverse-mode order: its backward is `tensor_product_bwd`, whose own
backward is one `tensor_product_bwd` and two `tensor_product` calls
(`src/e3j/ops/tensor_product.py:571-591`).

Extensions over the reference's operator: any channel count (no power-of-two rule in
the trailing layout), MAP mode served directly in the leading layout, and a fused
backward in both layouts (the reference falls back to two forward products in the
leading layout).
"""

from __future__ import annotations

import ctypes
import dataclasses

import numpy as np
import torch

from . import _lib
from .coef import Coef
from .options import Layout, MixingMode, config

_VAL_DTYPES = {torch.float32: (_lib.F32, np.float32), torch.float64: (_lib.F64, np.float64),
               torch.float16: (_lib.F16, np.float16)}


@dataclasses.dataclass
class TensorProductParams:
    """Static description of the operator (`src/e3j/ops/tensor_product.py:41-45`)."""

    num_out: int
    mode: str | MixingMode = MixingMode.OUTER
    layout: str | Layout = Layout.LEADING_CHANNELS


#: name used by code written against the reference
CUDATensorProductParams = TensorProductParams


def _is_sorted(first_column: np.ndarray) -> bool:
    return bool(np.all(np.diff(first_column.astype(np.int64)) >= 0))


class _Table:
    """A packed rank-3 coefficient table, its two transposes and their device copies."""

    _cache: dict = {}

    def __init__(self, packed: np.ndarray, val_np_dtype):
        self.packed = np.ascontiguousarray(packed)
        self.idx_bytes = self.packed.dtype.itemsize
        self.val_np_dtype = np.dtype(val_np_dtype)
        self.num_coef = int(self.packed.shape[0])
        c = Coef.unpack(self.packed, self.val_np_dtype)
        self.sorted = _is_sorted(c.idx[:, 0]) if self.num_coef else True
        # dx and dy tables: columns (j, i, k) and (k, i, j), stable-sorted by the new first
        # column (src/e3j/ops/tensor_product.py:331-338); always sorted, whatever the input
        self.packed_bwd = np.ascontiguousarray(np.stack(
            [c.transpose((1, 0, 2)).pack(), c.transpose((2, 0, 1)).pack()]))
        self._device = {}
        self._signature = {}

    def signature(self, num_x: int, num_y: int, num_out: int, channels: int, kind: int,
                  layout: Layout = Layout.TRAILING_CHANNELS):
        """`(id, scale)` of a built-in unrolled kernel, `(-1, 1.0)` if none matches.  `kind`: 0 MAP,
        1 OUTER with a channel-free y, 2 INNER.  For a float64 table `scale` is the ctypes array of
        its coefficient classes (`e3j_amd_tp_params.coef_classes`)."""
        kind = int(kind)
        key = (num_x, num_y, num_out, channels, kind, layout, config().jit)
        hit = self._signature.get(key)
        if hit is None:
            scale = ctypes.c_float(1.0)
            classes = (ctypes.c_double * _lib.F64_CLASSES)()
            f64 = self.val_np_dtype == np.float64
            sig = -1

            def find():
                if f64:
                    return int(_lib.load().e3j_amd_tp_find_signature_f64(
                        self.packed.ctypes.data, self.idx_bytes, self.num_coef, num_x, num_y, num_out, channels,
                        kind, layout.value, classes))
                code = _lib.F16 if self.val_np_dtype == np.float16 else _lib.F32
                return int(_lib.load().e3j_amd_tp_find_signature(
                    self.packed.ctypes.data, self.idx_bytes, code, self.num_coef, num_x, num_y, num_out,
                    channels, kind, layout.value, ctypes.byref(scale)))

            if self.num_coef > 0:
                sig = find()
                if sig < 0 and config().jit:
                    # not built in: generate and compile the kernels of this table, then look again
                    from . import jit as _jit
                    c = Coef.unpack(self.packed, self.val_np_dtype)
                    trailing = layout == Layout.TRAILING_CHANNELS
                    if (channels % 64 == 0 or channels in (16, 32) or not trailing) and _jit.register_tp(
                            c.val, c.idx.astype(np.int64), (num_out, num_x, num_y), channels if trailing else 0):
                        sig = find()
            hit = self._signature[key] = (sig, classes if f64 else float(scale.value))
        return hit

    @classmethod
    def get(cls, coef, val_np_dtype) -> "_Table":
        if isinstance(coef, torch.Tensor):
            raise TypeError("`coef` must be concrete: it is read on the host.")
        packed = np.asarray(coef)
        if packed.dtype not in (np.dtype(np.uint8), np.dtype(np.int32)):
            raise TypeError(f"unsupported coefficient index dtype {packed.dtype}")
        key = (packed.dtype.str, packed.shape, packed.tobytes(), np.dtype(val_np_dtype).str)
        table = cls._cache.get(key)
        if table is None:
            if len(cls._cache) > 256:
                cls._cache.clear()
            table = cls._cache[key] = cls(packed, val_np_dtype)
        return table

    def device(self, device: torch.device, backward: bool = False) -> torch.Tensor:
        key = (device, backward)
        t = self._device.get(key)
        if t is None:
            host = self.packed_bwd if backward else self.packed
            t = torch.from_numpy(host.view(np.uint8).reshape(-1).copy()).to(device)
            self._device[key] = t
        return t


@dataclasses.dataclass
class _Meta:
    """Everything static about one call."""

    table: _Table
    num_out: int
    mode: MixingMode
    layout: Layout
    has_cx: bool
    has_cy: bool

    def dims(self, t: torch.Tensor, has_c: bool):
        """`(dim, channels)` of an operand."""
        if not has_c:
            return int(t.shape[1]), 1
        if self.layout == Layout.TRAILING_CHANNELS:
            return int(t.shape[1]), int(t.shape[2])
        return int(t.shape[2]), int(t.shape[1])

    def out_shape(self, rows: int, cx: int, cy: int):
        if self.mode == MixingMode.INNER:
            chans = []
        elif self.mode == MixingMode.MAP:
            chans = [cx]
        else:
            chans = ([cx] if self.has_cx else []) + ([cy] if self.has_cy else [])
        if self.layout == Layout.TRAILING_CHANNELS:
            return (rows, self.num_out, *chans)
        return (rows, *chans, self.num_out)


def _stream(device) -> int:
    return int(torch.cuda.current_stream(device).cuda_stream)


def _params(meta: _Meta, x: torch.Tensor, y: torch.Tensor, backward: bool, dz=None) -> _lib.TpParams:
    num_x, cx = meta.dims(x, meta.has_cx)
    num_y, cy = meta.dims(y, meta.has_cy)
    # unrolled kernels: float32, MAP, OUTER with a channel-free y, or INNER; the leading-layout ones
    # need 64 columns in all and 16-byte aligned operands
    sig, scale = -1, 1.0
    # (float16 / float64: trailing layout, whole waves of channels; the look-up knows)
    usable = (meta.layout == Layout.TRAILING_CHANNELS or
              (x.dtype == torch.float32 and int(x.shape[0]) * cx >= 64 and
               all(t.data_ptr() % 16 == 0 for t in (x, y, dz) if t is not None)))
    if usable and meta.mode == MixingMode.MAP:
        sig, scale = meta.table.signature(num_x, num_y, meta.num_out, cx, 0, meta.layout)
    elif usable and meta.mode == MixingMode.OUTER and cy == 1 and cx > 1:
        sig, scale = meta.table.signature(num_x, num_y, meta.num_out, cx, 1, meta.layout)
    elif usable and meta.mode == MixingMode.INNER:
        sig, scale = meta.table.signature(num_x, num_y, meta.num_out, cx, 2, meta.layout)
    classes = None
    if not isinstance(scale, float):   # float64: the coefficient classes take the place of the factor
        classes, scale = scale, 1.0
    p = _lib.TpParams(
        signature=sig, coef_scale=scale,
        num_rows=int(x.shape[0]), num_coef=meta.table.num_coef, num_x=num_x, num_y=num_y,
        num_out=meta.num_out, channels_x=cx, channels_y=cy, mode=meta.mode.value, layout=meta.layout.value,
        val_dtype=_VAL_DTYPES[x.dtype][0], coef_idx_bytes=meta.table.idx_bytes,
        coef_sorted=1 if (backward or meta.table.sorted) else 0, debug=int(config().debug_level))
    if classes is not None and sig >= 0:
        p.coef_classes = ctypes.cast(classes, ctypes.c_void_p).value   # (kept alive by the table's cache)
    return p


def _raw_forward(meta: _Meta, x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    x, y = x.contiguous(), y.contiguous()
    p = _params(meta, x, y, backward=False)
    z = torch.empty(meta.out_shape(int(x.shape[0]), p.channels_x, p.channels_y), dtype=x.dtype, device=x.device)
    lib = _lib.load()
    with torch.cuda.device(x.device):
        _lib.check(lib.e3j_amd_tensor_product_fwd(
            ctypes.byref(p), meta.table.device(x.device).data_ptr(), x.data_ptr(), y.data_ptr(), z.data_ptr(),
            _stream(x.device)))
    return z


def _raw_backward(meta: _Meta, x: torch.Tensor, y: torch.Tensor, dz: torch.Tensor):
    x, y, dz = x.contiguous(), y.contiguous(), dz.contiguous()
    p = _params(meta, x, y, backward=True, dz=dz)
    if tuple(dz.shape) != meta.out_shape(int(x.shape[0]), p.channels_x, p.channels_y):
        raise ValueError(f"cotangent shape {tuple(dz.shape)} does not match the output of the product")
    dx, dy = torch.empty_like(x), torch.empty_like(y)
    lib = _lib.load()
    with torch.cuda.device(x.device):
        _lib.check(lib.e3j_amd_tensor_product_bwd(
            ctypes.byref(p), meta.table.device(x.device, backward=True).data_ptr(), x.data_ptr(), y.data_ptr(),
            dz.data_ptr(), dx.data_ptr(), dy.data_ptr(), _stream(x.device)))
    return dx, dy


def _sum(*terms):
    terms = [t for t in terms if t is not None]
    if not terms:
        return None
    total = terms[0]
    for t in terms[1:]:
        total = total + t
    return total


def _lead(t: torch.Tensor, dim, batch: int) -> torch.Tensor:
    """Batch axis first; an operand that is not batched is broadcast over the batch."""
    if dim is None:
        return t.unsqueeze(0).expand((batch,) + tuple(t.shape))
    return t.movedim(dim, 0)


def _fold(t: torch.Tensor) -> torch.Tensor:
    return t.reshape((t.shape[0] * t.shape[1],) + tuple(t.shape[2:]))


def _unfold(t: torch.Tensor, batch: int) -> torch.Tensor:
    return t.reshape((batch, t.shape[0] // batch) + tuple(t.shape[1:]))


class _TensorProduct(torch.autograd.Function):
    """Differentiable to any reverse-mode order; composes with `torch.func` transforms (the
    batching rule folds the batch into the rows, `src/e3j/ops/tensor_product.py:251-268`)."""

    @staticmethod
    def forward(x, y, meta):
        return _raw_forward(meta, x, y)

    @staticmethod
    def setup_context(ctx, inputs, output):
        x, y, meta = inputs
        ctx.meta = meta
        ctx.save_for_backward(x, y)

    @staticmethod
    def backward(ctx, dz):
        x, y = ctx.saved_tensors
        meta = ctx.meta
        if meta.mode == MixingMode.OUTER and meta.has_cx and meta.has_cy:
            raise NotImplementedError("Cannot backpropagate through 'OUTER' tensor product "
                                      "with channel axes on both inputs.")
        dx, dy = _TensorProductBwd.apply(x, y, dz, meta)
        return dx, dy, None

    @staticmethod
    def vmap(info, in_dims, x, y, meta):
        batch = info.batch_size
        out = _TensorProduct.apply(_fold(_lead(x, in_dims[0], batch)), _fold(_lead(y, in_dims[1], batch)), meta)
        return _unfold(out, batch), 0


class _TensorProductBwd(torch.autograd.Function):
    @staticmethod
    def forward(x, y, dz, meta):
        return _raw_backward(meta, x, y, dz)

    @staticmethod
    def setup_context(ctx, inputs, output):
        x, y, dz, meta = inputs
        ctx.meta = meta
        ctx.save_for_backward(x, y, dz)

    @staticmethod
    def backward(ctx, ddx, ddy):
        # (dx, dy) is bilinear in (dz, y) and (dz, x): cotangents of x, y through one backward
        # product in (ddx, ddy), of dz through two forward products
        # (src/e3j/ops/tensor_product.py:576-591)
        x, y, dz = ctx.saved_tensors
        meta = ctx.meta
        ddx = torch.zeros_like(x) if ddx is None else ddx
        ddy = torch.zeros_like(y) if ddy is None else ddy
        gx = gy = gdz = None
        if ctx.needs_input_grad[0] or ctx.needs_input_grad[1]:
            gx, gy = _TensorProductBwd.apply(ddx, ddy, dz, meta)
        if ctx.needs_input_grad[2]:
            gdz = _sum(_TensorProduct.apply(x, ddy, meta), _TensorProduct.apply(ddx, y, meta))
        return gx, gy, gdz, None

    @staticmethod
    def vmap(info, in_dims, x, y, dz, meta):
        batch = info.batch_size
        dx, dy = _TensorProductBwd.apply(_fold(_lead(x, in_dims[0], batch)), _fold(_lead(y, in_dims[1], batch)),
                                         _fold(_lead(dz, in_dims[2], batch)), meta)
        return (_unfold(dx, batch), _unfold(dy, batch)), (0, 0)


def _check(x: torch.Tensor, y: torch.Tensor):
    for name, t in (("x", x), ("y", y)):
        if not isinstance(t, torch.Tensor):
            raise TypeError(f"`{name}` must be a torch tensor")
        if t.ndim not in (2, 3):
            raise ValueError(f"Expected {name} rank 2 or 3, got {tuple(t.shape)}")
    if x.dtype != y.dtype:
        raise TypeError(f"x and y must share a dtype, got {x.dtype} and {y.dtype}")
    if x.dtype not in _VAL_DTYPES:
        raise NotImplementedError(f"the HIP tensor product runs in float16, float32 or float64, got {x.dtype}")
    if not x.is_cuda or x.device != y.device:
        raise ValueError("x and y must live on the same GPU: the tensor product has no CPU path")
    if x.shape[0] != y.shape[0]:
        raise ValueError(f"x and y must have as many rows, got {x.shape[0]} and {y.shape[0]}")


def _make_meta(coef, x, y, params: TensorProductParams) -> _Meta:
    layout = Layout.parse(params.layout)
    mode = MixingMode.parse(params.mode)
    has_cx, has_cy = x.ndim > 2, y.ndim > 2
    meta = _Meta(table=_Table.get(coef, _VAL_DTYPES[x.dtype][1]), num_out=int(params.num_out), mode=mode,
                 layout=layout, has_cx=has_cx, has_cy=has_cy)
    _, cx = meta.dims(x, has_cx)
    _, cy = meta.dims(y, has_cy)
    if mode != MixingMode.OUTER:
        if not (has_cx and has_cy):
            raise ValueError(f"{mode.name} mode requires channel dims on both x and y")
        if cx != cy:
            raise ValueError("MAP and INNER modes require same number of LHS and RHS channels. "
                             f"Got ({cx, cy}).")
    return meta


def tensor_product(coef, x: torch.Tensor, y: torch.Tensor, params: TensorProductParams) -> torch.Tensor:
    """Contraction of the sparse 3-D coefficient table with `x` and `y`, row by row.

    Args:
        coef: packed `Coef` table `(val, i, j, k)` (host numpy array, opaque index dtype).
        x: `(rows, num_x, channels_x)` or `(rows, num_x)` [leading layout: `(rows, channels_x, num_x)`].
        y: `(rows, num_y, channels_y)` or `(rows, num_y)` [leading: `(rows, channels_y, num_y)`].
        params: `TensorProductParams(num_out, mode, layout)`.

    Returns `(rows, num_out, *channels_z)` [leading: `(rows, *channels_z, num_out)`] with
    `channels_z` = the channel axes of x then y (OUTER), none (INNER), the shared one (MAP).
    """
    _check(x, y)
    meta = _make_meta(coef, x, y, params)
    return _TensorProduct.apply(x, y, meta)


def tensor_product_bwd(coef, x: torch.Tensor, y: torch.Tensor, ct_z: torch.Tensor, params: TensorProductParams):
    """Cotangents `(ct_x, ct_y)` of `tensor_product` for the output cotangent `ct_z`; the
    cotangent is read by one call for both results."""
    _check(x, y)
    meta = _make_meta(coef, x, y, params)
    if meta.mode == MixingMode.OUTER and meta.has_cx and meta.has_cy:
        raise NotImplementedError("The `tensor_product_bwd` handler requires either LHS or RHS to have one "
                                  f"channel for now, got ({meta.dims(x, True)[1], meta.dims(y, True)[1]}).")
    return _TensorProductBwd.apply(x, y, ct_z, meta)


def tensor_product_batched(coef, x: torch.Tensor, y: torch.Tensor, params: TensorProductParams,
                            x_batched: bool = True, y_batched: bool = True) -> torch.Tensor:
    """Batch on a leading axis, folded into the rows: the counterpart of the reference's batching
    rule (`src/e3j/ops/tensor_product.py:251-268`).  An operand that is not batched is broadcast
    over the batch (the asymmetric pattern a Jacobian produces)."""
    if not (x_batched or y_batched):
        return tensor_product(coef, x, y, params)
    batch = x.shape[0] if x_batched else y.shape[0]
    if not x_batched:
        x = x.unsqueeze(0).expand((batch,) + tuple(x.shape))
    if not y_batched:
        y = y.unsqueeze(0).expand((batch,) + tuple(y.shape))
    if x.shape[0] != y.shape[0] or x.shape[1] != y.shape[1]:
        raise ValueError(f"batched operands disagree: x {tuple(x.shape)}, y {tuple(y.shape)}")
    rows = x.shape[1]
    out = tensor_product(coef, x.reshape((batch * rows,) + tuple(x.shape[2:])),
                         y.reshape((batch * rows,) + tuple(y.shape[2:])), params)
    return out.reshape((batch, rows) + tuple(out.shape[1:]))


tensor_product.Params = TensorProductParams
