"""View / layout / indexing ops.

Mirrors nabla/ops/view/shape.py (broadcast_to 56-158, reshape 161-390,
slice_update 393-583, slice_tensor 586-818, concatenate / stack 821-980 and
1095-1110, pad 1313-1398), nabla/ops/view/axes.py (unsqueeze, squeeze,
swap_axes, moveaxis, permute 43-868) and nabla/ops/view/indexing.py (gather
27-447).  None of the pure views runs a kernel: the lowering folds them into
the strides of their consumers.
"""
from __future__ import annotations

from typing import Any, Sequence

from ..backend import ir
from ..core.dtype import DType
from ..core.tensor import Tensor
from .base import AxisOp, Operation, ShapeOp, ensure_tensor


def _norm_axis(axis: int, rank: int, extra: int = 0) -> int:
    n = rank + extra
    a = axis + n if axis < 0 else axis
    if not 0 <= a < max(n, 1):
        raise ValueError(f"axis {axis} out of range for rank {rank}")
    return a


# ---------------------------------------------------------------- broadcast_to
class BroadcastToOp(ShapeOp):
    @property
    def name(self) -> str:
        return "broadcast_to"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x = args[0]
        return [tuple(kwargs["shape"])], [x.dtype], [x.device]

    def kernel(self, args, kwargs):
        return [ir.broadcast_to(args[0], kwargs["shape"])]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        # sum over the added leading dims, then over the dims that were 1 (shape.py:131-152)
        from .reduction import reduce_sum
        x, g = primals[0], cotangents[0]
        diff = len(g.shape) - len(x.shape)
        if diff > 0:
            g = reduce_sum(g, axis=list(range(diff)))
        axes = [i for i, (c, a) in enumerate(zip(g.shape, x.shape)) if a == 1 and c > 1]
        if axes:
            g = reduce_sum(g, axis=axes, keepdims=True)
        return [g]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        return [broadcast_to(tangents[0], kwargs["shape"])]


_broadcast_to_op = BroadcastToOp()


def broadcast_to(x: Tensor, shape) -> Tensor:
    shape = tuple(int(d) for d in shape)
    x = ensure_tensor(x)
    if tuple(x.shape) == shape:
        return x
    if len(shape) < len(x.shape):
        raise ValueError(f"Cannot broadcast shape {x.shape} to {shape}")
    for a, b in zip(x.shape[::-1], shape[::-1]):
        if a != b and a != 1:
            raise ValueError(f"Cannot broadcast shape {x.shape} to {shape}")
    return _broadcast_to_op([x], {"shape": shape})[0]


# ---------------------------------------------------------------------- reshape
class ReshapeOp(ShapeOp):
    @property
    def name(self) -> str:
        return "reshape"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x = args[0]
        return [tuple(kwargs["shape"])], [x.dtype], [x.device]

    def kernel(self, args, kwargs):
        return [ir.reshape(args[0], kwargs["shape"])]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        return [reshape(cotangents[0], primals[0].shape)]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        return [reshape(tangents[0], kwargs["shape"])]


_reshape_op = ReshapeOp()


def reshape(x: Tensor, shape) -> Tensor:
    shape = tuple(int(d) for d in shape)
    n = 1
    for d in x.shape:
        n *= d
    if -1 in shape:
        known = 1
        for d in shape:
            if d != -1:
                known *= d
        shape = tuple(n // max(known, 1) if d == -1 else d for d in shape)
    m = 1
    for d in shape:
        m *= d
    if m != n:
        raise ValueError(f"Cannot reshape tensor of shape {x.shape} to {shape}")
    if shape == tuple(x.shape):
        return x
    return _reshape_op([x], {"shape": shape})[0]


def flatten(x: Tensor, start_dim: int = 0, end_dim: int = -1) -> Tensor:
    r = len(x.shape)
    if r == 0:
        return reshape(x, (1,))
    s = _norm_axis(start_dim, r)
    e = _norm_axis(end_dim, r)
    mid = 1
    for d in x.shape[s:e + 1]:
        mid *= d
    return reshape(x, tuple(x.shape[:s]) + (mid,) + tuple(x.shape[e + 1:]))


def unsqueeze(x: Tensor, axis: int = 0) -> Tensor:
    a = _norm_axis(axis, len(x.shape), extra=1)
    return reshape(x, tuple(x.shape[:a]) + (1,) + tuple(x.shape[a:]))


def squeeze(x: Tensor, axis: Any = 0) -> Tensor:
    r = len(x.shape)
    if axis is None:
        return reshape(x, tuple(d for d in x.shape if d != 1))
    axes = [axis] if isinstance(axis, int) else list(axis)
    axes = {_norm_axis(a, r) for a in axes}
    for a in axes:
        if x.shape[a] != 1:
            raise ValueError(f"cannot squeeze axis {a} of shape {x.shape}")
    return reshape(x, tuple(d for i, d in enumerate(x.shape) if i not in axes))


# ---------------------------------------------------------------------- permute
class PermuteOp(ShapeOp):
    @property
    def name(self) -> str:
        return "permute"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x = args[0]
        order = kwargs["order"]
        return [tuple(x.shape[p] for p in order)], [x.dtype], [x.device]

    def kernel(self, args, kwargs):
        return [ir.permute(args[0], kwargs["order"])]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        order = kwargs["order"]
        inv = [0] * len(order)
        for i, p in enumerate(order):
            inv[p] = i
        return [permute(cotangents[0], tuple(inv))]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        return [permute(tangents[0], kwargs["order"])]


_permute_op = PermuteOp()


def permute(x: Tensor, order) -> Tensor:
    r = len(x.shape)
    order = tuple(_norm_axis(int(p), r) for p in order)
    if sorted(order) != list(range(r)):
        raise ValueError(f"permute: {order} is not a permutation of {r} axes")
    if order == tuple(range(r)):
        return x
    return _permute_op([x], {"order": order})[0]


def swap_axes(x: Tensor, axis1: int, axis2: int) -> Tensor:
    r = len(x.shape)
    a, b = _norm_axis(axis1, r), _norm_axis(axis2, r)
    order = list(range(r))
    order[a], order[b] = order[b], order[a]
    return permute(x, order)


transpose = swap_axes


def moveaxis(x: Tensor, source: int, destination: int) -> Tensor:
    r = len(x.shape)
    s, d = _norm_axis(source, r), _norm_axis(destination, r)
    order = [i for i in range(r) if i != s]
    order.insert(d, s)
    return permute(x, order)


# ----------------------------------------------------------------- slice_tensor
class SliceTensorOp(ShapeOp):
    @property
    def name(self) -> str:
        return "slice_tensor"

    @staticmethod
    def _norm(x_shape, start, size):
        start = [int(s) + d if int(s) < 0 else int(s) for s, d in zip(start, x_shape)]
        size = [int(s) for s in size]
        for s, n, d in zip(start, size, x_shape):
            if s < 0 or n < 0 or s + n > d:
                raise ValueError(f"slice [{s}:{s + n}] out of bounds for extent {d}")
        return tuple(start), tuple(size)

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x = args[0]
        _, size = self._norm(x.shape, kwargs["start"], kwargs["size"])
        return [size], [x.dtype], [x.device]

    def kernel(self, args, kwargs):
        x = args[0]
        start, size = self._norm(x.shape, kwargs["start"], kwargs["size"])
        return [ir.slice(x, start, tuple(a + n for a, n in zip(start, size)))]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        x = primals[0]
        start, size = self._norm(x.shape, kwargs["start"], kwargs["size"])
        paddings = [(a, d - a - n) for a, n, d in zip(start, size, x.shape)]
        return [pad(cotangents[0], paddings)]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        return [slice_tensor(tangents[0], kwargs["start"], kwargs["size"])]


_slice_tensor_op = SliceTensorOp()


def slice_tensor(x: Tensor, start, size) -> Tensor:
    return _slice_tensor_op([x], {"start": tuple(start), "size": tuple(size)})[0]


# ----------------------------------------------------------------- slice_update
class SliceUpdateOp(Operation):
    @property
    def name(self) -> str:
        return "slice_update"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x = args[0]
        return [tuple(x.shape)], [x.dtype], [x.device]

    def kernel(self, args, kwargs):
        x, u = args
        start, size = SliceTensorOp._norm(x.shape, kwargs["start"], kwargs["size"])
        if tuple(u.shape) != size:
            raise ValueError(f"slice_update: update shape {u.shape} != size {size}")
        return [ir.slice_update(x, ir.cast(u, x.dtype), start)]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        from .creation import zeros
        x, u = primals
        g = cotangents[0]
        gx = slice_update(g, zeros(u.shape, dtype=g.dtype, device=g.device), kwargs["start"],
                          kwargs["size"])
        gu = slice_tensor(g, kwargs["start"], kwargs["size"])
        return [gx, gu]


_slice_update_op = SliceUpdateOp()


def slice_update(x: Tensor, update: Tensor, start, size) -> Tensor:
    x = ensure_tensor(x)
    update = ensure_tensor(update, x)
    return _slice_update_op([x, update], {"start": tuple(start), "size": tuple(size)})[0]


# -------------------------------------------------------------------------- pad
class PadOp(Operation):
    @property
    def name(self) -> str:
        return "pad"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x = args[0]
        shape = tuple(d + int(a) + int(b) for d, (a, b) in zip(x.shape, kwargs["paddings"]))
        return [shape], [x.dtype], [x.device]

    def kernel(self, args, kwargs):
        pads = kwargs["paddings"]
        if kwargs.get("mode", "constant") != "constant":
            raise ValueError("pad: only mode='constant' is supported")
        return [ir.pad(args[0], [int(a) for a, _ in pads], [int(b) for _, b in pads],
                       kwargs.get("value", 0.0))]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        x = primals[0]
        start = [int(a) for a, _ in kwargs["paddings"]]
        return [slice_tensor(cotangents[0], start, x.shape)]


_pad_op = PadOp()


def pad(x: Tensor, paddings=None, mode: str = "constant", value: float = 0.0, **kwargs) -> Tensor:
    paddings = paddings if paddings is not None else kwargs.get("pad_width")
    if paddings is None:
        raise ValueError("pad() requires paddings or pad_width")
    paddings = tuple((int(a), int(b)) for a, b in paddings)
    if len(paddings) != len(x.shape):
        raise ValueError(f"pad: {len(paddings)} padding pairs for rank {len(x.shape)}")
    if all(a == 0 and b == 0 for a, b in paddings):
        return x
    return _pad_op([x], {"paddings": paddings, "mode": mode, "value": float(value)})[0]


# ------------------------------------------------------------------ concatenate
class ConcatenateOp(AxisOp):
    @property
    def name(self) -> str:
        return "concatenate"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        axis = self._norm_axis(kwargs.get("axis", 0), len(args[0].shape))
        total = sum(a.shape[axis] for a in args)
        base = args[0].shape
        return [tuple(base[:axis]) + (total,) + tuple(base[axis + 1:])], [args[0].dtype], [args[0].device]

    def kernel(self, args, kwargs):
        axis = self._norm_axis(kwargs.get("axis", 0), args[0].rank)
        return [ir.concat(args, axis)]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        axis = self._norm_axis(kwargs.get("axis", 0), len(primals[0].shape))
        g = cotangents[0]
        outs = []
        pos = 0
        for p in primals:
            start = [0] * len(g.shape)
            start[axis] = pos
            outs.append(slice_tensor(g, start, p.shape))
            pos += p.shape[axis]
        return outs


_concatenate_op = ConcatenateOp()


def concatenate(tensors: Sequence[Tensor], axis: int = 0) -> Tensor:
    tensors = list(tensors)
    if not tensors:
        raise ValueError("concatenate: needs at least one tensor")
    if len(tensors) == 1:
        return tensors[0]
    return _concatenate_op(tensors, {"axis": axis})[0]


def stack(tensors, axis: int = 0) -> Tensor:
    return concatenate([unsqueeze(t, axis=axis) for t in tensors], axis=axis)


# ----------------------------------------------------------------------- gather
class GatherOp(AxisOp):
    """``take`` along ``axis`` (indexing.py:100-171)."""

    @property
    def name(self) -> str:
        return "gather"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x, idx = args
        axis = self._norm_axis(kwargs.get("axis", 0), len(x.shape))
        shape = tuple(x.shape[:axis]) + tuple(idx.shape) + tuple(x.shape[axis + 1:])
        return [shape], [x.dtype], [x.device]

    def kernel(self, args, kwargs):
        x, idx = args
        if not idx.dtype.is_integral():
            raise TypeError(f"gather: indices must be integers, got {idx.dtype}")
        return [ir.gather(x, idx, self._norm_axis(kwargs.get("axis", 0), x.rank))]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        # the reference scatters the cotangent into zeros (indexing.py:173-182); the
        # node stays lazy and is dropped as dead code unless the table gradient is
        # actually requested
        from .creation import zeros_like
        x, idx = primals
        return [_scatter_op([zeros_like(x), idx, cotangents[0]], dict(kwargs))[0], None]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        # linear in the table: the same rows of the tangent (indexing.py:183-190)
        return [_gather_op([tangents[0], primals[1]], dict(kwargs))[0]]


class ScatterOp(AxisOp):
    """``x`` with the rows selected by ``indices`` along ``axis`` replaced by ``updates``
    (indexing.py:185-447); the VJP of gather scatters the cotangent into zeros with it
    (173-182).  A row named more than once takes the LAST update (numpy's assignment rule);
    the reference leaves that order to its backend."""

    @property
    def name(self) -> str:
        return "scatter"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x = args[0]
        return [tuple(x.shape)], [x.dtype], [x.device]

    def kernel(self, args, kwargs):
        x, idx, upd = args
        if not idx.dtype.is_integral():
            raise TypeError(f"scatter: indices must be integers, got {idx.dtype}")
        if upd.dtype is not x.dtype:
            upd = ir.cast(upd, x.dtype)
        return [ir.scatter(x, idx, upd, self._norm_axis(kwargs.get("axis", 0), x.rank))]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        # the replaced rows of x receive nothing; every update receives the row it was written
        # to (for a row named twice that is exact for the update that won)
        from .creation import zeros_like
        x, idx, upd = primals
        g = cotangents[0]
        gx = _scatter_op([g, idx, zeros_like(upd)], dict(kwargs))[0]
        return [gx, None, _gather_op([g, idx], dict(kwargs))[0]]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        return [_scatter_op([tangents[0], primals[1], tangents[2]], dict(kwargs))[0]]


_gather_op = GatherOp()
_scatter_op = ScatterOp()


def gather(x: Tensor, indices: Tensor | None = None, axis: int = 0) -> Tensor:
    if indices is None:
        raise ValueError("gather: indices are required")
    indices = ensure_tensor(indices)
    return _gather_op([x, indices], {"axis": axis})[0]


take = gather


def scatter(x: Tensor, indices: Tensor, updates: Tensor, axis: int = 0) -> Tensor:
    """Out-of-place ``out = x.copy(); out[indices] = updates`` along ``axis``
    (indexing.py:483-504)."""
    x, indices, updates = ensure_tensor(x), ensure_tensor(indices), ensure_tensor(updates)
    return _scatter_op([x, indices, updates], {"axis": axis})[0]


# ------------------------------------------------------------------ __getitem__
def getitem(x: Tensor, key) -> Tensor:
    """Basic indexing with ints, slices, None and Ellipsis (api.py:1079-1297)."""
    if not isinstance(key, tuple):
        key = (key,)
    n_specified = sum(1 for k in key if k is not None and k is not Ellipsis)
    if n_specified > len(x.shape):
        raise IndexError(f"too many indices for tensor of rank {len(x.shape)}")
    if Ellipsis in key:
        i = key.index(Ellipsis)
        key = key[:i] + (slice(None),) * (len(x.shape) - n_specified) + key[i + 1:]
    starts, sizes, steps = [], [], []
    squeeze_axes, new_axes = [], []
    dim = 0
    out_pos = 0
    for k in key:
        if k is None:
            new_axes.append(out_pos)
            out_pos += 1
            continue
        d = x.shape[dim]
        if isinstance(k, int):
            kk = k + d if k < 0 else k
            if not 0 <= kk < d:
                raise IndexError(f"index {k} out of range for axis {dim} with size {d}")
            starts.append(kk); sizes.append(1); steps.append(1)
            squeeze_axes.append(dim)
        elif isinstance(k, slice):
            a, b, s = k.indices(d)
            if s <= 0:
                raise IndexError("negative slice steps are not supported")
            n = max(0, (b - a + s - 1) // s)
            starts.append(a); sizes.append(n); steps.append(s)
            out_pos += 1
        elif isinstance(k, Tensor):
            if len(key) != 1:
                raise IndexError("tensor indices cannot be mixed with other indices")
            return gather(x, k, axis=0)
        else:
            raise IndexError(f"unsupported index {k!r}")
        dim += 1
    while dim < len(x.shape):
        starts.append(0); sizes.append(x.shape[dim]); steps.append(1)
        dim += 1
    if any(s != 1 for s in steps):
        raise IndexError("strided slices are not supported; use slice_tensor and reshape")
    y = slice_tensor(x, starts, sizes)
    if squeeze_axes:
        y = squeeze(y, tuple(squeeze_axes))
    for a in new_axes:
        y = unsqueeze(y, a)
    return y
